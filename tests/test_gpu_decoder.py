"""The compressed cache inside a decoder loop (packkv_amd/decoder.py): the fused decode step against the
reference's decompress-then-attend on the same cache contents, across compression cuts."""
import pytest
import torch

from packkv_amd.cache import PackKVCacheConfig
from packkv_amd.decoder import DecoderShape, ShapedDecoder

pytestmark = pytest.mark.gpu


def _say(*a):
    print(*a, flush=True)


@pytest.mark.parametrize("dtype,head_norm", [(torch.float16, False), (torch.bfloat16, True)])
def test_fused_decode_follows_decompress_then_attend(cuda, dtype, head_norm):
    """Two decoders with the same weights decode the same forced token ids, one through cache.attend, one through
    materialize + eager attention.  Layer 0 sees identical cache contents in both, so its attention output must meet
    the contract of the attention kernel (with the widened absolute term of short, peaky contexts); deeper layers
    quantise slightly different K / V, so the logits are compared in norm.  130 steps cross two cuts."""
    shape = DecoderShape(layers=3, hidden=256, q_heads=4, kv_heads=2, mlp=512, vocab=640, head_norm=head_norm)
    model = ShapedDecoder(shape, dtype=dtype, device=cuda, seed=5)
    B, prompt, steps = 2, 330, 130
    g = torch.Generator().manual_seed(6)
    ids = torch.randint(0, shape.vocab, (B, prompt), generator=g).to(cuda)
    forced = torch.randint(0, shape.vocab, (B, steps), generator=g).to(cuda)
    c_f = model.new_cache(B, 1024, PackKVCacheConfig())
    c_d = model.new_cache(B, 1024, PackKVCacheConfig())
    lf, ld = model.prefill(ids, c_f), model.prefill(ids, c_d)
    assert torch.equal(lf, ld)
    assert c_f.get_seq_length() == prompt and c_f.layers[0].k.tokens == 128      # 192 cut, 64 of them pending
    abs_tol = {torch.float16: 8e-3, torch.bfloat16: 6e-2}[dtype]
    worst_a, worst_l = 0.0, 0.0
    for t in range(steps):
        tf, td = [], []
        lf = model.forward(forced[:, t:t + 1], c_f, attention="fused", taps=tf)
        ld = model.forward(forced[:, t:t + 1], c_d, attention="dense", taps=td)
        a_f, a_d = tf[0].float(), td[0].float()
        err = ((a_f - a_d).abs() - 1e-3 * a_d.abs()).max().item()
        worst_a = max(worst_a, err)
        assert err <= abs_tol, ("layer-0 attention", t, err)
        rel = ((lf - ld).norm() / ld.norm()).item()
        worst_l = max(worst_l, rel)
        assert rel < 0.05, ("logits", t, rel)
    assert c_f.get_seq_length() == prompt + steps
    assert c_f.layers[0].k.tokens == c_d.layers[0].k.tokens == 256
    _say("decoder", dtype, "layer-0 attention err", worst_a, "logit rel err", worst_l,
         "cache bytes", c_f.cache_bytes(), "fp16 bytes", 2 * shape.layers * B * shape.kv_heads * (prompt + steps) * 128 * 2)


def test_greedy_runs_and_accounts(cuda):
    shape = DecoderShape(layers=2, hidden=256, q_heads=8, kv_heads=2, mlp=512, vocab=512)
    model = ShapedDecoder(shape, dtype=torch.bfloat16, device=cuda, seed=7)
    ids = torch.randint(0, shape.vocab, (3, 256), generator=torch.Generator().manual_seed(8)).to(cuda)
    cache = model.new_cache(3, 512)
    out = model.greedy(ids, cache, 40)
    assert out.shape == (3, 40) and int(out.min()) >= 0 and int(out.max()) < shape.vocab
    assert cache.get_seq_length() == 256 + 40          # every generated token but the last one's successor is cached
