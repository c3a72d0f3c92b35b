"""The compressed cache inside a decoder loop (packkv_amd/decoder.py): the fused decode step against the
reference's decompress-then-attend path, restated on the CPU, on the cache's own contents, across compression cuts."""
import pytest
import torch

from oracle import quant as oq
from packkv_amd import ops
from packkv_amd.cache import PackKVCacheConfig
from packkv_amd.decoder import DecoderShape, ShapedDecoder
from attn_bounds import check_fast, check_reference_mode, say as _say

pytestmark = pytest.mark.gpu


def _exact_view(cache, layer):
    """(K, V) [B, H, T, 128] in fp64 as the fused kernel attends them: (code + zero) * scale WITHOUT the rounding to
    16 bits for the tokens in the streams (codes from the unpack kernel, which other tests hold bit-exact; arithmetic
    on the CPU), the 16-bit window as it is."""
    L = cache.layers[layer]
    out = []
    for side, win in ((L.k, L.k_win), (L.v, L.v_win)):
        parts = []
        if side.tokens:
            hidden = side.B * side.H * 128
            codes = torch.empty(side.tokens, hidden, dtype=torch.uint8, device=win.device)
            (ops.k_decode if side.is_k else ops.v_decode)(side.stream, side.info[:side.tokens // 128 * side.blocks_per_tile],
                                                          codes, bits=side.bits)
            c = codes.cpu().double().view(side.tokens, side.B, side.H, 128).permute(1, 2, 0, 3)
            sc = side.scale[:, :side.tokens].cpu().double()[:, None, :, None]
            ze = side.zero[:, :side.tokens].cpu().double()[:, None, :, None]
            parts.append((c + ze) * sc)
        if L.win_len:
            parts.append(win[:, :, :L.win_len].cpu().double())
        out.append(torch.cat(parts, dim=2))
    return out[0], out[1]


def _layer0_parity(cache, q, a, dtype, label):
    """Layer 0's decode-step attention `a` for the rotated query `q` (both [B, Hq, 1, 128]): the reference path is
    the oracle's fp32-accumulating attention on the dense view the cache returns (the tensors the reference's
    update hands to eager attention; tests/test_gpu_cache.py holds that view bit-identical to the restated cache)."""
    gk, gv = cache.materialize(0)
    ref = oq.attention_f32(q.cpu(), gk.cpu(), gv.cpu())
    ek, ev = _exact_view(cache, 0)
    exact = oq.attention_f64_np(q.cpu(), ek, ev)
    chk = cache.attend(q, 0, variant=1, ref_rounding=True, out_f32=True)
    check_reference_mode(chk, ref, label)
    check_fast(a, ref, exact, dtype, label=label)


@pytest.mark.parametrize("dtype,head_norm", [(torch.float16, False), (torch.bfloat16, True)])
def test_fused_decode_follows_decompress_then_attend(cuda, dtype, head_norm):
    """Two decoders with the same weights decode the same forced token ids, one through cache.attend, one through
    materialize + eager attention.  Layer 0's fused attention output is checked against the oracle on the cache's
    contents at every step; deeper layers quantise slightly different K / V in the two decoders, so the logits are
    compared in norm.  130 steps cross two cuts."""
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
    worst_l = 0.0
    for t in range(steps):
        tf = []
        lf = model.forward(forced[:, t:t + 1], c_f, attention="fused", taps=tf)
        ld = model.forward(forced[:, t:t + 1], c_d, attention="dense")
        _layer0_parity(c_f, tf[0][0], tf[0][1], dtype, "step %d" % t)
        rel = ((lf - ld).norm() / ld.norm()).item()
        worst_l = max(worst_l, rel)
        assert rel < 0.05, ("logits", t, rel)
    assert c_f.get_seq_length() == prompt + steps
    assert c_f.layers[0].k.tokens == c_d.layers[0].k.tokens == 256
    _say("decoder", dtype, "logit rel err", worst_l, "cache bytes", c_f.cache_bytes(), "fp16 bytes",
         2 * shape.layers * B * shape.kv_heads * (prompt + steps) * 128 * 2)


def test_decoder_at_the_benchmark_head_shape(cuda):
    """The end-to-end configuration's own attention shape -- 32 query / 8 KV heads of 128, hidden 4096, MLP 12288,
    bf16, batch 4, an 8192-token prompt (8064 tokens compressed by the prompt pass, 128 buffered) -- with two layers and a
    small vocabulary so that it runs in seconds.  132 greedy-free steps (forced ids) cross the cuts at steps 63 and
    127; layer 0's fused attention is checked against the oracle on the cache's contents around both."""
    dtype = torch.bfloat16
    shape = DecoderShape(layers=2, hidden=4096, q_heads=32, kv_heads=8, mlp=12288, vocab=4096, head_norm=True)
    model = ShapedDecoder(shape, dtype=dtype, device=cuda, seed=11)
    B, prompt, steps = 4, 8192, 132
    g = torch.Generator().manual_seed(12)
    ids = torch.randint(0, shape.vocab, (B, prompt), generator=g).to(cuda)
    forced = torch.randint(0, shape.vocab, (B, steps), generator=g).to(cuda)
    cache = model.new_cache(B, prompt + 512, PackKVCacheConfig())
    model.prefill(ids, cache)
    assert cache.layers[0].k.tokens == 8064 and cache.layers[0].win_len == 128
    check_at = {0, 1, 62, 63, 64, 100, 126, 127, 128, 131}
    for t in range(steps):
        taps = []
        logits = model.forward(forced[:, t:t + 1], cache, attention="fused", taps=taps)
        assert bool(torch.isfinite(logits).all())
        if t in check_at:
            L = cache.layers[0]
            _say("benchmark-shape decoder step", t, "compressed", L.k.tokens, "pending", L.pend, "window", L.win_len)
            _layer0_parity(cache, taps[0][0], taps[0][1], dtype, "step %d" % t)
    L = cache.layers[0]
    assert cache.get_seq_length() == prompt + steps
    assert L.k.tokens == 8064 + 128 and L.pend == 0 and L.win_len == prompt + steps - L.k.tokens
    fp16_bytes = 2 * shape.layers * B * shape.kv_heads * (prompt + steps) * 128 * 2
    _say("benchmark-shape decoder: cache bytes", cache.cache_bytes(), "vs 16-bit", fp16_bytes)
    assert cache.cache_bytes() < 0.3 * fp16_bytes


def test_greedy_runs_and_accounts(cuda):
    shape = DecoderShape(layers=2, hidden=256, q_heads=8, kv_heads=2, mlp=512, vocab=512)
    model = ShapedDecoder(shape, dtype=torch.bfloat16, device=cuda, seed=7)
    ids = torch.randint(0, shape.vocab, (3, 256), generator=torch.Generator().manual_seed(8)).to(cuda)
    cache = model.new_cache(3, 512)
    out = model.greedy(ids, cache, 40)
    assert out.shape == (3, 40) and int(out.min()) >= 0 and int(out.max()) < shape.vocab
    assert cache.get_seq_length() == 256 + 40          # every generated token but the last one's successor is cached
