"""The compressed cache that grows (packkv_amd/cache.py) against the restated reference cache
(oracle/cache.py): dense view bit-exact, decode step within the attention tolerance, streams equal to a
one-shot encode."""
import numpy as np
import pytest
import torch

from oracle import cache as oc
from oracle import quant as oq
from packkv_amd import ops, synth
from packkv_amd.cache import PackKVCacheConfig, PackKVCompressedCache
from attn_bounds import check_fast, check_reference_mode, say as _say

pytestmark = pytest.mark.gpu


def _attend_parity(cache, layer, q, wk, wv, ek, ev, dtype, cuda, label):
    """cache.attend in the checking mode against the reference path at the contract, and the fast decode step
    against exact arithmetic, its distance to the reference path printed beside the contract (tests/attn_bounds.py).
    wk, wv: what the reference's update returns; ek, ev: the same tokens before their rounding to 16 bits (fp64).
    Only the tokens already in the streams are attended unrounded: a pending 64-token cut sits in the 16-bit window
    in dequantised form, like the buffer."""
    n = cache.layers[layer].k.tokens
    ek, ev = torch.cat([ek[:, :, :n], wk[:, :, n:].double()], dim=2), torch.cat([ev[:, :, :n], wv[:, :, n:].double()], dim=2)
    ref = oq.attention_f32(q.unsqueeze(2), wk, wv).squeeze(2)
    exact = oq.attention_f64_np(q.unsqueeze(2), ek, ev).squeeze(2)
    chk = cache.attend(q.to(cuda), layer, variant=1, ref_rounding=True, out_f32=True)
    check_reference_mode(chk, ref, label)
    check_fast(cache.attend(q.to(cuda), layer), ref, exact, dtype, label=label)


def _rope_tables(B, pos0, n, dtype):
    pos = torch.arange(pos0, pos0 + n, dtype=torch.float32)
    inv = 1.0 / (10000.0 ** (torch.arange(0, 128, 2, dtype=torch.float32) / 128))
    f = torch.outer(pos, inv)
    emb = torch.cat((f, f), dim=-1)
    return emb.cos().to(dtype).expand(B, n, 128).contiguous(), emb.sin().to(dtype).expand(B, n, 128).contiguous()


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("rope", [False, True])
def test_cache_matches_restated_reference(cuda, dtype, rope):
    B, Hq, H, T0, steps = 2, 8, 4, 300, 200
    k, v = synth.make_kv(B, H, T0 + steps, seed=90, dtype=dtype)
    want = oc.SimulatedCache(1, 64, 192, 0.1, 0.1, track_exact=True)
    got = PackKVCompressedCache(B, H, 128, 1, PackKVCacheConfig(64, 192, 0.1, 0.1), max_tokens=1024, dtype=dtype,
                                device=cuda)
    check_at = {0, 1, 18, 19, 20, 82, 83, 84, 146, 147, 148, 199}   # around the cuts at steps 19, 83, 147
    pos, tok = 0, 0
    for step in range(-1, steps):
        n = T0 if step < 0 else 1
        ks, vs = k[:, :, tok:tok + n], v[:, :, tok:tok + n]
        cos = sin = None
        if rope:
            cos, sin = _rope_tables(B, pos, n, dtype)
        wk, wv = want.update(ks, vs, 0, cos, sin)
        kw = {"cos": cos.to(cuda), "sin": sin.to(cuda)} if rope else None
        got.update(ks.to(cuda), vs.to(cuda), 0, kw, return_dense=False)
        tok += n
        pos += n
        assert got.get_seq_length(0) == want.get_seq_length(0) == tok
        if step in check_at or step < 0:
            _say("cache case", dtype, "rope" if rope else "plain", "step", step, "tokens", tok,
                 "compressed", got.layers[0].k.tokens, "window", got.layers[0].win_len)
            gk, gv = got.materialize(0)
            assert torch.equal(gk.cpu().view(torch.int16), wk.view(torch.int16))
            assert torch.equal(gv.cpu().view(torch.int16), wv.view(torch.int16))
            q = synth.make_q(B, Hq, seed=300 + step, dtype=dtype)
            ek, ev = want.exact(0)
            _attend_parity(got, 0, q, wk, wv, ek, ev, dtype, cuda, "step %d" % step)
    L = got.layers[0]
    # 500 tokens: 320 have been cut (128 at the prefill, then at steps 19, 83, 147) = 2 tiles + one pending cut
    assert L.k.tokens == L.v.tokens == 256 and L.pend == 64 and L.win_len == T0 + steps - 256


def test_append_equals_one_shot_encode(cuda):
    """Chunk-by-chunk append (K in cuts of 64 and 128 tokens, V of 128 and 256) gives the stream, block_info and
    parameters of one encode over all tokens."""
    B, H, T = 2, 4, 512
    k, v = synth.make_kv(B, H, T, seed=95, device=cuda)
    for is_k, x, chunks in ((True, k, (64, 128, 64, 256)), (False, v, (128, 256, 128))):
        one = ops.k_quant_encode(x, 0.1) if is_k else ops.v_quant_encode(x, 0.1)
        per_tok = (B * H) if is_k else (B * H * 2)
        nblk = T // (64 if is_k else 128) * per_tok
        stream = torch.zeros(one["size"] + 64, dtype=torch.uint8, device=cuda)
        info = torch.zeros(nblk, 2, dtype=torch.uint32, device=cuda)
        scale = torch.zeros(B, T + 128, dtype=x.dtype, device=cuda)     # rows longer than the token count
        zero = torch.zeros_like(scale)
        used, tok = 0, 0
        for n in chunks:
            _say("append case", "K" if is_k else "V", "tokens", tok, "+", n)
            used = ops.quant_encode_append(is_k, x[:, :, tok:tok + n].contiguous(), 0.1, one["bits"], stream, used,
                                           info, tok, scale, zero)
            tok += n
        assert tok == T and used == one["size"]
        assert torch.equal(stream[:used], one["stream"][:used])
        assert torch.equal(info.view(torch.int32), one["info"].view(torch.int32))
        assert torch.equal(scale[:, :T].view(torch.int16), one["scale"].view(torch.int16))
        assert torch.equal(zero[:, :T].view(torch.int16), one["zero"].view(torch.int16))


def test_append_reports_a_full_buffer(cuda):
    B, H = 1, 2
    k, _ = synth.make_kv(B, H, 128, seed=96, device=cuda)
    stream = torch.zeros(256, dtype=torch.uint8, device=cuda)
    info = torch.zeros(4, 2, dtype=torch.uint32, device=cuda)
    scale = torch.zeros(B, 128, dtype=k.dtype, device=cuda)
    with pytest.raises(RuntimeError):
        ops.quant_encode_append(True, k, 0.1, 4, stream, 0, info, 0, scale, torch.zeros_like(scale))


def test_cache_bytes_and_prefill_only(cuda):
    """A prompt below buffer_size stays uncompressed (utils/compute.py:54-67); a long prefill compresses all but
    128..191 tokens, in whole tiles."""
    B, H = 1, 8
    k, v = synth.make_kv(B, H, 1000, seed=97, device=cuda)
    c = PackKVCompressedCache(B, H, 128, 2, max_tokens=2048, device=cuda)
    c.update(k[:, :, :191], v[:, :, :191], 0, return_dense=False)
    assert c.layers[0].k.tokens == 0 and c.layers[0].win_len == 191
    assert c.cache_bytes(0) == 2 * B * H * 191 * 128 * 2
    c.update(k, v, 1, return_dense=False)     # 1000 tokens: 832 cut = 6 tiles + one pending cut of 64, 168 buffered
    L = c.layers[1]
    assert L.k.tokens == 768 and L.pend == 64 and L.win_len == 64 + 168 and c.get_seq_length(1) == 1000
    fp16_bytes = 2 * B * H * 1000 * 128 * 2
    assert c.cache_bytes(1) < 0.45 * fp16_bytes
    q = synth.make_q(B, 32, seed=98, device=cuda)
    gk, gv = c.materialize(1)
    ref = oq.attention_f32(q.cpu().unsqueeze(2), gk.cpu(), gv.cpu()).squeeze(2)
    out = c.attend(q.unsqueeze(2), 1)
    assert out.shape == (B, 32, 1, 128)
    # the reference path on the dense view: the checking mode at the contract; the fast step within the bound the
    # oracle gives (exact arithmetic = the restated quantiser's unrounded values for the 832 cut tokens)
    sim = oc.SimulatedCache(1, 64, 192, 0.1, 0.1, track_exact=True)
    wk, wv = sim.update(k.cpu(), v.cpu(), 0)
    assert torch.equal(gk.cpu().view(torch.int16), wk.view(torch.int16))
    ek, ev = sim.exact(0)
    ek, ev = torch.cat([ek[:, :, :768], wk[:, :, 768:].double()], dim=2), torch.cat([ev[:, :, :768], wv[:, :, 768:].double()], dim=2)
    exact = oq.attention_f64_np(q.cpu().unsqueeze(2), ek, ev).squeeze(2)
    check_reference_mode(c.attend(q, 1, variant=1, ref_rounding=True, out_f32=True), ref, "prefill 1000")
    check_fast(out[:, :, 0], ref, exact, torch.float16, label="prefill 1000")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_window_append_is_the_reference_chain_bit_for_bit(cuda, dtype):
    """Rotary embedding of the new keys + append, one launch, against the reference's chain of 16-bit elementwise ops
    (utils/compute.py:35-43, restated in oracle/cache.py) evaluated by torch on the device: equal bits; contiguous
    and strided inputs (a transposed projection output, an expanded cos / sin table), one and several new tokens,
    with and without the embedding."""
    from oracle import cache as oc
    g = torch.Generator().manual_seed(400)
    B, H, cap = 3, 4, 40
    for n, pos, strided in ((1, 0, False), (1, 17, True), (5, 30, True), (8, 32, False)):
        _say("append case", dtype, n, pos, strided)
        if strided:     # [B, n, H, 128] storage seen as [B, H, n, 128], like a projection output after transpose(1, 2)
            k = (torch.randn(B, n, H, 128, generator=g) * 3).to(dtype).to(cuda).transpose(1, 2)
            v = torch.randn(B, n, H, 128, generator=g).to(dtype).to(cuda).transpose(1, 2)
            cos1, sin1 = _rope_tables(1, 100 + pos, n, dtype)
            cos, sin = cos1.to(cuda).expand(B, n, 128), sin1.to(cuda).expand(B, n, 128)
        else:
            k = (torch.randn(B, H, n, 128, generator=g) * 3).to(dtype).to(cuda)
            v = torch.randn(B, H, n, 128, generator=g).to(dtype).to(cuda)
            cos, sin = (t.to(cuda) for t in _rope_tables(B, 100 + pos, n, dtype))
        for rotary in (True, False):
            k_win = torch.full((B, H, cap, 128), 7.0, dtype=dtype, device=cuda)
            v_win = torch.full((B, H, cap, 128), 7.0, dtype=dtype, device=cuda)
            ops.window_append(k, v, cos if rotary else None, sin if rotary else None, k_win, v_win, pos)
            want_k = oc.apply_rotary_pos_emb_single(k, cos, sin) if rotary else k
            assert torch.equal(k_win[:, :, pos:pos + n].view(torch.int16), want_k.contiguous().view(torch.int16))
            assert torch.equal(v_win[:, :, pos:pos + n], v)
            rest = torch.ones(cap, dtype=torch.bool)
            rest[pos:pos + n] = False
            assert (k_win[:, :, rest] == 7.0).all() and (v_win[:, :, rest] == 7.0).all()     # nothing else written
    with pytest.raises(Exception):
        ops.window_append(k, v, None, None, k_win, v_win, cap - 2)                           # 8 rows do not fit


def test_cache_with_five_bit_codes(cuda):
    """rel 0.05 (5-bit codes, the format extension) through the growing cache: the fused encoders append, the
    asynchronous-copy attention kernel reads; dense view bit-exact with the restated reference cache, the decode
    step within the attention tolerance, across one cut."""
    B, Hq, H, T0, steps = 2, 8, 4, 300, 40
    dtype = torch.float16
    k, v = synth.make_kv(B, H, T0 + steps, seed=96, dtype=dtype)
    want = oc.SimulatedCache(1, 64, 192, 0.05, 0.05, track_exact=True)
    got = PackKVCompressedCache(B, H, 128, 1, PackKVCacheConfig(64, 192, 0.05, 0.05), max_tokens=1024, dtype=dtype,
                                device=cuda)
    assert got.config.k_bits == 5 and got.config.v_bits == 5
    tok = 0
    for step in range(-1, steps):
        n = T0 if step < 0 else 1
        ks, vs = k[:, :, tok:tok + n], v[:, :, tok:tok + n]
        wk, wv = want.update(ks, vs, 0, None, None)
        got.update(ks.to(cuda), vs.to(cuda), 0, None, return_dense=False)
        tok += n
        if step in (-1, 0, 19, 20, 39):
            _say("5-bit cache case step", step, "tokens", tok, "compressed", got.layers[0].k.tokens)
            gk, gv = got.materialize(0)
            assert torch.equal(gk.cpu().view(torch.int16), wk.view(torch.int16))
            assert torch.equal(gv.cpu().view(torch.int16), wv.view(torch.int16))
            q = synth.make_q(B, Hq, seed=500 + step, dtype=dtype)
            ek, ev = want.exact(0)
            _attend_parity(got, 0, q, wk, wv, ek, ev, dtype, cuda, "5-bit step %d" % step)
    assert got.layers[0].k.tokens == 128 and got.layers[0].pend == 64      # 128 at the prefill, one more cut waiting for its partner


def test_reference_cache_class_and_its_two_line_hook(cuda):
    """The reference builds ``PackKVCache(batch, heads, head_dim, layers)`` (models/llama.py:830-833), configured
    through ``PackKVCacheConfigStatic.config``, and its attention modules run (models/llama.py:260-261)

        cache_kwargs = {"sin": sin, "cos": cos, "cache_position": cache_position}
        key_states, value_states = past_key_value.update(key_states, value_states, self.layer_idx, cache_kwargs)

    The drop-in class takes both lines as they stand: it is a transformers.Cache, and update returns the dense K and V
    of the restated reference cache bit for bit -- prompt pass and decode steps across a cut, two layers."""
    import transformers
    from packkv_amd.cache import PackKVCache, PackKVCacheConfigStatic
    dtype = torch.float16
    B, H, T0, steps, layers = 2, 4, 300, 70, 2
    k, v = synth.make_kv(B, H, T0 + steps, seed=610, dtype=dtype)
    PackKVCacheConfigStatic.config = PackKVCacheConfig(64, 192, 0.1, 0.1)
    PackKVCacheConfigStatic.max_tokens = 1024
    try:
        past_key_value = PackKVCache(B, H, 128, layers)
        assert isinstance(past_key_value, transformers.Cache)
        want = oc.SimulatedCache(layers, 64, 192, 0.1, 0.1)
        pos = 0
        for step in range(-1, steps):
            n = T0 if step < 0 else 1
            cos, sin = _rope_tables(B, pos, n, dtype)
            cache_position = torch.arange(pos, pos + n)
            for layer_idx in range(layers):
                key_states = (k[:, :, pos:pos + n] * (1 + layer_idx)).to(cuda)
                value_states = v[:, :, pos:pos + n].to(cuda)
                wk, wv = want.update(key_states.cpu(), value_states.cpu(), layer_idx, cos, sin)
                sin_d, cos_d = sin.to(cuda), cos.to(cuda)
                # the reference's two lines, with sin / cos on the device
                cache_kwargs = {"sin": sin_d, "cos": cos_d, "cache_position": cache_position}
                key_states, value_states = past_key_value.update(key_states, value_states, layer_idx, cache_kwargs)
                if step < 0 or step in (0, 18, 19, 20, 69):
                    _say("reference hook: step", step, "layer", layer_idx, "K", tuple(key_states.shape))
                    assert key_states.shape == wk.shape and value_states.shape == wv.shape
                    assert torch.equal(key_states.cpu().view(torch.int16), wk.view(torch.int16))
                    assert torch.equal(value_states.cpu().view(torch.int16), wv.view(torch.int16))
            pos += n
            assert past_key_value.get_seq_length(0) == past_key_value.get_seq_length(1) == pos
    finally:
        PackKVCacheConfigStatic.config = None
        PackKVCacheConfigStatic.max_tokens = 32768
