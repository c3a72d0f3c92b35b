"""GPU parity of the fused decompress-attention decode against the reference
decompress-then-attend path restated on the CPU (quantize -> dequantise to the storage dtype ->
attention with fp32 accumulation).

How the contract (2e-3 absolute + 1e-3 relative, element-wise) is applied to the checking mode and to
the fast kernels is written down once, in tests/attn_bounds.py; no case here widens it."""
import numpy as np
import pytest
import torch

from oracle import quant as oq
from packkv_amd import ops, synth
from attn_bounds import check_fast, check_reference_mode, contract_holds, say as _say

pytestmark = pytest.mark.gpu


def _parity(cuda, q, ke, ve, ref, exact, dtype, variants, k_win=None, v_win=None, label="", contract_too=False):
    """The checking mode against the reference path at the contract; every fast variant against exact arithmetic,
    its distance to the reference path printed beside the contract (asserted where `contract_too` says it holds)."""
    qd = q.to(cuda)
    chk = ops.attn_decode(qd, ke, ve, k_win, v_win, variant=1, ref_rounding=True, out_f32=True)
    check_reference_mode(chk, ref, label)
    outs = {}
    for variant in variants:
        got = ops.attn_decode(qd, ke, ve, k_win, v_win, variant=variant)
        check_fast(got, ref, exact, dtype, variant, label="%s variant %d" % (label, variant))
        if contract_too:
            assert contract_holds(got, ref)
        outs[variant] = got.float()
    return outs


def _exact(q, k, v, rel_k, rel_v, k_win=None, v_win=None):
    """fp64 attention on the UNROUNDED dequantised values (code + zero) * scale."""
    ck, zk, sk = oq.quant_ints(k, 64, rel_k)
    cv, zv, sv = oq.quant_ints(v, 64, rel_v)
    kd = ((ck.double() + zk.double()) * sk.double()).reshape(k.shape)
    vd = ((cv.double() + zv.double()) * sv.double()).reshape(v.shape)
    if k_win is not None:
        kd, vd = torch.cat([kd, k_win.double()], dim=2), torch.cat([vd, v_win.double()], dim=2)
    return oq.attention_f64_np(q.unsqueeze(2), kd, vd).squeeze(2)


def _reference(q, k, v, rel_k, rel_v, k_win=None, v_win=None):
    ck, zk, sk = oq.quant_ints(k, 64, rel_k)
    cv, zv, sv = oq.quant_ints(v, 64, rel_v)
    kd, vd = oq.dequant(ck, zk, sk), oq.dequant(cv, zv, sv)
    if k_win is not None:
        kd, vd = torch.cat([kd, k_win], dim=2), torch.cat([vd, v_win], dim=2)
    return oq.attention_f32(q.unsqueeze(2), kd, vd).squeeze(2)


CASES = [
    # B, Hq, Hkv, T, rel_k, rel_v
    (1, 32, 32, 256, 0.1, 0.1),
    (2, 32, 8, 1024, 0.1, 0.1),
    (1, 8, 8, 128, 0.2, 0.2),
    (2, 16, 2, 2048, 0.1, 0.2),
    (1, 16, 8, 512, 0.34, 0.1),
    (3, 4, 4, 384, 0.1, 0.1),
]


@pytest.mark.parametrize("variant", [0, 1, 2])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_attn_decode_matches_decompress_then_attend(cuda, dtype, variant):
    for (B, Hq, Hkv, T, rk, rv) in CASES:
        _say("attn case", dtype, "variant", variant, B, Hq, Hkv, T, rk, rv)
        k, v = synth.make_kv(B, Hkv, T, seed=50 + T, dtype=dtype)
        q = synth.make_q(B, Hq, seed=51, dtype=dtype)
        want = _reference(q, k, v, rk, rv)
        ke = ops.k_quant_encode(k.to(cuda), rk)
        ve = ops.v_quant_encode(v.to(cuda), rv)
        _parity(cuda, q, ke, ve, want, _exact(q, k, v, rk, rv), dtype, [variant], label="T=%d" % T)


# The shapes the benchmarks are quoted on (one or two sequences of them, so that the CPU oracle
# finishes in seconds).  In fp16 the fast kernels meet the contract against the reference path directly.
BASELINE_SHAPES = [
    ("config0: Llama-2-7B layer", 1, 32, 32, 4096),
    ("config1: Llama-3-8B GQA, 2 of 16 sequences", 2, 32, 8, 32768),
    ("config4: Mistral-7B long context, 1 of 4 sequences at 65536 tokens", 1, 32, 8, 65536),
]


@pytest.mark.parametrize("variant", [0, 1, 2])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_attn_decode_baseline_shapes_contract_tolerance(cuda, dtype, variant):
    for (name, B, Hq, Hkv, T) in BASELINE_SHAPES:
        if dtype == torch.bfloat16 and T > 32768:
            continue
        _say("attn baseline shape", name, dtype, "variant", variant)
        k, v = synth.make_kv(B, Hkv, T, seed=90, dtype=dtype)
        q = synth.make_q(B, Hq, seed=91, dtype=dtype)
        want = _reference(q, k, v, 0.1, 0.1)
        ke = ops.k_quant_encode(k.to(cuda), 0.1)
        ve = ops.v_quant_encode(v.to(cuda), 0.1)
        _parity(cuda, q, ke, ve, want, _exact(q, k, v, 0.1, 0.1), dtype, [variant], label=name.split(":")[0],
                contract_too=dtype == torch.float16)


@pytest.mark.parametrize("variant", [0, 1, 2])
def test_attn_decode_with_tail_window(cuda, variant):
    dtype = torch.float16
    # the default kernel spreads the window over its splits: cover pieces of unequal size, more splits than
    # window tokens (empty pieces), the largest piece that fits and one that does not (window kernel of its own)
    for (B, Hq, Hkv, T, Tw) in ((2, 32, 8, 512, 150), (1, 8, 8, 0, 191), (1, 16, 4, 128, 1), (1, 8, 2, 1024, 3),
                                (1, 8, 1, 256, 2048), (1, 8, 1, 128, 2048)):
        _say("attn window case", B, Hq, Hkv, T, Tw)
        k, v = synth.make_kv(B, Hkv, T + Tw, seed=60 + Tw, dtype=dtype)
        q = synth.make_q(B, Hq, seed=61, dtype=dtype)
        kc, kw = k[:, :, :T].contiguous(), k[:, :, T:].contiguous()
        vc, vw = v[:, :, :T].contiguous(), v[:, :, T:].contiguous()
        if T > 0:
            want = _reference(q, kc, vc, 0.1, 0.1, kw, vw)
            exact = _exact(q, kc, vc, 0.1, 0.1, kw, vw)
            ke = ops.k_quant_encode(kc.to(cuda), 0.1)
            ve = ops.v_quant_encode(vc.to(cuda), 0.1)
        else:
            want = oq.attention_f32(q.unsqueeze(2), kw, vw).squeeze(2)
            exact = oq.attention_f64_np(q.unsqueeze(2), kw, vw).squeeze(2)
            ke = ve = None
        _parity(cuda, q, ke, ve, want, exact, dtype, [variant], kw.to(cuda), vw.to(cuda), label="T=%d+%d" % (T, Tw))


@pytest.mark.parametrize("variant", [0, 1, 2])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_attn_decode_group_sizes_that_are_no_power_of_two(cuda, dtype, variant):
    """3, 5, 6 and 7 query heads per KV head (24 q / 8 KV, 28 q / 4 KV, ...): the kernels of 4 and 8 with idle head
    slots.  Same bars as every other case, with and without a tail window."""
    for (B, Hq, Hkv, T, Tw) in ((2, 24, 8, 512, 0), (1, 28, 4, 1024, 37), (2, 10, 2, 384, 0), (1, 12, 2, 640, 130), (1, 3, 1, 256, 0)):
        _say("odd group case", dtype, "variant", variant, B, Hq, Hkv, T, Tw)
        k, v = synth.make_kv(B, Hkv, T + Tw, seed=520 + Hq, dtype=dtype)
        q = synth.make_q(B, Hq, seed=521, dtype=dtype)
        kc, vc = k[:, :, :T].contiguous(), v[:, :, :T].contiguous()
        kw, vw = (k[:, :, T:].contiguous(), v[:, :, T:].contiguous()) if Tw else (None, None)
        want = _reference(q, kc, vc, 0.1, 0.1, kw, vw)
        exact = _exact(q, kc, vc, 0.1, 0.1, kw, vw)
        ke, ve = ops.k_quant_encode(kc.to(cuda), 0.1), ops.v_quant_encode(vc.to(cuda), 0.1)
        _parity(cuda, q, ke, ve, want, exact, dtype, [variant], kw.to(cuda) if Tw else None, vw.to(cuda) if Tw else None,
                label="group of %d" % (Hq // Hkv))


def test_attn_decode_close_to_reference_fp16_eager(cuda):
    """Against the literal 16-bit eager path (models/llama.py:189-212), which also rounds the logits and the softmax
    weights to fp16: the kernel may differ from it by the contract plus what those two extra roundings moved, a
    distance the oracle gives (eager path against the fp32-accumulating path on the same tensors)."""
    B, Hq, Hkv, T = 2, 32, 8, 1024
    k, v = synth.make_kv(B, Hkv, T, seed=70)
    q = synth.make_q(B, Hq, seed=71)
    ck, zk, sk = oq.quant_ints(k, 64, 0.1)
    cv, zv, sv = oq.quant_ints(v, 64, 0.1)
    kd, vd = oq.dequant(ck, zk, sk), oq.dequant(cv, zv, sv)
    eager = oq.eager_attention(q.unsqueeze(2), kd, vd).squeeze(2).double().numpy()
    ref = oq.attention_f32(q.unsqueeze(2), kd, vd).squeeze(2).double().numpy()
    chk = ops.attn_decode(q.to(cuda), ops.k_quant_encode(k.to(cuda), 0.1), ops.v_quant_encode(v.to(cuda), 0.1),
                          variant=1, ref_rounding=True, out_f32=True).double().cpu().numpy()
    _say("   eager 16-bit path vs fp32-accumulating path: %.3e; checking mode vs eager: %.3e"
         % (np.abs(eager - ref).max(), np.abs(chk - eager).max()))
    assert (np.abs(chk - eager) <= np.abs(eager - ref) + 2e-3 + 1e-3 * np.abs(ref)).all()


def test_attn_decode_full_size_property(cuda):
    """At the benchmark's shape (batch 16, 32 q / 8 KV heads, 32768 tokens) the oracle is too slow;
    use properties instead: (i) a query of zeros gives uniform weights, so the output equals the
    mean of the dequantised V, which the unpack + dequantize kernels provide independently;
    (ii) splitting the cache into compressed part + 16-bit tail gives the same answer as
    compressing everything up to quantisation error bounds."""
    B, Hq, Hkv, T = 16, 32, 8, 32768
    k, v = synth.make_kv(B, Hkv, T, seed=80, device=cuda)
    ke = ops.k_quant_encode(k, 0.1)
    ve = ops.v_quant_encode(v, 0.1)
    q0 = torch.zeros(B, Hq, 128, dtype=torch.float16, device=cuda)
    got = ops.attn_decode(q0, ke, ve)
    codes = torch.empty(T, B * Hkv * 128, dtype=torch.uint8, device=cuda)
    ops.v_decode(ve["stream"], ve["info"], codes, 128, 64, ve["bits"])
    vd = ops.dequantize(codes, ve["scale"], ve["zero"], B, Hkv)
    want = vd.float().mean(dim=2).repeat_interleave(Hq // Hkv, dim=1)
    err = (got.float() - want).abs().max().item()
    _say("   zero-query mean-of-V check: err %.3e, max|ref| %.3e" % (err, want.abs().max().item()))
    assert err <= 1e-3 * want.abs().max().item() + 2 ** -11 * want.abs().max().item() + 2e-5


@pytest.mark.parametrize("dtype,hq,rel", [(torch.float16, 32, 0.1), (torch.bfloat16, 32, 0.1), (torch.float16, 8, 0.1),
                                          (torch.float16, 16, 0.1), (torch.bfloat16, 64, 0.1), (torch.float16, 32, 0.05),
                                          (torch.bfloat16, 32, 0.03), (torch.float16, 32, 0.2)])
def test_attn_decode_tiles_handed_out_by_counter(cuda, dtype, hq, rel):
    """Shapes at which the members of a (sequence, KV head) take their tiles from the head's counter (eight members
    with twelve tiles each and more): random queries, every group size, both dtypes, the reference's widths and the
    extension widths, against the plain kernel, whose workgroups own fixed tile ranges.  The two kernels differ by
    their own rounding only.  Three steps in a row: the counters must come back to zero after each."""
    B, Hkv, T = 16, 8, 12288
    k, v = synth.make_kv(B, Hkv, T, seed=410, dtype=dtype, device=cuda)
    ke, ve = ops.k_quant_encode(k, rel), ops.v_quant_encode(v, rel)
    del k, v
    half_ulp = 2.0 ** -11 if dtype == torch.float16 else 2.0 ** -8
    for rep in range(3):
        q = synth.make_q(B, hq, seed=411 + rep, dtype=dtype, device=cuda)
        fast = ops.attn_decode(q, ke, ve, variant=0).float()
        plain = ops.attn_decode(q, ke, ve, variant=1).float()
        err = (fast - plain).abs()
        _say("tiles by counter", dtype, "group of", hq // Hkv, "rel", rel, "step", rep, "max diff %.3e" % err.max().item())
        assert bool(torch.isfinite(fast).all())
        assert bool((err <= 2 * 5e-4 + 2.1 * half_ulp * plain.abs()).all())


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_long_context_layer_at_its_own_size(cuda, dtype):
    """One layer of the long-context configuration at its own size -- batch 4, 32 query / 8 KV heads, 131072 cached
    tokens per sequence, 1 GiB each of K and V -- where the oracle is far too slow; size-independent properties
    instead: (i) the fused encoders' streams unpack to the codes of the stand-alone quantizer (which the small tests
    hold bit-exact against the oracle), K and V; (ii) a query of zeros weighs all tokens alike, so the output is the
    mean of the dequantised V; (iii) the last 128 tokens handed over as a 16-bit window holding their dequantised
    values give the output of the all-compressed cache up to the contract; (iv) the stream sizes add up
    (offsets = running sums of sizes, the last block ends the stream)."""
    B, Hq, Hkv, T = 4, 32, 8, 131072
    k, v = synth.make_kv(B, Hkv, T, seed=330, dtype=dtype, device=cuda)
    hidden = B * Hkv * 128
    ke, ve = ops.k_quant_encode(k, 0.1), ops.v_quant_encode(v, 0.1)
    codes = torch.empty(T, hidden, dtype=torch.uint8, device=cuda)
    deq = {}
    for name, x, e, dec, cb, hb in (("K", k, ke, ops.k_decode, 64, 128), ("V", v, ve, ops.v_decode, 128, 64)):
        _say("long context", dtype, name, "stream", e["size"], "bytes, ratio %.2f" % (x.numel() * 2 / e["size"]))
        dec(e["stream"], e["info"], codes, cb, hb, e["bits"])
        scale, zero = ops.quant_params(x, 0.1)
        want_codes, _ = ops.quantize(x, scale, zero)
        assert torch.equal(scale.view(torch.int16), e["scale"].view(torch.int16))
        assert torch.equal(zero.view(torch.int16), e["zero"].view(torch.int16))
        assert torch.equal(codes, want_codes)                                                       # (i)
        del want_codes
        info = e["info"].view(torch.int32).to(torch.int64) & 0xFFFFFFFF
        assert int(info[0, 0]) == 0 and bool((info[1:, 0] == info[:-1, 0] + info[:-1, 1]).all())    # (iv)
        assert int(info[-1, 0] + info[-1, 1]) == e["size"]
        deq[name] = ops.dequantize(codes, e["scale"], e["zero"], B, Hkv)
    del k, v, codes
    q0 = torch.zeros(B, Hq, 128, dtype=dtype, device=cuda)
    got = ops.attn_decode(q0, ke, ve).float()
    want = deq["V"].float().mean(dim=2).repeat_interleave(Hq // Hkv, dim=1)
    half_ulp = 2.0 ** -11 if dtype == torch.float16 else 2.0 ** -8
    err = (got - want).abs()
    _say("   zero-query mean-of-V: max err %.3e, max|ref| %.3e" % (err.max().item(), want.abs().max().item()))
    assert bool((err <= 5e-4 + 1.05 * half_ulp * want.abs() + 2.0 ** -9 * want.abs().max()).all())      # (ii)
    # (iii) all tokens compressed against [T - 128 compressed | the last 128 as a 16-bit window of their dequantised
    # values]: the same numbers reach the kernel both ways, up to the 16-bit rounding of 128 tokens
    q = synth.make_q(B, Hq, seed=331, dtype=dtype, device=cuda)
    full = ops.attn_decode(q, ke, ve, out_f32=True)
    kw, vw = deq["K"][:, :, T - 128:].contiguous(), deq["V"][:, :, T - 128:].contiguous()
    ke_c, ve_c = dict(ke, tokens=T - 128, heads=Hkv), dict(ve, tokens=T - 128, heads=Hkv)
    part = ops.attn_decode(q, ke_c, ve_c, kw, vw, out_f32=True)
    err = (part - full).abs()
    _say("   compressed + window vs all compressed: max err %.3e, max|ref| %.3e" % (err.max().item(), full.abs().max().item()))
    assert bool((err <= 2e-3 + 1e-3 * full.abs()).all())


def test_attn_decode_replays_in_a_hip_graph(cuda):
    """A decode step launches only kernels on the caller's stream (no memset nodes), and while a stream is capturing it
    allocates nothing: a capture stream that has no scratch of its own yet (torch captures on a side stream) keeps its
    partials in the library's fixed device array, like pkv_attn_decode_noalloc.  Four layers' worth of calls in one
    graph, replayed with new queries and eager work in between, must reproduce the eager results every time."""
    B, Hq, Hkv, T, Tw = 2, 16, 4, 1024, 150
    layers = []
    for i in range(4):
        k, v = synth.make_kv(B, Hkv, T + Tw, seed=110 + i, device=cuda)
        layers.append((ops.k_quant_encode(k[:, :, :T].contiguous(), 0.1), ops.v_quant_encode(v[:, :, :T].contiguous(), 0.1),
                       k[:, :, T:].contiguous(), v[:, :, T:].contiguous()))
    q = synth.make_q(B, Hq, seed=120, device=cuda)
    outs = [torch.empty_like(q) for _ in layers]
    for (ke, ve, kw, vw), o in zip(layers, outs):       # warm-up: sizes the library's scratch outside the capture
        ops.attn_decode(q, ke, ve, kw, vw, out=o)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for (ke, ve, kw, vw), o in zip(layers, outs):
            ops.attn_decode(q, ke, ve, kw, vw, out=o)
    for rep in range(3):
        q.copy_(synth.make_q(B, Hq, seed=121 + rep, device=cuda))
        want = [ops.attn_decode(q, ke, ve, kw, vw) for (ke, ve, kw, vw) in layers]     # eager, own outputs
        torch.cuda.synchronize()
        for o in outs:
            o.zero_()
        graph.replay()
        torch.cuda.synchronize()
        for o, w in zip(outs, want):
            assert torch.equal(o, w)


def test_attn_decode_takes_buffers_that_end_with_their_stream(cuda):
    """Stream buffers without a byte of slack behind the encoded size (sizes that end in the middle of a dword and of
    a 16-byte copy unit included) give the results of generously sized buffers, on every variant."""
    for seed, (B, Hq, Hkv, T) in enumerate([(1, 8, 2, 128), (2, 16, 4, 512), (1, 32, 8, 1024), (1, 4, 1, 256), (3, 12, 3, 384)]):
        k, v = synth.make_kv(B, Hkv, T, seed=900 + seed, device=cuda)
        q = synth.make_q(B, Hq, seed=950 + seed, device=cuda)
        ke, ve = ops.k_quant_encode(k, 0.1), ops.v_quant_encode(v, 0.1)
        ke2, ve2 = dict(ke), dict(ve)
        ke2["stream"], ve2["stream"] = ke["stream"][:ke["size"]].clone(), ve["stream"][:ve["size"]].clone()
        _say("exact buffers: K size %% 16 = %d, V size %% 16 = %d" % (ke["size"] % 16, ve["size"] % 16))
        for variant in (0, 1, 2):
            want = ops.attn_decode(q, ke, ve, variant=1 if variant == 2 else variant)     # variant 2 falls back to 1
            assert torch.equal(ops.attn_decode(q, ke2, ve2, variant=variant), want)


def test_two_streams_do_not_share_scratch(cuda):
    """The library keeps its scratch memory (attention partials and tile counters, the encoders' look-back state) per
    stream: encodes on one stream and decode steps on another may overlap.  Forty rounds of both at once must give
    the results of running them one after the other."""
    B, Hq, Hkv, T = 4, 32, 8, 4096
    k, v = synth.make_kv(B, Hkv, T, seed=300, device=cuda)
    q = synth.make_q(B, Hq, seed=301, device=cuda)
    ke, ve = ops.k_quant_encode(k, 0.1), ops.v_quant_encode(v, 0.1)
    want_out = ops.attn_decode(q, ke, ve)
    k2, _ = synth.make_kv(B, Hkv, T, seed=302, device=cuda)
    want_enc = ops.k_quant_encode(k2, 0.1)
    torch.cuda.synchronize()
    s_enc, s_att = torch.cuda.Stream(), torch.cuda.Stream()
    outs, encs = [], []
    for _ in range(40):
        with torch.cuda.stream(s_att):
            outs.append(ops.attn_decode(q, ke, ve))
        with torch.cuda.stream(s_enc):
            encs.append(ops.k_quant_encode(k2, 0.1, want_size=False))      # no host synchronisation: the streams overlap
    torch.cuda.synchronize()
    n = want_enc["size"]
    for o in outs:
        assert torch.equal(o, want_out)
    for e in encs:
        assert torch.equal(e["stream"][:n], want_enc["stream"][:n])
        assert torch.equal(e["info"].view(torch.int32), want_enc["info"].view(torch.int32))


def test_stream_release_gives_the_scratch_back(cuda):
    """A stream's workspace (partials, tile counters, encoder state, outgrown buffers) is freed by
    pkv_stream_release and allocated afresh on the next call; results do not change, and a hundred streams that
    come and go leave no memory behind."""
    B, Hq, Hkv, T = 4, 32, 8, 4096
    k, v = synth.make_kv(B, Hkv, T, seed=310, device=cuda)
    q = synth.make_q(B, Hq, seed=311, device=cuda)
    ke, ve = ops.k_quant_encode(k, 0.1), ops.v_quant_encode(v, 0.1)
    want = ops.attn_decode(q, ke, ve)
    torch.cuda.synchronize()
    ops.stream_release(torch.cuda.Stream())                 # a stream the library has never seen: not an error

    def one_stream():
        st = torch.cuda.Stream()
        with torch.cuda.stream(st):
            got = ops.attn_decode(q, ke, ve)
            enc = ops.k_quant_encode(k, 0.1)
        st.synchronize()
        ops.stream_release(st)
        return got, enc

    got, enc = one_stream()
    assert torch.equal(got, want) and enc["size"] == ke["size"]
    del got, enc
    for _ in range(40):                                      # torch hands out streams from a pool of 32 that it creates
        one_stream()                                         # lazily, and the runtime allocates for every new stream
    torch.cuda.synchronize()
    torch.cuda.empty_cache()           # torch caches freed blocks per stream: take them out of the picture
    free0 = torch.cuda.mem_get_info()[0]
    for _ in range(100):
        got, enc = one_stream()
        del got, enc
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    leaked = free0 - torch.cuda.mem_get_info()[0]
    _say("   100 streams created, used and released: free memory moved by %d bytes" % leaked)
    assert leaked < (8 << 20)                                # an unreleased workspace is > 1 MiB per stream
    st = torch.cuda.Stream()                                 # released and used again
    with torch.cuda.stream(st):
        a = ops.attn_decode(q, ke, ve)
        ops.stream_release(st)
        b = ops.attn_decode(q, ke, ve)
    st.synchronize()
    assert torch.equal(a, want) and torch.equal(b, want)
    ops.stream_release(st)


@pytest.mark.parametrize("rel,bits", [(0.05, 5), (0.03, 6)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_attn_decode_wide_codes(cuda, rel, bits, dtype):
    """rel 0.05 gives 22 code levels, rel 0.03 gives 35: 5- and 6-bit codes, outside the reference's format and
    inside this build's extension (three-kernel encode).  The asynchronous-copy kernel takes them with two-token
    windows (variant 0); the plain kernel (variant 1) is the cross-check.  Same contract against
    decompress-then-attend, with a tail window and a context that is not a multiple of the split size."""
    B, Hq, Hkv, T, Tw = 2, 16, 4, 1152, 70
    k, v = synth.make_kv(B, Hkv, T + Tw, seed=180, dtype=dtype)
    q = synth.make_q(B, Hq, seed=181, dtype=dtype)
    k_c, v_c, k_w, v_w = k[:, :, :T].contiguous(), v[:, :, :T].contiguous(), k[:, :, T:].contiguous(), v[:, :, T:].contiguous()
    want = _reference(q, k_c, v_c, rel, rel, k_w, v_w)
    exact = _exact(q, k_c, v_c, rel, rel, k_w, v_w)
    kc, vc = k_c.to(cuda), v_c.to(cuda)
    ke = ops.k_quant_encode(kc, rel)
    ve = ops.v_quant_encode(vc, rel)
    assert ke["bits"] == bits and ve["bits"] == bits
    ck, _, _ = oq.quant_ints(k_c, 64, rel)
    codes = torch.empty(T, B * Hkv * 128, dtype=torch.uint8, device=cuda)
    ops.k_decode(ke["stream"], ke["info"], codes, bits=bits)
    assert torch.equal(codes.cpu(), oq.code_matrix(ck))
    kw, vw = k_w.to(cuda), v_w.to(cuda)
    _say("wide attention case", dtype, "bits", bits)
    outs = _parity(cuda, q, ke, ve, want, exact, dtype, [0, 1], kw, vw, label="%d-bit" % bits)
    _say("  fast vs plain kernel: max diff", (outs[0] - outs[1]).abs().max().item())


@pytest.mark.parametrize("hq", [4, 8, 32])
def test_attn_decode_wide_codes_group_sizes(cuda, hq):
    """The 5-bit path for groups of 1, 2 and 8 query heads per KV head (the case above has 4), no tail window."""
    B, Hkv, T = 1, 4, 640
    k, v = synth.make_kv(B, Hkv, T, seed=185)
    q = synth.make_q(B, hq, seed=186)
    want = _reference(q, k, v, 0.05, 0.05)
    exact = _exact(q, k, v, 0.05, 0.05)
    ke = ops.k_quant_encode(k.to(cuda), 0.05)
    ve = ops.v_quant_encode(v.to(cuda), 0.05)
    assert ke["bits"] == 5 and ve["bits"] == 5
    _say("wide attention case: group of", hq // Hkv)
    _parity(cuda, q, ke, ve, want, exact, torch.float16, [0], label="5-bit, group of %d" % (hq // Hkv))


@pytest.mark.parametrize("rel_k,rel_v,bits", [(0.05, 0.1, (5, 4)), (0.1, 0.05, (4, 5)), (0.03, 0.05, (6, 5)), (0.03, 0.1, (6, 4))])
def test_attn_decode_mixed_widths(cuda, rel_k, rel_v, bits):
    """K and V at different error bounds, one of them (or both) at an extension width: the asynchronous-copy kernel
    windows each side on its own.  Checked against decompress-then-attend and against the plain kernel."""
    B, Hq, Hkv, T = 2, 16, 4, 896
    k, v = synth.make_kv(B, Hkv, T, seed=187)
    q = synth.make_q(B, Hq, seed=188)
    want = _reference(q, k, v, rel_k, rel_v)
    exact = _exact(q, k, v, rel_k, rel_v)
    ke = ops.k_quant_encode(k.to(cuda), rel_k)
    ve = ops.v_quant_encode(v.to(cuda), rel_v)
    assert (ke["bits"], ve["bits"]) == bits
    _say("mixed widths case", bits)
    outs = _parity(cuda, q, ke, ve, want, exact, torch.float16, [0, 1], label="K %d / V %d bits" % bits)
    # the two kernels differ by their own rounding only: twice the allowance of the faster one + an output rounding
    assert (outs[0] - outs[1]).abs().max().item() <= 2 * 5e-4 + 2 ** -10 * outs[1].abs().max().item()


@pytest.mark.parametrize("variant", [0, 1, 2])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_attn_decode_with_values_of_large_and_mixed_magnitude(cuda, dtype, variant):
    """V of large magnitude (v_scale in the thousands: a fixed weight scale overflowed fp16 there) and V whose
    magnitude jumps by 2^17 inside one split (the running exponent of the weight scale grows mid-stream).
    Attention is linear in V and powers of two commute with the quantiser (same codes, scaled parameters), so the
    outputs are held to the usual bounds after division by the power of two that sets the outputs' magnitude."""
    B, Hq, Hkv, T = 2, 16, 4, 1024
    k, v = synth.make_kv(B, Hkv, T, seed=700, dtype=dtype)
    q = synth.make_q(B, Hq, seed=701, dtype=dtype)
    big = 2048.0 if dtype == torch.float16 else 4096.0
    cases = {"large": v.float() * big}
    mixed = v.float().clone()
    mixed[:, :, :192] *= 2.0 ** -6          # the first tile and a half: small values, then 2^11 times larger ones
    mixed[:, :, 192:] *= 2.0 ** 11
    cases["mixed"] = mixed
    ke = ops.k_quant_encode(k.to(cuda), 0.1)
    for name, vv in cases.items():
        vv = vv.to(dtype)
        c = big if name == "large" else 2.0 ** 11
        _say("large-V case", name, dtype, "variant", variant, "max |v| %.0f" % float(vv.abs().max()))
        want = _reference(q, k, vv, 0.1, 0.1).double() / c
        exact = _exact(q, k, vv, 0.1, 0.1) / c
        ve = ops.v_quant_encode(vv.to(cuda), 0.1)
        assert float(ve["scale"].float().max()) > 250.0
        qd = q.to(cuda)
        chk = ops.attn_decode(qd, ke, ve, variant=1, ref_rounding=True, out_f32=True)
        assert bool(torch.isfinite(chk).all())
        check_reference_mode(chk.double().cpu() / c, want, name)
        got = ops.attn_decode(qd, ke, ve, variant=variant)
        assert bool(torch.isfinite(got).all()), (name, variant)
        check_fast(got.double().cpu() / c, want, exact, dtype, variant, label="%s variant %d" % (name, variant))


@pytest.mark.parametrize("variant", [0, 1, 2])
def test_attn_decode_survives_damaged_block_info(cuda, variant):
    """block_info entries that point outside the streams or claim absurd sizes: the step returns (with arbitrary
    numbers for the heads concerned); no kernel reads outside the buffers it was given."""
    dtype = torch.float16
    B, Hq, Hkv, T = 2, 16, 4, 1024
    k, v = synth.make_kv(B, Hkv, T, seed=77, dtype=dtype)
    q = synth.make_q(B, Hq, seed=78, dtype=dtype).to(cuda)
    ke = ops.k_quant_encode(k.to(cuda), 0.1)
    ve = ops.v_quant_encode(v.to(cuda), 0.1)
    good = ops.attn_decode(q, ke, ve, variant=variant).float().cpu()
    for side in (ke, ve):
        info = side["info"].cpu().numpy().astype(np.int64)
        info[1] = (side["stream"].numel() + 4096, 3000)
        info[10] = (0xFFFFFFF0, 0xFFFFFFFF)
        info[17] = (side["size"] - 5, 0xFFFF)
        side["info"] = torch.from_numpy(info.astype(np.uint32)).to(cuda)
    got = ops.attn_decode(q, ke, ve, variant=variant)
    torch.cuda.synchronize()
    assert got.shape == good.shape
    # blocks 1, 10, 17 belong to (sequence, KV head) (0, 1), (0, 2), (0, 1) in K's block_info [8 blocks per 64 tokens]
    # and to (0, 0), (1, 1), (0, 0) in V's [16 per 128 tokens]: KV heads 0 and 3 of sequence 1 are untouched
    G = Hq // Hkv
    for h in (0, 3):
        assert torch.equal(got.float().cpu()[1, h * G:(h + 1) * G], good[1, h * G:(h + 1) * G])
