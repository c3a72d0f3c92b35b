"""Token repacking and the analytic size model on the device against the NumPy restatement (oracle/repack.py):
integers throughout, so everything is compared exactly."""
import numpy as np
import pytest
import torch

from oracle import quant as oq
from oracle import repack as orp
from packkv_amd import ops, synth

from attn_bounds import check_fast, check_reference_mode

pytestmark = pytest.mark.gpu


def _say(*a):
    print(*a, flush=True)


def _codes(B, H, T, rel, seed, k_mode="outliers"):
    k, v = synth.make_kv(B, H, T, seed=seed, k_mode=k_mode)
    ck, _, _ = oq.quant_ints(k, 64, rel)
    cv, _, _ = oq.quant_ints(v, 64, rel)
    return oq.code_matrix(ck), oq.code_matrix(cv)


@pytest.mark.parametrize("rel", [0.1, 0.05, 0.02])
def test_bit_pack_sizes_match_for_every_pack_length(cuda, rel):
    """rel 0.05 / 0.02 give code widths up to 6 / 7 bits: the size model has no width limit."""
    kc, vc = _codes(1, 8, 2048, rel, seed=130, k_mode="channel_scale")
    kd, vd = kc.to(cuda), vc.to(cuda)
    blocks = orp.blocks_from_code_matrices(kc.numpy(), vc.numpy(), 64)
    for pack_len in (16, 32, 64, 128, 256):
        want = orp.bit_pack(blocks, pack_len)
        got = ops.bit_pack(kd, vd, pack_len)
        _say("bit_pack case rel", rel, "pack", pack_len, "->", got, "max code", int(kc.max()), int(vc.max()))
        assert got == want


def test_code_stats_shapes_against_closed_forms(cuda):
    """Narrow, wide and very long code matrices (more packs along the context than one grid dimension holds, fewer
    items than one workgroup, 16 channels, byte values up to 255) against numpy on the same codes."""
    rng = np.random.default_rng(77)
    for (T, hid, top, pack) in ((65552 * 16, 16, 32, 16), (48, 16, 256, 16), (4096, 1024, 40, 32), (512, 16384, 6, 64),
                                (640, 48, 256, 128)):
        _say("code_stats case", T, hid, top, pack)
        c = rng.integers(0, top, size=(T, hid), dtype=np.uint8)
        c[T // 2, hid // 3] = top - 1
        r = c.reshape(T // pack, pack, hid).astype(np.int64)
        span = r.max(axis=1) - r.min(axis=1)
        want = (int(np.where(span > 0, np.floor(np.log2(np.maximum(span, 1))) + 1, 0).sum()), int(np.unique(c).size))
        assert ops.code_stats(torch.from_numpy(c).to(cuda), pack) == want


def test_median_repacking_matches_restatement(cuda):
    for (B, H, T, bs) in ((1, 2, 256, 64), (2, 8, 512, 64), (1, 1, 384, 128), (3, 2, 128, 16)):
        _say("repack case", B, H, T, bs)
        kc, vc = _codes(B, H, T, 0.1, seed=140 + B)
        blocks = orp.blocks_from_code_matrices(kc.numpy(), vc.numpy(), bs)
        want, order = orp.median_repacking(blocks)
        k_out, v_out, perm = ops.median_repacking(kc.to(cuda), vc.to(cuda), bs)
        hid = kc.shape[1]
        assert (perm.cpu().numpy().reshape(-1, bs) == order).all()
        assert (k_out.cpu().numpy().reshape(-1, bs, hid) == want[:, :, :hid]).all()
        assert (v_out.cpu().numpy().reshape(-1, bs, hid) == want[:, :, hid:]).all()
        for pack in (16, 64):
            assert ops.repack_and_encode(kc.to(cuda), vc.to(cuda), pack, "median", bs) == \
                   orp.repack_and_encode(kc.numpy(), vc.numpy(), pack, "median", bs)
            assert ops.repack_and_encode(kc.to(cuda), vc.to(cuda), pack, "none", bs) == \
                   orp.repack_and_encode(kc.numpy(), vc.numpy(), pack, "none", bs)


def test_repacked_codes_encode_and_round_trip(cuda):
    """Repacked code matrices go through the codecs like any other: stream decodes to the repacked codes, and the
    real K stream of 16-token packs is priced by bit_pack up to the block headers."""
    B, H, T = 1, 8, 512
    kc, vc = _codes(B, H, T, 0.1, seed=150)
    k_rep, v_rep, _ = ops.median_repacking(kc.to(cuda), vc.to(cuda), 64)
    hid = kc.shape[1]
    stream = torch.empty(T * hid, dtype=torch.uint8, device=cuda)
    info = torch.empty((T // 64) * (hid // 128), 2, dtype=torch.uint32, device=cuda)
    size = ops.k_encode(k_rep, stream, info, bits=4)
    back = torch.empty_like(k_rep)
    ops.k_decode(stream, info, back, bits=4)
    assert torch.equal(back, k_rep)
    # real stream = analytic payload and metadata (4 + 3 bits per pack at W = 4) + 8 header bytes per block
    n_packs = (T // 16) * hid
    analytic_bits = ops.bit_pack_bytes(k_rep, 16) * 8
    w = int(np.ceil(np.log2(len(torch.unique(k_rep)))))
    payload_bits = analytic_bits - n_packs * (w + int(np.ceil(np.log2(w + 1))))
    assert abs(size - ((payload_bits + n_packs * 7) // 8 + 8 * info.size(0))) <= 1


def test_full_size_properties(cuda):
    """configs[2] shape (8 KV heads x 128 x 16384 tokens): the oracle is slow there, so check what must hold:
    perm is a permutation inside every block, rows move with it, medians come out non-increasing, and repacking
    leaves the multiset of codes (hence the histogram and W) unchanged."""
    T, hid, bs = 16384, 1024, 64
    g = torch.Generator(device="cpu").manual_seed(160)
    kc = torch.randint(0, 16, (T, hid), dtype=torch.uint8, generator=g).to(cuda)
    vc = (torch.randn(T, 1, generator=g).mul(2).add(8).round().clamp(0, 15) +
          torch.randint(-2, 3, (T, hid), generator=g)).clamp(0, 15).to(torch.uint8).to(cuda)
    k_out, v_out, perm = ops.median_repacking(kc, vc, bs)
    p = perm.view(-1, bs).long()
    assert torch.equal(torch.sort(p, dim=1).values, torch.arange(bs, device=cuda).expand_as(p))
    src = (torch.arange(T, device=cuda).view(-1, bs)[:, :1] + p).view(-1)
    assert torch.equal(k_out, kc[src]) and torch.equal(v_out, vc[src])
    med = torch.median(v_out.view(-1, bs, hid).to(torch.int16), dim=2).values
    assert (med[:, :-1] >= med[:, 1:]).all()
    assert torch.equal(torch.bincount(v_out.view(-1).long(), minlength=16), torch.bincount(vc.view(-1).long(), minlength=16))
    assert ops.bit_pack_bytes(v_out, 16) <= ops.bit_pack_bytes(vc, 16)     # sorting by level helps this input


def test_median_repacking_wide_codes_and_wide_rows(cuda):
    """Codes of 128 and above and rows longer than 16384 channels take the kernel's histogram path; a row of
    exactly 16384 codes below 128 fills the register path completely."""
    g = torch.Generator(device="cpu").manual_seed(170)
    for (T, hid, top, bs) in ((128, 256, 256, 64), (64, 32768, 16, 64), (64, 16384, 128, 32), (128, 1040, 100, 64)):
        _say("repack wide case", T, hid, top, bs)
        kc = torch.randint(0, top, (T, hid), dtype=torch.uint8, generator=g)
        vc = torch.randint(0, top, (T, hid), dtype=torch.uint8, generator=g)
        vc[::3] //= 2                                   # spread the medians
        blocks = orp.blocks_from_code_matrices(kc.numpy(), vc.numpy(), bs)
        want, order = orp.median_repacking(blocks)
        k_out, v_out, perm = ops.median_repacking(kc.to(cuda), vc.to(cuda), bs)
        assert (perm.cpu().numpy().reshape(-1, bs) == order).all()
        assert (v_out.cpu().numpy().reshape(-1, bs, hid) == want[:, :, hid:]).all()
        assert (k_out.cpu().numpy().reshape(-1, bs, hid) == want[:, :, :hid]).all()


def test_greedy_repacking_matches_restatement(cuda):
    """The greedy order (seed by cosine to the rounded mean, then fewest added bits) on the device against the
    integer restatement: same permutation, same rows, same priced sizes; quantised K/V and plain random codes
    (which tie often: ties must go to the earlier token on both sides)."""
    cases = []
    for (B, H, T, bs, pack) in ((1, 2, 256, 64, 16), (2, 4, 256, 64, 16), (1, 1, 128, 32, 8), (1, 2, 128, 64, 64)):
        kc, vc = _codes(B, H, T, 0.1, seed=240 + B + H)
        cases.append((kc, vc, bs, pack, "quantised %dx%dx%d" % (B, H, T)))
    g = torch.Generator(device="cpu").manual_seed(241)
    # (the last two have more blocks than the device holds at once as groups of workgroups: 72 blocks of 8 slices and
    # 520 blocks of one slice, so a group walks several blocks)
    for (T, hid, top, bs, pack) in ((64, 16, 4, 16, 4), (128, 48, 2, 64, 16), (256, 2064, 200, 256, 32), (64, 32768, 16, 64, 16),
                                    (576, 8192, 6, 8, 4), (33280, 128, 6, 64, 16),
                                    # two slices with blocks of 32 tokens; a last slice of 32 channels only; 8-bit codes in two slices
                                    (96, 4096, 5, 32, 8), (128, 2064, 9, 64, 16), (64, 4096, 256, 64, 32)):
        kc = torch.randint(0, top, (T, hid), dtype=torch.uint8, generator=g)
        vc = torch.randint(0, top, (T, hid), dtype=torch.uint8, generator=g)
        cases.append((kc, vc, bs, pack, "random %dx%d below %d" % (T, hid, top)))
    zero = torch.zeros(64, 128, dtype=torch.uint8)
    cases.append((zero, zero.clone(), 64, 16, "all zero"))
    for kc, vc, bs, pack, name in cases:
        _say("greedy case", name, "block", bs, "pack", pack)
        hid = kc.shape[1]
        blocks = orp.blocks_from_code_matrices(kc.numpy(), vc.numpy(), bs)
        want, order = orp.greedy_repacking(blocks, pack)
        k_out, v_out, perm = ops.greedy_repacking(kc.to(cuda), vc.to(cuda), pack, bs)
        assert (perm.cpu().numpy().reshape(-1, bs) == order).all()
        assert (k_out.cpu().numpy().reshape(-1, bs, hid) == want[:, :, :hid]).all()
        assert (v_out.cpu().numpy().reshape(-1, bs, hid) == want[:, :, hid:]).all()
        if kc.max() > 0:
            assert ops.repack_and_encode(kc.to(cuda), vc.to(cuda), pack, "greedy", bs) == \
                   orp.repack_and_encode(kc.numpy(), vc.numpy(), pack, "greedy", bs)


def test_greedy_repacking_shrinks_shifted_tokens_and_feeds_attention(cuda):
    """Tokens with a token-wise level shift: grouping similar tokens must shrink the priced V size, and the cache
    encoded in greedy order must attend like the cache in natural order (attention ignores token order)."""
    B, Hq, Hkv, T = 1, 8, 2, 512
    k, v = synth.make_kv(B, Hkv, T, seed=250)
    g = torch.Generator().manual_seed(251)
    v = (v.float() * 0.3 + torch.randn(1, 1, T, 1, generator=g) * 2.0).to(torch.float16)
    q = synth.make_q(B, Hq, seed=252)
    kd, vd = k.to(cuda), v.to(cuda)
    ke, ve, perm = ops.repack_quant_encode(kd, vd, 0.1, 0.1, "greedy")
    kn, vn, _ = ops.repack_quant_encode(kd, vd, 0.1, 0.1, "none")
    assert sorted(perm.cpu().numpy().reshape(-1, 64)[0].tolist()) == list(range(64))
    _say("greedy sizes", ke["size"], ve["size"], "natural", kn["size"], vn["size"])
    assert ve["size"] < vn["size"]
    out_g = ops.attn_decode(q.to(cuda), ke, ve).float().cpu()
    out_n = ops.attn_decode(q.to(cuda), kn, vn).float().cpu()
    diff = (out_g - out_n).abs().max().item()
    _say("greedy order vs natural order: max|diff| = %.2e, max|out| = %.2e" % (diff, out_n.abs().max().item()))
    assert diff <= 2 ** -9 * max(out_n.abs().max().item(), 1.0)      # the same terms in another order: an output rounding or two apart


def test_repacked_cache_attends_like_the_original(cuda):
    """Attention does not depend on the order of the cached tokens, so a cache whose 64-token blocks were reordered
    by median repacking (K, V and their per-token parameters together) must give the output of the cache in natural
    order, and both must meet the contract against decompress-then-attend."""
    B, Hq, Hkv, T = 2, 16, 4, 1024
    k, v = synth.make_kv(B, Hkv, T, seed=190)
    g = torch.Generator().manual_seed(191)
    v = (v.float() * 0.3 + torch.randn(1, 1, T, 1, generator=g) * 2.0).to(torch.float16)   # token-wise level shift
    q = synth.make_q(B, Hq, seed=192)
    ck, zk, sk = oq.quant_ints(k, 64, 0.1)
    cv, zv, sv = oq.quant_ints(v, 64, 0.1)
    want = oq.attention_f32(q.unsqueeze(2), oq.dequant(ck, zk, sk), oq.dequant(cv, zv, sv)).squeeze(2).double().numpy()
    kd, vd, qd = k.to(cuda), v.to(cuda), q.to(cuda)
    kr, vr, perm = ops.repack_quant_encode(kd, vd, 0.1, 0.1, "median")
    kn, vn, ident = ops.repack_quant_encode(kd, vd, 0.1, 0.1, "none")
    assert torch.equal(ident.view(-1, 64), torch.arange(64, dtype=torch.int32, device=cuda).expand(T // 64, 64))
    plain_k = ops.k_quant_encode(kd, 0.1)
    assert kn["size"] == plain_k["size"] and torch.equal(kn["stream"][:kn["size"]], plain_k["stream"][:kn["size"]])
    # the repacked streams hold the oracle's repacked codes
    blocks = orp.blocks_from_code_matrices(oq.code_matrix(ck).numpy(), oq.code_matrix(cv).numpy(), 64)
    rep, order = orp.median_repacking(blocks)
    assert (perm.cpu().numpy().reshape(-1, 64) == order).all()
    hid = B * Hkv * 128
    codes = torch.empty(T, hid, dtype=torch.uint8, device=cuda)
    ops.v_decode(vr["stream"], vr["info"], codes, bits=vr["bits"])
    assert (codes.cpu().numpy().reshape(-1, 64, hid) == rep[:, :, hid:]).all()
    assert vr["size"] <= vn["size"]                      # tokens of similar level side by side: no wider packs
    out_r = ops.attn_decode(qd, kr, vr).double().cpu().numpy()
    out_n = ops.attn_decode(qd, kn, vn).double().cpu().numpy()
    _say("repacked cache: V bytes %d -> %d, max|out_r - out_n| = %.2e" % (vn["size"], vr["size"], np.abs(out_r - out_n).max()))
    exact = oq.attention_f64_np(q.unsqueeze(2), ((ck.double() + zk.double()) * sk.double()).reshape(k.shape),
                                ((cv.double() + zv.double()) * sv.double()).reshape(v.shape)).squeeze(2)
    for name, (ke_, ve_), out in (("repacked", (kr, vr), out_r), ("natural order", (kn, vn), out_n)):
        chk = ops.attn_decode(qd, ke_, ve_, variant=1, ref_rounding=True, out_f32=True)
        check_reference_mode(chk, want, name)          # the contract, on the checking mode
        check_fast(out, want, exact, torch.float16, label=name)
    # the two orders add the same terms in a different sequence: at most an output rounding apart
    assert np.abs(out_r - out_n).max() <= 2 ** -10 * np.abs(out_n).max()


def test_pack_sweep_rows_match_restatement(cuda):
    """The sweep mode of bench.py (pack sizes x code widths x repacking methods on one layer) on a small layer:
    every row's sizes equal the restated size model on the restated quantiser's codes, and the real codec's stream at
    every pack length (bench.py asserts it while it runs) is that model's bytes plus 8 per block."""
    import importlib.util
    import os
    spec = importlib.util.spec_from_file_location("bench_mod", os.path.join(os.path.dirname(__file__), "..", "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    H, T = 2, 2048
    k, v = synth.make_kv(1, H, T, seed=2, k_mode="channel_scale")
    rels, packs = (0.2, 0.05, 0.0125), (16, 64, 256)
    res = bench.pack_sweep(torch, H, T, cuda, rels=rels, packs=packs, kv=(k.to(cuda), v.to(cuda)))
    assert len(res["rows"]) == len(rels) * len(packs) * 3 and len(res["codec"]) == len(rels) * len(packs)
    mats = {}
    for rel in rels:
        ck, _, _ = oq.quant_ints(k, 64, rel)
        cv, _, _ = oq.quant_ints(v, 64, rel)
        mats[rel] = (oq.code_matrix(ck).numpy(), oq.code_matrix(cv).numpy())
    for row in res["rows"]:
        _say("sweep row", row["rel"], row["pack"], row["method"])
        kc, vc = mats[row["rel"]]
        want = orp.repack_and_encode(kc, vc, row["pack"], row["method"], row["block"])
        assert (row["k_bytes"], row["v_bytes"]) == (want[2], want[3])
        assert row["bits"] >= int(max(kc.max(), vc.max())).bit_length()
    for c in res["codec"]:
        none = [r for r in res["rows"] if (r["rel"], r["pack"], r["method"]) == (c["rel"], c["pack"], "none")][0]
        nk, nv = (T // (4 * c["pack"])) * H, (T // (8 * c["pack"])) * 2 * H
        assert (c["k_stream_bytes"] - 8 * nk, c["v_stream_bytes"] - 8 * nv) == (none["k_bytes"], none["v_bytes"])
        assert c["k_cr"] > 1.0 and c["v_cr"] > 1.0 and c["k_decode_gbs_codes"] > 0


def _same_encoding(a, b, label):
    assert a["size"] == b["size"], label
    assert torch.equal(a["info"], b["info"]), label
    assert torch.equal(a["stream"][:a["size"]], b["stream"][:b["size"]]), label
    assert torch.equal(a["scale"].view(torch.int16), b["scale"].view(torch.int16)), label
    assert torch.equal(a["zero"].view(torch.int16), b["zero"].view(torch.int16)), label


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_median_repack_inside_the_fused_encode_equals_the_code_matrix_path(cuda, dtype):
    """repack_quant_encode("median") with the order counted straight from V and the fused encoders gathering the
    permuted rows (no code matrix) against the path through the code matrices (quantize, median repack, block codec):
    the same permutation, streams, block_info and parameters.  The permutation is also checked against the NumPy
    restatement on the restated quantiser's codes."""
    cases = [(2, 4, 512, 0.1, 0.1, 64), (3, 8, 256, 0.2, 0.05, 64), (1, 2, 1024, 0.1, 0.2, 128), (2, 8, 512, 0.05, 0.1, 256),
             (1, 1, 256, 0.5, 0.1, 64), (2, 8, 256, 0.03, 0.03, 64)]      # the last: 6-bit codes, the widest the fused path takes
    for n, (B, H, T, k_rel, v_rel, bs) in enumerate(cases):
        _say("fused median case", dtype, B, H, T, k_rel, v_rel, bs)
        k, v = synth.make_kv(B, H, T, seed=300 + n)
        g = torch.Generator().manual_seed(400 + n)
        v = v.float() * 0.4 + torch.randn(1, 1, T, 1, generator=g) * 1.5       # token-wise level shifts: medians differ
        if n == 0 and dtype == torch.float16:
            # every third token far from zero with a small range: its zero point (about 100 / (range * rel)) leaves
            # the span of the usual quantisation sequence, so wavefronts hold tokens of both kinds
            v[:, :, ::3] = 100.0 + 0.1 * torch.randn(B, H, (T + 2) // 3, 128, generator=g)
            k[:, :, 1::3] = -60.0 + 0.05 * torch.randn(B, H, (T + 1) // 3, 128, generator=g)
        k, v = k.to(dtype), v.to(dtype)
        kd, vd = k.to(cuda), v.to(cuda)
        kf, vf, pf = ops.repack_quant_encode(kd, vd, k_rel, v_rel, "median", bs, fused=True)
        km, vm, pm = ops.repack_quant_encode(kd, vd, k_rel, v_rel, "median", bs, fused=False)
        assert torch.equal(pf.view(torch.int32), pm.view(torch.int32))
        assert not torch.equal(pf.view(-1, bs), torch.arange(bs, dtype=torch.int32, device=cuda).expand(T // bs, bs))
        _same_encoding(kf, km, "K")
        _same_encoding(vf, vm, "V")
        cv, _, _ = oq.quant_ints(v, 64, v_rel)
        ck, _, _ = oq.quant_ints(k, 64, k_rel)
        blocks = orp.blocks_from_code_matrices(oq.code_matrix(ck).numpy(), oq.code_matrix(cv).numpy(), bs)
        _, order = orp.median_repacking(blocks)
        assert np.array_equal(pf.cpu().numpy().reshape(-1, bs), order)
    # the default takes the fused path where it applies and the code matrices elsewhere (here: 7-bit codes)
    k, v = synth.make_kv(1, 2, 256, seed=9)
    a = ops.repack_quant_encode(k.to(cuda), v.to(cuda), 0.1, 0.0125, "median")
    b = ops.repack_quant_encode(k.to(cuda), v.to(cuda), 0.1, 0.0125, "median", fused=False)
    _same_encoding(a[0], b[0], "K 7-bit V")
    _same_encoding(a[1], b[1], "V 7-bit")
    with pytest.raises(Exception):
        ops.repack_quant_encode(k.to(cuda), v.to(cuda), 0.1, 0.0125, "median", fused=True)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_greedy_order_inside_the_fused_encode_equals_the_code_matrix_path(cuda, dtype):
    """repack_quant_encode("greedy") with the fused encoders gathering the rows in the greedy order (the code matrices
    serve the order only) against the path that repacks the code matrices and runs the block codec: the same
    permutation, streams, block_info and parameters; the permutation also against the restatement."""
    cases = [(2, 4, 512, 0.1, 0.1, 64), (1, 8, 256, 0.2, 0.05, 64), (1, 2, 512, 0.1, 0.2, 128), (3, 8, 256, 0.1, 0.1, 256)]
    for n, (B, H, T, k_rel, v_rel, bs) in enumerate(cases):
        _say("fused greedy case", dtype, B, H, T, k_rel, v_rel, bs)
        k, v = synth.make_kv(B, H, T, seed=500 + n)
        g = torch.Generator().manual_seed(600 + n)
        v = v.float() * 0.4 + torch.randn(1, 1, T, 1, generator=g) * 1.5       # token-wise level shifts: an order that matters
        k, v = k.to(dtype), v.to(dtype)
        kd, vd = k.to(cuda), v.to(cuda)
        kf, vf, pf = ops.repack_quant_encode(kd, vd, k_rel, v_rel, "greedy", bs, fused=True)
        km, vm, pm = ops.repack_quant_encode(kd, vd, k_rel, v_rel, "greedy", bs, fused=False)
        assert torch.equal(pf.view(torch.int32), pm.view(torch.int32))
        assert not torch.equal(pf.view(-1, bs), torch.arange(bs, dtype=torch.int32, device=cuda).expand(T // bs, bs))
        _same_encoding(kf, km, "K")
        _same_encoding(vf, vm, "V")
        cv, _, _ = oq.quant_ints(v, 64, v_rel)
        ck, _, _ = oq.quant_ints(k, 64, k_rel)
        blocks = orp.blocks_from_code_matrices(oq.code_matrix(ck).numpy(), oq.code_matrix(cv).numpy(), bs)
        _, order = orp.greedy_repacking(blocks, 16)
        assert np.array_equal(pf.cpu().numpy().reshape(-1, bs), order)


def test_fused_median_repack_at_the_benchmark_shape(cuda):
    """16 sequences x 8 KV heads x 32768 tokens: the fused path's streams decode (unpack kernels) to codes whose
    every 64-token block is the natural-order block permuted by perm, and the medians along the new order descend."""
    B, H, T = 16, 8, 32768
    k, v = synth.make_kv(B, H, T, seed=0, device=cuda)
    kf, vf, perm = ops.repack_quant_encode(k, v, 0.1, 0.1, "median")
    kn, vn = ops.k_quant_encode(k, 0.1), ops.v_quant_encode(v, 0.1)
    del k, v
    hidden = B * H * 128
    src = (torch.arange(T, device=cuda) // 64) * 64 + perm.to(torch.int64)
    assert torch.equal(torch.sort(perm.view(-1, 64).to(torch.int64), dim=1).values,
                       torch.arange(64, device=cuda).expand(T // 64, 64))
    for (f, n, dec) in ((kf, kn, ops.k_decode), (vf, vn, ops.v_decode)):
        cf = torch.empty(T, hidden, dtype=torch.uint8, device=cuda)
        cn = torch.empty(T, hidden, dtype=torch.uint8, device=cuda)
        dec(f["stream"], f["info"], cf, bits=f["bits"])
        dec(n["stream"], n["info"], cn, bits=n["bits"])
        for lo in range(0, T, 8192):
            assert torch.equal(cf[lo:lo + 8192], cn[src[lo:lo + 8192]])
        assert torch.equal(f["scale"], n["scale"][:, src]) and torch.equal(f["zero"].view(torch.int16), n["zero"][:, src].view(torch.int16))
        med = torch.sort(cf[:4096].to(torch.int16), dim=1).values[:, (hidden - 1) // 2] if dec is ops.v_decode else None
        if med is not None:
            m = med.view(-1, 64)
            assert bool((m[:, 1:] <= m[:, :-1]).all())
        del cf, cn
