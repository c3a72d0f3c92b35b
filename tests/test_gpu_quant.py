"""GPU parity of the quantizer and the fused quantize+encode kernels: integer codes, scale, zero,
dequantised values and the packed stream are bit-exact against the CPU oracle."""
import numpy as np
import pytest
import torch

from oracle import quant as oq
from packkv_amd import ops, synth

pytestmark = pytest.mark.gpu


def _say(*a):
    print(*a, flush=True)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("rel", [0.1, 0.2, 0.14])
def test_quantizer_bit_exact(cuda, dtype, rel):
    B, H, T = 2, 8, 256
    k, v = synth.make_kv(B, H, T, seed=21, dtype=dtype)
    for name, x in (("k", k), ("v", v)):
        _say("quant case", name, dtype, rel)
        c, z, s = oq.quant_ints(x, 64, rel)
        want_codes = oq.code_matrix(c)
        xd = x.to(cuda)
        scale, zero = ops.quant_params(xd, rel)
        assert torch.equal(scale.cpu().view(torch.int16), s.reshape(B, T).view(torch.int16))
        assert torch.equal(zero.cpu().view(torch.int16), z.reshape(B, T).view(torch.int16))
        codes, mx = ops.quantize(xd, scale, zero)
        assert torch.equal(codes.cpu(), want_codes)
        assert mx == int(want_codes.max())
        y = ops.dequantize(codes, scale, zero, B, H)
        want_y = oq.dequant(c, z, s)
        assert torch.equal(y.cpu().view(torch.int16), want_y.view(torch.int16))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_fused_quant_encode_stream_bit_exact(cuda, oracle_codec, dtype):
    for (B, H, T, rel) in ((1, 2, 128, 0.1), (2, 8, 256, 0.1), (1, 32, 128, 0.1), (2, 4, 256, 0.2), (1, 8, 128, 0.34),
                           (1, 3, 128, 0.1), (2, 5, 256, 0.14), (3, 1, 128, 0.1),
                           # five to eight heads: the kernels that read x once as cells (unused head slots repeat a head)
                           (1, 6, 256, 0.1), (3, 7, 128, 0.2), (2, 7, 256, 0.05), (1, 6, 128, 0.03),
                           # few heads: several groups to a workgroup, the last workgroup partly filled
                           (3, 2, 384, 0.1), (5, 1, 256, 0.1), (3, 3, 384, 0.2), (3, 4, 128, 0.1),
                           # widths 5 and 6 (format extension): cells / round-major kernels up to eight heads, runs of eight beyond
                           (2, 8, 256, 0.05), (1, 4, 384, 0.03), (1, 3, 128, 0.05), (1, 16, 128, 0.05), (2, 12, 256, 0.03)):
        k, v = synth.make_kv(B, H, T, seed=31 + H, dtype=dtype)
        for is_k, x in ((1, k), (0, v)):
            _say("fused quant+encode", "K" if is_k else "V", dtype, B, H, T, rel)
            c, z, s = oq.quant_ints(x, 64, rel)
            cm = oq.code_matrix(c).numpy()
            W = ops.bits_for_rel(rel)
            assert oq.bits_for_codes(torch.from_numpy(cm)) <= W
            cb, hb = (64, 128) if is_k else (128, 64)
            so, io, zo = oracle_codec.encode(is_k, cm, cb, hb, W)
            r = (ops.k_quant_encode if is_k else ops.v_quant_encode)(x.to(cuda), rel, W)
            assert r["size"] == zo
            assert np.array_equal(r["info"].cpu().numpy(), io)
            assert np.array_equal(r["stream"][:zo].cpu().numpy(), so[:zo])
            assert torch.equal(r["scale"].cpu().view(torch.int16), s.reshape(B, T).view(torch.int16))
            assert torch.equal(r["zero"].cpu().view(torch.int16), z.reshape(B, T).view(torch.int16))


def test_fused_quant_encode_more_than_eight_heads(cuda, oracle_codec):
    """More than eight KV heads: the heads of a (context block, sequence) are cut into runs of eight, one workgroup
    each, that exchange their minima and maxima through memory; hundreds of runs in flight, groups of 3, 4 and 5 runs,
    a last run of fewer than eight heads."""
    for (B, H, T, rel, dtype) in ((4, 32, 2048, 0.1, torch.float16), (2, 24, 1024, 0.2, torch.bfloat16),
                                  (1, 40, 512, 0.1, torch.float16), (3, 20, 512, 0.05, torch.float16)):
        k, v = synth.make_kv(B, H, T, seed=3 + H, dtype=dtype)
        for is_k, x in ((1, k), (0, v)):
            _say("fused quant+encode, many heads", "K" if is_k else "V", dtype, B, H, T, rel)
            c, z, s = oq.quant_ints(x, 64, rel)
            cm = oq.code_matrix(c).numpy()
            W = ops.bits_for_rel(rel)
            cb, hb = (64, 128) if is_k else (128, 64)
            so, io, zo = oracle_codec.encode(is_k, cm, cb, hb, W)
            for rep in range(2):                      # (twice: the exchange words of the first call must not leak into the second)
                r = (ops.k_quant_encode if is_k else ops.v_quant_encode)(x.to(cuda), rel, W)
                assert r["size"] == zo
                assert np.array_equal(r["info"].cpu().numpy(), io)
                assert np.array_equal(r["stream"][:zo].cpu().numpy(), so[:zo])
                assert torch.equal(r["scale"].cpu().view(torch.int16), s.reshape(B, T).view(torch.int16))
                assert torch.equal(r["zero"].cpu().view(torch.int16), z.reshape(B, T).view(torch.int16))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_fused_quant_encode_offset_rows_bit_exact(cuda, oracle_codec, dtype):
    """Rows far from zero: the zero point is large (here about -750 and +750, and a few hundred for the smaller
    shift), which takes the encoders' general rounding sequence for some tokens and the short one for others;
    ties (quotients at exactly k + 0.5) are common because the shifted fp16 values are multiples of 0.5."""
    B, H, T, rel = 2, 4, 256, 0.1
    k, v = synth.make_kv(B, H, T, seed=77)
    shift = torch.zeros(B, 1, T, 1)
    big, small = (600.0, 150.0) if dtype == torch.float16 else (48.0, 12.0)    # bf16 keeps 8 bits: stay where it resolves the rows
    shift[:, :, 0:128:3] = -big          # first half: every 16-token round holds tokens of both kinds
    shift[:, :, 1:128:3] = big
    shift[:, :, 2:128:6] = small
    shift[:, :, 128::2] = big            # second half: large positive zero points only (the short sequence)
    shift[:, :, 129::4] = small
    for is_k, x0 in ((1, v), (0, v)):          # unit-variance rows, so that the codes stay within 4 bits
        x = (x0.float() + shift).to(dtype)
        c, z, s = oq.quant_ints(x, 64, rel)
        zi = z.float().flatten()
        if dtype == torch.float16:
            assert (zi.abs() > 600).any() and (zi.abs() < 400).any()
        else:
            assert (zi.abs() > 40).any()
        cm = oq.code_matrix(c).numpy()
        assert int(cm.max()) <= 15
        cb, hb = (64, 128) if is_k else (128, 64)
        so, io, zo = oracle_codec.encode(is_k, cm, cb, hb, 4)
        r = (ops.k_quant_encode if is_k else ops.v_quant_encode)(x.to(cuda), rel, 4)
        assert r["size"] == zo
        assert np.array_equal(r["stream"][:zo].cpu().numpy(), so[:zo])
        assert torch.equal(r["zero"].cpu().view(torch.int16), z.reshape(B, T).view(torch.int16))
        codes, _ = ops.quantize(x.to(cuda), r["scale"], r["zero"])
        assert np.array_equal(codes.cpu().numpy(), cm)


def test_code_wider_than_bits_is_reported(cuda):
    k, _ = synth.make_kv(1, 2, 128, seed=5)
    with pytest.raises(ops.PackKVError) as e:
        ops.k_quant_encode(k.to(cuda), 0.1, 3)     # codes reach 10..11: needs 4 bits
    assert e.value.code == 1 and "does not fit" in str(e.value)


@pytest.mark.gpu
def test_fused_quant_encode_round_trip_medium(cuda):
    """Size-independent property at a size the CPU oracle would take minutes for: unpacking the fused
    encoder's stream gives back exactly the codes of the stand-alone quantizer."""
    B, H, T, rel = 4, 8, 4096, 0.1
    k, v = synth.make_kv(B, H, T, seed=77)
    for is_k, x in ((True, k), (False, v)):
        x = x.to(cuda)
        r = (ops.k_quant_encode if is_k else ops.v_quant_encode)(x, rel, 4)
        scale, zero = ops.quant_params(x, rel)
        assert torch.equal(scale, r["scale"]) and torch.equal(zero, r["zero"])
        codes, _ = ops.quantize(x, scale, zero)
        back = torch.empty_like(codes)
        if is_k:
            ops.k_decode(r["stream"], r["info"], back, 64, 128, 4)
        else:
            ops.v_decode(r["stream"], r["info"], back, 128, 64, 4)
        assert torch.equal(back, codes)


@pytest.mark.gpu
def test_fused_quant_encode_round_trip_full_size(cuda):
    """The benchmark workload itself (16 x 8 heads x 32768 tokens, 1 GiB of fp16 per tensor): block_info tiles the
    stream without gaps, and unpacking the stream reproduces the stand-alone quantizer's codes."""
    B, H, T, rel = 16, 8, 32768, 0.1
    k, v = synth.make_kv(B, H, T, seed=0, device=cuda)
    for is_k, x in ((True, k), (False, v)):
        r = (ops.k_quant_encode if is_k else ops.v_quant_encode)(x, rel, 4)
        info = r["info"].view(-1, 2).to(torch.int64)
        assert int(info[0, 0]) == 0
        assert torch.equal(info[1:, 0], torch.cumsum(info[:-1, 1], 0))          # back to back, in block order
        assert int(info[-1, 0] + info[-1, 1]) == r["size"]
        scale, zero = ops.quant_params(x, rel)
        assert torch.equal(scale, r["scale"]) and torch.equal(zero, r["zero"])
        codes, _ = ops.quantize(x, scale, zero)
        back = torch.empty_like(codes)
        if is_k:
            ops.k_decode(r["stream"], r["info"], back, 64, 128, 4)
        else:
            ops.v_decode(r["stream"], r["info"], back, 128, 64, 4)
        assert torch.equal(back, codes)
        del r, codes, back


@pytest.mark.parametrize("B,H,T,dtype,rel", [(16, 8, 32768, torch.bfloat16, 0.1), (8, 7, 16384, torch.bfloat16, 0.2),
                                             (2, 40, 8192, torch.float16, 0.05)])
def test_fused_quant_encode_large_shapes_repeat_and_round_trip(cuda, B, H, T, dtype, rel):
    """Thousands of workgroups in flight (the in-order stream offsets, the exchange between runs of eight heads, the
    wavefronts' shared minima and maxima): three launches give the same bytes, the parameters are the stand-alone
    quantizer's, and the stream unpacks to its codes."""
    k, v = synth.make_kv(B, H, T, seed=5, device=cuda, dtype=dtype)
    bits = ops.bits_for_rel(rel)
    for is_k, x in ((True, k), (False, v)):
        scale, zero = ops.quant_params(x, rel)
        codes, _ = ops.quantize(x, scale, zero)
        first = None
        for _ in range(3):
            r = (ops.k_quant_encode if is_k else ops.v_quant_encode)(x, rel, bits)
            assert torch.equal(scale, r["scale"]) and torch.equal(zero, r["zero"])
            got = (r["size"], r["stream"][:r["size"]].clone(), r["info"].clone())
            if first is None:
                first = got
            else:
                assert got[0] == first[0] and torch.equal(got[1], first[1]) and torch.equal(got[2], first[2])
        back = torch.empty_like(codes)
        if is_k:
            ops.k_decode(r["stream"], r["info"], back, 64, 128, bits)
        else:
            ops.v_decode(r["stream"], r["info"], back, 128, 64, bits)
        assert torch.equal(back, codes)
        del r, codes, back, first, got


def test_asynchronous_encode_reports_through_encode_status(cuda):
    """want_size=False keeps the launch asynchronous and reports nothing by itself; ops.encode_status then gives the
    size, or raises what the synchronous form raises: a stream that does not fit, a code wider than bits_len.  A
    compressed buffer at an odd address is refused up front (blocks are written in 2-byte units)."""
    B, H, T = 2, 4, 512
    k, _ = synth.make_kv(B, H, T, seed=620, device=cuda)
    sync = ops.k_quant_encode(k, 0.1)
    a = ops.k_quant_encode(k, 0.1, want_size=False)
    assert a["size"] == 0
    q = synth.make_q(B, 4 * H, seed=621, device=cuda)
    ops.attn_decode(q, sync, ops.v_quant_encode(k, 0.1))          # other work on the stream does not disturb the status
    assert ops.encode_status(cuda, bits=4) == sync["size"]
    assert torch.equal(a["stream"][:sync["size"]], sync["stream"][:sync["size"]])
    small = torch.empty(1024, dtype=torch.uint8, device=cuda)
    ops.k_quant_encode(k, 0.1, stream=small, want_size=False)     # does not fit: silent until asked
    with pytest.raises(ops.PackKVError) as e:
        ops.encode_status(cuda)
    assert e.value.code == 4
    ops.k_quant_encode(k, 0.1, bits=2, want_size=False)           # codes up to 11 do not fit 2 bits
    with pytest.raises(ops.PackKVError) as e:
        ops.encode_status(cuda, bits=2)
    assert e.value.code == 1
    odd = torch.empty(B * H * T * 128 + 1, dtype=torch.uint8, device=cuda)[1:]
    with pytest.raises(ops.PackKVError) as e:
        ops.k_quant_encode(k, 0.1, stream=odd)
    assert e.value.code == 2 and "even address" in str(e.value)
    codes = torch.zeros(64, 128, dtype=torch.uint8, device=cuda)
    with pytest.raises(RuntimeError, match="even address"):
        ops.k_encode(codes, odd, torch.zeros(1, 2, dtype=torch.uint32, device=cuda))
