"""GPU parity of the bit-pack / bit-unpack kernels against the CPU oracle: bit-exact stream,
block_info, size and decoded codes, through the C ABI (packkv_amd.ops -> libpackkv_hip.so)."""
import numpy as np
import pytest
import torch

from oracle import codec
from oracle import quant as oq
from packkv_amd import ops

pytestmark = pytest.mark.gpu


def _say(*a):
    print(*a, flush=True)


def _rand_codes(rng, T, H, W, kind):
    if kind == "uniform":
        c = rng.integers(0, 1 << W, (T, H))
    elif kind == "const":
        c = np.full((T, H), (1 << W) - 1)
    elif kind == "narrow":
        c = rng.integers(0, 2, (T, H)) + rng.integers(0, (1 << W) - 1, (1, H))
    else:
        c = np.clip(np.rint(rng.normal(1 << (W - 1), 1.0, (T, H))), 0, (1 << W) - 1)
    return c.astype(np.uint8)


def _gpu_encode(cuda, is_k, c, cb, hb, W):
    T, H = c.shape
    d_codes = torch.from_numpy(c).to(cuda)
    d_stream = torch.zeros(T * H, dtype=torch.uint8, device=cuda)
    d_info = torch.zeros((T // cb) * (H // hb), 2, dtype=torch.uint32, device=cuda)
    fn = ops.k_encode if is_k else ops.v_encode
    size = fn(d_codes, d_stream, d_info, cb, hb, W)
    return d_stream, d_info, size


# (192, 640) and (256, 320): 15 and 10 blocks, so the eight-blocks-per-workgroup encoder ends on a partial group
SHAPES = {1: [(64, 128, 64, 128), (256, 512, 64, 128), (128, 4096, 64, 128), (64, 256, 32, 128),
              (256, 128, 128, 128), (32, 128, 16, 128), (192, 640, 64, 128)],
          0: [(128, 64, 128, 64), (512, 512, 128, 64), (128, 4096, 128, 64), (256, 128, 128, 32),
              (128, 256, 128, 128), (256, 320, 128, 64)]}


@pytest.mark.parametrize("is_k", [1, 0])
@pytest.mark.parametrize("W", [2, 3, 4])
def test_encode_decode_bit_exact_vs_oracle(cuda, oracle_codec, is_k, W):
    rng = np.random.default_rng(100 + 10 * is_k + W)
    for (T, H, cb, hb) in SHAPES[is_k]:
        for kind in ("uniform", "const", "narrow", "gauss"):
            _say("codec case", "K" if is_k else "V", T, H, cb, hb, W, kind)
            c = _rand_codes(rng, T, H, W, kind)
            so, io, zo = oracle_codec.encode(is_k, c, cb, hb, W)
            d_stream, d_info, size = _gpu_encode(cuda, is_k, c, cb, hb, W)
            assert size == zo
            assert np.array_equal(d_info.cpu().numpy(), io)
            assert np.array_equal(d_stream[:size].cpu().numpy(), so[:zo])
            # unpack both the GPU stream and (independently) the oracle stream
            d_out = torch.zeros(T, H, dtype=torch.uint8, device=cuda)
            (ops.k_decode if is_k else ops.v_decode)(d_stream, d_info, d_out, cb, hb, W)
            assert np.array_equal(d_out.cpu().numpy(), c)
            d_out.zero_()
            s2 = torch.from_numpy(so[:zo].copy()).to(cuda)      # exactly-sized stream buffer
            (ops.k_decode if is_k else ops.v_decode)(s2, torch.from_numpy(io).to(cuda), d_out, cb, hb, W)
            assert np.array_equal(d_out.cpu().numpy(), c)


ODD_SHAPES = {1: [(96, 128, 48, 128), (160, 256, 80, 128), (512, 128, 256, 128), (112, 384, 112, 128)],
              0: [(128, 96, 128, 96), (256, 320, 128, 160), (128, 512, 128, 256), (128, 448, 128, 224)]}


@pytest.mark.parametrize("is_k", [1, 0])
def test_block_shapes_off_the_beaten_track(cuda, oracle_codec, is_k):
    """K blocks of 48, 80, 112 and 256 tokens and V blocks of 96, 160, 224 and 256 channels (3, 5, 7 and 8 units per
    block), at every code width from 2 to 8 bits: stream, block_info and the decoded codes against the restatement."""
    rng = np.random.default_rng(300 + is_k)
    for (T, H, cb, hb) in ODD_SHAPES[is_k]:
        for W in range(2, 9):
            kind = ("uniform", "gauss", "narrow")[W % 3]
            _say("odd block case", "K" if is_k else "V", T, H, cb, hb, W, kind)
            c = _rand_codes(rng, T, H, W, kind)
            so, io, zo = oracle_codec.encode(is_k, c, cb, hb, W)
            d_stream, d_info, size = _gpu_encode(cuda, is_k, c, cb, hb, W)
            assert size == zo
            assert np.array_equal(d_info.cpu().numpy(), io)
            assert np.array_equal(d_stream[:size].cpu().numpy(), so[:zo])
            d_out = torch.zeros(T, H, dtype=torch.uint8, device=cuda)
            (ops.k_decode if is_k else ops.v_decode)(d_stream, d_info, d_out, cb, hb, W)
            assert np.array_equal(d_out.cpu().numpy(), c)


def test_encode_from_a_misaligned_code_matrix(cuda, oracle_codec):
    """A code matrix that does not start on a 16-byte boundary takes the one-block-per-workgroup encoder; same
    stream."""
    rng = np.random.default_rng(77)
    for is_k, (T, H, cb, hb) in ((1, (128, 256, 64, 128)), (0, (128, 256, 128, 64))):
        c = _rand_codes(rng, T, H, 4, "gauss")
        so, io, zo = oracle_codec.encode(is_k, c, cb, hb, 4)
        flat = torch.zeros(T * H + 16, dtype=torch.uint8, device=cuda)
        d_codes = flat[3:3 + T * H].view(T, H)
        d_codes.copy_(torch.from_numpy(c))
        assert d_codes.data_ptr() % 16 != 0 and d_codes.is_contiguous()
        d_stream = torch.zeros(T * H, dtype=torch.uint8, device=cuda)
        d_info = torch.zeros((T // cb) * (H // hb), 2, dtype=torch.uint32, device=cuda)
        size = (ops.k_encode if is_k else ops.v_encode)(d_codes, d_stream, d_info, cb, hb, 4)
        assert size == zo and np.array_equal(d_info.cpu().numpy(), io)
        assert np.array_equal(d_stream[:size].cpu().numpy(), so[:zo])


def test_golden_vectors_from_reference_codec(cuda, golden):
    for name in [str(n) for n in golden["cases"]]:
        is_k, T, H, cb, hb, W, size = [int(x) for x in golden[name + "_meta"]]
        _say("golden", name)
        c = golden[name + "_codes"]
        d_stream, d_info, got = _gpu_encode(cuda, is_k, c, cb, hb, W)
        assert got == size
        assert np.array_equal(d_info.cpu().numpy(), golden[name + "_info"])
        assert np.array_equal(d_stream[:size].cpu().numpy(), golden[name + "_stream"])
        d_out = torch.zeros(T, H, dtype=torch.uint8, device=cuda)
        (ops.k_decode if is_k else ops.v_decode)(torch.from_numpy(golden[name + "_stream"]).to(cuda),
                                                 torch.from_numpy(golden[name + "_info"]).to(cuda),
                                                 d_out, cb, hb, W)
        assert np.array_equal(d_out.cpu().numpy(), c)


def test_drop_in_cpu_signatures_round_trip(cuda, oracle_codec):
    """The reference call sequence (evaluation/evaluation.py:419-456) with host tensors."""
    import packkv_cuda
    rng = np.random.default_rng(7)
    for is_k, (cb, hb, W) in ((1, (64, 128, 4)), (0, (128, 64, 3))):
        T, H = 256, 1024
        block = torch.from_numpy(_rand_codes(rng, T, H, W, "gauss"))
        info = torch.zeros((T // cb) * (H // hb), 2, dtype=torch.uint32)
        comp = torch.zeros_like(block)
        enc = packkv_cuda.k_encode_cpu if is_k else packkv_cuda.v_encode_cpu
        dec = packkv_cuda.k_decode_cpu if is_k else packkv_cuda.v_decode_cpu
        size = enc(block, comp, info, T, H, cb, hb, W)
        so, io, zo = oracle_codec.encode(is_k, block.numpy(), cb, hb, W)
        assert size == zo and np.array_equal(info.numpy(), io)
        assert np.array_equal(comp.flatten()[:size].numpy(), so[:zo])
        back = torch.zeros_like(block)
        dec(comp, info, back, T, H, cb, hb, W)
        assert (block == back).all()


def test_error_conventions(cuda):
    c = torch.zeros(64, 128, dtype=torch.uint8, device=cuda)
    s = torch.zeros(64 * 128, dtype=torch.uint8, device=cuda)
    i = torch.zeros(1, 2, dtype=torch.uint32, device=cuda)
    with pytest.raises(RuntimeError, match="not supported"):
        ops.k_encode(c, s, i, 64, 128, 1)
    with pytest.raises(RuntimeError, match="bits_len"):
        ops.k_encode(c, s, i, 64, 128, 9)
    with pytest.raises(RuntimeError, match="bits_len"):        # the drop-in functions keep the reference's limit
        ops.k_encode_cpu(c, s, i, 64, 128, 64, 128, 5)
    with pytest.raises(RuntimeError, match="block num mismatch"):
        ops.k_encode(c, s, torch.zeros(2, 2, dtype=torch.uint32, device=cuda), 64, 128, 4)
    with pytest.raises(RuntimeError, match="UInt8"):
        ops.k_encode(c.to(torch.int32), s, i, 64, 128, 4)
    # output buffer too small for the stream: reported, nothing written out of bounds
    rnd = torch.randint(0, 16, (64, 128), dtype=torch.uint8, device=cuda)
    small = torch.zeros(1000, dtype=torch.uint8, device=cuda)
    with pytest.raises(ops.PackKVError) as e:
        ops.k_encode(rnd, small, i, 64, 128, 4)
    assert e.value.code == 4


def test_round_trip_at_bench_scale(cuda):
    """Size-independent property at a full-size shape (8 KV heads x 128 x 32768 tokens x batch 4):
    decode(encode(x)) == x, offsets are the prefix sum of sizes, sizes are within the block bounds."""
    T, H = 32768, 4 * 8 * 128
    g = torch.Generator(device=cuda)
    g.manual_seed(11)
    x = torch.randn(T, H, device=cuda, generator=g)
    codes = ((x - x.amin(1, keepdim=True)) / (x.amax(1, keepdim=True) - x.amin(1, keepdim=True)) * 10).round().to(torch.uint8)
    del x
    for is_k, (cb, hb) in ((1, (64, 128)), (0, (128, 64))):
        stream = torch.empty(T * H, dtype=torch.uint8, device=cuda)
        info = torch.empty((T // cb) * (H // hb), 2, dtype=torch.uint32, device=cuda)
        size = (ops.k_encode if is_k else ops.v_encode)(codes, stream, info, cb, hb, 4)
        inf = info.cpu().numpy().astype(np.int64)
        assert int(inf[:, 1].sum()) == size
        assert np.array_equal(inf[:, 0], np.concatenate([[0], np.cumsum(inf[:, 1])[:-1]]))
        assert inf[:, 1].min() >= (456 if is_k else 8 + 4 * 112) and inf[:, 1].max() <= 4552
        out = torch.zeros_like(codes)
        (ops.k_decode if is_k else ops.v_decode)(stream, info, out, cb, hb, 4)
        assert torch.equal(out, codes)
        _say("bench-scale", "K" if is_k else "V", "ratio uint8/stream = %.3f" % (T * H / size))


@pytest.mark.parametrize("W", [5, 6, 7, 8])
def test_wide_codes_stream_matches_restatement(cuda, oracle_codec, W):
    """Widths 5..8 are this build's extension of the format (pack words of up to 128 bits; the reference's
    templates stop at 4).  There is no reference for them: the device codec is held to the restated C codec byte for
    byte, to an exact round trip, and the stream size to the closed form (payload 2 * len bytes per pack, W + LB bits
    of metadata per pack, 8 header bytes per block)."""
    rng = np.random.default_rng(40 + W)
    # (rows of 1024 and 2048 channels: the kernels that read the code matrix as cells)
    for is_k, (cb, hb), (T, H) in ((1, (64, 128), (128, 256)), (0, (128, 64), (256, 192)), (1, (32, 128), (96, 128)),
                                   (1, (64, 128), (128, 2048)), (0, (128, 64), (256, 1024))):
        codes = rng.integers(0, 2 ** W, size=(T, H), dtype=np.uint8)
        codes[: T // 2, ::2] //= 8                 # mixed widths: some packs narrow, some constant
        codes[:16, :32] = 7
        _say("wide codec case W", W, "K" if is_k else "V", cb, hb, T, H)
        so, io, zo = oracle_codec.encode(is_k, codes, cb, hb, W)
        nblk = (T // cb) * (H // hb)
        LB = int(np.ceil(np.log2(W + 1)))
        packs = codes.reshape(T // 16, 16, H)
        lens = np.ceil(np.log2(packs.max(1).astype(np.int64) - packs.min(1) + 1)).astype(np.int64)
        assert zo == int(lens.sum()) * 2 + lens.size * (W + LB) // 8 + (2 * (cb // 16) if is_k else 4 * (hb // 32)) * nblk
        d = torch.from_numpy(codes).to(cuda)
        stream = torch.zeros(nblk * ops.block_bound(is_k, cb, hb, W) + 16, dtype=torch.uint8, device=cuda)
        info = torch.zeros(nblk, 2, dtype=torch.uint32, device=cuda)
        size = (ops.k_encode if is_k else ops.v_encode)(d, stream, info, cb, hb, W)
        assert size == zo
        assert np.array_equal(info.cpu().numpy(), io)
        assert np.array_equal(stream[:zo].cpu().numpy(), so[:zo])
        back = torch.zeros_like(d)
        (ops.k_decode if is_k else ops.v_decode)(stream, info, back, cb, hb, W)
        assert torch.equal(back, d)


# ---- packs longer than 16 tokens (this build's extension of the format; the oracle's restatement of it is pinned
# on the CPU by tests/test_oracle_codec.py) ---------------------------------------------------------------------

def _gpu_encode_p(cuda, is_k, c, P, W):
    ctx_blk, hid_blk = ops.long_block_shape(is_k, P)
    nblk = (c.shape[0] // ctx_blk) * (c.shape[1] // hid_blk)
    d_codes = torch.from_numpy(c).to(cuda)
    d_stream = torch.zeros(nblk * ops.block_bound_p(P, W), dtype=torch.uint8, device=cuda)
    d_info = torch.zeros(nblk, 2, dtype=torch.uint32, device=cuda)
    size = ops.encode_p(is_k, d_codes, d_stream, d_info, P, W)
    return d_codes, d_stream, d_info, size


@pytest.mark.parametrize("is_k", [1, 0])
@pytest.mark.parametrize("P", [32, 64, 128, 256])
def test_long_packs_bit_exact_vs_oracle(cuda, oracle_codec, is_k, P):
    rng = np.random.default_rng(500 + 10 * is_k + P)
    ctx_blk, hid_blk = ops.long_block_shape(is_k, P)
    for W in (2, 3, 4, 5, 6, 7, 8):
        for kind in ("uniform", "const", "narrow", "gauss"):
            # five blocks to a row: V rows of 320 channels (one block per workgroup, plain decoder); six: whole 128-byte
            # lines (two V blocks per workgroup in the encoder, the staged decoder)
            # (packs of 32 tokens, K: 20 or 24 blocks at even widths -- four to a workgroup -- and 15 or 18 at odd widths,
            # one or two to a workgroup)
            rows_of_blocks = (4 if W % 2 == 0 else 3) if P == 32 else 3 if P == 64 else 2
            T, H = ctx_blk * rows_of_blocks, hid_blk * (5 if kind in ("uniform", "narrow") else 6)
            _say("long-pack case", "K" if is_k else "V", "pack", P, "bits", W, kind, (T, H))
            c = _rand_codes(rng, T, H, W, kind)
            so, io, zo = codec.long_encode(is_k, c, P, W)
            d_codes, d_stream, d_info, size = _gpu_encode_p(cuda, is_k, c, P, W)
            assert size == zo
            assert np.array_equal(d_info.cpu().numpy(), io)
            assert np.array_equal(d_stream[:size].cpu().numpy(), so[:zo])
            assert size - 8 * len(io) == oq.bit_pack_bytes(c, P, W)
            back = torch.full_like(d_codes, 0xEE)
            ops.decode_p(is_k, d_stream, d_info, back, P, W)
            assert torch.equal(back, d_codes)
            # the oracle's stream decodes on the GPU too
            back.fill_(0xEE)
            ops.decode_p(is_k, torch.from_numpy(so).to(cuda), torch.from_numpy(io).to(cuda), back, P, W)
            assert torch.equal(back, d_codes)


def test_long_v_packs_from_a_code_matrix_that_is_not_16_byte_aligned(cuda):
    """V's long-pack encoder loads 16 bytes per lane; a code matrix that starts elsewhere takes the plain kernel and
    must give the same stream."""
    g = torch.Generator().manual_seed(11)
    for P, W in ((32, 4), (128, 3), (256, 6)):
        ctx_blk, hid_blk = ops.long_block_shape(0, P)
        T, H = 2 * ctx_blk, 3 * hid_blk
        c = torch.randint(0, 1 << W, (T, H), generator=g, dtype=torch.uint8).to(cuda)
        buf = torch.empty(T * H + 16, dtype=torch.uint8, device=cuda)
        shifted = buf[3:3 + T * H].view(T, H)
        shifted.copy_(c)
        assert shifted.data_ptr() % 16 != 0 and shifted.is_contiguous()
        nblk = (T // ctx_blk) * (H // hid_blk)
        out = []
        for m in (c, shifted):
            stream = torch.zeros(nblk * ops.block_bound_p(P, W), dtype=torch.uint8, device=cuda)
            info = torch.zeros(nblk, 2, dtype=torch.uint32, device=cuda)
            size = ops.encode_p(0, m, stream, info, P, W)
            out.append((size, stream[:size].clone(), info.clone()))
        assert out[0][0] == out[1][0]
        assert torch.equal(out[0][1], out[1][1]) and torch.equal(out[0][2].view(torch.int32), out[1][2].view(torch.int32))


def test_long_packs_of_16_tokens_forward_to_the_reference_format(cuda, oracle_codec):
    rng = np.random.default_rng(77)
    for is_k, (cb, hb) in ((1, (64, 128)), (0, (128, 64))):
        c = _rand_codes(rng, 256, 512, 4, "gauss")
        so, io, zo = oracle_codec.encode(is_k, c, cb, hb, 4)
        d_codes, d_stream, d_info, size = _gpu_encode_p(cuda, is_k, c, 16, 4)
        assert size == zo and np.array_equal(d_info.cpu().numpy(), io)
        assert np.array_equal(d_stream[:size].cpu().numpy(), so[:zo])
        back = torch.zeros_like(d_codes)
        ops.decode_p(is_k, d_stream, d_info, back, 16, 4)
        assert torch.equal(back, d_codes)


def test_long_packs_sweep_layer_round_trip_and_size_model(cuda):
    """The sweep's layer (8 KV heads x 128 x 16384 tokens) at every pack length: round trip, and stream bytes - 8 per
    block equal to the size model with the pack widths counted on the GPU (ops.code_stats, itself checked against the
    oracle in tests/test_gpu_repack.py)."""
    g = torch.Generator().manual_seed(3)
    for W in (3, 4, 6):
        c = torch.clamp(torch.round(torch.randn(16384, 1024, generator=g) * 1.5 + (1 << (W - 1))), 0, (1 << W) - 1).to(torch.uint8).to(cuda)
        for P in (32, 64, 128, 256):
            for is_k in (1, 0):
                ctx_blk, hid_blk = ops.long_block_shape(is_k, P)
                nblk = (16384 // ctx_blk) * (1024 // hid_blk)
                stream = torch.empty(nblk * ops.block_bound_p(P, W), dtype=torch.uint8, device=cuda)
                info = torch.empty(nblk, 2, dtype=torch.uint32, device=cuda)
                size = ops.encode_p(is_k, c, stream, info, P, W)
                len_sum, _ = ops.code_stats(c, P)                 # sum of the packs' widths, counted on the GPU
                lb = max(1, int(W).bit_length())
                assert size - 8 * nblk == (len_sum * P + (16384 // P) * 1024 * (W + lb)) // 8, (W, P, is_k)
                back = torch.zeros_like(c)
                ops.decode_p(is_k, stream, info, back, P, W)
                assert torch.equal(back, c), (W, P, is_k)


def test_long_pack_argument_checks(cuda):
    c = torch.zeros(1024, 128, dtype=torch.uint8, device=cuda)
    stream = torch.zeros(1 << 20, dtype=torch.uint8, device=cuda)
    with pytest.raises(Exception):
        ops.encode_p(1, c, stream, torch.zeros(2, 2, dtype=torch.uint32, device=cuda), 48, 4)      # pack length
    with pytest.raises(Exception):
        ops.encode_p(1, c[:1000], stream, torch.zeros(1, 2, dtype=torch.uint32, device=cuda), 256, 4)   # tokens
    with pytest.raises(Exception):
        ops.encode_p(1, c, stream[:64], torch.zeros(1, 2, dtype=torch.uint32, device=cuda), 256, 4)   # capacity
    # a block_info row that points outside the stream decodes nothing and faults nothing
    info = torch.tensor([[1 << 30, 4096]], dtype=torch.int64).to(torch.uint32).to(cuda)
    out = torch.full_like(c, 7)
    ops.decode_p(1, stream, info, out, 256, 4)
    torch.cuda.synchronize()
    assert int(out.min()) == 7 and int(out.max()) == 7


@pytest.mark.parametrize("is_k", [1, 0])
def test_damaged_block_info_is_survived(cuda, is_k):
    """block_info is device data the decoders do not own: entries that point outside the stream, or claim absurd
    sizes, yield arbitrary codes for their own blocks and nothing else -- the other blocks decode as before."""
    rng = np.random.default_rng(5)
    cb, hb = (64, 128) if is_k else (128, 64)
    T, H, W = 2 * cb, 4 * hb, 4
    c = _rand_codes(rng, T, H, W, "normal")
    d_stream, d_info, size = _gpu_encode(cuda, is_k, c, cb, hb, W)
    stream = d_stream[:size].clone()                      # a buffer that ends with the stream
    info = d_info.cpu().numpy().astype(np.int64)
    bad = info.copy()
    bad[1] = (size + 12345, 4000)                         # behind the buffer
    bad[2] = (0xFFFFFFF0, 0xFFFFFFFF)                     # far outside, absurd size
    bad[5] = (size - 3, 0xFFFF)                           # starts inside, runs out
    bad[6] = (size, 16)                                   # exactly at the end
    d_bad = torch.from_numpy(bad.astype(np.uint32)).to(cuda)
    out = torch.zeros(T, H, dtype=torch.uint8, device=cuda)
    (ops.k_decode if is_k else ops.v_decode)(stream, d_bad, out, cb, hb, W)
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    n_hid = H // hb
    for b in range(info.shape[0]):
        if b in (1, 2, 5, 6):
            continue
        r, h = b // n_hid, b % n_hid
        assert np.array_equal(got[r * cb:(r + 1) * cb, h * hb:(h + 1) * hb], c[r * cb:(r + 1) * cb, h * hb:(h + 1) * hb]), b
