"""Pins the restated CPU codec (oracle/packkv_oracle.c): golden vectors made by the compiled
reference codec, the compiled reference itself where it is built, and closed-form answers
that follow from the stream layout."""
import numpy as np
import pytest

from oracle import codec
from oracle import quant as oq


def _case(golden, name):
    is_k, T, H, cb, hb, W, size = [int(x) for x in golden[name + "_meta"]]
    return is_k, T, H, cb, hb, W, size, golden[name + "_codes"], golden[name + "_stream"], golden[name + "_info"]


def test_oracle_matches_reference_golden_vectors(golden, oracle_codec):
    names = [str(n) for n in golden["cases"]]
    assert len(names) == 24
    for name in names:
        is_k, T, H, cb, hb, W, size, codes, stream, info = _case(golden, name)
        s, i, z = oracle_codec.encode(is_k, codes, cb, hb, W)
        assert z == size, name
        assert np.array_equal(i, info), name
        assert np.array_equal(s[:z], stream), name
        back = oracle_codec.decode(is_k, stream, info, T, H, cb, hb, W)
        assert np.array_equal(back, codes), name


@pytest.mark.skipif(not codec.have_ref(), reason="reference codec build (oracle/_ref) not present")
def test_oracle_matches_compiled_reference(oracle_codec):
    ref = codec.ref()
    rng = np.random.default_rng(1)
    shapes = {1: [(64, 128, 64, 128), (128, 1024, 64, 128), (64, 256, 32, 128), (256, 128, 128, 128)],
              0: [(128, 128, 128, 64), (256, 1024, 128, 64), (128, 128, 128, 32), (128, 256, 128, 128)]}
    for is_k, lst in shapes.items():
        for (T, H, cb, hb) in lst:
            for W in (2, 3, 4):
                for kind in range(3):
                    if kind == 0:
                        c = rng.integers(0, 1 << W, (T, H))
                    elif kind == 1:
                        c = rng.integers(0, 2, (T, H)) + rng.integers(0, (1 << W) - 1, (1, H))
                    else:
                        c = np.clip(np.rint(rng.normal(1 << (W - 1), 1.0, (T, H))), 0, (1 << W) - 1)
                    c = c.astype(np.uint8)
                    so, io, zo = oracle_codec.encode(is_k, c, cb, hb, W)
                    sr, ir, zr = ref.encode(is_k, c, cb, hb, W)
                    assert zo == zr and np.array_equal(io, ir) and np.array_equal(so, sr)
                    assert np.array_equal(ref.decode(is_k, so, io, T, H, cb, hb, W), c)
                    assert np.array_equal(oracle_codec.decode(is_k, sr, ir, T, H, cb, hb, W), c)


def test_constant_block_closed_form(oracle_codec):
    # every pack has len 0: K block = 8 + 4 * (64 + 48) bytes, header = cumulative 112s
    c = np.full((64, 128), 9, dtype=np.uint8)
    s, info, size = oracle_codec.encode(1, c, 64, 128, 4)
    assert size == 456 and tuple(info[0]) == (0, 456)
    assert list(s[:8].view(np.uint16)) == [112, 224, 336, 448]
    assert (s[8:8 + 64] == 0x99).all()          # mins nibble = the constant
    assert (s[8 + 64:8 + 112] == 0).all()       # lens all zero
    c = np.full((128, 64), 5, dtype=np.uint8)
    s, info, size = oracle_codec.encode(0, c, 128, 64, 3)
    assert size == 328
    assert list(s[:8].view(np.uint16)) == [80, 160, 240, 320]


def test_alternating_pack_bytes(oracle_codec):
    # one pack (round 2, channel 37) alternates m, m+1: contributes exactly 0x55 0x55 at the start
    # of round 2's payload (every other pack has len 0)
    c = np.full((64, 128), 3, dtype=np.uint8)
    c[32:48, 37] = np.array([3, 4] * 8, dtype=np.uint8)
    s, info, size = oracle_codec.encode(1, c, 64, 128, 4)
    assert size == 456 + 2
    cum = list(s[:8].view(np.uint16))
    assert cum == [112, 224, 338, 450]
    r2 = 8 + 224
    assert list(s[r2 + 112:r2 + 114]) == [0x55, 0x55]
    lens = s[r2 + 64:r2 + 112]
    bit = 37 * 3
    val = (int(lens[bit // 8]) | (int(lens[bit // 8 + 1]) << 8)) >> (bit % 8) & 7
    assert val == 1


def test_full_range_pack_nibbles_and_payload_order(oracle_codec):
    # channel c(j) = (j % 32) * 4 + j // 32 ; packs appear in j order.  Give two channels a full-range
    # pack and check where their 8 bytes land and that token 0 sits in the top nibble.
    c = np.zeros((64, 128), dtype=np.uint8)
    toks = np.arange(16, dtype=np.uint8)           # 0..15 -> len 4
    c[0:16, 4] = toks                              # j = 1  (lane 1, slot 0)
    c[0:16, 1] = toks[::-1]                        # j = 32 (lane 0, slot 1)
    s, info, size = oracle_codec.encode(1, c, 64, 128, 4)
    assert size == 456 + 16
    pay = s[8 + 112:8 + 112 + 16]
    w0 = int.from_bytes(bytes(pay[:8]), "little")
    w1 = int.from_bytes(bytes(pay[8:]), "little")
    assert [(w0 >> (4 * (15 - k))) & 15 for k in range(16)] == list(range(16))
    assert [(w1 >> (4 * (15 - k))) & 15 for k in range(16)] == list(range(15, -1, -1))


def test_sizes_offsets_and_bit_pack_parity(oracle_codec):
    rng = np.random.default_rng(5)
    for is_k, (T, H, cb, hb) in ((1, (256, 256, 64, 128)), (0, (256, 256, 128, 64))):
        for W in (2, 3, 4):
            c = np.clip(np.rint(rng.normal(1 << (W - 1), 1.2, (T, H))), 0, (1 << W) - 1).astype(np.uint8)
            s, info, size = oracle_codec.encode(is_k, c, cb, hb, W)
            assert int(info[:, 1].sum()) == size
            assert np.array_equal(info[:, 0], np.concatenate([[0], np.cumsum(info[:, 1])[:-1]]))
            # analytic size model (utils/compute.py:272-297): payload + (W + LB) bits per pack;
            # the encoder adds an 8-byte header per block
            nblk = info.shape[0]
            assert size - 8 * nblk == oq.bit_pack_bytes(c, 16, W=W)
            assert np.array_equal(oracle_codec.decode(is_k, s, info, T, H, cb, hb, W), c)


def test_unsupported_shapes_raise(oracle_codec):
    c = np.zeros((64, 128), dtype=np.uint8)
    with pytest.raises(RuntimeError):
        oracle_codec.encode(1, c, 64, 128, 9)
    with pytest.raises(RuntimeError):
        oracle_codec.encode(1, c, 64, 64, 4)
    with pytest.raises(RuntimeError):
        oracle_codec.encode(0, c, 64, 64, 3)


# ---- packs longer than 16 tokens: this build's extension of the format (no reference: parity unpinned) ----------
# Pinned by (i) the definition restated here with Python integers (a different formulation from the C restatement's
# bit writes), (ii) the reference's size model, (iii) P = 16 reproducing the reference-pinned format, (iv) round trips.

def _random_codes(rng, T, H, W, kind):
    if kind == 0:
        return rng.integers(0, 1 << W, (T, H)).astype(np.uint8)
    if kind == 1:                                  # narrow, slowly varying: short packs
        base = rng.integers(0, (1 << W) - 1, (1, H))
        return np.minimum(base + rng.integers(0, 2, (T, H)), (1 << W) - 1).astype(np.uint8)
    c = np.full((T, H), (1 << W) - 1, dtype=np.uint8)   # constant columns with a few spikes
    c[rng.integers(0, T, 8), rng.integers(0, H, 8)] = 0
    return c


def _long_block_by_definition(is_k, tile, P, W):
    """One block's bytes from the written definition: header of four u16 cumulative unit sizes (in 4-byte words for
    P >= 32), then per unit the LSB-first bit arrays of minima and widths and the pack words, slot-major and
    lane-minor, each word = sum_k (code_k - min) << ((P - 1 - k) * len) as P * len / 8 little-endian bytes."""
    LB = max(1, int(W).bit_length())
    units, cum = [], []
    total = 0
    for u in range(4):
        mins = lens = 0
        payload = b""
        for i in range(4):
            for t in range(32):
                if is_k:
                    tok0, ch = u * P, 4 * t + i
                else:
                    tok0, ch = ((u % 2) * 4 + i) * P, (u // 2) * 32 + t
                col = [int(x) for x in tile[tok0:tok0 + P, ch]]
                mn, ln = min(col), (max(col) - min(col)).bit_length()
                mins |= mn << ((4 * t + i) * W)
                lens |= ln << ((4 * t + i) * LB)
                word = 0
                for k, c in enumerate(col):
                    word |= (c - mn) << ((P - 1 - k) * ln)
                payload += word.to_bytes(P * ln // 8, "little")
        body = mins.to_bytes(128 * W // 8, "little") + lens.to_bytes(128 * LB // 8, "little") + payload
        total += len(body)
        cum.append(total if P == 16 else total // 4)
        assert P == 16 or total % 4 == 0
        units.append(body)
    return b"".join(int(c).to_bytes(2, "little") for c in cum) + b"".join(units)


@pytest.mark.parametrize("is_k", [1, 0])
def test_long_packs_follow_their_definition(is_k, oracle_codec):
    rng = np.random.default_rng(7)
    for P in (16, 32, 64, 128, 256):
        for W in (2, 3, 4, 5, 8):
            ctx_blk, hid_blk = ((4 * P, 128) if is_k else (8 * P, 64))
            codes = _random_codes(rng, 2 * ctx_blk, 2 * hid_blk, W, (P + W) % 3)
            stream, info, size = codec.long_encode(is_k, codes, P, W)
            want = b""
            for cb in range(2):
                for hb in range(2):
                    blk = _long_block_by_definition(is_k, codes[cb * ctx_blk:(cb + 1) * ctx_blk, hb * hid_blk:(hb + 1) * hid_blk], P, W)
                    assert tuple(info[2 * cb + hb]) == (len(want), len(blk)), (P, W)
                    want += blk
            assert size == len(want) and bytes(stream[:size]) == want, (P, W)
            assert np.array_equal(codec.long_decode(is_k, stream, info, *codes.shape, P, W), codes), (P, W)


def test_long_packs_of_16_tokens_are_the_reference_format(oracle_codec):
    rng = np.random.default_rng(8)
    for is_k, (cb, hb) in ((1, (64, 128)), (0, (128, 64))):
        for W in (2, 3, 4, 6):
            codes = _random_codes(rng, 256, 256, W, W % 3)
            s0, i0, z0 = oracle_codec.encode(is_k, codes, cb, hb, W)
            s1, i1, z1 = codec.long_encode(is_k, codes, 16, W)
            assert z0 == z1 and np.array_equal(i0, i1) and np.array_equal(s0[:z0], s1[:z1]), (is_k, W)


def test_long_pack_sizes_equal_the_size_model(oracle_codec):
    """stream bytes - 8 per block == the reference's analytic size (utils/compute.py:272-297) for the same codes,
    pack length and width, whatever the pack length."""
    rng = np.random.default_rng(9)
    for is_k in (1, 0):
        for P in (16, 32, 64, 128, 256):
            for W in (2, 3, 4, 5, 6, 7, 8):
                T, H = (8 if is_k else 8) * P, 256
                codes = _random_codes(rng, T, H, W, (P // 16 + W) % 3)
                _, info, size = codec.long_encode(is_k, codes, P, W)
                assert size - 8 * len(info) == oq.bit_pack_bytes(codes, P, W), (is_k, P, W)


def test_long_pack_header_counts_words_where_bytes_would_overflow(oracle_codec):
    codes = np.random.default_rng(10).integers(0, 256, (1024, 128)).astype(np.uint8)   # every pack at 8 bits
    stream, info, size = codec.long_encode(1, codes, 256, 8)
    unit = 128 + 64 + 128 * 256                      # minima, widths, 128 packs of 256 bytes
    assert size == 8 + 4 * unit == codec.long_block_bound(256, 8)
    assert [int(x) for x in stream[:8].view(np.uint16)] == [unit * (u + 1) // 4 for u in range(4)]
    assert np.array_equal(codec.long_decode(1, stream, info, 1024, 128, 256, 8), codes)
    with pytest.raises(RuntimeError):
        codec.long_encode(1, codes, 48, 4)           # not a supported pack length
    with pytest.raises(RuntimeError):
        codec.long_encode(1, codes[:1000], 256, 4)   # tokens not a multiple of the block
