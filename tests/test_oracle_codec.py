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
