"""TEST INFRASTRUCTURE ONLY: ctypes front ends for the two CPU codecs.

* ``oracle``  -- the restated codec in ``packkv_oracle.c`` (always available once built)
* ``ref``     -- the reference's own scalar codec (``packkv_cuda_ext/src/*_cpu.cpp``)
                 compiled by ``oracle/Makefile`` into ``oracle/_ref``; present only
                 where that build ran.

Both expose ``encode(is_k, codes, ctx_blk, hid_blk, W)`` and ``decode(...)`` on numpy
arrays, with the buffer conventions of the reference call sites
(evaluation/evaluation.py:419-456): ``codes`` is uint8 ``[ctx_len, hidden_dim]``, the
stream buffer has ``ctx_len * hidden_dim`` bytes of capacity, ``block_info`` is uint32
``[n_blocks, 2]`` holding (byte offset, byte size).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_ORACLE_SO = os.path.join(_HERE, "libpackkv_oracle.so")
_REF_SO = os.path.join(_HERE, "_ref", "libpackkv_ref.so")

_u8p = ctypes.POINTER(ctypes.c_uint8)
_u32p = ctypes.POINTER(ctypes.c_uint32)


def build(with_ref=True):
    """Compile the checker libraries (the restated C codec, and the reference build
    when the reference checkout is present)."""
    subprocess.check_call(["make", "-s", "-C", _HERE, "oracle"])
    if with_ref:
        subprocess.check_call(["make", "-s", "-C", _HERE, "ref"])


class _Codec:
    def __init__(self, path, prefix):
        self.lib = ctypes.CDLL(path)
        self.enc = getattr(self.lib, prefix + "_encode")
        self.dec = getattr(self.lib, prefix + "_decode")
        self.enc.restype = ctypes.c_uint64
        self.enc.argtypes = [ctypes.c_int, _u8p, _u8p, _u32p] + [ctypes.c_int] * 5
        self.dec.restype = ctypes.c_int
        self.dec.argtypes = [ctypes.c_int, _u8p, _u32p, _u8p] + [ctypes.c_int] * 5
        self.bound = getattr(self.lib, prefix + "_block_bound", None)     # the restated codec only
        if self.bound is not None:
            self.bound.restype = ctypes.c_uint64
            self.bound.argtypes = [ctypes.c_int] * 4

    def encode(self, is_k, codes, ctx_blk, hid_blk, W):
        codes = np.ascontiguousarray(codes, dtype=np.uint8)
        ctx_len, hidden = codes.shape
        nblk = (ctx_len // ctx_blk) * (hidden // hid_blk)
        # the reference sizes the buffer like the code matrix (evaluation/evaluation.py:426); widths above 4
        # (this build's extension) can exceed that, so take the worst case when it is larger
        bound = int(self.bound(int(is_k), ctx_blk, hid_blk, W)) if self.bound is not None else 0
        stream = np.zeros(max(ctx_len * hidden, nblk * bound), dtype=np.uint8)
        info = np.zeros((nblk, 2), dtype=np.uint32)
        size = self.enc(int(is_k), codes.ctypes.data_as(_u8p), stream.ctypes.data_as(_u8p),
                        info.ctypes.data_as(_u32p), ctx_len, hidden, ctx_blk, hid_blk, W)
        if size == 2 ** 64 - 1:
            raise RuntimeError("not supported")
        return stream, info, int(size)

    def decode(self, is_k, stream, info, ctx_len, hidden, ctx_blk, hid_blk, W):
        stream = np.ascontiguousarray(stream, dtype=np.uint8)
        info = np.ascontiguousarray(info, dtype=np.uint32)
        out = np.zeros((ctx_len, hidden), dtype=np.uint8)
        rc = self.dec(int(is_k), stream.ctypes.data_as(_u8p), info.ctypes.data_as(_u32p),
                      out.ctypes.data_as(_u8p), ctx_len, hidden, ctx_blk, hid_blk, W)
        if rc != 0:
            raise RuntimeError("not supported")
        return out


_cache = {}


def oracle():
    if "oracle" not in _cache:
        if not os.path.exists(_ORACLE_SO):
            build(with_ref=False)
        c = _Codec(_ORACLE_SO, "pkv_oracle")
        c.lib.pkv_oracle_block_bound.restype = ctypes.c_uint64
        c.lib.pkv_oracle_block_bound.argtypes = [ctypes.c_int] * 4
        _cache["oracle"] = c
    return _cache["oracle"]


def have_ref():
    return os.path.exists(_REF_SO)


def ref():
    if "ref" not in _cache:
        _cache["ref"] = _Codec(_REF_SO, "pkv_ref")
    return _cache["ref"]


def block_bound(is_k, ctx_blk, hid_blk, W):
    return int(oracle().lib.pkv_oracle_block_bound(int(is_k), ctx_blk, hid_blk, W))


# ---- packs longer than 16 tokens (this build's extension of the format; see packkv_oracle.c) ----

def long_block_bound(pack_len, W):
    lib = oracle().lib
    lib.pkv_oracle_long_block_bound.restype = ctypes.c_uint64
    lib.pkv_oracle_long_block_bound.argtypes = [ctypes.c_int] * 2
    return int(lib.pkv_oracle_long_block_bound(pack_len, W))


def long_encode(is_k, codes, pack_len, W):
    """codes uint8 [ctx_len, hidden] -> (stream, block_info [n_blocks, 2], size) with packs of `pack_len` tokens:
    K blocks of 4 pack_len x 128, V blocks of 8 pack_len x 64."""
    lib = oracle().lib
    lib.pkv_oracle_long_encode.restype = ctypes.c_uint64
    lib.pkv_oracle_long_encode.argtypes = [ctypes.c_int, _u8p, _u8p, ctypes.c_uint64, _u32p] + [ctypes.c_int] * 4
    codes = np.ascontiguousarray(codes, dtype=np.uint8)
    ctx_len, hidden = codes.shape
    nblk = (ctx_len // ((4 if is_k else 8) * pack_len)) * (hidden // (128 if is_k else 64))
    stream = np.zeros(nblk * long_block_bound(pack_len, W), dtype=np.uint8)
    info = np.zeros((nblk, 2), dtype=np.uint32)
    size = lib.pkv_oracle_long_encode(int(is_k), codes.ctypes.data_as(_u8p), stream.ctypes.data_as(_u8p), stream.size,
                                      info.ctypes.data_as(_u32p), ctx_len, hidden, pack_len, W)
    if size == 2 ** 64 - 1:
        raise RuntimeError("not supported")
    return stream, info, int(size)


def long_decode(is_k, stream, info, ctx_len, hidden, pack_len, W):
    lib = oracle().lib
    lib.pkv_oracle_long_decode.restype = ctypes.c_int
    lib.pkv_oracle_long_decode.argtypes = [ctypes.c_int, _u8p, _u32p, _u8p] + [ctypes.c_int] * 4
    stream = np.ascontiguousarray(stream, dtype=np.uint8)
    info = np.ascontiguousarray(info, dtype=np.uint32)
    out = np.zeros((ctx_len, hidden), dtype=np.uint8)
    if lib.pkv_oracle_long_decode(int(is_k), stream.ctypes.data_as(_u8p), info.ctypes.data_as(_u32p),
                                  out.ctypes.data_as(_u8p), ctx_len, hidden, pack_len, W) != 0:
        raise RuntimeError("not supported")
    return out
