"""ctypes binding of libpackkv_hip.so (the C ABI declared in include/packkv.h).

The library is the product: there is no fallback.  If it has not been built, or cannot be
loaded, importing the op surface fails with instructions instead of silently running
something else.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# PACKKV_HIP_LIB names another build of the same library (kernel development: A/B runs of two builds)
LIB_PATH = os.environ.get("PACKKV_HIP_LIB") or os.path.join(_HERE, "libpackkv_hip.so")

F16, BF16 = 0, 1
OK, ERR_UNSUPPORTED, ERR_INVALID, ERR_HIP, ERR_CAPACITY, ERR_INTERNAL = range(6)
ATTN_REF_ROUNDING, ATTN_OUT_F32 = 1, 2

_vp = ctypes.c_void_p
_i = ctypes.c_int
_u64 = ctypes.c_uint64
_f = ctypes.c_float
_fp = ctypes.POINTER(ctypes.c_float)
_u64p = ctypes.POINTER(ctypes.c_uint64)


class AttnArgs(ctypes.Structure):
    _fields_ = [
        ("k_stream", _vp), ("k_info", _vp), ("v_stream", _vp), ("v_info", _vp),
        ("k_bytes", _u64), ("v_bytes", _u64),
        ("k_scale", _vp), ("k_zero", _vp), ("v_scale", _vp), ("v_zero", _vp),
        ("q", _vp), ("out", _vp), ("k_win", _vp), ("v_win", _vp),
        ("B", _i), ("Hq", _i), ("Hkv", _i), ("T_c", _i), ("T_w", _i),
        ("k_bits", _i), ("v_bits", _i), ("dtype", _i), ("sm_scale", _f), ("variant", _i),
        ("par_stride", _i), ("win_stride", _i), ("flags", _i),
    ]


# name -> (restype, argtypes); every symbol include/packkv.h declares
SIGNATURES = {
    "pkv_abi_version": (_i, []),
    "pkv_last_error": (ctypes.c_char_p, []),
    "pkv_block_bound": (_u64, [_i, _i, _i, _i]),
    "pkv_k_encode": (_i, [_vp, _vp, _u64, _vp, _i, _i, _i, _i, _i, _u64p, _fp, _vp]),
    "pkv_v_encode": (_i, [_vp, _vp, _u64, _vp, _i, _i, _i, _i, _i, _u64p, _fp, _vp]),
    "pkv_encode_status": (_i, [_vp, _i, _u64p]),
    "pkv_k_encode_p": (_i, [_vp, _vp, _u64, _vp, _i, _i, _i, _i, _u64p, _fp, _vp]),
    "pkv_v_encode_p": (_i, [_vp, _vp, _u64, _vp, _i, _i, _i, _i, _u64p, _fp, _vp]),
    "pkv_k_decode_p": (_i, [_vp, _u64, _vp, _vp, _i, _i, _i, _i, _fp, _vp]),
    "pkv_v_decode_p": (_i, [_vp, _u64, _vp, _vp, _i, _i, _i, _i, _fp, _vp]),
    "pkv_block_bound_p": (_u64, [_i, _i]),
    "pkv_k_decode": (_i, [_vp, _u64, _vp, _vp, _i, _i, _i, _i, _i, _fp, _vp]),
    "pkv_v_decode": (_i, [_vp, _u64, _vp, _vp, _i, _i, _i, _i, _i, _fp, _vp]),
    "pkv_quant_params": (_i, [_vp, _i, _i, _i, _i, _f, _vp, _vp, _fp, _vp]),
    "pkv_quantize": (_i, [_vp, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _fp, _vp]),
    "pkv_dequantize": (_i, [_vp, _i, _i, _i, _i, _vp, _vp, _vp, _fp, _vp]),
    "pkv_median_order": (_i, [_vp, _i, _i, _i, _i, _f, _i, _i, _vp, _vp, _vp, _fp, _vp]),
    "pkv_k_quant_encode_perm": (_i, [_vp, _i, _i, _i, _i, _f, _i, _vp, _i, _vp, _u64, _vp, _vp, _vp, _u64p, _fp, _vp]),
    "pkv_v_quant_encode_perm": (_i, [_vp, _i, _i, _i, _i, _f, _i, _vp, _i, _vp, _vp, _vp, _u64, _vp, _vp, _vp, _u64p, _fp, _vp]),
    "pkv_k_quant_encode": (_i, [_vp, _i, _i, _i, _i, _f, _i, _vp, _u64, _vp, _vp, _vp, _u64p, _fp, _vp]),
    "pkv_v_quant_encode": (_i, [_vp, _i, _i, _i, _i, _f, _i, _vp, _u64, _vp, _vp, _vp, _u64p, _fp, _vp]),
    "pkv_k_quant_encode_append": (_i, [_vp, _i, _i, _i, _i, _f, _i, _vp, _u64, _u64, _vp, _vp, _vp, _i, _u64p, _fp, _vp]),
    "pkv_v_quant_encode_append": (_i, [_vp, _i, _i, _i, _i, _f, _i, _vp, _u64, _u64, _vp, _vp, _vp, _i, _u64p, _fp, _vp]),
    "pkv_window_append": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64,
                               ctypes.c_int64, _vp, _vp, _i, _i, _vp]),
    "pkv_bit_pack_size": (_i, [_vp, _i, _i, _i, _u64p, ctypes.POINTER(ctypes.c_uint32), _fp, _vp]),
    "pkv_median_repack": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _fp, _vp]),
    "pkv_greedy_repack": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _fp, _vp]),
    "pkv_kq_mat_vec_mul": (_i, [_vp, _u64, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _fp, _vp]),
    "pkv_wv_mat_vec_mul": (_i, [_vp, _u64, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _fp, _vp]),
    "pkv_fused_kq": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _fp, _vp]),
    "pkv_fused_wv": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _fp, _vp]),
    "pkv_attn_decode": (_i, [ctypes.POINTER(AttnArgs), _fp, _vp]),
    "pkv_attn_decode_noalloc": (_i, [ctypes.POINTER(AttnArgs), _vp]),
    "pkv_stream_release": (_i, [_vp]),
}

_lib = None


class PackKVError(RuntimeError):
    """A C-ABI call returned a non-zero status; ``code`` holds the PKV_ERR_* value."""

    def __init__(self, code, message):
        super().__init__(message)
        self.code = code


def load():
    """Load the library once and attach prototypes.  Raises ImportError when it is missing."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            "libpackkv_hip.so is not built (%s). Build it with `python -m packkv_amd.build` "
            "(needs hipcc, targets gfx950); there is no CPU fallback." % LIB_PATH)
    try:
        lib = ctypes.CDLL(LIB_PATH)
    except OSError as e:  # pragma: no cover - depends on the machine
        raise ImportError("cannot load %s: %s" % (LIB_PATH, e))
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(rc):
    if rc != 0:
        msg = load().pkv_last_error().decode("utf-8", "replace")
        raise PackKVError(rc, msg or ("packkv error %d" % rc))
