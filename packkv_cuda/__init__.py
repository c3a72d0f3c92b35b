"""Drop-in for the reference's native module ``packkv_cuda`` (packkv_cuda_ext/setup.py:18-21,
packkv_cuda_ext/export_packkv.cpp:9-18): the same eight callables with the same positional
arguments, implemented by hand-written HIP kernels for gfx950.

    from packkv_cuda import k_encode_cpu, k_decode_cpu, kq_mat_vec_mul, ...   # unchanged caller code
"""
from packkv_amd.ops import (  # noqa: F401
    fused_kq,
    fused_wv,
    k_decode_cpu,
    k_encode_cpu,
    kq_mat_vec_mul,
    v_decode_cpu,
    v_encode_cpu,
    wv_mat_vec_mul,
)

__all__ = [
    "kq_mat_vec_mul", "wv_mat_vec_mul", "k_encode_cpu", "k_decode_cpu",
    "v_encode_cpu", "v_decode_cpu", "fused_kq", "fused_wv",
]
