"""PackKV compressed KV-cache hot path for AMD MI355X (gfx950).

Hand-written HIP kernels behind a C ABI (include/packkv.h, libpackkv_hip.so) and a Python op
surface that mirrors the reference's ``packkv_cuda`` module.
"""
from . import _lib  # noqa: F401

__all__ = ["ops", "synth"]
