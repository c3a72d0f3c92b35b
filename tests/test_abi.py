"""The C-ABI library loads and exports every symbol include/packkv.h declares (no compute calls:
this runs without a GPU)."""
import ctypes
import os
import re

from packkv_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "packkv.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(pkv_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported_and_bound():
    names = _declared()
    assert "pkv_attn_decode" in names and "pkv_k_quant_encode" in names and len(names) >= 17
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), "missing export " + n
        assert n in _lib.SIGNATURES, "python binding lacks " + n
    assert sorted(_lib.SIGNATURES) == names


def test_version_bounds_and_error_text():
    lib = _lib.load()
    assert lib.pkv_abi_version() == 3
    assert lib.pkv_block_bound(1, 64, 128, 4) == 4552      # 8 + 4*112 + 512*8
    assert lib.pkv_block_bound(0, 128, 64, 3) == 3400      # 8 + 4*80 + 512*6
    # argument validation happens before any GPU call: a bad width is reported, not crashed on
    rc = lib.pkv_k_decode(None, 0, None, None, 64, 128, 64, 128, 4, None, None)
    assert rc == _lib.ERR_INVALID
    assert b"null" in lib.pkv_last_error()
    one = ctypes.c_void_p(16)
    rc = lib.pkv_k_encode(one, one, 1, one, 64, 128, 64, 128, 9, None, None, None)
    assert rc == _lib.ERR_UNSUPPORTED and b"not supported" in lib.pkv_last_error()
    rc = lib.pkv_k_encode(one, one, 1, one, 64, 128, 64, 64, 4, None, None, None)
    assert rc == _lib.ERR_UNSUPPORTED
    rc = lib.pkv_v_encode(one, one, 1, one, 100, 128, 128, 64, 3, None, None, None)
    assert rc == _lib.ERR_INVALID


def test_drop_in_module_exports_reference_names():
    import packkv_cuda
    # packkv_cuda_ext/export_packkv.cpp:9-18
    for n in ("kq_mat_vec_mul", "wv_mat_vec_mul", "k_encode_cpu", "k_decode_cpu", "v_encode_cpu",
              "v_decode_cpu", "fused_kq", "fused_wv"):
        assert callable(getattr(packkv_cuda, n))


def test_bits_for_rel():
    from packkv_amd.ops import bits_for_rel
    assert [bits_for_rel(r) for r in (0.1, 0.14, 0.2, 0.25, 0.34)] == [4, 4, 3, 3, 3]
    assert bits_for_rel(0.05) == 5
