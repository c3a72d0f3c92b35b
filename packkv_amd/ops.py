"""Python op surface over the C ABI: the reference's eight ``packkv_cuda`` functions with the
same positional signatures (packkv_cuda_ext/packkv_cuda.pyi:4-86, bound in
packkv_cuda_ext/export_packkv.cpp:9-18), plus the device-native ops the reference does not
have (GPU encode / unpack, fused quantize+encode, fused decompress-attention).

All tensors are caller-allocated and written in place, as in the reference.  PyTorch is used
for device memory and the current stream only; every computation happens in
libpackkv_hip.so.
"""
import ctypes
import math

import torch

from . import _lib
from ._lib import AttnArgs, PackKVError  # noqa: F401  (re-exported)

__all__ = [
    "k_encode_cpu", "k_decode_cpu", "v_encode_cpu", "v_decode_cpu",
    "kq_mat_vec_mul", "wv_mat_vec_mul", "fused_kq", "fused_wv",
    "k_encode", "v_encode", "k_decode", "v_decode",
    "quant_params", "quantize", "dequantize", "k_quant_encode", "v_quant_encode",
    "attn_decode", "AttnPlan", "block_bound", "bits_for_rel", "repack_quant_encode", "encode_status",
]


def _dtype_code(t):
    if t.dtype == torch.float16:
        return _lib.F16
    if t.dtype == torch.bfloat16:
        return _lib.BF16
    raise RuntimeError("Unsupported data type")


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)


def _stream(dev):
    return ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)


def _require(cond, msg):
    if not cond:
        raise RuntimeError("PackKV Assertion failed: " + msg)


def _device_of(*tensors):
    dev = None
    for t in tensors:
        if t.is_cuda:
            dev = t.device
    if dev is None:
        if not torch.cuda.is_available():
            raise RuntimeError("packkv needs a GPU: the ops run in libpackkv_hip.so, there is no CPU path")
        dev = torch.device("cuda", torch.cuda.current_device())
    return dev


def block_bound(is_k, ctx_blk, hid_blk, bits):
    return int(_lib.load().pkv_block_bound(int(is_k), ctx_blk, hid_blk, bits))


def bits_for_rel(rel):
    """Raw code width W for a relative quant step: codes span 0..ceil(1/rel), plus at most one
    more level from rounding the quotient to the storage type."""
    import math
    top = math.ceil(1.0 / rel - 1e-9) + 1
    return max(2, top.bit_length())


# ------------------------------------------------------------------ codec ------------

def _check_codec_args(codes, stream, info, ctx_len, hidden_dim, ctx_blk, hid_blk, bits, is_k, max_bits=4):
    # mirrors k_encode_cpu_assert / v_encode_cpu_assert (src/k_encode_cpu.cpp:247-284,
    # src/v_encode_cpu.cpp:262-299); raises instead of aborting the process
    _require(codes.dim() == 2 and codes.size(0) == ctx_len, "ctx_len mismatch")
    _require(codes.size(1) == hidden_dim, "hidden_dim mismatch")
    _require(ctx_blk > 0, "ctx_len_block_size must be greater than 0")
    _require(hid_blk > 0, "hidden_dim_block_size must be greater than 0")
    _require(ctx_len % ctx_blk == 0, "ctx_len must be divisible by ctx_len_block_size")
    _require(hidden_dim % hid_blk == 0, "hidden_dim must be divisible by hidden_dim_block_size")
    nblk = (ctx_len // ctx_blk) * (hidden_dim // hid_blk)
    _require(info.dim() == 2 and info.size(0) == nblk, "block_info_buffer block num mismatch")
    _require(info.size(1) == 2, "block_info_buffer.size(1) must be 2")
    _require(bits <= max_bits, "bits_len must be less than or equal to %d" % max_bits)
    _require(ctx_blk % 16 == 0, "ctx_len_block_size must be divisible by PACK_ELE_NUM")
    if is_k:
        _require(hid_blk == 128, "hidden_dim_block_size must be 128, because this is most common head dim")
    _require(codes.dtype == torch.uint8, "quant_ints_tensor must be a UInt8 tensor")
    _require(stream.dtype == torch.uint8, "compressed_buffer must be a UInt8 tensor")
    _require(stream.numel() > 0, "compressed_buffer must be a non-empty tensor")
    _require(info.dtype == torch.uint32, "block_info_buffer must be a UInt32 tensor")
    _require(codes.is_contiguous() and stream.is_contiguous() and info.is_contiguous(),
             "tensors must be contiguous")
    _require(not stream.is_cuda or stream.data_ptr() % 2 == 0, "compressed_buffer must start at an even address")


def _encode(is_k, codes, stream, info, ctx_len, hidden_dim, ctx_blk, hid_blk, bits, want_size=True,
            timed=False, max_bits=4):
    _check_codec_args(codes, stream, info, ctx_len, hidden_dim, ctx_blk, hid_blk, bits, is_k, max_bits)
    lib = _lib.load()
    dev = _device_of(codes, stream, info)
    on_host = not codes.is_cuda
    _require(stream.is_cuda != on_host and info.is_cuda != on_host, "all tensors must be on one device")
    d_codes = codes.to(dev) if on_host else codes
    d_stream = torch.empty(stream.numel(), dtype=torch.uint8, device=dev) if on_host else stream
    d_info = torch.empty_like(info, device=dev) if on_host else info
    size = ctypes.c_uint64(0)
    ms = ctypes.c_float(0.0)
    fn = lib.pkv_k_encode if is_k else lib.pkv_v_encode
    with torch.cuda.device(dev):
        rc = fn(_ptr(d_codes), _ptr(d_stream), d_stream.numel() * d_stream.element_size(), _ptr(d_info), ctx_len, hidden_dim,
                ctx_blk, hid_blk, bits, ctypes.byref(size) if (want_size or on_host) else None,
                ctypes.byref(ms) if timed else None, _stream(dev))
    _lib.check(rc)
    if on_host:
        n = int(size.value)
        stream.view(-1)[:n].copy_(d_stream[:n].cpu())
        info.copy_(d_info.cpu())
    return (int(size.value), float(ms.value)) if timed else int(size.value)


def _decode(is_k, stream, info, codes, ctx_len, hidden_dim, ctx_blk, hid_blk, bits, timed=False, max_bits=4):
    _check_codec_args(codes, stream, info, ctx_len, hidden_dim, ctx_blk, hid_blk, bits, is_k, max_bits)
    lib = _lib.load()
    dev = _device_of(codes, stream, info)
    on_host = not codes.is_cuda
    _require(stream.is_cuda != on_host and info.is_cuda != on_host, "all tensors must be on one device")
    d_stream = stream.to(dev) if on_host else stream
    d_info = info.to(dev) if on_host else info
    d_codes = torch.empty_like(codes, device=dev) if on_host else codes
    ms = ctypes.c_float(0.0)
    fn = lib.pkv_k_decode if is_k else lib.pkv_v_decode
    with torch.cuda.device(dev):
        rc = fn(_ptr(d_stream), d_stream.numel() * d_stream.element_size(), _ptr(d_info), _ptr(d_codes), ctx_len, hidden_dim, ctx_blk, hid_blk, bits,
                ctypes.byref(ms) if timed else None, _stream(dev))
    _lib.check(rc)
    if on_host:
        codes.copy_(d_codes.cpu())
    return float(ms.value) if timed else None


def stream_release(stream=None):
    """Gives back the device memory the library keeps for `stream` (a torch.cuda.Stream; default: the current one) --
    scratch buffers, tile counters and the buffers it has outgrown.  For callers that create and destroy streams:
    call it before the stream goes away, and only when no HIP graph captured on it will be replayed again."""
    st = torch.cuda.current_stream() if stream is None else stream
    with torch.cuda.device(st.device):
        rc = _lib.load().pkv_stream_release(ctypes.c_void_p(st.cuda_stream))
    _lib.check(rc)


def encode_status(device=None, bits=0):
    """Stream size of the last encode launched on the current stream of `device` with want_size=False; waits for the
    stream and raises what the encode would have raised (a stream that did not fit, a code wider than `bits`)."""
    dev = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
    size = ctypes.c_uint64(0)
    with torch.cuda.device(dev):
        rc = _lib.load().pkv_encode_status(_stream(dev), int(bits), ctypes.byref(size))
    _lib.check(rc)
    return int(size.value)


def k_encode_cpu(quant_ints_tensor, compressed_buffer, block_info_buffer, ctx_len, hidden_dim,
                 ctx_len_block_size, hidden_dim_block_size, bits_len):
    """Drop-in for packkv_cuda.k_encode_cpu (packkv_cuda.pyi:4-13): host tensors in, host tensors
    written in place, stream size returned -- but encoded on the GPU (staged through device
    memory).  Device tensors are accepted too and then nothing is copied."""
    return _encode(True, quant_ints_tensor, compressed_buffer, block_info_buffer, ctx_len, hidden_dim,
                   ctx_len_block_size, hidden_dim_block_size, bits_len)


def v_encode_cpu(quant_ints_tensor, compressed_buffer, block_info_buffer, ctx_len, hidden_dim,
                 ctx_len_block_size, hidden_dim_block_size, bits_len):
    """Drop-in for packkv_cuda.v_encode_cpu (packkv_cuda.pyi:38-47)."""
    return _encode(False, quant_ints_tensor, compressed_buffer, block_info_buffer, ctx_len, hidden_dim,
                   ctx_len_block_size, hidden_dim_block_size, bits_len)


def k_decode_cpu(compressed_buffer, block_info_buffer, quant_ints_tensor, ctx_len, hidden_dim,
                 ctx_len_block_size, hidden_dim_block_size, bits_len):
    """Drop-in for packkv_cuda.k_decode_cpu (packkv_cuda.pyi:15-24)."""
    _decode(True, compressed_buffer, block_info_buffer, quant_ints_tensor, ctx_len, hidden_dim,
            ctx_len_block_size, hidden_dim_block_size, bits_len)


def v_decode_cpu(compressed_buffer, block_info_buffer, quant_ints_tensor, ctx_len, hidden_dim,
                 ctx_len_block_size, hidden_dim_block_size, bits_len):
    """Drop-in for packkv_cuda.v_decode_cpu (packkv_cuda.pyi:49-58)."""
    _decode(False, compressed_buffer, block_info_buffer, quant_ints_tensor, ctx_len, hidden_dim,
            ctx_len_block_size, hidden_dim_block_size, bits_len)


MAX_BITS = 8     # widths 5..8 are this library's extension of the format (the reference stops at 4)


def k_encode(codes, stream, info, ctx_blk=64, hid_blk=128, bits=4, want_size=True, timed=False):
    """Device encode of a uint8 code matrix [ctx_len, hidden]; returns the stream size (and ms).  bits 2..8."""
    return _encode(True, codes, stream, info, codes.size(0), codes.size(1), ctx_blk, hid_blk, bits,
                   want_size, timed, MAX_BITS)


def v_encode(codes, stream, info, ctx_blk=128, hid_blk=64, bits=4, want_size=True, timed=False):
    return _encode(False, codes, stream, info, codes.size(0), codes.size(1), ctx_blk, hid_blk, bits,
                   want_size, timed, MAX_BITS)


def k_decode(stream, info, codes, ctx_blk=64, hid_blk=128, bits=4, timed=False):
    return _decode(True, stream, info, codes, codes.size(0), codes.size(1), ctx_blk, hid_blk, bits, timed, MAX_BITS)


def v_decode(stream, info, codes, ctx_blk=128, hid_blk=64, bits=4, timed=False):
    return _decode(False, stream, info, codes, codes.size(0), codes.size(1), ctx_blk, hid_blk, bits, timed, MAX_BITS)


# ---- packs longer than 16 tokens (an extension of the format: the reference only prices them, utils/compute.py:272-297) ----

PACK_LENS = (16, 32, 64, 128, 256)


def long_block_shape(is_k, pack_len):
    """(tokens, channels) of a block with packs of `pack_len` tokens: the reference's 64 x 128 / 128 x 64 scaled."""
    return ((4 * pack_len, 128) if is_k else (8 * pack_len, 64))


def block_bound_p(pack_len, bits):
    return int(_lib.load().pkv_block_bound_p(pack_len, bits))


def _check_long(is_k, codes, stream, info, pack_len, bits):
    _require(pack_len in PACK_LENS, "not supported: pack_len %d (16, 32, 64, 128 or 256)" % pack_len)
    ctx_blk, hid_blk = long_block_shape(is_k, pack_len)
    _require(codes.dim() == 2 and codes.dtype == torch.uint8, "quant_ints_tensor must be a 2-D UInt8 tensor")
    _require(codes.size(0) % ctx_blk == 0, "ctx_len must be divisible by %d (the block's tokens at this pack_len)" % ctx_blk)
    _require(codes.size(1) % hid_blk == 0, "hidden_dim must be divisible by hidden_dim_block_size")
    nblk = (codes.size(0) // ctx_blk) * (codes.size(1) // hid_blk)
    _require(info.dim() == 2 and info.size(0) == nblk and info.size(1) == 2, "block_info_buffer block num mismatch")
    _require(stream.dtype == torch.uint8 and stream.numel() > 0, "compressed_buffer must be a non-empty UInt8 tensor")
    _require(info.dtype == torch.uint32, "block_info_buffer must be a UInt32 tensor")
    _require(2 <= bits <= MAX_BITS, "bits_len must be 2..%d" % MAX_BITS)
    _require(codes.is_cuda and stream.is_cuda and info.is_cuda, "tensors must be on the GPU")
    _require(codes.is_contiguous() and stream.is_contiguous() and info.is_contiguous(), "tensors must be contiguous")
    _require(stream.data_ptr() % 2 == 0, "compressed_buffer must start at an even address")


def encode_p(is_k, codes, stream, info, pack_len, bits, want_size=True, timed=False):
    """Encode a uint8 code matrix [ctx_len, hidden] with packs of `pack_len` tokens (16 = the reference's format with
    its block shapes).  Returns the stream size (and ms)."""
    _check_long(is_k, codes, stream, info, pack_len, bits)
    dev = _device_of(codes, stream, info)
    size, ms = ctypes.c_uint64(0), ctypes.c_float(0.0)
    fn = _lib.load().pkv_k_encode_p if is_k else _lib.load().pkv_v_encode_p
    with torch.cuda.device(dev):
        rc = fn(_ptr(codes), _ptr(stream), stream.numel(), _ptr(info), codes.size(0), codes.size(1), pack_len, bits,
                ctypes.byref(size) if want_size else None, ctypes.byref(ms) if timed else None, _stream(dev))
    _lib.check(rc)
    return (int(size.value), float(ms.value)) if timed else int(size.value)


def decode_p(is_k, stream, info, codes, pack_len, bits, timed=False):
    _check_long(is_k, codes, stream, info, pack_len, bits)
    dev = _device_of(codes, stream, info)
    ms = ctypes.c_float(0.0)
    fn = _lib.load().pkv_k_decode_p if is_k else _lib.load().pkv_v_decode_p
    with torch.cuda.device(dev):
        rc = fn(_ptr(stream), stream.numel(), _ptr(info), _ptr(codes), codes.size(0), codes.size(1), pack_len, bits,
                ctypes.byref(ms) if timed else None, _stream(dev))
    _lib.check(rc)
    return float(ms.value) if timed else None


# --------------------------------------------------------------- quantizer -----------

def _check_x(x):
    _require(x.is_cuda and x.dim() == 4 and x.size(3) == 128 and x.is_contiguous(),
             "x must be a contiguous device tensor [B, H, T, 128]")
    return x.size(0), x.size(1), x.size(2)


def _check_params(scale, zero, B, T, dtype, device):
    for name, t in (("scale", scale), ("zero", zero)):
        _require(t.is_cuda and t.device == device and t.dtype == dtype and t.dtype in (torch.float16, torch.bfloat16) and
                 t.numel() == B * T and t.is_contiguous(),
                 name + " must be a contiguous device tensor of B*T values in the tensor's 16-bit dtype")


def quant_params(x, rel, timed=False):
    """Per-(batch, token) scale and zero of quant_ints(TokenQuant) (utils/compute.py:84-112);
    returns (scale, zero) as [B, T] tensors of x.dtype."""
    B, H, T = _check_x(x)
    scale = torch.empty(B, T, dtype=x.dtype, device=x.device)
    zero = torch.empty(B, T, dtype=x.dtype, device=x.device)
    ms = ctypes.c_float(0.0)
    with torch.cuda.device(x.device):
        rc = _lib.load().pkv_quant_params(_ptr(x), _dtype_code(x), B, H, T, float(rel), _ptr(scale),
                                          _ptr(zero), ctypes.byref(ms) if timed else None, _stream(x.device))
    _lib.check(rc)
    return (scale, zero, float(ms.value)) if timed else (scale, zero)


def quantize(x, scale, zero):
    """uint8 code matrix [T, B*H*128] (layout of evaluation/evaluation.py:406) and the largest code."""
    B, H, T = _check_x(x)
    _check_params(scale, zero, B, T, x.dtype, x.device)
    codes = torch.empty(T, B * H * 128, dtype=torch.uint8, device=x.device)
    mx = torch.zeros(1, dtype=torch.int32, device=x.device)
    with torch.cuda.device(x.device):
        rc = _lib.load().pkv_quantize(_ptr(x), _dtype_code(x), B, H, T, _ptr(scale), _ptr(zero), _ptr(codes),
                                      _ptr(mx), None, _stream(x.device))
    _lib.check(rc)
    return codes, int(mx.item())


def dequantize(codes, scale, zero, B, H):
    """(code + zero) * scale in the storage dtype -> [B, H, T, 128] (utils/compute.py:173-179)."""
    _require(codes.is_cuda and codes.dtype == torch.uint8 and codes.dim() == 2 and codes.is_contiguous() and
             codes.size(1) == B * H * 128, "codes must be a contiguous uint8 device tensor [T, B*H*128]")
    T = codes.size(0)
    _check_params(scale, zero, B, T, scale.dtype, codes.device)
    x = torch.empty(B, H, T, 128, dtype=scale.dtype, device=codes.device)
    with torch.cuda.device(codes.device):
        rc = _lib.load().pkv_dequantize(_ptr(codes), _dtype_code(scale), B, H, T, _ptr(scale), _ptr(zero),
                                        _ptr(x), None, _stream(codes.device))
    _lib.check(rc)
    return x


def _quant_encode(is_k, x, rel, bits, stream, info, want_size, timed, perm=None, perm_block=0, params=None):
    B, H, T = _check_x(x)
    _require(perm is None or (bits <= 6 and H <= 8), "a token order is taken by the fused encoders only (bits <= 6, H <= 8)")
    hidden = B * H * 128
    ctx_blk, hid_blk = (64, 128) if is_k else (128, 64)
    nblk = (T // ctx_blk) * (hidden // hid_blk)
    if stream is None:     # sized like the code matrix as the reference does; the extension widths can need more
        stream = torch.empty(max(T * hidden, nblk * block_bound(is_k, ctx_blk, hid_blk, bits) + 16) if bits > 4
                             else T * hidden, dtype=torch.uint8, device=x.device)
    if info is None:
        info = torch.empty(nblk, 2, dtype=torch.uint32, device=x.device)
    _require(info.numel() == 2 * nblk and info.dtype == torch.uint32, "block_info_buffer block num mismatch")
    if bits > 6:
        # widths 7..8 (format extension): quantize to the code matrix, then the block codec -- three kernels instead
        # of the fused one
        scale, zero = quant_params(x, rel)
        codes, mx = quantize(x, scale, zero)
        if mx >= (1 << bits):
            raise PackKVError(1, "not supported: code %d does not fit bits_len %d" % (mx, bits))
        res = _encode(is_k, codes, stream, info, T, hidden, ctx_blk, hid_blk, bits, want_size, timed, MAX_BITS)
        size, ms = res if timed else (res, 0.0)
        return {"stream": stream, "info": info, "scale": scale, "zero": zero, "size": int(size), "ms": float(ms),
                "bits": bits}
    scale = torch.empty(B, T, dtype=x.dtype, device=x.device)
    zero = torch.empty(B, T, dtype=x.dtype, device=x.device)
    size = ctypes.c_uint64(0)
    ms = ctypes.c_float(0.0)
    with torch.cuda.device(x.device):
        tail = (_ptr(stream), stream.numel(), _ptr(info), _ptr(scale), _ptr(zero), ctypes.byref(size) if want_size else None,
                ctypes.byref(ms) if timed else None, _stream(x.device))
        if perm is None:
            fn = _lib.load().pkv_k_quant_encode if is_k else _lib.load().pkv_v_quant_encode
            rc = fn(_ptr(x), _dtype_code(x), B, H, T, float(rel), bits, *tail)
        else:
            _require(perm.is_cuda and perm.dtype in (torch.uint32, torch.int32) and perm.numel() == T and perm.is_contiguous(),
                     "perm must hold one 32-bit index per token")
            if is_k:
                rc = _lib.load().pkv_k_quant_encode_perm(_ptr(x), _dtype_code(x), B, H, T, float(rel), bits, _ptr(perm),
                                                         int(perm_block), *tail)
            else:       # params: V's (scale, zero) [B, T] in the order of x, as median_order writes them
                sp, zp = (None, None) if params is None else (_ptr(params[0]), _ptr(params[1]))
                rc = _lib.load().pkv_v_quant_encode_perm(_ptr(x), _dtype_code(x), B, H, T, float(rel), bits, _ptr(perm),
                                                         int(perm_block), sp, zp, *tail)
    _lib.check(rc)
    return {"stream": stream, "info": info, "scale": scale, "zero": zero, "size": int(size.value),
            "ms": float(ms.value), "bits": bits}


def k_quant_encode(x, rel, bits=None, stream=None, info=None, want_size=True, timed=False):
    """Fused quantize + K encode of x [B, H, T, 128]; returns a dict with stream, info (block_info),
    scale, zero [B, T], size (bytes), ms and bits."""
    return _quant_encode(True, x, rel, bits or bits_for_rel(rel), stream, info, want_size, timed)


def v_quant_encode(x, rel, bits=None, stream=None, info=None, want_size=True, timed=False):
    return _quant_encode(False, x, rel, bits or bits_for_rel(rel), stream, info, want_size, timed)


def quant_encode_append(is_k, x, rel, bits, stream, used, info, tokens, scale, zero):
    """Append the tokens x [B, H, n, 128] (n a multiple of 64 for K, 128 for V) to a stream that holds
    ``tokens`` tokens in its first ``used`` bytes.  ``info`` [blocks, 2] and ``scale`` / ``zero``
    [B, row] are allocated for the cache's full length and filled behind what is there; the new blocks'
    offsets count from the start of ``stream``.  Returns the bytes in use afterwards."""
    B, H, n = _check_x(x)
    ctx_blk, hid_blk = (64, 128) if is_k else (128, 64)
    per_row = B * H * 128 // hid_blk
    _require(n % ctx_blk == 0 and tokens % ctx_blk == 0, "token counts must be multiples of the block length")
    nblk_done, nblk_new = tokens // ctx_blk * per_row, n // ctx_blk * per_row
    _require(info.is_cuda and info.dtype == torch.uint32 and info.is_contiguous()
             and info.numel() >= 2 * (nblk_done + nblk_new), "block_info_buffer too small")
    _require(scale.shape == zero.shape and scale.dim() == 2 and scale.size(0) == B and scale.dtype == x.dtype
             and zero.dtype == x.dtype and scale.is_contiguous() and zero.is_contiguous()
             and scale.size(1) >= tokens + n, "scale / zero must be contiguous [B, row] with room for the new tokens")
    _require(stream.is_cuda and stream.dtype == torch.uint8 and stream.is_contiguous() and 0 <= used <= stream.numel(),
             "compressed_buffer must be a contiguous device UInt8 tensor holding the bytes in use")
    es = scale.element_size()
    size = ctypes.c_uint64(0)
    fn = _lib.load().pkv_k_quant_encode_append if is_k else _lib.load().pkv_v_quant_encode_append
    with torch.cuda.device(x.device):
        rc = fn(_ptr(x), _dtype_code(x), B, H, n, float(rel), int(bits), _ptr(stream), stream.numel(), int(used),
                ctypes.c_void_p(info.data_ptr() + 8 * nblk_done), ctypes.c_void_p(scale.data_ptr() + es * tokens),
                ctypes.c_void_p(zero.data_ptr() + es * tokens), scale.size(1), ctypes.byref(size), None,
                _stream(x.device))
    _lib.check(rc)
    return int(size.value)


def window_append(k_new, v_new, cos, sin, k_win, v_win, win_pos):
    """Write the new tokens k_new / v_new [B, H, n, 128] into rows win_pos.. of the 16-bit windows k_win / v_win
    [B, H, cap, 128]; with cos / sin [B, n, 128] the keys get the rotary embedding first, rounded like the reference's
    chain of 16-bit elementwise ops (utils/compute.py:35-43).  One launch; strided views (a transposed projection
    output, an expanded cos / sin table) are read in place."""
    B, H, n, D = k_new.shape
    _require(D == 128 and v_new.shape == k_new.shape and k_new.is_cuda and v_new.dtype == k_new.dtype,
             "K and V must be device tensors [B, H, n, 128] of one dtype")
    _require(k_win.is_contiguous() and v_win.is_contiguous() and k_win.shape == v_win.shape and k_win.dim() == 4
             and k_win.size(0) == B and k_win.size(1) == H and k_win.size(3) == 128 and k_win.dtype == k_new.dtype,
             "windows must be contiguous [B, H, cap, 128] of the tokens' dtype")
    if k_new.stride(3) != 1 or k_new.stride() != v_new.stride():
        k_new, v_new = k_new.contiguous(), v_new.contiguous()
    rot_sb = 0
    if cos is not None:
        _require(cos.shape == (B, n, 128) and sin.shape == (B, n, 128) and cos.dtype == k_new.dtype
                 and sin.dtype == k_new.dtype, "cos / sin must be [B, n, 128] of the tokens' dtype")
        if cos.stride(2) != 1 or (n > 1 and cos.stride(1) != 128) or cos.stride() != sin.stride():
            cos, sin = cos.contiguous(), sin.contiguous()
        rot_sb = cos.stride(0) if B > 1 else 0
    with torch.cuda.device(k_new.device):
        rc = _lib.load().pkv_window_append(_ptr(k_new), _ptr(v_new), _ptr(cos) if cos is not None else None,
                                           _ptr(sin) if cos is not None else None, _dtype_code(k_new), B, H, n,
                                           k_new.stride(0), k_new.stride(1), k_new.stride(2), rot_sb, _ptr(k_win),
                                           _ptr(v_win), int(win_pos), k_win.size(2), _stream(k_new.device))
    _lib.check(rc)


# ------------------------------------------------- repacking and analytic size ------

def _check_code_matrix(c, name):
    _require(c.is_cuda and c.dim() == 2 and c.dtype == torch.uint8 and c.is_contiguous(),
             "%s must be a contiguous device UInt8 code matrix [ctx_len, hidden]" % name)


def code_stats(codes, pack_len, timed=False):
    """(sum over packs of bit_length(max - min), number of distinct code values) of a code matrix [ctx_len, hidden]
    for packs of `pack_len` consecutive tokens of one channel: the two data-dependent terms of `bit_pack`
    (utils/compute.py:272-297)."""
    _check_code_matrix(codes, "codes")
    ctx, hidden = codes.shape
    len_sum, n_unique, ms = ctypes.c_uint64(0), ctypes.c_uint32(0), ctypes.c_float(0.0)
    with torch.cuda.device(codes.device):
        rc = _lib.load().pkv_bit_pack_size(_ptr(codes), ctx, hidden, int(pack_len), ctypes.byref(len_sum),
                                           ctypes.byref(n_unique), ctypes.byref(ms) if timed else None,
                                           _stream(codes.device))
    _lib.check(rc)
    out = (int(len_sum.value), int(n_unique.value))
    return out + (float(ms.value),) if timed else out


def bit_pack_bytes(codes, pack_len, timed=False):
    """Analytic size of ONE code matrix [ctx_len, hidden] in bytes, as `bit_pack` prices each half
    (utils/compute.py:272-297): packs of `pack_len` consecutive tokens of one channel cost
    pack_len * bit_length(max - min) payload bits + W + ceil(log2(W + 1)) metadata bits, W = ceil(log2(#codes))."""
    len_sum, n_unique, ms = code_stats(codes, pack_len, timed=True)
    ctx, hidden = codes.shape
    w = math.ceil(math.log2(n_unique))
    n_packs = (ctx // pack_len) * hidden
    size = (len_sum * pack_len + n_packs * (w + math.ceil(math.log2(w + 1)))) // 8
    return (size, ms) if timed else size


def bit_pack(k_codes, v_codes, pack_len):
    """(k_bytes, v_bytes) of `bit_pack(blocks, pack_len)` (utils/compute.py:272-297) for blocks = K and V codes
    side by side."""
    return bit_pack_bytes(k_codes, pack_len), bit_pack_bytes(v_codes, pack_len)


def median_repacking(k_codes, v_codes, block_size=64, timed=False):
    """`median_repacking` (utils/compute.py:262-270) on the device: inside every block of `block_size` tokens, K and
    V rows are reordered together by descending median of the token's V codes; equal medians keep their order.
    Returns (k_repacked, v_repacked, perm) with perm [ctx_len] int32: perm[blk * block_size + r] = position inside the
    block the token at r came from."""
    _check_code_matrix(k_codes, "k_codes")
    _check_code_matrix(v_codes, "v_codes")
    _require(k_codes.shape == v_codes.shape, "K and V code matrices must have one shape")
    ctx, hidden = k_codes.shape
    k_out, v_out = torch.empty_like(k_codes), torch.empty_like(v_codes)
    perm = torch.empty(ctx, dtype=torch.int32, device=k_codes.device)
    ms = ctypes.c_float(0.0)
    with torch.cuda.device(k_codes.device):
        rc = _lib.load().pkv_median_repack(_ptr(k_codes), _ptr(v_codes), _ptr(k_out), _ptr(v_out), _ptr(perm), ctx,
                                           hidden, int(block_size), ctypes.byref(ms) if timed else None,
                                           _stream(k_codes.device))
    _lib.check(rc)
    return (k_out, v_out, perm, float(ms.value)) if timed else (k_out, v_out, perm)


def greedy_repacking(k_codes, v_codes, pack_len=16, block_size=64, timed=False):
    """`greedy_repacking` (utils/compute.py:210-260) on the device: every block of `block_size` tokens is rebuilt pack
    by pack -- seed = the remaining token closest (cosine) to the rounded mean of the remaining tokens, then
    pack_len - 1 times the remaining token that adds the fewest payload bits -- jointly for K and V.  Exact integer
    arithmetic; ties go to the earlier token.  Returns (k_repacked, v_repacked, perm) like median_repacking."""
    _check_code_matrix(k_codes, "k_codes")
    _check_code_matrix(v_codes, "v_codes")
    _require(k_codes.shape == v_codes.shape, "K and V code matrices must have one shape")
    ctx, hidden = k_codes.shape
    k_out, v_out = torch.empty_like(k_codes), torch.empty_like(v_codes)
    perm = torch.empty(ctx, dtype=torch.int32, device=k_codes.device)
    ms = ctypes.c_float(0.0)
    with torch.cuda.device(k_codes.device):
        rc = _lib.load().pkv_greedy_repack(_ptr(k_codes), _ptr(v_codes), _ptr(k_out), _ptr(v_out), _ptr(perm), ctx,
                                           hidden, int(block_size), int(pack_len), ctypes.byref(ms) if timed else None,
                                           _stream(k_codes.device))
    _lib.check(rc)
    return (k_out, v_out, perm, float(ms.value)) if timed else (k_out, v_out, perm)


def greedy_order(k_codes, v_codes, pack_len=16, block_size=64):
    """perm [ctx] int32 of greedy_repacking without the repacked matrices (for the fused encoders, which gather the
    rows of K and V themselves)."""
    _check_code_matrix(k_codes, "k_codes")
    _check_code_matrix(v_codes, "v_codes")
    _require(k_codes.shape == v_codes.shape, "K and V code matrices must have one shape")
    ctx, hidden = k_codes.shape
    perm = torch.empty(ctx, dtype=torch.int32, device=k_codes.device)
    with torch.cuda.device(k_codes.device):
        rc = _lib.load().pkv_greedy_repack(_ptr(k_codes), _ptr(v_codes), None, None, _ptr(perm), ctx, hidden,
                                           int(block_size), int(pack_len), None, _stream(k_codes.device))
    _lib.check(rc)
    return perm


def repack_and_encode(k_codes, v_codes, pack_size, repack_method="none", block_size=64):
    """`repack_and_encode` (utils/compute.py:329-357) on code matrices: (k_size_pre, v_size_pre, k_size_aft,
    v_size_aft) in bytes.  repack_method: "none", "median" or "greedy"."""
    k_pre, v_pre = bit_pack(k_codes, v_codes, pack_size)
    if repack_method == "median":
        k_codes, v_codes, _ = median_repacking(k_codes, v_codes, block_size)
    elif repack_method == "greedy":
        k_codes, v_codes, _ = greedy_repacking(k_codes, v_codes, pack_size, block_size)
    elif repack_method != "none":
        raise ValueError("repack_method must be one of none, median, greedy")
    k_aft, v_aft = bit_pack(k_codes, v_codes, pack_size)
    return k_pre, v_pre, k_aft, v_aft


def median_order(v, rel, bits=None, block_size=64, timed=False, want_params=False):
    """perm [T] int32 of `median_repacking` (utils/compute.py:262-270) for V [B, H, T, 128] quantised at `rel`,
    counted straight from V: perm[blk * block_size + r] = index inside the block of the token that moves to r."""
    B, H, T = _check_x(v)
    bits = bits or bits_for_rel(rel)
    perm = torch.empty(T, dtype=torch.int32, device=v.device)
    scale = torch.empty(B, T, dtype=v.dtype, device=v.device) if want_params else None
    zero = torch.empty(B, T, dtype=v.dtype, device=v.device) if want_params else None
    ms = ctypes.c_float(0.0)
    with torch.cuda.device(v.device):
        rc = _lib.load().pkv_median_order(_ptr(v), _dtype_code(v), B, H, T, float(rel), bits, int(block_size), _ptr(perm),
                                          _ptr(scale) if want_params else None, _ptr(zero) if want_params else None,
                                          ctypes.byref(ms) if timed else None, _stream(v.device))
    _lib.check(rc)
    out = (perm, scale, zero) if want_params else perm          # want_params: V's (scale, zero) in the order of v
    return (out, float(ms.value)) if timed else out


def repack_quant_encode(k, v, k_rel, v_rel, repack_method="median", block_size=64, k_bits=None, v_bits=None, fused=None):
    """Quantize K and V [B, H, T, 128], reorder the tokens of every quantisation block (jointly for K and V, as the
    reference's repacking does before it prices the packs, utils/compute.py:329-357) and encode.  Returns (k, v,
    perm): dicts like k_quant_encode / v_quant_encode -- stream, info, scale, zero in the REPACKED token order, so
    attn_decode takes them as they are (attention does not depend on the order of the cached tokens) -- and the
    permutation [T] int32 (perm[blk * block_size + r] = position inside the block the token at r came from).
    `fused` (default: whenever it applies -- median or greedy method, H <= 8, codes of at most 6 bits) runs the fused
    encoders on the permuted tokens: the median order is counted from V itself (median_order, no code matrix at all),
    the greedy order from the code matrices (greedy_order), which are then dropped instead of being repacked and
    encoded; fused=False goes through the code matrices (quantize, repack, block codec), which gives the same streams."""
    B, H, T = _check_x(k)
    _require(v.shape == k.shape and v.dtype == k.dtype and v.is_cuda and v.is_contiguous(), "K and V must have one shape")
    _require(T % 128 == 0 and T % block_size == 0, "the token count must be a multiple of 128 and of block_size")
    k_bits, v_bits = k_bits or bits_for_rel(k_rel), v_bits or bits_for_rel(v_rel)
    can_fuse = (repack_method in ("median", "greedy") and H <= 8 and max(k_bits, v_bits) <= 6 and block_size % 64 == 0 and
                block_size <= (1024 if repack_method == "median" else 256))
    if fused is None:
        fused = can_fuse
    if fused:
        # the order from V itself, then the fused encoders on the tokens in that order: no code matrix in HBM
        _require(can_fuse, "the fused path takes the median or greedy method, at most 8 KV heads, codes of at most 6 bits and "
                           "blocks of a multiple of 64 tokens")
        if repack_method == "median":
            perm, vs, vz = median_order(v, v_rel, v_bits, block_size, want_params=True)
        else:
            ks, kz = quant_params(k, k_rel)
            vs, vz = quant_params(v, v_rel)
            kc, kmx = quantize(k, ks, kz)
            vc, vmx = quantize(v, vs, vz)
            for mx, bits in ((kmx, k_bits), (vmx, v_bits)):
                if mx >= (1 << bits):
                    raise PackKVError(1, "not supported: code %d does not fit bits_len %d" % (mx, bits))
            perm = greedy_order(kc, vc, 16, block_size)      # the codecs' packs are 16 tokens
            del kc, vc
        ke = _quant_encode(True, k, k_rel, k_bits, None, None, True, False, perm, block_size)
        ve = _quant_encode(False, v, v_rel, v_bits, None, None, True, False, perm, block_size, (vs, vz))
        return ke, ve, perm
    ks, kz = quant_params(k, k_rel)
    vs, vz = quant_params(v, v_rel)
    kc, kmx = quantize(k, ks, kz)
    vc, vmx = quantize(v, vs, vz)
    for mx, bits in ((kmx, k_bits), (vmx, v_bits)):
        if mx >= (1 << bits):
            raise PackKVError(1, "not supported: code %d does not fit bits_len %d" % (mx, bits))
    if repack_method in ("median", "greedy"):
        if repack_method == "median":
            kc, vc, perm = median_repacking(kc, vc, block_size)
        else:
            kc, vc, perm = greedy_repacking(kc, vc, 16, block_size)      # the codecs' packs are 16 tokens
        src = (torch.arange(T, device=k.device, dtype=torch.int64) // block_size) * block_size + perm.to(torch.int64)
        ks, kz, vs, vz = (p[:, src].contiguous() for p in (ks, kz, vs, vz))
    elif repack_method == "none":
        perm = (torch.arange(T, device=k.device, dtype=torch.int32) % block_size)
    else:
        raise ValueError("repack_method must be one of none, median, greedy")
    hidden = B * H * 128
    out = []
    for is_k, codes, scale, zero, bits in ((True, kc, ks, kz, k_bits), (False, vc, vs, vz, v_bits)):
        ctx_blk, hid_blk = (64, 128) if is_k else (128, 64)
        nblk = (T // ctx_blk) * (hidden // hid_blk)
        stream = torch.empty(max(T * hidden, nblk * block_bound(is_k, ctx_blk, hid_blk, bits) + 16) if bits > 4
                             else T * hidden, dtype=torch.uint8, device=k.device)
        info = torch.empty(nblk, 2, dtype=torch.uint32, device=k.device)
        size = _encode(is_k, codes, stream, info, T, hidden, ctx_blk, hid_blk, bits, True, False, MAX_BITS)
        out.append({"stream": stream, "info": info, "scale": scale, "zero": zero, "size": int(size), "ms": 0.0,
                    "bits": bits})
    return out[0], out[1], perm


# ------------------------------------------------------- reference GEMV surface ------

def _require_cuda(*ts):
    for t in ts:
        if not t.is_cuda:
            raise RuntimeError("tensor must be a CUDA tensor")


def kq_mat_vec_mul(compressed_buffer, block_info_buffer, q, kq_out, ctx_len, hidden_dim,
                   ctx_len_block_size, hidden_dim_block_size, bits_len, q_interleaved=True):
    """Drop-in for packkv_cuda.kq_mat_vec_mul (packkv_cuda.pyi:26-36): kq_out[h, tok] =
    sum_d q[h, d] * code[tok, h*128 + d]; returns kernel milliseconds.  `q` is expected in the
    reference's lane-interleaved layout (evaluation/evaluation.py:465-468) unless
    q_interleaved=False.  Like the reference, an unsupported shape or dtype prints a message
    and returns 0.0 (src/kernels.cu:586-589, :626-629)."""
    _require_cuda(compressed_buffer, block_info_buffer, q, kq_out)
    if q.dtype not in (torch.float16, torch.bfloat16):
        print("Unsupported data type")
        return 0.0
    ms = ctypes.c_float(0.0)
    with torch.cuda.device(q.device):
        rc = _lib.load().pkv_kq_mat_vec_mul(_ptr(compressed_buffer), compressed_buffer.numel() * compressed_buffer.element_size(), _ptr(block_info_buffer), _ptr(q),
                                            _ptr(kq_out), ctx_len, hidden_dim, ctx_len_block_size,
                                            hidden_dim_block_size, bits_len, _dtype_code(q),
                                            int(bool(q_interleaved)), ctypes.byref(ms), _stream(q.device))
    if rc == _lib.ERR_UNSUPPORTED:
        print("no such case")
        return 0.0
    _lib.check(rc)
    return float(ms.value)


def wv_mat_vec_mul(compressed_buffer, block_info_buffer, w, wv_out, ctx_len, hidden_dim,
                   ctx_len_block_size, hidden_dim_block_size, bits_len):
    """Drop-in for packkv_cuda.wv_mat_vec_mul (packkv_cuda.pyi:60-70): wv_out (fp32, caller-zeroed,
    [hidden_dim] or [H, 128]) += sum_tok w[c // 128, tok] * code[tok, c]; returns milliseconds."""
    _require_cuda(compressed_buffer, block_info_buffer, w, wv_out)
    if w.dtype not in (torch.float16, torch.bfloat16):
        print("Unsupported data type")
        return 0.0
    if wv_out.dtype != torch.float32:
        raise RuntimeError("wv_out must be a float32 tensor")
    ms = ctypes.c_float(0.0)
    with torch.cuda.device(w.device):
        rc = _lib.load().pkv_wv_mat_vec_mul(_ptr(compressed_buffer), compressed_buffer.numel() * compressed_buffer.element_size(), _ptr(block_info_buffer), _ptr(w),
                                            _ptr(wv_out), ctx_len, hidden_dim, ctx_len_block_size,
                                            hidden_dim_block_size, bits_len, _dtype_code(w),
                                            ctypes.byref(ms), _stream(w.device))
    if rc == _lib.ERR_UNSUPPORTED:
        print("no such case")
        return 0.0
    _lib.check(rc)
    return float(ms.value)


def fused_kq(our_kq, q, k_quant_zero, k_quant_scale, t):
    """Drop-in for packkv_cuda.fused_kq (packkv_cuda.pyi:72-78; checks of
    src/fused_kernels.cu:90-108): our_kq[m, n] = (sum(q[m]) * zero[n] + t[m, n]) * scale[n]."""
    if q.dtype not in (torch.float16, torch.bfloat16):
        raise RuntimeError("Unsupported data type for fused_kq_launcher")
    if q.dim() != 2: raise RuntimeError("q must be a 2D tensor")
    if t.dim() != 2: raise RuntimeError("t must be a 2D tensor")
    if k_quant_zero.dim() != 1: raise RuntimeError("k_quant_zero must be a 1D tensor")
    if k_quant_scale.dim() != 1: raise RuntimeError("k_quant_scale must be a 1D tensor")
    if our_kq.dim() != 2: raise RuntimeError("our_kq must be a 2D tensor")
    M, K = q.shape
    N = t.size(1)
    if t.size(0) != M: raise RuntimeError("t.size(0) must be equal to q.size(0)")
    if k_quant_zero.size(0) != N: raise RuntimeError("k_quant_zero.size(0) must be equal to t.size(1)")
    if k_quant_scale.size(0) != N: raise RuntimeError("k_quant_scale.size(0) must be equal to t.size(1)")
    if our_kq.size(0) != M: raise RuntimeError("our_kq.size(0) must be equal to q.size(0)")
    if our_kq.size(1) != N: raise RuntimeError("our_kq.size(1) must be equal to t.size(1)")
    for name, x in (("q", q), ("t", t), ("k_quant_zero", k_quant_zero), ("k_quant_scale", k_quant_scale),
                    ("our_kq", our_kq)):
        if not x.is_cuda:
            raise RuntimeError("%s must be a CUDA tensor" % name)
    if not our_kq.is_contiguous(): raise RuntimeError("our_kq must be contiguous")
    ms = ctypes.c_float(0.0)
    # contiguous copies of strided inputs must outlive the call: a temporary released between two .contiguous() calls
    # can be handed the same memory again
    q_c, z_c, s_c, t_c = q.contiguous(), k_quant_zero.contiguous(), k_quant_scale.contiguous(), t.contiguous()
    with torch.cuda.device(q.device):
        rc = _lib.load().pkv_fused_kq(_ptr(our_kq), _ptr(q_c), _ptr(z_c), _ptr(s_c), _ptr(t_c), M, K, N,
                                      _dtype_code(q), ctypes.byref(ms), _stream(q.device))
    del q_c, z_c, s_c, t_c
    _lib.check(rc)
    return float(ms.value)


def fused_wv(our_wv, w, v_quant_zero, v_quant_scale, term1):
    """Drop-in for packkv_cuda.fused_wv (packkv_cuda.pyi:80-86; checks of
    src/fused_kernels.cu:275-293): our_wv[m, d] = sum_n w[m, n] * zero[n] * scale[n] + term1[m, d]."""
    if w.dtype not in (torch.float16, torch.bfloat16):
        raise RuntimeError("Unsupported data type for fused_wv_launcher")
    if w.dim() != 2: raise RuntimeError("w must be a 2D tensor")
    if term1.dim() != 2: raise RuntimeError("term1 must be a 2D tensor")
    if v_quant_zero.dim() != 1: raise RuntimeError("v_quant_zero must be a 1D tensor")
    if v_quant_scale.dim() != 1: raise RuntimeError("v_quant_scale must be a 1D tensor")
    if our_wv.dim() != 2: raise RuntimeError("our_wv must be a 2D tensor")
    M, N = w.shape
    D = term1.size(1)
    if term1.size(0) != M: raise RuntimeError("term1.size(0) must be equal to w.size(0)")
    if v_quant_zero.size(0) != N: raise RuntimeError("v_quant_zero.size(0) must be equal to w.size(1)")
    if v_quant_scale.size(0) != N: raise RuntimeError("v_quant_scale.size(0) must be equal to w.size(1)")
    if tuple(our_wv.shape) != (M, D): raise RuntimeError("our_wv shape must match term1")
    if term1.dtype != w.dtype: raise RuntimeError("term1 must have the dtype of w")
    for name, x in (("w", w), ("term1", term1), ("v_quant_zero", v_quant_zero),
                    ("v_quant_scale", v_quant_scale), ("our_wv", our_wv)):
        if not x.is_cuda:
            raise RuntimeError("%s must be a CUDA tensor" % name)
    if not our_wv.is_contiguous(): raise RuntimeError("our_wv must be contiguous")
    ms = ctypes.c_float(0.0)
    w_c, z_c, s_c, t_c = w.contiguous(), v_quant_zero.contiguous(), v_quant_scale.contiguous(), term1.contiguous()
    with torch.cuda.device(w.device):
        rc = _lib.load().pkv_fused_wv(_ptr(our_wv), _ptr(w_c), _ptr(z_c), _ptr(s_c), _ptr(t_c), M, N, D,
                                      _dtype_code(w), ctypes.byref(ms), _stream(w.device))
    del w_c, z_c, s_c, t_c
    _lib.check(rc)
    return float(ms.value)


# ------------------------------------------------- fused decompress-attention --------

class AttnPlan:
    """The checked, filled-in arguments of one decode step, kept for callers that repeat it (a decode loop over the
    same layer): ``plan()`` launches again without re-validating; ``plan(q=..., out=...)`` swaps the query / output
    tensors (same shape and dtype).  The tensors given at construction must stay alive and in place; build a new
    plan when a buffer is reallocated or the token counts change."""

    def __init__(self, q, k, v, k_win=None, v_win=None, sm_scale=None, out=None, variant=0, win_len=None,
                 ref_rounding=False, out_f32=False, noalloc=False):
        _require(q.is_cuda and q.dim() == 3 and q.size(2) == 128 and q.is_contiguous(),
                 "q must be a contiguous device tensor [B, Hq, 128]")
        B, Hq, _ = q.shape
        a = AttnArgs()
        T_c = 0
        Hkv = None
        if k is not None:
            T_c = int(k.get("tokens", k["scale"].size(1)))
            _require(int(v.get("tokens", v["scale"].size(1))) == T_c, "K and V hold different token counts")
            _require(0 < T_c <= k["scale"].size(1) and k["scale"].shape == v["scale"].shape,
                     "scale / zero rows shorter than the token count")
            a.par_stride = k["scale"].size(1)
            for name, d in (("k", k), ("v", v)):
                for f in ("stream", "info", "scale", "zero"):
                    _require(d[f].is_cuda and d[f].is_contiguous(), "%s.%s must be a contiguous device tensor" % (name, f))
            nblk_k = k["info"].numel() // 2
            Hkv = int(k["heads"]) if "heads" in k else nblk_k // (T_c // 64) // B
            _require(nblk_k >= (T_c // 64) * B * Hkv and v["info"].numel() // 2 >= (T_c // 128) * B * Hkv * 2,
                     "block_info_buffer block num mismatch")
            a.k_stream, a.k_info = _ptr(k["stream"]), _ptr(k["info"])
            a.v_stream, a.v_info = _ptr(v["stream"]), _ptr(v["info"])
            # readable bytes of each buffer.  The default kernel copies whole dwords and needs no slack; the gather
            # kernel (variant 2, and variant 0 on streams that are not 16-byte aligned) fetches pack words as whole
            # 8-byte words and needs 7 readable bytes behind the encoded size: without them the plain kernel runs
            gathers = int(variant) == 2 or (int(variant) == 0 and (k["stream"].data_ptr() | v["stream"].data_ptr()) % 16 != 0)
            if gathers and any(d.get("size") and d["stream"].numel() < int(d["size"]) + 7 for d in (k, v)):
                variant = 1
            a.k_bytes, a.v_bytes = k["stream"].numel(), v["stream"].numel()
            a.k_scale, a.k_zero = _ptr(k["scale"]), _ptr(k["zero"])
            a.v_scale, a.v_zero = _ptr(v["scale"]), _ptr(v["zero"])
            a.k_bits, a.v_bits = int(k["bits"]), int(v["bits"])
        T_w = 0
        if k_win is not None:
            _require(k_win.is_cuda and v_win.is_cuda and k_win.is_contiguous() and v_win.is_contiguous()
                     and k_win.shape == v_win.shape and k_win.dim() == 4 and k_win.size(3) == 128
                     and k_win.dtype == q.dtype and v_win.dtype == q.dtype,
                     "window tensors must be contiguous [B, Hkv, T_w, 128] of q's dtype")
            T_w = k_win.size(2) if win_len is None else int(win_len)
            _require(0 < T_w <= k_win.size(2), "win_len outside the window tensors")
            a.win_stride = k_win.size(2)
            _require(Hkv is None or Hkv == k_win.size(1), "window head count mismatch")
            Hkv = k_win.size(1)
            a.k_win, a.v_win = _ptr(k_win), _ptr(v_win)
        _require(Hkv is not None, "empty cache")
        out_dtype = torch.float32 if out_f32 else q.dtype
        if out is None:
            out = torch.empty(q.shape, dtype=out_dtype, device=q.device)
        _require(out.is_cuda and out.shape == q.shape and out.dtype == out_dtype and out.is_contiguous(),
                 "out must be a contiguous device tensor of q's shape (fp32 with out_f32, else q's dtype)")
        a.flags = (_lib.ATTN_REF_ROUNDING if ref_rounding else 0) | (_lib.ATTN_OUT_F32 if out_f32 else 0)
        a.q, a.out = _ptr(q), _ptr(out)
        a.B, a.Hq, a.Hkv, a.T_c, a.T_w = B, Hq, Hkv, T_c, T_w
        a.dtype = _dtype_code(q)
        a.sm_scale = float(sm_scale if sm_scale is not None else 128 ** -0.5)
        a.variant = int(variant)
        self.args, self.out, self.device = a, out, q.device
        self._shape, self._dtype, self._out_dtype = q.shape, q.dtype, out_dtype
        self._keep = (q, k, v, k_win, v_win, out)          # the buffers the pointers refer to
        self._fn = _lib.load().pkv_attn_decode
        self._fn_noalloc = _lib.load().pkv_attn_decode_noalloc if noalloc else None
        self._ref = ctypes.byref(a)

    def set_window_rows(self, win_len):
        """Window rows in use (the window tensors are allocated longer and fill up between cuts)."""
        self.args.T_w = int(win_len)

    def __call__(self, q=None, out=None, timed=False):
        a = self.args
        if q is not None:
            _require(q.is_cuda and q.shape == self._shape and q.dtype == self._dtype and q.is_contiguous(),
                     "q must match the plan's query tensor")
            a.q = _ptr(q)
        if out is not None:
            _require(out.is_cuda and out.shape == self._shape and out.dtype == self._out_dtype and out.is_contiguous(),
                     "out must match the plan's output tensor")
            a.out = _ptr(out)
            self.out = out
        ms = ctypes.c_float(0.0)
        with torch.cuda.device(self.device):
            if self._fn_noalloc is not None:
                _require(not timed, "the entry point that allocates nothing does not time its launch")
                rc = self._fn_noalloc(self._ref, _stream(self.device))
            else:
                rc = self._fn(self._ref, ctypes.byref(ms) if timed else None, _stream(self.device))
        if rc:
            _lib.check(rc)
        return (self.out, float(ms.value)) if timed else self.out


def attn_decode(q, k, v, k_win=None, v_win=None, sm_scale=None, out=None, variant=0, timed=False, win_len=None,
                ref_rounding=False, out_f32=False, noalloc=False):
    """One decode step over a compressed cache.

    q [B, Hq, 128]; k and v are the dicts returned by k_quant_encode / v_quant_encode (stream,
    info, scale, zero, bits) or None when only the 16-bit window exists; k_win / v_win are
    optional [B, Hkv, T_w, 128] tails.  Returns out [B, Hq, 128] (and ms when timed).

    Buffers allocated for a cache that grows: the dicts may carry ``tokens`` (compressed tokens in use;
    scale / zero rows and block_info are then longer than that) and ``heads`` (KV heads); ``win_len``
    gives the window rows in use when k_win / v_win are allocated longer.  AttnPlan keeps the checked
    arguments for callers that repeat the step.

    out_f32: the result as fp32, before its rounding to q's dtype.  ref_rounding (variant 1 only): the checking
    mode -- every K and V element is formed as the reference stores it, dtype(dtype(code + zero) * scale)
    (utils/compute.py:173-179), before the fp32 dot products.  noalloc: go through pkv_attn_decode_noalloc (the
    partial results in the library's fixed 8 MiB device array; the caller passes `out`, or torch allocates it)."""
    return AttnPlan(q, k, v, k_win, v_win, sm_scale, out, variant, win_len, ref_rounding, out_f32, noalloc)(timed=timed)
