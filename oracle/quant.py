"""TEST INFRASTRUCTURE ONLY: CPU restatement of the reference quantizer, layouts,
size model and the decompress-then-attend path.

Restates (PyTorch CPU ops, same op order as the reference so that every intermediate is
rounded to the tensor dtype exactly where the reference rounds it):
  quant_ints, TokenQuant mode       utils/compute.py:84-112, QUANT_DIM :405-410
  dequant (code + zero) * scale     utils/compute.py:173-179
  code-matrix layout                evaluation/evaluation.py:406-408 (K), :596-598 (V)
  q channel re-interleave           evaluation/evaluation.py:465-468
  bit_pack size model               utils/compute.py:272-297
  cut_tensor residual-window policy utils/compute.py:54-67
  eager attention                   models/llama.py:177-212

Pinned by: ``quant_ints_np`` below (an independent NumPy emulation that computes every
op in fp32 and rounds to the storage dtype by explicit bit manipulation), closed forms
in the tests, and fp64 NumPy attention.
"""
import math

import numpy as np
import torch


# --------------------------------------------------------------- quantizer ---

def quant_ints(x, block_size, rel):
    """x: [B, H, T, D] fp16/bf16.  Returns (codes, zero, scale) with codes float-typed
    [B, H, T/bs, bs, D] and zero/scale [B, 1, T/bs, bs, 1] (one pair per (batch, token),
    shared by all heads and channels)."""
    assert x.shape[2] % block_size == 0
    t = x.reshape(x.shape[0], x.shape[1], -1, block_size, x.shape[3])
    mn, mx = t, t
    for d in (1, 4):
        mn = mn.min(dim=d, keepdim=True).values
        mx = mx.max(dim=d, keepdim=True).values
    scale = (mx - mn) * rel
    zero = (mn / scale).round()
    codes = (t / scale).round() - zero
    return codes, zero, scale


def dequant(codes, zero, scale):
    """[B, H, nb, bs, D] -> [B, H, T, D] in the tensor dtype."""
    y = (codes + zero) * scale
    return y.reshape(y.shape[0], y.shape[1], -1, y.shape[4])


def code_matrix(codes):
    """[B, H, nb, bs, D] float codes -> uint8 [ctx_len, B*H*D], channel = (b*H + h)*D + d."""
    return codes.flatten(2, 3).permute(2, 0, 1, 3).flatten(1, 3).contiguous().to(torch.uint8)


def bits_for_codes(code_mat):
    """ceil(log2(#distinct codes)) -- how the reference call sites derive bits_len
    (evaluation/evaluation.py:416, :607)."""
    n = int(torch.unique(code_mat).numel())
    return max(1, math.ceil(math.log2(n))) if n > 1 else 1


def q_interleave(q):
    """q [H, 128] -> lane-ordered layout expected by the reference K kernel."""
    h = q.shape[0]
    r = q.view(h, 32, 4)
    return torch.cat([r[:, :, :2].contiguous().view(h, -1), r[:, :, 2:].contiguous().view(h, -1)], dim=1)


# ---- independent emulation used to pin quant_ints ----------------------------

def _round_to(x32, dtype):
    """Round an fp32 array to fp16/bf16 (nearest even), back as fp32."""
    if dtype == "fp16":
        return x32.astype(np.float16).astype(np.float32)
    u = x32.view(np.uint32).astype(np.uint64)
    lsb = (u >> 16) & 1
    u = (u + 0x7FFF + lsb) & 0xFFFF0000
    return u.astype(np.uint32).view(np.float32)


def quant_ints_np(x32, dtype, block_size, rel):
    """x32: fp32 array [B, H, T, D] whose values are exactly representable in ``dtype``.
    Returns codes [B, H, T, D], zero [B, T], scale [B, T] as fp32 arrays holding the
    dtype-rounded values."""
    f = np.float32
    mn = x32.min(axis=(1, 3))
    mx = x32.max(axis=(1, 3))
    rng = _round_to((mx - mn).astype(f), dtype)
    scale = _round_to(rng * f(rel), dtype)
    zero = _round_to(np.rint(_round_to(mn / scale, dtype)), dtype)
    s = scale[:, None, :, None]
    z = zero[:, None, :, None]
    codes = _round_to(_round_to(np.rint(_round_to(x32 / s, dtype)), dtype) - z, dtype)
    return codes, zero, scale


# ----------------------------------------------------------- size model -------

def bit_pack_bytes(code_mat, pack_len, W=None):
    """Closed form of the reference's analytic size for ONE tensor: code_mat is an integer
    array [ctx_len, channels]; packs are ``pack_len`` consecutive tokens of one channel."""
    c = np.asarray(code_mat).astype(np.int64)
    if W is None:
        W = math.ceil(math.log2(len(np.unique(c))))
    p = c.reshape(-1, pack_len, c.shape[1])
    rng = p.max(axis=1) - p.min(axis=1)
    lens = np.ceil(np.log2(rng + 1)).astype(np.int64)
    bits = int(lens.sum()) * pack_len + rng.size * (W + math.ceil(math.log2(W + 1)))
    return bits // 8


def cut_counts(buffered, new, block_size, recent_size):
    """(tokens to compress now, tokens left in the fp16 window) after appending ``new``
    tokens to a window holding ``buffered``."""
    n = buffered + new
    blocks = (n + block_size - n % block_size - recent_size) // block_size
    blocks = max(blocks, 0)
    return blocks * block_size, n - blocks * block_size


# ------------------------------------------------------------ attention -------

def repeat_kv(x, n_rep):
    b, h, t, d = x.shape
    if n_rep == 1:
        return x
    return x[:, :, None, :, :].expand(b, h, n_rep, t, d).reshape(b, h * n_rep, t, d)


def eager_attention(q, k, v, scaling=None):
    """The reference's eager path for one decode step, in the storage dtype:
    q [B, Hq, 1, D], k/v [B, Hkv, T, D] -> [B, Hq, 1, D]."""
    g = q.shape[1] // k.shape[1]
    scaling = q.shape[-1] ** -0.5 if scaling is None else scaling
    ks, vs = repeat_kv(k, g), repeat_kv(v, g)
    w = torch.matmul(q, ks.transpose(2, 3)) * scaling
    w = torch.nn.functional.softmax(w, dim=-1, dtype=torch.float32).to(q.dtype)
    return torch.matmul(w, vs)


def attention_f32(q, k, v, scaling=None):
    """Same attention on the same (already dequantised, dtype-rounded) K/V but with fp32
    products, accumulation and softmax -- the comparison target for the fused kernel."""
    g = q.shape[1] // k.shape[1]
    scaling = q.shape[-1] ** -0.5 if scaling is None else scaling
    ks, vs = repeat_kv(k.float(), g), repeat_kv(v.float(), g)
    w = torch.matmul(q.float(), ks.transpose(2, 3)) * scaling
    w = torch.softmax(w, dim=-1)
    return torch.matmul(w, vs)


def attention_f64_np(q, k, v, scaling=None):
    """fp64 NumPy attention used to pin the two torch versions above."""
    q = q.double().numpy(); k = k.double().numpy(); v = v.double().numpy()
    g = q.shape[1] // k.shape[1]
    scaling = q.shape[-1] ** -0.5 if scaling is None else scaling
    k = np.repeat(k, g, axis=1); v = np.repeat(v, g, axis=1)
    s = np.einsum("bhqd,bhtd->bhqt", q, k) * scaling
    s = s - s.max(axis=-1, keepdims=True)
    p = np.exp(s); p /= p.sum(axis=-1, keepdims=True)
    return np.einsum("bhqt,bhtd->bhqd", p, v)
