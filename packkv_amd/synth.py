"""Seeded synthetic K / V / q tensors of the shapes the benchmarks are quoted on.

K ~ N(0,1) with four fixed outlier channels per head scaled x10 (or a per-channel log-uniform
scale), V ~ N(0,1), q ~ N(0,1); 16-bit storage.  Generated on the requested device with a
seeded torch.Generator so that a run is reproducible; small test cases generate on the CPU and
copy, so that the CPU checker and the GPU see identical bits.
"""
import math

import torch

OUTLIER_CHANNELS = (3, 40, 77, 120)


def make_kv(B, Hkv, T, seed=0, dtype=torch.float16, device="cpu", k_mode="outliers", chunk_tokens=8192):
    """Returns (k, v), each [B, Hkv, T, 128] in `dtype` on `device`."""
    dev = torch.device(device)
    gen = torch.Generator(device=dev)
    gen.manual_seed(seed)
    k = torch.empty(B, Hkv, T, 128, dtype=dtype, device=dev)
    v = torch.empty(B, Hkv, T, 128, dtype=dtype, device=dev)
    if k_mode == "channel_scale":
        u = torch.rand(Hkv, 128, generator=gen, device=dev)
        ch_scale = torch.exp(math.log(0.1) + u * (math.log(10.0) - math.log(0.1)))
    for t0 in range(0, T, chunk_tokens):      # chunked: fp32 temporaries stay small
        t1 = min(T, t0 + chunk_tokens)
        kc = torch.randn(B, Hkv, t1 - t0, 128, generator=gen, device=dev)
        if k_mode == "outliers":
            kc[..., list(OUTLIER_CHANNELS)] *= 10.0
        elif k_mode == "channel_scale":
            kc *= ch_scale[None, :, None, :]
        k[:, :, t0:t1] = kc.to(dtype)
        v[:, :, t0:t1] = torch.randn(B, Hkv, t1 - t0, 128, generator=gen, device=dev).to(dtype)
    return k, v


def make_q(B, Hq, seed=1, dtype=torch.float16, device="cpu"):
    dev = torch.device(device)
    gen = torch.Generator(device=dev)
    gen.manual_seed(seed)
    return torch.randn(B, Hq, 128, generator=gen, device=dev).to(dtype)
