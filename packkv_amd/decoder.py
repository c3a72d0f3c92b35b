"""A random-init decoder of Qwen3 / Llama shape around the compressed cache: the caller side of the hot path.

This is measurement and test scaffolding in plain torch, not a model implementation: projections, norms and the
MLP are library GEMMs and elementwise ops; what it exercises is the place where the reference's attention module
meets its cache (models/llama.py:242-294, and models/qwen3.py:175-198 for the per-head q / k norms):

    q, k, v = projections; q, k = head norms (Qwen3 shape only); q = rotary(q)
    K, V = cache.update(k, v, layer, {"cos", "sin"})        # the cache applies the rotary embedding to K
    out  = eager_attention(q, K, V)                           # decompress-then-attend

At decode time (one new token) ``attention="fused"`` replaces the last two lines by ``cache.update(...,
return_dense=False)`` and ``cache.attend(q, layer)``, the fused decompress-attention kernel;
``attention="dense"`` keeps the reference's decompress-then-attend through ``cache.materialize``.  Prefill always
attends to the dense tensors the cache returns, as the reference does.
"""
import math

import torch
import torch.nn.functional as F

from .cache import PackKVCompressedCache, PackKVCacheConfig, rotate_half


class DecoderShape:
    """Qwen3-8B by default: 36 layers, hidden 4096, 32 query / 8 KV heads of 128, MLP 12288, vocabulary 151936."""

    def __init__(self, layers=36, hidden=4096, q_heads=32, kv_heads=8, head_dim=128, mlp=12288, vocab=151936,
                 rope_theta=1.0e6, rms_eps=1.0e-6, head_norm=True):
        self.layers, self.hidden, self.q_heads, self.kv_heads, self.head_dim = layers, hidden, q_heads, kv_heads, head_dim
        self.mlp, self.vocab, self.rope_theta, self.rms_eps, self.head_norm = mlp, vocab, rope_theta, rms_eps, head_norm


def _rms(x, w, eps):
    """RMS norm over the last dimension in fp32, one library kernel (models/qwen3.py:53-58 rounds to the storage
    dtype before the weight multiply; the two agree wherever the weight is exactly representable times the value,
    as for the unit weights used here)."""
    return F.rms_norm(x, (x.size(-1),), w, eps)


class ShapedDecoder:
    """Weights ~ N(0, 0.02), norm weights 1, in `dtype` on `device`; no gradients anywhere."""

    def __init__(self, shape=None, dtype=torch.bfloat16, device="cuda", seed=0):
        self.shape = s = shape or DecoderShape()
        self.dtype, self.device = dtype, torch.device(device)
        g = torch.Generator(device=self.device).manual_seed(seed)

        def w(*dims):
            return (torch.randn(*dims, generator=g, device=self.device, dtype=torch.float32) * 0.02).to(dtype)

        one = lambda n: torch.ones(n, dtype=dtype, device=self.device)
        self.embed = w(s.vocab, s.hidden)
        self.lm_head = w(s.vocab, s.hidden)
        self.final_norm = one(s.hidden)
        self.blocks = []
        for _ in range(s.layers):
            # q, k, v projections as one weight [Hq*128 + 2*Hkv*128, hidden] and gate, up as one [2*mlp, hidden]:
            # a decode step is launch-bound around the cache, so every projection pair that shares its input is
            # one library GEMM
            blk = {"in_norm": one(s.hidden), "post_norm": one(s.hidden)}
            blk["qkv"] = torch.cat((w(s.q_heads * s.head_dim, s.hidden), w(s.kv_heads * s.head_dim, s.hidden),
                                    w(s.kv_heads * s.head_dim, s.hidden)), dim=0)
            blk["o"] = w(s.hidden, s.q_heads * s.head_dim)
            blk["q_norm"], blk["k_norm"] = one(s.head_dim), one(s.head_dim)
            blk["gate_up"] = torch.cat((w(s.mlp, s.hidden), w(s.mlp, s.hidden)), dim=0)
            blk["down"] = w(s.hidden, s.mlp)
            self.blocks.append(blk)
        inv = 1.0 / (s.rope_theta ** (torch.arange(0, s.head_dim, 2, device=self.device, dtype=torch.float32) / s.head_dim))
        self.inv_freq = inv

    def new_cache(self, batch, max_tokens, config=None):
        s = self.shape
        return PackKVCompressedCache(batch, s.kv_heads, s.head_dim, s.layers, config or PackKVCacheConfig(),
                                     max_tokens=max_tokens, dtype=self.dtype, device=self.device)

    def _rotary(self, pos0, n, batch):
        t = torch.arange(pos0, pos0 + n, device=self.device, dtype=torch.float32)
        f = torch.outer(t, self.inv_freq)
        emb = torch.cat((f, f), dim=-1)
        cos, sin = emb.cos().to(self.dtype), emb.sin().to(self.dtype)
        return cos.unsqueeze(0).expand(batch, n, -1), sin.unsqueeze(0).expand(batch, n, -1)

    @staticmethod
    def _rotate_q(q, cos, sin_signed):
        """q [B, n, Hq, 128] * cos + rotate_half(q) * sin with the reference's roundings (each product rounded,
        then the sum; utils/compute.py:35-43): rotate_half(q) * sin = roll(q, 64) * (-sin | sin), sign changes
        being exact."""
        t = q * cos.unsqueeze(2)
        t += torch.roll(q, q.size(-1) // 2, -1) * sin_signed.unsqueeze(2)
        return t

    def _dense_attention(self, q, k, v, scaling):
        """Decode step (one query token): the reference's eager attention (models/llama.py:189-212: fp32 softmax
        cast back to the storage dtype), with the query heads of a group stacked instead of K / V repeated.
        Prompt pass: the library's causal attention, a few sequences at a time."""
        B, Hq, n, D = q.shape
        Hkv = k.size(1)
        if n == 1:
            qg = q.reshape(B, Hkv, Hq // Hkv, D)
            w = torch.matmul(qg, k.transpose(2, 3)) * scaling
            w = F.softmax(w, dim=-1, dtype=torch.float32).to(q.dtype)
            return torch.matmul(w, v).reshape(B, Hq, 1, D)
        out = torch.empty_like(q)
        for b in range(0, B, 4):
            out[b:b + 4] = F.scaled_dot_product_attention(q[b:b + 4], k[b:b + 4], v[b:b + 4], is_causal=True,
                                                          scale=scaling, enable_gqa=True)
        return out

    @torch.no_grad()
    def forward(self, ids, cache, attention="fused", taps=None):
        """ids [B, n] continue the sequences held in `cache`; returns the logits of the last position [B, vocab]
        (fp32).  `taps`, a list, receives every layer's (rotated query, attention output), both [B, Hq, n, 128],
        when given."""
        s = self.shape
        B, n = ids.shape
        pos0 = cache.get_seq_length(0)
        cos, sin = self._rotary(pos0, n, B)
        fused = attention == "fused" and n == 1
        scaling = 1.0 / math.sqrt(s.head_dim)
        half = s.head_dim // 2
        sin_signed = torch.cat((-sin[..., :half], sin[..., half:]), dim=-1)
        nq = s.q_heads * s.head_dim
        kw = {"cos": cos, "sin": sin}
        h = self.embed[ids].view(B * n, s.hidden)
        for li, blk in enumerate(self.blocks):
            x = _rms(h, blk["in_norm"], s.rms_eps)
            qkv = F.linear(x, blk["qkv"]).view(B, n, s.q_heads + 2 * s.kv_heads, s.head_dim)
            q, k, v = qkv[:, :, :s.q_heads], qkv[:, :, s.q_heads:s.q_heads + s.kv_heads], qkv[:, :, s.q_heads + s.kv_heads:]
            if s.head_norm:
                q, k = _rms(q, blk["q_norm"], s.rms_eps), _rms(k, blk["k_norm"], s.rms_eps)
                v = v.contiguous()                        # the cache reads K and V with one set of strides
            q = self._rotate_q(q, cos, sin_signed).transpose(1, 2)                 # [B, Hq, n, 128]
            k, v = k.transpose(1, 2), v.transpose(1, 2)
            if fused:
                cache.update(k, v, li, kw, return_dense=False)
                a = cache.attend(q, li, sm_scale=scaling)                          # [B, Hq, 1, 128]
            else:
                kd, vd = cache.update(k, v, li, kw, return_dense=True)
                a = self._dense_attention(q, kd, vd, scaling)
            if taps is not None:
                taps.append((q, a))
            h = torch.addmm(h, a.transpose(1, 2).reshape(B * n, nq), blk["o"].t())
            x = _rms(h, blk["post_norm"], s.rms_eps)
            gu = F.linear(x, blk["gate_up"])
            h = torch.addmm(h, F.silu(gu[:, :s.mlp]) * gu[:, s.mlp:], blk["down"].t())
        h = h.view(B, n, s.hidden)
        h = _rms(h[:, -1], self.final_norm, s.rms_eps)
        return F.linear(h, self.lm_head).float()

    @torch.no_grad()
    def prefill(self, ids, cache):
        """Prompt pass: attends to the dense tensors the cache returns, as the reference does."""
        return self.forward(ids, cache, attention="dense")

    @torch.no_grad()
    def greedy(self, ids, cache, steps, attention="fused"):
        """Prefill `ids` [B, n], then `steps` greedy tokens.  Returns the generated ids [B, steps]."""
        logits = self.prefill(ids, cache)
        out = []
        for _ in range(steps):
            nxt = logits.argmax(dim=-1, keepdim=True)
            out.append(nxt)
            logits = self.forward(nxt, cache, attention=attention)
        return torch.cat(out, dim=1)
