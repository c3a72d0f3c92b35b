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
    v = x.float()
    return (v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps)).to(x.dtype) * w


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
            self.blocks.append({
                "in_norm": one(s.hidden), "post_norm": one(s.hidden),
                "q": w(s.q_heads * s.head_dim, s.hidden), "k": w(s.kv_heads * s.head_dim, s.hidden),
                "v": w(s.kv_heads * s.head_dim, s.hidden), "o": w(s.hidden, s.q_heads * s.head_dim),
                "q_norm": one(s.head_dim), "k_norm": one(s.head_dim),
                "gate": w(s.mlp, s.hidden), "up": w(s.mlp, s.hidden), "down": w(s.hidden, s.mlp),
            })
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
        h = self.embed[ids]
        for li, blk in enumerate(self.blocks):
            x = _rms(h, blk["in_norm"], s.rms_eps)
            q = F.linear(x, blk["q"]).view(B, n, s.q_heads, s.head_dim).transpose(1, 2)
            k = F.linear(x, blk["k"]).view(B, n, s.kv_heads, s.head_dim).transpose(1, 2)
            v = F.linear(x, blk["v"]).view(B, n, s.kv_heads, s.head_dim).transpose(1, 2)
            if s.head_norm:
                q, k = _rms(q, blk["q_norm"], s.rms_eps), _rms(k, blk["k_norm"], s.rms_eps)
            q = q * cos.unsqueeze(1) + rotate_half(q) * sin.unsqueeze(1)
            kw = {"cos": cos, "sin": sin}
            if fused:
                cache.update(k, v, li, kw, return_dense=False)
                a = cache.attend(q, li, sm_scale=scaling)                          # [B, Hq, 1, 128]
            else:
                kd, vd = cache.update(k, v, li, kw, return_dense=True)
                a = self._dense_attention(q, kd, vd, scaling)
            if taps is not None:
                taps.append((q, a))
            h = h + F.linear(a.transpose(1, 2).reshape(B, n, s.q_heads * s.head_dim), blk["o"])
            x = _rms(h, blk["post_norm"], s.rms_eps)
            h = h + F.linear(F.silu(F.linear(x, blk["gate"])) * F.linear(x, blk["up"]), blk["down"])
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
