"""Compressed KV cache that grows: the device-side counterpart of the reference's simulated cache
(models/cache/packkv_quant.py:30-131, ``PackKVCachePytorchQuant``; wrapper models/cache/packkv_cache.py:22-38).

The reference keeps the quantised prefix in DEQUANTISED 16-bit form and returns ``cat(prefix, buffer)``
from ``update`` for eager attention.  This class keeps the prefix as PackKV streams and answers a decode
step with the fused decompress-attention kernel; ``update`` has the reference's signature and policy:

  * K gets its rotary embedding inside the cache when ``cache_kwargs`` holds cos / sin
    (packkv_quant.py:59-60, utils/compute.py:35-43);
  * residual window per utils/compute.py:54-67 (``cut_tensor``): after appending the new tokens,
    ``n_blk = (len + bs - len % bs - buffer_size) // bs`` blocks of ``bs`` tokens leave the 16-bit buffer
    and are quantised (per token, so cutting chunk by chunk gives the codes of a one-shot quantisation);
  * the streams are append-only.  The attention kernel walks tiles of 128 tokens (one V block), so an odd
    64-token cut waits for its partner: until then it sits in the 16-bit window in DEQUANTISED form -- the
    values the reference attends over -- and its original values are kept aside for the encode.

``materialize`` rebuilds what the reference's ``update`` returns (for parity tests and for callers that still
want dense tensors); ``attend`` is the hot path.  There is no CPU path: every operation runs through the HIP
library.
"""
import torch

from . import ops


class PackKVCacheConfig:
    """The fields of the reference's cache configuration this path reads (block_size, buffer_size,
    k_quant_scale_rel, v_quant_scale_rel: models/cache/packkv_quant.py:62-82;
    scripts/throughput_config_test.py:16-24 uses 64 / 192 / 0.1 / 0.1)."""

    def __init__(self, block_size=64, buffer_size=192, k_quant_scale_rel=0.1, v_quant_scale_rel=0.1,
                 k_bits=None, v_bits=None, enable_quant=True):
        self.enable_quant = enable_quant
        if block_size != 64:
            raise RuntimeError("not supported: block_size %d (the K block is 64 tokens)" % block_size)
        if buffer_size < block_size or buffer_size + 2 * block_size > 2048:
            raise RuntimeError("not supported: buffer_size %d" % buffer_size)
        self.block_size, self.buffer_size = block_size, buffer_size
        self.k_quant_scale_rel, self.v_quant_scale_rel = k_quant_scale_rel, v_quant_scale_rel
        self.k_bits = k_bits or ops.bits_for_rel(k_quant_scale_rel)
        self.v_bits = v_bits or ops.bits_for_rel(v_quant_scale_rel)


def rotate_half(x):
    h = x.shape[-1] // 2
    return torch.cat((-x[..., h:], x[..., :h]), dim=-1)


def apply_rotary_pos_emb_single(t, cos, sin, unsqueeze_dim=1):
    """utils/compute.py:35-43: t [B, H, n, D], cos / sin [B, n, D]."""
    cos, sin = cos.unsqueeze(unsqueeze_dim), sin.unsqueeze(unsqueeze_dim)
    return (t * cos) + (rotate_half(t) * sin)


class _Side:
    """The compressed state of K or of V of one layer."""

    def __init__(self, is_k, B, H, rel, bits, max_tokens, dtype, device):
        self.is_k, self.B, self.H, self.rel, self.bits = is_k, B, H, rel, bits
        ctx_blk, hid_blk = (64, 128) if is_k else (128, 64)
        self.blocks_per_tile = (128 // ctx_blk) * (B * H * 128 // hid_blk)
        self.bound = ops.block_bound(is_k, ctx_blk, hid_blk, bits)
        self.par_stride = (max_tokens + 127) // 128 * 128
        self.info = torch.empty(self.par_stride // 128 * self.blocks_per_tile, 2, dtype=torch.uint32, device=device)
        self.scale = torch.zeros(B, self.par_stride, dtype=dtype, device=device)
        self.zero = torch.zeros(B, self.par_stride, dtype=dtype, device=device)
        self.stream = torch.empty(0, dtype=torch.uint8, device=device)
        self.used = 0          # bytes of the stream in use
        self.tokens = 0        # tokens encoded

    def _reserve(self, n_tiles):
        """Room for n_tiles more tiles at their worst-case size, plus the slack the readers ask for."""
        need = self.used + n_tiles * self.blocks_per_tile * self.bound + 16
        if need > self.stream.numel():
            # grow by what the cache has needed so far per token, at least half as much again
            grown = torch.empty(max(need, self.stream.numel() * 3 // 2), dtype=torch.uint8, device=self.stream.device)
            grown[: self.used] = self.stream[: self.used]
            self.stream = grown

    def append(self, x):
        """x [B, H, n, 128], n a multiple of 128: encode and append."""
        n = x.size(2)
        if self.tokens + n > self.par_stride:
            raise RuntimeError("compressed cache is full (%d tokens)" % self.par_stride)
        self._reserve(n // 128)
        self.used = ops.quant_encode_append(self.is_k, x, self.rel, self.bits, self.stream, self.used, self.info,
                                            self.tokens, self.scale, self.zero)
        self.tokens += n

    def as_dict(self):
        return {"stream": self.stream, "info": self.info, "scale": self.scale, "zero": self.zero, "bits": self.bits,
                "size": self.used, "tokens": self.tokens, "heads": self.H}


class _Layer:
    def __init__(self, B, H, cfg, max_tokens, dtype, device):
        self.k = _Side(True, B, H, cfg.k_quant_scale_rel, cfg.k_bits, max_tokens, dtype, device)
        self.v = _Side(False, B, H, cfg.v_quant_scale_rel, cfg.v_bits, max_tokens, dtype, device)
        # 16-bit window [pending 64-token cut, dequantised | buffer]; rows hold `cap` tokens
        self.cap = 64 + cfg.buffer_size + 64
        self.k_win = torch.empty(B, H, self.cap, 128, dtype=dtype, device=device)
        self.v_win = torch.empty(B, H, self.cap, 128, dtype=dtype, device=device)
        self.win_len = 0
        self.pend = 0                      # 0 or 64: tokens at the head of the window that are a quantised cut
        self.k_pend = self.v_pend = None   # their original values
        self.plan = None                   # checked arguments of the decode step, valid until the next cut


class PackKVCompressedCache:
    """``update`` / ``get_seq_length`` as in the reference's cache classes, plus ``attend``."""

    def __init__(self, batch_size, head_num, head_dim, layer_num, config=None, max_tokens=32768,
                 dtype=torch.float16, device="cuda"):
        if head_dim != 128:
            raise RuntimeError("not supported: head_dim %d" % head_dim)
        self.config = config or PackKVCacheConfig()
        self.batch_size, self.head_num, self.head_dim = batch_size, head_num, head_dim
        self.max_tokens, self.dtype, self.device = max_tokens, dtype, torch.device(device)
        self.layers = [None] * layer_num

    def _layer(self, i):
        if self.layers[i] is None:
            self.layers[i] = _Layer(self.batch_size, self.head_num, self.config, self.max_tokens, self.dtype,
                                    self.device)
        return self.layers[i]

    # -- reference contract --------------------------------------------------------------------------
    def update(self, key_states, value_states, layer_idx, cache_kwargs=None, return_dense=True):
        """Append key_states / value_states [B, H, n, 128].  Returns the dense (K, V) [B, H, T, 128] the reference's
        update returns (packkv_quant.py:84-85), so that the caller's eager attention runs unchanged
        (models/llama.py:261); a caller that attends through ``attend`` passes return_dense=False and gets None --
        building the dense view decompresses the whole layer."""
        L = self._layer(layer_idx)
        cfg = self.config
        rotary = bool(cache_kwargs) and cache_kwargs.get("cos") is not None
        n = key_states.size(2)
        buf_len = L.win_len - L.pend
        total = buf_len + n
        n_blk = max((total + cfg.block_size - total % cfg.block_size - cfg.buffer_size) // cfg.block_size, 0)
        n_cut = n_blk * cfg.block_size
        if n_cut == 0 and L.win_len + n <= L.cap:                 # the common decode step: rotary + the new rows, one launch
            ops.window_append(key_states, value_states, cache_kwargs["cos"] if rotary else None,
                              cache_kwargs["sin"] if rotary else None, L.k_win, L.v_win, L.win_len)
            L.win_len += n
        else:
            if rotary:
                key_states = apply_rotary_pos_emb_single(key_states, cache_kwargs["cos"], cache_kwargs["sin"])
            kbuf = torch.cat([L.k_win[:, :, L.pend:L.win_len], key_states], dim=2)
            vbuf = torch.cat([L.v_win[:, :, L.pend:L.win_len], value_states], dim=2)
            k_cut, v_cut = kbuf[:, :, :n_cut], vbuf[:, :, :n_cut]
            if L.pend:
                k_cut, v_cut = torch.cat([L.k_pend, k_cut], dim=2), torch.cat([L.v_pend, v_cut], dim=2)
            whole = k_cut.size(2) // 128 * 128
            if whole:
                L.k.append(k_cut[:, :, :whole].contiguous())
                L.v.append(v_cut[:, :, :whole].contiguous())
            L.pend = k_cut.size(2) - whole
            left = total - n_cut
            if L.pend + left > L.cap:
                raise RuntimeError("not supported: %d tokens left in the 16-bit window" % (L.pend + left))
            if L.pend:
                L.k_pend, L.v_pend = k_cut[:, :, whole:].contiguous(), v_cut[:, :, whole:].contiguous()
                L.k_win[:, :, :L.pend] = self._quant_dequant(L.k_pend, cfg.k_quant_scale_rel)
                L.v_win[:, :, :L.pend] = self._quant_dequant(L.v_pend, cfg.v_quant_scale_rel)
            else:
                L.k_pend = L.v_pend = None
            L.k_win[:, :, L.pend:L.pend + left] = kbuf[:, :, n_cut:]
            L.v_win[:, :, L.pend:L.pend + left] = vbuf[:, :, n_cut:]
            L.win_len = L.pend + left
            L.plan = None                  # token counts (and possibly the stream buffers) changed
        if return_dense:
            return self.materialize(layer_idx)
        return None

    def get_seq_length(self, layer_idx=0):
        L = self.layers[layer_idx or 0]
        return 0 if L is None else L.k.tokens + L.win_len

    # -- hot path ------------------------------------------------------------------------------------
    def attend(self, query_states, layer_idx, sm_scale=None, out=None, variant=0, ref_rounding=False, out_f32=False):
        """One decode step: query_states [B, Hq, 128] (or [B, Hq, 1, 128]) against everything cached in the
        layer; returns [B, Hq, 128] (same rank as given).  variant / ref_rounding / out_f32 select the checking
        kernels of ops.attn_decode (not cached as a plan)."""
        L = self._layer(layer_idx)
        q = query_states
        squeeze = q.dim() == 4
        if squeeze:
            q = q[:, :, 0]
        q = q.contiguous()
        if variant or ref_rounding or out_f32:
            res = ops.attn_decode(q, L.k.as_dict() if L.k.tokens else None, L.v.as_dict() if L.v.tokens else None,
                                  L.k_win if L.win_len else None, L.v_win if L.win_len else None, sm_scale=sm_scale,
                                  out=out, variant=variant, win_len=L.win_len or None, ref_rounding=ref_rounding,
                                  out_f32=out_f32)
            return res.unsqueeze(2) if squeeze else res
        if out is None:
            out = torch.empty_like(q)
        plan = L.plan
        if plan is None or plan.sm_scale_arg != sm_scale or not L.win_len or plan._shape != q.shape or plan._dtype != q.dtype:
            k = L.k.as_dict() if L.k.tokens else None
            v = L.v.as_dict() if L.v.tokens else None
            plan = ops.AttnPlan(q, k, v, L.k_win if L.win_len else None, L.v_win if L.win_len else None,
                                sm_scale=sm_scale, out=out, win_len=L.win_len)
            plan.sm_scale_arg = sm_scale
            L.plan = plan if L.win_len else None      # between cuts only the window rows in use change
        else:
            plan.set_window_rows(L.win_len)
        res = plan(q=q, out=out)
        return res.unsqueeze(2) if squeeze else res

    # -- dense view and accounting ---------------------------------------------------------------------
    @staticmethod
    def _quant_dequant(x, rel):
        scale, zero = ops.quant_params(x, rel)
        codes, _ = ops.quantize(x, scale, zero)
        return ops.dequantize(codes, scale, zero, x.size(0), x.size(1))

    def materialize(self, layer_idx):
        """(K, V) [B, H, T, 128]: the dequantised prefix followed by the window, i.e. the tensors the reference's
        ``update`` returns for decompress-then-attend."""
        L = self._layer(layer_idx)
        out = []
        for side, win in ((L.k, L.k_win), (L.v, L.v_win)):
            parts = []
            if side.tokens:
                hidden = side.B * side.H * 128
                codes = torch.empty(side.tokens, hidden, dtype=torch.uint8, device=win.device)
                dec = ops.k_decode if side.is_k else ops.v_decode
                nblk = side.tokens // 128 * side.blocks_per_tile
                dec(side.stream, side.info[:nblk], codes, bits=side.bits)
                sc = side.scale[:, :side.tokens].contiguous()
                ze = side.zero[:, :side.tokens].contiguous()
                parts.append(ops.dequantize(codes, sc, ze, side.B, side.H))
            if L.win_len:
                parts.append(win[:, :, :L.win_len])
            out.append(torch.cat(parts, dim=2) if parts else None)
        return out[0], out[1]

    def cache_bytes(self, layer_idx=None):
        """Bytes the cache holds (streams in use, block_info and parameters of the encoded tokens, the 16-bit
        window rows in use, the originals of a pending cut) -- per layer or summed."""
        idx = range(len(self.layers)) if layer_idx is None else [layer_idx]
        total = 0
        for i in idx:
            L = self.layers[i]
            if L is None:
                continue
            for side in (L.k, L.v):
                total += side.used + side.tokens // 128 * side.blocks_per_tile * 8 + side.B * side.tokens * 4
            es = L.k_win.element_size()
            total += 2 * self.batch_size * self.head_num * (L.win_len + L.pend) * 128 * es
        return total


# ---- the reference's own class names ------------------------------------------------------------------

class PackKVCacheConfigStatic:
    """The process-wide configuration slot the reference's caches read (models/cache/packkv_quant.py:10-12):
    ``PackKVCacheConfigStatic.config`` holds an object with block_size, buffer_size, k_quant_scale_rel,
    v_quant_scale_rel (and optionally enable_quant) -- the reference's utils/config.py ``PackKVCacheConfig`` or this
    module's ``PackKVCacheConfig``.  ``max_tokens`` sizes the per-layer tables of the compressed cache."""
    config = None
    max_tokens = 32768


try:                                    # the reference's caches are transformers.Cache subclasses
    from transformers import Cache as _HFCache
except Exception:                       # pragma: no cover - transformers is an optional dependency of this class only
    _HFCache = object


class PackKVCache(_HFCache):
    """Drop-in for the reference's ``PackKVCache`` (models/cache/packkv_cache.py:22-38; built by
    models/llama.py:830-833 as ``PackKVCache(batch, heads, head_dim, layers)`` and called by its attention modules as
    ``key_states, value_states = past_key_value.update(key_states, value_states, layer_idx, cache_kwargs)``,
    models/llama.py:261): same constructor, same ``update`` return value (the dense K and V, the quantised prefix in
    dequantised form followed by the 16-bit buffer), same ``get_seq_length``.  The quantised prefix is held as PackKV
    streams on the device; ``attend`` / ``materialize`` / ``cache_bytes`` of the compressed cache are passed through
    for callers that replace the eager attention of a decode step.  The compressed cache is created at the first
    ``update`` (dtype and device of the tensors it is given; head_num is the number of KV heads those tensors have)."""

    def __init__(self, batch_size, head_num, head_dim, layer_num, config=None, max_tokens=None):
        if _HFCache is not object:
            try:
                super().__init__(layers=[])          # transformers 5: a Cache is a list of layers
            except TypeError:
                super().__init__()                   # transformers 4 (the reference pins 4.52)
        # (transformers.Cache defines read-only properties of its own under some of the reference's attribute names)
        self._shape = (batch_size, head_num, head_dim)
        self._layer_num = layer_num
        self._config, self._max_tokens = config, max_tokens
        self.cache_instance = None
        self._plain_k = [None] * layer_num           # enable_quant = False: everything stays in 16 bits
        self._plain_v = [None] * layer_num

    def _cfg(self):
        cfg = self._config or PackKVCacheConfigStatic.config
        if cfg is None:
            raise ValueError("PackKVCacheConfigStatic.config is not set. Please set it before using PackKVCache.")
        return cfg

    def _instance(self, key_states):
        if self.cache_instance is None:
            cfg = self._cfg()
            own = cfg if isinstance(cfg, PackKVCacheConfig) else PackKVCacheConfig(
                cfg.block_size, cfg.buffer_size, cfg.k_quant_scale_rel, cfg.v_quant_scale_rel)
            self.cache_instance = PackKVCompressedCache(
                key_states.size(0), key_states.size(1), key_states.size(3), self._layer_num, own,
                max_tokens=self._max_tokens or PackKVCacheConfigStatic.max_tokens, dtype=key_states.dtype,
                device=key_states.device)
        return self.cache_instance

    def update(self, key_states, value_states, layer_idx, cache_kwargs=None, return_dense=True):
        if getattr(self._cfg(), "enable_quant", True) is False:          # packkv_quant.py:87-99 (update_disable)
            if cache_kwargs and cache_kwargs.get("cos") is not None:
                key_states = apply_rotary_pos_emb_single(key_states, cache_kwargs["cos"], cache_kwargs["sin"])
            k, v = self._plain_k[layer_idx], self._plain_v[layer_idx]
            self._plain_k[layer_idx] = key_states if k is None else torch.cat([k, key_states], dim=2)
            self._plain_v[layer_idx] = value_states if v is None else torch.cat([v, value_states], dim=2)
            return self._plain_k[layer_idx], self._plain_v[layer_idx]
        return self._instance(key_states).update(key_states, value_states, layer_idx, cache_kwargs, return_dense)

    def get_seq_length(self, layer_idx=0):
        if self.cache_instance is None:
            k = self._plain_k[layer_idx or 0]
            return 0 if k is None else k.shape[2]
        return self.cache_instance.get_seq_length(layer_idx)

    def attend(self, query_states, layer_idx, **kw):
        return self.cache_instance.attend(query_states, layer_idx, **kw)

    def materialize(self, layer_idx):
        return self.cache_instance.materialize(layer_idx)

    def cache_bytes(self, layer_idx=None):
        return self.cache_instance.cache_bytes(layer_idx)
