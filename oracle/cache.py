"""TEST INFRASTRUCTURE -- CPU restatement of the reference's simulated compressed cache.

Follows models/cache/packkv_quant.py:45-85 (``PackKVCachePytorchQuant.update``),
utils/compute.py:149-181 (``quant_error``), :54-67 (``cut_tensor``), :22-43 (rotary embedding
of K inside the cache).  The reference keeps, per layer, the already quantised-and-dequantised
prefix plus a 16-bit buffer, and hands ``cat(prefix, buffer)`` to eager attention.  Only tests,
the smoke check and the CPU-baseline leg of the benchmark may import this module.

Pinned by: ``cut_counts`` against the closed-form buffer cycle (a window of 192 with blocks of 64
holds 128..191 tokens and cuts one block every 64 steps, scripts/throughput_config_test.py:16-17)
in tests/test_oracle_quant.py, and ``quant_ints`` / ``dequant`` by the checks listed in
oracle/quant.py; the class below only composes them.
"""
import torch

from . import quant as oq


def rotate_half(x):
    """utils/compute.py:22-26."""
    h = x.shape[-1] // 2
    return torch.cat((-x[..., h:], x[..., :h]), dim=-1)


def apply_rotary_pos_emb_single(t, cos, sin, unsqueeze_dim=1):
    """utils/compute.py:35-43; cos/sin [B, n, D], t [B, H, n, D]."""
    cos = cos.unsqueeze(unsqueeze_dim)
    sin = sin.unsqueeze(unsqueeze_dim)
    return (t * cos) + (rotate_half(t) * sin)


def _cat(a, b):
    """utils/compute.py:45-52 (safe_cat)."""
    if a is None:
        return None if b is None else b.clone()
    if b is None:
        return a.clone()
    return torch.cat([a, b], dim=2)


class SimulatedCache:
    """One layer list of (dequantised prefix, 16-bit buffer) pairs; ``update`` returns what
    the reference's ``update`` returns: K and V [B, H, T, D] for decompress-then-attend."""

    def __init__(self, layer_num, block_size=64, buffer_size=192, k_rel=0.1, v_rel=0.1):
        self.block_size, self.buffer_size = block_size, buffer_size
        self.k_rel, self.v_rel = k_rel, v_rel
        self.ck = [None] * layer_num
        self.cv = [None] * layer_num
        self.bk = [None] * layer_num
        self.bv = [None] * layer_num

    def _quant_error(self, done, buf, new, rel):
        """utils/compute.py:149-181."""
        buf = _cat(buf, new)
        n_cut, _ = oq.cut_counts(0, buf.shape[2], self.block_size, self.buffer_size)
        to_compress = None
        if n_cut > 0:
            to_compress, buf = buf[:, :, :n_cut], buf[:, :, n_cut:]
            codes, zero, scale = oq.quant_ints(to_compress, self.block_size, rel)
            to_compress = oq.dequant(codes, zero, scale)
        return _cat(done, to_compress), buf

    def update(self, key_states, value_states, layer_idx, cos=None, sin=None):
        if cos is not None:
            key_states = apply_rotary_pos_emb_single(key_states, cos, sin)
        self.ck[layer_idx], self.bk[layer_idx] = self._quant_error(self.ck[layer_idx], self.bk[layer_idx],
                                                                   key_states, self.k_rel)
        self.cv[layer_idx], self.bv[layer_idx] = self._quant_error(self.cv[layer_idx], self.bv[layer_idx],
                                                                   value_states, self.v_rel)
        return _cat(self.ck[layer_idx], self.bk[layer_idx]), _cat(self.cv[layer_idx], self.bv[layer_idx])

    def get_seq_length(self, layer_idx=0):
        n = 0
        for t in (self.ck[layer_idx], self.bk[layer_idx]):
            n += 0 if t is None else t.shape[2]
        return n
