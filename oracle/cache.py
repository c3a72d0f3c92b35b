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

    def __init__(self, layer_num, block_size=64, buffer_size=192, k_rel=0.1, v_rel=0.1, track_exact=False):
        self.block_size, self.buffer_size = block_size, buffer_size
        self.k_rel, self.v_rel = k_rel, v_rel
        # track_exact: also keep the quantised prefix BEFORE its rounding to 16 bits, (code + zero) * scale in fp64
        # -- not something the reference holds; the tests use it to measure what that rounding moves
        self.track_exact = track_exact
        self.xk = [None] * layer_num
        self.xv = [None] * layer_num
        self.ck = [None] * layer_num
        self.cv = [None] * layer_num
        self.bk = [None] * layer_num
        self.bv = [None] * layer_num

    def _quant_error(self, done, buf, new, rel, exact=None):
        """utils/compute.py:149-181.  `exact` (a one-element list, or None) accumulates the unrounded prefix."""
        buf = _cat(buf, new)
        n_cut, _ = oq.cut_counts(0, buf.shape[2], self.block_size, self.buffer_size)
        to_compress = None
        if n_cut > 0:
            to_compress, buf = buf[:, :, :n_cut], buf[:, :, n_cut:]
            codes, zero, scale = oq.quant_ints(to_compress, self.block_size, rel)
            to_compress = oq.dequant(codes, zero, scale)
            if exact is not None:
                x = (codes.double() + zero.double()) * scale.double()
                exact[0] = _cat(exact[0], x.reshape(x.shape[0], x.shape[1], -1, x.shape[4]))
        return _cat(done, to_compress), buf

    def update(self, key_states, value_states, layer_idx, cos=None, sin=None):
        if cos is not None:
            key_states = apply_rotary_pos_emb_single(key_states, cos, sin)
        xk = [self.xk[layer_idx]] if self.track_exact else None
        xv = [self.xv[layer_idx]] if self.track_exact else None
        self.ck[layer_idx], self.bk[layer_idx] = self._quant_error(self.ck[layer_idx], self.bk[layer_idx],
                                                                   key_states, self.k_rel, xk)
        self.cv[layer_idx], self.bv[layer_idx] = self._quant_error(self.cv[layer_idx], self.bv[layer_idx],
                                                                   value_states, self.v_rel, xv)
        if self.track_exact:
            self.xk[layer_idx], self.xv[layer_idx] = xk[0], xv[0]
        return _cat(self.ck[layer_idx], self.bk[layer_idx]), _cat(self.cv[layer_idx], self.bv[layer_idx])

    def exact(self, layer_idx):
        """(K, V) [B, H, T, D] in fp64 with the quantised prefix unrounded (needs track_exact)."""
        bk, bv = self.bk[layer_idx], self.bv[layer_idx]
        return (_cat(self.xk[layer_idx], None if bk is None else bk.double()),
                _cat(self.xv[layer_idx], None if bv is None else bv.double()))

    def get_seq_length(self, layer_idx=0):
        n = 0
        for t in (self.ck[layer_idx], self.bk[layer_idx]):
            n += 0 if t is None else t.shape[2]
        return n
