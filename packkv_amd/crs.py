"""Compression-ratio evaluation of dumped KV caches on the device.

The reference collects the K and V tensors of every layer during a forward pass, writes them as
``<root>/<model>/<ctx_len>/<round>/{k,v}/<layer>.pt`` (``save_extract_cache``, evaluation/evaluation.py:160-185)
and prices them with ``crs_evaluation_with_data`` (evaluation/evaluation.py:188-250): original size, size after
quantisation alone, and the analytic pack sizes before and after token repacking.  This module reads and writes
that tree and computes the same record with the library's kernels: per-token parameters and codes from
``quant_params`` / ``quantize``, the number of distinct codes and the pack sizes from ``pkv_bit_pack_size``, the
token orders from ``pkv_median_repack`` / ``pkv_greedy_repack``.  Everything is integer arithmetic on the codes, so
the record equals the reference's wherever the codes and the token order are defined by it (RepackMethod.NONE
always; the repacked sizes up to the tie order the reference leaves to its backend).
"""
import math
import os

import torch

from . import ops


class CRConfig:
    """The fields of the reference's PackKVCacheConfig that the size evaluation reads
    (evaluation/evaluation.py:220-238): block_size, pack_size, the two relative scales and the repacking method
    ("none", "median" or "greedy")."""

    def __init__(self, block_size=64, pack_size=16, k_quant_scale_rel=0.1, v_quant_scale_rel=0.1, repack_method="none"):
        if repack_method not in ("none", "median", "greedy"):
            raise ValueError("repack_method must be one of none, median, greedy")
        self.block_size, self.pack_size = int(block_size), int(pack_size)
        self.k_quant_scale_rel, self.v_quant_scale_rel = k_quant_scale_rel, v_quant_scale_rel
        self.repack_method = repack_method


def save_kv_dump(root_dir, model_name, ctx_len, key_caches, value_caches):
    """Write the tree of evaluation/evaluation.py:160-185.  key_caches / value_caches: one list of per-layer
    tensors [B, H, T, D] per collection round."""
    for round_i, (ks, vs) in enumerate(zip(key_caches, value_caches)):
        for side, tensors in (("k", ks), ("v", vs)):
            d = os.path.join(root_dir, model_name, str(ctx_len), str(round_i), side)
            os.makedirs(d, exist_ok=True)
            for i, t in enumerate(tensors):
                torch.save(t.detach().cpu(), os.path.join(d, "%d.pt" % i))


def load_kv_dump(root_dir, model_name, ctx_len, round_i=0, device="cpu"):
    """Read one round of the tree back: (key_caches, value_caches), lists over layers.  Files are read with
    weights_only=True: a dump holds plain tensors, nothing in it is executed."""
    out = []
    for side in ("k", "v"):
        d = os.path.join(root_dir, model_name, str(ctx_len), str(round_i), side)
        layers = sorted(int(f[:-3]) for f in os.listdir(d) if f.endswith(".pt") and f[:-3].isdigit())
        if layers != list(range(len(layers))):
            raise RuntimeError("KV dump %s: layer files must be 0.pt .. n-1.pt, found %s" % (d, layers))
        out.append([torch.load(os.path.join(d, "%d.pt" % i), map_location=device, weights_only=True) for i in layers])
    return out[0], out[1]


def _bit_num(n_unique):
    return math.ceil(math.log2(n_unique))


def crs_evaluation_with_data(config, key_caches, value_caches, device="cuda"):
    """The record of evaluation/evaluation.py:188-250 (same keys, one entry per layer) for K / V tensors
    [B, H, T, 128] whose T is a multiple of config.block_size."""
    res = {k: [] for k in (
        "k_original_size", "v_original_size", "k_quant_size", "v_quant_size",
        "k_encode_size_before_repack", "v_encode_size_before_repack", "k_encode_size_after_repack",
        "v_encode_size_after_repack", "k_quant_cr", "v_quant_cr", "k_encode_before_repack_cr",
        "v_encode_before_repack_cr", "k_encode_after_repack_cr", "v_encode_after_repack_cr")}
    for k, v in zip(key_caches, value_caches):
        if k.shape != v.shape or k.dim() != 4 or k.size(2) % config.block_size:
            raise RuntimeError("K and V must be [B, H, T, D] of one shape with T a multiple of block_size")
        codes, orig = {}, {}
        for side, x, rel in (("k", k, config.k_quant_scale_rel), ("v", v, config.v_quant_scale_rel)):
            xd = x.to(device).contiguous()
            scale, zero = ops.quant_params(xd, rel)
            c, _ = ops.quantize(xd, scale, zero)
            codes[side] = c
            orig[side] = x.numel() * x.element_size()
            # every code at quant_bit_num bits plus one zero and one scale per (batch, token) in the storage dtype
            n_unique = ops.code_stats(c, config.pack_size)[1]
            quant_size = c.numel() * _bit_num(n_unique) // 8 + (zero.numel() + scale.numel()) * x.element_size()
            res[side + "_original_size"].append(orig[side])
            res[side + "_quant_size"].append(quant_size)
            res[side + "_quant_cr"].append(orig[side] / quant_size)
        k_pre, v_pre, k_aft, v_aft = ops.repack_and_encode(codes["k"], codes["v"], config.pack_size,
                                                           config.repack_method, config.block_size)
        for side, pre, aft in (("k", k_pre, k_aft), ("v", v_pre, v_aft)):
            res[side + "_encode_size_before_repack"].append(pre)
            res[side + "_encode_size_after_repack"].append(aft)
            res[side + "_encode_before_repack_cr"].append(orig[side] / pre)
            res[side + "_encode_after_repack_cr"].append(orig[side] / aft)
    return res


def crs_evaluation_detail(config, key_caches, value_caches, device="cuda"):
    """The split of the packed size into its three parts (crs_evaluation_with_data_detail_rebuttal,
    evaluation/evaluation.py:253-299, with bit_pack_detail_rebuttal, utils/compute.py:299-327): quantiser
    parameters, pack minima, pack widths and payload, after median repacking as there."""
    keys = ("original_size", "quant_zero_point_size", "quant_scale_size", "bitpack_min_value_size",
            "bitpack_encode_len_size", "bitpack_encoded_size")
    res = {s + "_" + k: [] for k in keys for s in ("k", "v")}
    for k, v in zip(key_caches, value_caches):
        codes, pars = {}, {}
        for side, x, rel in (("k", k, config.k_quant_scale_rel), ("v", v, config.v_quant_scale_rel)):
            xd = x.to(device).contiguous()
            scale, zero = ops.quant_params(xd, rel)
            codes[side], _ = ops.quantize(xd, scale, zero)
            pars[side] = (zero.numel() * x.element_size(), scale.numel() * x.element_size())
            res[side + "_original_size"].append(x.numel() * x.element_size())
        kc, vc, _ = ops.median_repacking(codes["k"], codes["v"], config.block_size)
        for side, c in (("k", kc), ("v", vc)):
            len_sum, n_unique = ops.code_stats(c, config.pack_size)
            w = _bit_num(n_unique)
            n_packs = (c.size(0) // config.pack_size) * c.size(1)
            res[side + "_quant_zero_point_size"].append(pars[side][0])
            res[side + "_quant_scale_size"].append(pars[side][1])
            res[side + "_bitpack_min_value_size"].append(n_packs * w // 8)
            res[side + "_bitpack_encode_len_size"].append(n_packs * math.ceil(math.log2(w + 1)) // 8)
            res[side + "_bitpack_encoded_size"].append(len_sum * config.pack_size // 8)
    return res
