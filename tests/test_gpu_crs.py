"""Compression-ratio evaluation of a dumped KV cache (packkv_amd/crs.py) against the restatement of the reference's
record (oracle/repack.py::crs_record): a synthetic dump tree is written, read back and priced on the device."""
import math

import pytest
import torch

from oracle import quant as oq
from oracle import repack as orp
from packkv_amd import crs, ops, synth

pytestmark = pytest.mark.gpu


def _say(*a):
    print(*a, flush=True)


def _layers(n, B, H, T, seed):
    ks, vs = [], []
    for i in range(n):
        k, v = synth.make_kv(B, H, T, seed=seed + i, k_mode="outliers" if i % 2 == 0 else "channel_scale")
        ks.append(k)
        vs.append(v)
    return ks, vs


@pytest.mark.parametrize("method", ["none", "median", "greedy"])
def test_record_matches_restatement(cuda, tmp_path, method):
    B, H, T = 2, 4, 512
    ks, vs = _layers(2, B, H, T, seed=310)
    crs.save_kv_dump(str(tmp_path), "toy-model", T, [ks], [vs])
    kl, vl = crs.load_kv_dump(str(tmp_path), "toy-model", T, 0)
    for pack in (16, 64):
        cfg = crs.CRConfig(block_size=64, pack_size=pack, k_quant_scale_rel=0.1, v_quant_scale_rel=0.14, repack_method=method)
        _say("crs case", method, "pack", pack)
        got = crs.crs_evaluation_with_data(cfg, kl, vl, device=cuda)
        for layer, (k, v) in enumerate(zip(ks, vs)):
            want = orp.crs_record(k, v, 64, pack, 0.1, 0.14, method)
            for key, val in want.items():
                assert got[key][layer] == val, (key, layer)
            assert got["k_quant_cr"][layer] == want["k_original_size"] / want["k_quant_size"]
            assert got["v_encode_after_repack_cr"][layer] == want["v_original_size"] / want["v_encode_size_after_repack"]
        _say("  K CR", got["k_encode_before_repack_cr"], "->", got["k_encode_after_repack_cr"],
             " V CR", got["v_encode_before_repack_cr"], "->", got["v_encode_after_repack_cr"])


def test_detail_adds_up(cuda):
    """The three parts of the packed size, each floored to bytes, bracket the size bit_pack reports after median
    repacking; the parameter sizes are 2 bytes per (batch, token) each."""
    B, H, T = 1, 8, 1024
    ks, vs = _layers(1, B, H, T, seed=320)
    cfg = crs.CRConfig(repack_method="median")
    d = crs.crs_evaluation_detail(cfg, ks, vs, device=cuda)
    r = crs.crs_evaluation_with_data(cfg, ks, vs, device=cuda)
    for s in ("k", "v"):
        parts = d[s + "_bitpack_min_value_size"][0] + d[s + "_bitpack_encode_len_size"][0] + d[s + "_bitpack_encoded_size"][0]
        total = r[s + "_encode_size_after_repack"][0]
        assert total - 2 <= parts <= total
        assert d[s + "_quant_zero_point_size"][0] == d[s + "_quant_scale_size"][0] == B * T * 2
        assert d[s + "_original_size"][0] == B * H * T * 128 * 2
