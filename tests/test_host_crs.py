"""The KV dump tree (evaluation/evaluation.py:160-185) is written and read back without a GPU."""
import pytest
import torch

from packkv_amd import crs, synth


def _layers(n, B, H, T, seed):
    ks, vs = [], []
    for i in range(n):
        k, v = synth.make_kv(B, H, T, seed=seed + i)
        ks.append(k)
        vs.append(v)
    return ks, vs


def test_dump_tree_round_trips(tmp_path):
    ks, vs = _layers(3, 1, 2, 128, seed=300)
    crs.save_kv_dump(str(tmp_path), "toy-model", 128, [ks, ks[:2]], [vs, vs[:2]])
    assert (tmp_path / "toy-model" / "128" / "1" / "v" / "1.pt").exists()
    k0, v0 = crs.load_kv_dump(str(tmp_path), "toy-model", 128, 0)
    k1, _ = crs.load_kv_dump(str(tmp_path), "toy-model", 128, 1)
    assert len(k0) == 3 and len(k1) == 2
    assert all(torch.equal(a, b) for a, b in zip(k0, ks)) and all(torch.equal(a, b) for a, b in zip(v0, vs))
    (tmp_path / "toy-model" / "128" / "0" / "k" / "1.pt").unlink()
    with pytest.raises(RuntimeError):
        crs.load_kv_dump(str(tmp_path), "toy-model", 128, 0)
