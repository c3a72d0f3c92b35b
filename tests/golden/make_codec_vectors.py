"""Writes tests/golden/codec_vectors.npz from the REFERENCE codec build (oracle/_ref), i.e. from
the reference's own k/v_encode_cpu templates compiled by oracle/Makefile.  Run in the container
that has the reference checkout:

    make -C oracle ref && python tests/golden/make_codec_vectors.py

The file holds, per case, the uint8 code matrix, the stream bytes the reference produced, its
block_info and the returned size.  Inputs are small on purpose (a few blocks per case).
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import codec  # noqa: E402


def gaussian_codes(rng, T, H, W, outliers):
    """Codes of a per-token min/max quantizer applied to N(0,1) data (what real K/V looks like)."""
    x = rng.normal(size=(T, H)).astype(np.float32)
    if outliers:
        x[:, 3::32] *= 10.0
    levels = (1 << W) - 1
    mn = x.min(axis=1, keepdims=True)
    mx = x.max(axis=1, keepdims=True)
    return np.clip(np.rint((x - mn) / (mx - mn) * levels), 0, levels).astype(np.uint8)


def main():
    assert codec.have_ref(), "build oracle/_ref first (make -C oracle ref)"
    ref = codec.ref()
    rng = np.random.default_rng(20240607)
    out = {}
    cases = []
    for is_k, (T, H, cb, hb) in ((1, (128, 256, 64, 128)), (0, (256, 128, 128, 64))):
        for W in (2, 3, 4):
            for kind in ("gauss", "gauss_outlier", "uniform", "const"):
                if kind == "uniform":
                    c = rng.integers(0, 1 << W, (T, H)).astype(np.uint8)
                elif kind == "const":
                    c = np.full((T, H), (1 << W) - 2, dtype=np.uint8)
                else:
                    c = gaussian_codes(rng, T, H, W, kind == "gauss_outlier")
                stream, info, size = ref.encode(is_k, c, cb, hb, W)
                name = "%s_W%d_%s" % ("k" if is_k else "v", W, kind)
                out[name + "_codes"] = c
                out[name + "_stream"] = stream[:size].copy()
                out[name + "_info"] = info
                out[name + "_meta"] = np.array([is_k, T, H, cb, hb, W, size], dtype=np.int64)
                cases.append(name)
    out["cases"] = np.array(cases)
    path = os.path.join(ROOT, "tests", "golden", "codec_vectors.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes,", len(cases), "cases")


if __name__ == "__main__":
    main()
