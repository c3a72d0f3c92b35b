"""TEST INFRASTRUCTURE -- CPU restatement (NumPy) of the reference's token repacking and analytic size model.

Follows utils/compute.py:262-270 (``median_repacking``), :272-297 (``bit_pack``) and :329-357
(``repack_and_encode``: K and V codes side by side, ``blocks`` [n_blocks, block tokens, 2 * B * H * D]).
``greedy_repacking`` (:210-260) is not restated.

Tie order.  The reference sorts the per-token medians with ``torch.sort(descending=True)`` without
``stable=True``; the order of equal medians is then whatever the backend does (medians of small integer codes tie
constantly), so repacked sizes are not uniquely defined by the reference: **parity unpinned** for
``RepackMethod.MEDIAN``.  This restatement, like the device kernels, keeps ties in their original order.

Pinned by (tests/test_oracle_quant.py): the median against ``torch.median`` (library routine: lower median on an
even count) and the order against ``torch.sort(descending=True, stable=True)``; ``bit_pack`` against the closed
form of oracle/quant.py::bit_pack_bytes and a hand-computed case.  Only tests, the smoke check and the CPU leg of
the benchmark may import this module.
"""
import math

import numpy as np


def blocks_from_code_matrices(k_codes, v_codes, block_size):
    """uint8 code matrices [ctx_len, hidden] (channel = (b * H + h) * D + d) -> blocks [n_blocks, block_size,
    2 * hidden], the tensor ``repack_and_encode`` builds with permute(2, 3, 0, 1, 4).flatten(2, 4) and cat
    (utils/compute.py:336-338)."""
    k = np.asarray(k_codes).astype(np.int64)
    v = np.asarray(v_codes).astype(np.int64)
    nb = k.shape[0] // block_size
    return np.concatenate([k.reshape(nb, block_size, -1), v.reshape(nb, block_size, -1)], axis=2)


def token_medians(blocks):
    """Lower median of the V half of every token (torch.median semantics), [n_blocks, N]."""
    half = blocks.shape[2] // 2
    v = np.sort(blocks[:, :, half:], axis=2)
    return v[:, :, (v.shape[2] - 1) // 2]


def median_repacking(blocks):
    """utils/compute.py:262-270 with a stable descending sort.  Returns (repacked blocks, order) where
    order[b, r] is the original position of the token now at position r."""
    med = token_medians(blocks)
    order = np.argsort(-med, axis=1, kind="stable")
    return np.take_along_axis(blocks, order[:, :, None], axis=1), order


def bit_pack(blocks, pack_len):
    """utils/compute.py:272-297: (k_bytes, v_bytes)."""
    half = blocks.shape[2] // 2
    flat = blocks.reshape(-1, blocks.shape[2]).astype(np.int64)
    out = []
    for part in (flat[:, :half], flat[:, half:]):
        packs = part.reshape(-1, pack_len, half)
        w = math.ceil(math.log2(np.unique(packs).size))
        mn, mx = packs.min(axis=1), packs.max(axis=1)
        bits = int(np.ceil(np.log2(mx - mn + 1)).astype(np.int64).sum()) * pack_len
        bits += mn.size * (w + math.ceil(math.log2(w + 1)))
        out.append(bits // 8)
    return out[0], out[1]


def repack_and_encode(k_codes, v_codes, pack_size, method="none", block_size=64):
    """utils/compute.py:329-357 on code matrices: (k_pre, v_pre, k_after, v_after) bytes."""
    blocks = blocks_from_code_matrices(k_codes, v_codes, block_size)
    k_pre, v_pre = bit_pack(blocks, pack_size)
    if method == "median":
        blocks, _ = median_repacking(blocks)
    elif method != "none":
        raise ValueError("repack_method must be one of none, median")
    k_aft, v_aft = bit_pack(blocks, pack_size)
    return k_pre, v_pre, k_aft, v_aft
