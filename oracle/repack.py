"""TEST INFRASTRUCTURE -- CPU restatement (NumPy) of the reference's token repacking and analytic size model.

Follows utils/compute.py:262-270 (``median_repacking``), :272-297 (``bit_pack``) and :329-357
(``repack_and_encode``: K and V codes side by side, ``blocks`` [n_blocks, block tokens, 2 * B * H * D]).
``greedy_repacking`` (:210-260, with ``_batched_pick`` :186-208) is restated in integers, see below.

Tie order.  The reference sorts the per-token medians with ``torch.sort(descending=True)`` without
``stable=True``; the order of equal medians is then whatever the backend does (medians of small integer codes tie
constantly), so repacked sizes are not uniquely defined by the reference: **parity unpinned** for
``RepackMethod.MEDIAN``.  This restatement, like the device kernels, keeps ties in their original order.

Greedy method.  Every pack starts from the remaining token most similar (cosine) to the rounded mean of the
remaining tokens and then takes, pack_len - 1 times, the remaining token that adds the fewest payload bits
(sum over channels of bit_length(max - min)).  The reference computes both criteria in fp32 and leaves ties to
``torch.argmax`` / ``torch.argmin``.  The bit counts are small integers, exact in fp32, so only the tie order of
the second criterion is open; the cosine, however, is a rounded fp32 quotient whose near-ties depend on the
backend's reduction order: **parity unpinned** for ``RepackMethod.GREEDY`` as well.  This restatement (and the
device kernel) compares the cosines exactly -- codes are non-negative integers, the mean is common to all
candidates, so cos_a > cos_b  <=>  dot_a^2 * |b|^2 > dot_b^2 * |a|^2 in integers -- and resolves every tie to the
token that comes first in the block.  Pinned by: a brute-force fp64 recomputation of both criteria on small random
blocks away from ties, the invariant that the result is a permutation that never raises the seed's own cost, and
the hand-built cases of tests/test_oracle_quant.py.

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


def _bit_length(a):
    """bit_length of non-negative integers below 2**16, elementwise (= ceil(log2(a + 1)))."""
    return np.frexp(np.asarray(a, dtype=np.float64))[1].astype(np.int64)    # a = m * 2**e, m in [0.5, 1): e = bit_length


def greedy_order(block, pack_len):
    """Order of ``greedy_repacking`` (utils/compute.py:210-260) for ONE block [N, D] of non-negative integer codes:
    order[r] = original position of the token picked r-th.  Ties go to the earlier token (see the module text)."""
    x = np.asarray(block, dtype=np.int64)
    n, _ = x.shape
    assert n % pack_len == 0, "the reference drops the tokens of an incomplete last pack"
    alive = list(range(n))          # _batched_pick keeps the remaining tokens in their original order
    order = []
    for _ in range(n // pack_len):
        rem = x[alive]
        # mean(dim=1).round() in fp32: sum / count, round half to even (compute.py:219)
        mean = np.rint(rem.sum(axis=0).astype(np.float32) / np.float32(len(alive))).astype(np.int64)
        dot = [int(v) for v in rem @ mean]
        nx = [int(v) for v in (rem * rem).sum(axis=1)]
        best = 0
        for i in range(1, len(alive)):   # cos_i > cos_best, exactly; a zero vector has cosine 0
            if nx[i] == 0:
                continue
            if (dot[i] > 0) if nx[best] == 0 else (dot[i] * dot[i] * nx[best] > dot[best] * dot[best] * nx[i]):
                best = i
        seed = alive.pop(best)
        order.append(seed)
        mn, mx = x[seed].copy(), x[seed].copy()
        for _ in range(pack_len - 1):
            rem = x[alive]
            # the bits before the pick are common to all candidates (compute.py:235-243): argmin of the new total
            cost = _bit_length(np.maximum(rem, mx) - np.minimum(rem, mn)).sum(axis=1)
            pick = alive.pop(int(np.argmin(cost)))          # np.argmin: first minimum
            order.append(pick)
            mn, mx = np.minimum(mn, x[pick]), np.maximum(mx, x[pick])
    return np.asarray(order, dtype=np.int64)


def greedy_repacking(blocks, pack_len):
    """utils/compute.py:210-260 on blocks [n_blocks, N, D].  Returns (repacked blocks, order)."""
    order = np.stack([greedy_order(b, pack_len) for b in blocks])
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
    elif method == "greedy":
        blocks, _ = greedy_repacking(blocks, pack_size)
    elif method != "none":
        raise ValueError("repack_method must be one of none, median, greedy")
    k_aft, v_aft = bit_pack(blocks, pack_size)
    return k_pre, v_pre, k_aft, v_aft


def crs_record(k, v, block_size, pack_size, k_rel, v_rel, method="none"):
    """One layer of ``crs_evaluation_with_data`` (evaluation/evaluation.py:188-250) for K, V torch tensors
    [B, H, T, D]: the sizes in bytes that the reference appends to its record, as a dict (the ratios are
    original / size and are left to the caller)."""
    import torch
    from oracle import quant as oq
    out, mats = {}, {}
    for side, x, rel in (("k", k, k_rel), ("v", v, v_rel)):
        codes, zero, scale = oq.quant_ints(x, block_size, rel)
        bit_num = math.ceil(math.log2(int(torch.unique(codes).numel())))
        out[side + "_original_size"] = x.numel() * x.element_size()
        out[side + "_quant_size"] = (codes.numel() * bit_num // 8 + zero.numel() * zero.element_size() +
                                     scale.numel() * scale.element_size())
        mats[side] = oq.code_matrix(codes).numpy()
    pre_k, pre_v, aft_k, aft_v = repack_and_encode(mats["k"], mats["v"], pack_size, method, block_size)
    out.update(k_encode_size_before_repack=pre_k, v_encode_size_before_repack=pre_v,
               k_encode_size_after_repack=aft_k, v_encode_size_after_repack=aft_v)
    return out
