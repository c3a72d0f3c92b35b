"""Pins the restated quantizer / attention (oracle/quant.py) against an independent NumPy
emulation with explicit rounding, closed forms, and fp64 attention."""
import numpy as np
import pytest
import torch

from oracle import quant as oq
from packkv_amd import synth


@pytest.mark.parametrize("dtype,name", [(torch.float16, "fp16"), (torch.bfloat16, "bf16")])
@pytest.mark.parametrize("rel", [0.05, 0.1, 0.14, 0.2])
def test_quant_chain_matches_explicit_rounding(dtype, name, rel):
    k, v = synth.make_kv(2, 4, 128, seed=3, dtype=dtype)
    for x in (k, v):
        c, z, s = oq.quant_ints(x, 64, rel)
        cn, zn, sn = oq.quant_ints_np(x.float().numpy(), name, 64, rel)
        assert np.array_equal(c.reshape(x.shape).float().numpy(), cn)
        assert np.array_equal(z.flatten().float().numpy(), zn.flatten())
        assert np.array_equal(s.flatten().float().numpy(), sn.flatten())
        assert cn.min() == 0
        assert cn.max() in (int(np.ceil(1 / rel - 1e-9)), int(np.ceil(1 / rel - 1e-9)) + 1)


def test_quant_is_per_batch_and_token():
    k, _ = synth.make_kv(2, 4, 64, seed=4)
    c, z, s = oq.quant_ints(k, 64, 0.1)
    assert tuple(z.shape) == (2, 1, 1, 64, 1) and tuple(s.shape) == (2, 1, 1, 64, 1)
    mn = k.float().amin(dim=(1, 3))
    mx = k.float().amax(dim=(1, 3))
    want = ((mx - mn).half().float() * np.float32(0.1)).half()
    assert torch.equal(s.flatten(), want.flatten())


def test_dequant_error_bound_and_layout():
    k, _ = synth.make_kv(1, 2, 64, seed=5)
    c, z, s = oq.quant_ints(k, 64, 0.1)
    y = oq.dequant(c, z, s)
    err = (y.float() - k.float()).abs()
    bound = 0.5 * s.flatten().float().view(1, 1, 64, 1) * 1.02 + 1e-2
    assert (err <= bound).all()
    m = oq.code_matrix(c)
    assert tuple(m.shape) == (64, 256)
    assert int(m[7, 1 * 128 + 5]) == int(c.reshape(1, 2, 64, 128)[0, 1, 7, 5])


def test_q_interleave_is_lane_order():
    q = torch.arange(128, dtype=torch.float32).view(1, 128)
    qi = oq.q_interleave(q)[0]
    for lane in range(32):
        assert qi[2 * lane].item() == 4 * lane and qi[2 * lane + 1].item() == 4 * lane + 1
        assert qi[64 + 2 * lane].item() == 4 * lane + 2 and qi[64 + 2 * lane + 1].item() == 4 * lane + 3


def test_cut_counts_residual_window():
    # block 64, buffer 192: a prompt below 192 tokens is never compressed; 8192 -> 8064 + 128; the
    # window then cycles 128..191
    assert oq.cut_counts(0, 191, 64, 192) == (0, 191)
    assert oq.cut_counts(0, 192, 64, 192) == (64, 128)
    assert oq.cut_counts(0, 8192, 64, 192) == (8064, 128)
    n = 128
    for _ in range(200):
        cut, n = oq.cut_counts(n, 1, 64, 192)
        assert cut in (0, 64) and 128 <= n <= 191


def test_bit_pack_closed_form():
    # 2 channels x 32 tokens: packs with ranges 0, 1, 3, 15 -> lens 0, 1, 2, 4
    c = np.zeros((32, 2), dtype=np.int64)
    c[16:, 0] = np.arange(16) % 2
    c[:16, 1] = np.arange(16) % 4
    c[16:, 1] = np.arange(16)
    bits = 16 * (0 + 1 + 2 + 4) + 4 * (4 + 3)
    assert oq.bit_pack_bytes(c, 16, W=4) == bits // 8


def test_attention_versions_agree_with_fp64():
    k, v = synth.make_kv(2, 2, 256, seed=6)
    q = synth.make_q(2, 8, seed=7).unsqueeze(2)
    ck, zk, sk = oq.quant_ints(k, 64, 0.1)
    cv, zv, sv = oq.quant_ints(v, 64, 0.1)
    kd, vd = oq.dequant(ck, zk, sk), oq.dequant(cv, zv, sv)
    want = oq.attention_f64_np(q, kd, vd)
    got32 = oq.attention_f32(q, kd, vd).double().numpy()
    got16 = oq.eager_attention(q, kd, vd).double().numpy()
    assert np.abs(got32 - want).max() < 1e-5
    assert np.abs(got16 - want).max() < 5e-3


def test_simulated_cache_follows_the_cut_policy():
    """The restated cache against facts that do not depend on it: (i) the lengths follow cut_tensor's
    closed form (prefix = cut tokens, buffer cycles 128..191); (ii) quantisation is per token, so the
    dequantised prefix equals a one-shot quantise -> dequantise of the same tokens however they were
    chunked; (iii) the buffer is the untouched tail; (iv) rotary embedding with cos = 1, sin = 0 is the
    identity and with cos = 0, sin = 1 is rotate_half."""
    from oracle import cache as oc
    B, H, T0, steps = 1, 2, 300, 150
    k, v = synth.make_kv(B, H, T0 + steps, seed=9)
    c = oc.SimulatedCache(1, 64, 192, 0.1, 0.2)
    kk, vv = c.update(k[:, :, :T0], v[:, :, :T0], 0)
    n_pref, n_buf = oq.cut_counts(0, T0, 64, 192)
    assert (n_pref, n_buf) == (128, 172) and kk.shape[2] == T0
    for i in range(steps):
        kk, vv = c.update(k[:, :, T0 + i:T0 + i + 1], v[:, :, T0 + i:T0 + i + 1], 0)
        cut, n_buf = oq.cut_counts(n_buf, 1, 64, 192)
        n_pref += cut
        assert c.ck[0].shape[2] == n_pref and c.bk[0].shape[2] == n_buf and 128 <= n_buf <= 191
    T = T0 + steps
    assert c.get_seq_length(0) == T and kk.shape[2] == T
    for got, x, rel in ((kk, k, 0.1), (vv, v, 0.2)):
        want = oq.dequant(*oq.quant_ints(x[:, :, :n_pref], 64, rel))
        assert torch.equal(got[:, :, :n_pref], want)
        assert torch.equal(got[:, :, n_pref:], x[:, :, n_pref:T])
    t = k[:, :, :8]
    one, nil = torch.ones(B, 8, 128, dtype=t.dtype), torch.zeros(B, 8, 128, dtype=t.dtype)
    assert torch.equal(oc.apply_rotary_pos_emb_single(t, one, nil), t)
    assert torch.equal(oc.apply_rotary_pos_emb_single(t, nil, one), torch.cat((-t[..., 64:], t[..., :64]), dim=-1))


def test_repack_restatement_against_library_routines():
    """median = torch.median (lower median on even counts), order = torch.sort(descending, stable); bit_pack =
    the single-tensor closed form; a hand-made block where the answer is known."""
    from oracle import repack as orp
    rng = np.random.default_rng(3)
    blocks = rng.integers(0, 6, size=(5, 64, 2 * 96))
    med = orp.token_medians(blocks)
    want = torch.median(torch.from_numpy(blocks[:, :, 96:]), dim=2).values.numpy()
    assert (med == want).all()
    rep, order = orp.median_repacking(blocks)
    _, idx = torch.sort(torch.from_numpy(med), dim=1, descending=True, stable=True)
    assert (order == idx.numpy()).all()
    assert (rep == np.take_along_axis(blocks, idx.numpy()[:, :, None], axis=1)).all()
    m2 = orp.token_medians(rep)
    assert (m2[:, :-1] >= m2[:, 1:]).all()                       # descending medians
    assert (np.sort(rep, axis=1) == np.sort(blocks, axis=1)).all()   # same tokens
    for pack_len in (16, 32, 64):
        kb, vb = orp.bit_pack(blocks, pack_len)
        flat = blocks.reshape(-1, 192)
        assert kb == oq.bit_pack_bytes(flat[:, :96], pack_len) and vb == oq.bit_pack_bytes(flat[:, 96:], pack_len)
    # 2 tokens-blocks of 4 tokens, 1 K + 1 V channel... token medians 3, 9, 9, 1 -> order 1, 2, 0, 3 (tie keeps 1 before 2)
    b = np.array([[[10, 3], [11, 9], [12, 9], [13, 1]]])
    rep, order = orp.median_repacking(b)
    assert order.tolist() == [[1, 2, 0, 3]] and rep[0, :, 0].tolist() == [11, 12, 10, 13]
    # packs of 2 tokens: K (11,12) (10,13) -> ranges 1, 3 -> 1 + 2 bits; 4 distinct values -> W = 2, 2 + 2 metadata bits
    kb, vb = orp.bit_pack(rep, 2)
    assert kb == ((1 + 2) * 2 + 2 * (2 + 2)) // 8


def test_greedy_repack_restatement_against_brute_force():
    """greedy_repacking (utils/compute.py:210-260): the integer restatement against a direct fp64 transcription of
    the two criteria (cosine to the rounded mean; added bits as ceil(log2(range + 1)) differences), on random blocks
    whose criteria have no ties, plus hand-built blocks with a known answer."""
    from oracle import repack as orp

    def brute(block, pack_len):
        x = block.astype(np.float64)
        alive, order = list(range(len(x))), []
        for _ in range(len(x) // pack_len):
            rem = x[alive]
            mean = np.round(rem.mean(axis=0))            # numpy rounds half to even, like torch
            cos = (rem @ mean) / np.maximum(np.linalg.norm(rem, axis=1) * np.linalg.norm(mean), 1e-8)
            gap = np.sort(cos)[::-1]
            assert len(gap) < 2 or gap[0] - gap[1] > 1e-9, "test data must not tie"
            seed = alive.pop(int(np.argmax(cos)))
            order.append(seed)
            mn, mx = x[seed].copy(), x[seed].copy()
            for _ in range(pack_len - 1):
                rem = x[alive]
                pre = np.ceil(np.log2(mx - mn + 1))
                inc = (np.ceil(np.log2(np.maximum(rem, mx) - np.minimum(rem, mn) + 1)) - pre).sum(axis=1)
                pick = alive.pop(int(np.argmin(inc)))      # ties: first, the documented rule
                order.append(pick)
                mn, mx = np.minimum(mn, x[pick]), np.maximum(mx, x[pick])
        return order

    rng = np.random.default_rng(11)
    for (n, d, pack, top) in ((16, 24, 4, 16), (32, 40, 8, 12), (64, 64, 16, 16), (12, 10, 3, 200)):
        for _ in range(3):
            block = rng.integers(0, top, size=(n, d))
            got = orp.greedy_order(block, pack)
            assert sorted(got.tolist()) == list(range(n))            # a permutation
            assert got.tolist() == brute(block, pack)
    # hand-built: 1 channel per half is too coarse for a cosine, so use 2 channels.  Tokens (rows):
    #   a = (4, 4)  b = (4, 5)  c = (0, 9)  d = (9, 0);  mean = (4.25, 4.5) -> rounds to (4, 4): a has cosine 1 -> seed a.
    #   pack_len 2: b adds bit_length(0) + bit_length(1) = 1 bit, c adds 3 + 3, d adds 3 + 3 -> b.  Second pack: remaining
    #   c, d: mean (4.5, 4.5) -> (4, 4) (half to even), cosines equal -> earlier token c, then d.
    block = np.array([[4, 4], [4, 5], [0, 9], [9, 0]])
    assert orp.greedy_order(block, 2).tolist() == [0, 1, 2, 3]
    assert orp.greedy_order(block[[2, 3, 1, 0]], 2).tolist() == [3, 2, 0, 1]      # same tokens, other positions
    # all-zero tokens: every cosine is 0, every cost 0 -> original order
    assert orp.greedy_order(np.zeros((8, 6), dtype=np.int64), 4).tolist() == list(range(8))
    # repacking by the greedy order never costs more payload bits than the seed packs' own lower bound and keeps the tokens
    blocks = rng.integers(0, 16, size=(3, 64, 2 * 32))
    rep, order = orp.greedy_repacking(blocks, 16)
    assert (np.sort(rep, axis=1) == np.sort(blocks, axis=1)).all()
    assert (rep == np.take_along_axis(blocks, order[:, :, None], axis=1)).all()
