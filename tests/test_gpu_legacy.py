"""GPU parity of the reference's GEMV surface (kq_mat_vec_mul, fused_kq, wv_mat_vec_mul, fused_wv),
following the reference call sequences (evaluation/evaluation.py:398-524, :587-715) and checked
against fp64 NumPy on the same codes."""
import numpy as np
import pytest
import torch

import packkv_cuda
from oracle import quant as oq
from packkv_amd import ops, synth

pytestmark = pytest.mark.gpu


def _setup(cuda, H, T, rel, is_k, dtype, seed):
    k, v = synth.make_kv(1, H, T, seed=seed, dtype=dtype)
    x = k if is_k else v
    c, z, s = oq.quant_ints(x, 64, rel)
    cm = oq.code_matrix(c)
    W = ops.bits_for_rel(rel)
    cb, hb = (64, 128) if is_k else (128, 64)
    info = torch.zeros((T // cb) * (H * 128 // hb), 2, dtype=torch.uint32)
    comp = torch.zeros_like(cm)
    size = (packkv_cuda.k_encode_cpu if is_k else packkv_cuda.v_encode_cpu)(cm, comp, info, T, H * 128, cb, hb, W)
    assert size > 0
    return cm, z.flatten(), s.flatten(), comp.to(cuda), info.to(cuda), W, cb, hb


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("H", [8, 32, 40])
def test_kq_path(cuda, dtype, H):
    T, rel = 512, 0.1
    cm, zero, scale, comp, info, W, cb, hb = _setup(cuda, H, T, rel, True, dtype, 41)
    torch.manual_seed(0)
    q = torch.randn(H, 128).to(dtype)
    t = torch.zeros(H, T, dtype=dtype, device=cuda)
    ms = packkv_cuda.kq_mat_vec_mul(comp, info, oq.q_interleave(q).to(cuda), t, T, H * 128, cb, hb, W)
    assert ms > 0
    codes = cm.numpy().astype(np.float64).reshape(T, H, 128)
    want_t = np.einsum("thd,hd->ht", codes, q.double().numpy())
    tol = 2 ** -9 if dtype == torch.float16 else 2 ** -6      # one rounding of the output to dtype
    assert np.abs(t.cpu().double().numpy() - want_t).max() <= tol * np.abs(want_t).max()
    # plain (non-interleaved) q gives the same result
    t2 = torch.zeros_like(t)
    ops.kq_mat_vec_mul(comp, info, q.to(cuda), t2, T, H * 128, cb, hb, W, q_interleaved=False)
    assert torch.equal(t, t2)
    our_kq = torch.empty_like(t)
    ms2 = packkv_cuda.fused_kq(our_kq, q.to(cuda), zero.to(cuda), scale.to(cuda), t)
    assert ms2 > 0
    want = (q.double().sum(1, keepdim=True) * zero.double()[None] + t.cpu().double()) * scale.double()[None]
    assert np.abs(our_kq.cpu().double().numpy() - want.numpy()).max() <= tol * want.abs().max().item()
    # against the dequantised-K matmul the reference uses as its target (10 % acceptance there)
    kd = ((cm.double().reshape(T, H, 128) + zero.double().view(T, 1, 1)) * scale.double().view(T, 1, 1))
    target = np.einsum("thd,hd->ht", kd.numpy(), q.double().numpy())
    assert np.abs(our_kq.cpu().double().numpy() - target).max() <= 4 * tol * np.abs(target).max()


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("H,rel", [(8, 0.2), (40, 0.2), (32, 0.1)])
def test_wv_path(cuda, dtype, H, rel):
    T = 512
    cm, zero, scale, comp, info, W, cb, hb = _setup(cuda, H, T, rel, False, dtype, 43)
    torch.manual_seed(1)
    w = torch.randn(H, T).to(dtype).pow(2).softmax(dim=1)
    w_prime = (w * scale.unsqueeze(0)).to(cuda)
    term1 = torch.zeros(H, 128, dtype=torch.float32, device=cuda)
    ms = packkv_cuda.wv_mat_vec_mul(comp, info, w_prime, term1, T, H * 128, cb, hb, W)
    assert ms > 0
    codes = cm.numpy().astype(np.float64).reshape(T, H, 128)
    want1 = np.einsum("ht,thd->hd", w_prime.cpu().double().numpy(), codes)
    assert np.abs(term1.cpu().double().numpy() - want1).max() <= 1e-5 * np.abs(want1).max()
    term1_t = term1.to(dtype)
    our_wv = torch.empty_like(term1_t)
    ms2 = packkv_cuda.fused_wv(our_wv, w.to(cuda), zero.to(cuda), scale.to(cuda), term1_t)
    assert ms2 > 0
    c_m = (w.double() * zero.double()[None] * scale.double()[None]).sum(1, keepdim=True)
    want = c_m + term1_t.cpu().double()
    tol = 2 ** -9 if dtype == torch.float16 else 2 ** -6
    assert np.abs(our_wv.cpu().double().numpy() - want.numpy()).max() <= tol * max(want.abs().max().item(), 1.0)


def test_unsupported_case_returns_zero(cuda, capsys):
    comp = torch.zeros(64 * 128, dtype=torch.uint8, device=cuda)
    info = torch.zeros(1, 2, dtype=torch.uint32, device=cuda)
    q = torch.zeros(1, 128, dtype=torch.float16, device=cuda)
    t = torch.zeros(1, 64, dtype=torch.float16, device=cuda)
    assert packkv_cuda.kq_mat_vec_mul(comp, info, q, t, 64, 128, 64, 128, 7) == 0.0
    assert "no such case" in capsys.readouterr().out
    assert packkv_cuda.kq_mat_vec_mul(comp, info, q.float(), t, 64, 128, 64, 128, 4) == 0.0
    assert "Unsupported data type" in capsys.readouterr().out
    with pytest.raises(RuntimeError, match="2D"):
        packkv_cuda.fused_kq(t, q[0], t[0], t[0], t)


def test_fused_fixups_take_strided_tensors(cuda):
    """fused_kq / fused_wv on transposed and sliced views (every operand non-contiguous at once): the contiguous
    copies the binding makes must all be alive during the call, so the results equal those of contiguous inputs."""
    g = torch.Generator().manual_seed(77)
    M, N = 8, 1024
    q = torch.randn(128, M, generator=g).to(torch.float16).to(cuda).t()                 # [M, 128] view of [128, M]
    t = torch.randn(N, M, generator=g).to(torch.float16).to(cuda).t()                   # [M, N] view
    zero = torch.randn(2 * N, generator=g).round().to(torch.float16).to(cuda)[::2]      # stride 2
    scale = (torch.rand(2 * N, generator=g) + 0.5).to(torch.float16).to(cuda)[::2]
    assert not (q.is_contiguous() or t.is_contiguous() or zero.is_contiguous() or scale.is_contiguous())
    got, want = torch.empty(M, N, dtype=torch.float16, device=cuda), torch.empty(M, N, dtype=torch.float16, device=cuda)
    packkv_cuda.fused_kq(got, q, zero, scale, t)
    packkv_cuda.fused_kq(want, q.contiguous(), zero.contiguous(), scale.contiguous(), t.contiguous())
    assert torch.equal(got, want)
    w = torch.rand(N, M, generator=g).to(torch.float16).to(cuda).t()
    term1 = torch.randn(128, M, generator=g).to(torch.float16).to(cuda).t()
    got, want = torch.empty(M, 128, dtype=torch.float16, device=cuda), torch.empty(M, 128, dtype=torch.float16, device=cuda)
    packkv_cuda.fused_wv(got, w, zero, scale, term1)
    packkv_cuda.fused_wv(want, w.contiguous(), zero.contiguous(), scale.contiguous(), term1.contiguous())
    assert torch.equal(got, want)


def test_damaged_block_info_is_survived(cuda):
    """Entries of block_info that point outside the compressed buffer give arbitrary products for their blocks;
    nothing outside the buffer is read and the other blocks' results stand."""
    H, T = 8, 512
    cm, zero, scale, comp, info, W, cb, hb = _setup(cuda, H, T, 0.1, True, torch.float16, 43)
    torch.manual_seed(1)
    q = torch.randn(H, 128).to(torch.float16).to(cuda)
    good = torch.zeros(H, T, dtype=torch.float16, device=cuda)
    ops.kq_mat_vec_mul(comp, info, q, good, T, H * 128, cb, hb, W, q_interleaved=False)
    bad_info = info.cpu().numpy().astype(np.int64)
    bad_info[3] = (comp.numel() + 999, 3000)
    bad_info[9] = (0xFFFFFFF0, 0xFFFFFFFF)
    t = torch.zeros(H, T, dtype=torch.float16, device=cuda)
    ops.kq_mat_vec_mul(comp, torch.from_numpy(bad_info.astype(np.uint32)).to(cuda), q, t, T, H * 128, cb, hb, W,
                       q_interleaved=False)
    torch.cuda.synchronize()
    keep = torch.ones(H, T, dtype=torch.bool)
    for b in (3, 9):                                      # block b = (context block b // H, head b % H)
        keep[b % H, (b // H) * cb:(b // H + 1) * cb] = False
    assert torch.equal(t.cpu()[keep], good.cpu()[keep])
    cm, zero, scale, comp, info, W, cb, hb = _setup(cuda, H, T, 0.1, False, torch.float16, 44)
    w = torch.rand(H, T).to(torch.float16).to(cuda)
    bad_info = info.cpu().numpy().astype(np.int64)
    bad_info[0] = (comp.numel(), 1 << 20)
    bad_info[7] = (comp.numel() - 1, 77)
    out = torch.zeros(H, 128, dtype=torch.float32, device=cuda)
    ops.wv_mat_vec_mul(comp, torch.from_numpy(bad_info.astype(np.uint32)).to(cuda), w, out, T, H * 128, cb, hb, W)
    torch.cuda.synchronize()
    assert out.shape == (H, 128)
