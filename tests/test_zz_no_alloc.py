"""pkv_attn_decode_noalloc (partials in the library's fixed device array, no allocation) against pkv_attn_decode:
same kernels, so the same bits -- on two calls in a row, the second with a smaller input (which leaves the first
call's partials behind it in the shared array), and the size limit is reported."""
import pytest
import torch

from packkv_amd import _lib, ops, synth

pytestmark = pytest.mark.gpu


def _case(cuda, B, Hq, Hkv, T, Tw, seed, dtype=torch.float16):
    k, v = synth.make_kv(B, Hkv, T + Tw, seed=seed, dtype=dtype, device=cuda)
    q = synth.make_q(B, Hq, seed=seed + 1, dtype=dtype, device=cuda)
    ke = ops.k_quant_encode(k[:, :, :T].contiguous(), 0.1)
    ve = ops.v_quant_encode(v[:, :, :T].contiguous(), 0.1)
    kw = k[:, :, T:].contiguous() if Tw else None
    vw = v[:, :, T:].contiguous() if Tw else None
    return q, ke, ve, kw, vw


def test_noalloc_entry_point_matches_the_allocating_one(cuda):
    big = _case(cuda, 4, 32, 8, 4096, 150, seed=700)
    small = _case(cuda, 1, 8, 2, 512, 3, seed=710, dtype=torch.bfloat16)
    want = [ops.attn_decode(*c) for c in (big, small)]
    torch.cuda.synchronize()
    for variant in (0, 1, 2):
        for c, w in zip((big, small), want):
            print("no-alloc case: variant", variant, "batch", c[0].shape[0], "tokens", c[1]["scale"].shape[1], flush=True)
            out = torch.full_like(c[0], 7.0)
            got = ops.attn_decode(*c, out=out, variant=variant, noalloc=True)
            ref = ops.attn_decode(*c, variant=variant)
            torch.cuda.synchronize()
            assert got.data_ptr() == out.data_ptr()
            assert torch.equal(got, ref)
            if variant == 0:
                assert torch.equal(got, w)


def test_noalloc_entry_point_with_tiles_handed_out_by_counter(cuda):
    """A step whose members take tiles from the heads' counters (8 members x 16 tiles) with the counters in the fixed
    array, behind the partials: twice in a row, then a smaller step, then again -- every launch must leave the
    counters at zero for the next.  Which member takes which tile depends on timing, and with it the running maxima
    against which the softmax weights are rounded to fp16, so two runs of such a step differ by that rounding (a few
    1e-5) and by a rounding of the 16-bit output; they are held to that, not to the bit (the small step has fixed
    shares and is compared bit for bit)."""
    big = _case(cuda, 16, 32, 8, 16384, 0, seed=730)
    small = _case(cuda, 2, 16, 4, 1024, 0, seed=740)
    want_big, want_small = ops.attn_decode(*big), ops.attn_decode(*small)
    torch.cuda.synchronize()
    for c, w in ((big, want_big), (big, want_big), (small, want_small), (big, want_big)):
        print("no-alloc case with tile counters: batch", c[0].shape[0], "tokens", c[1]["scale"].shape[1], flush=True)
        got = ops.attn_decode(*c, noalloc=True)
        torch.cuda.synchronize()
        if c is small:
            assert torch.equal(got, w)
        else:
            err = (got.float() - w.float()).abs()
            print("   largest difference between two runs of the step: %.3e" % err.max().item(), flush=True)
            assert bool((err <= 2.0 ** -10 * w.float().abs() + 2e-4).all())     # a lost or repeated tile would move them by 1e-2


def test_noalloc_entry_point_rejects_what_does_not_fit(cuda):
    """8 MiB hold B * Hq * partials * 520 bytes: batch 64 x 64 query heads with a window (2 x 2 partials... ) fits, a
    step with 64 sequences x 64 heads x 2 x 32 partials does not -- and says so instead of overrunning the array."""
    lib = _lib.load()
    B, Hq, Hkv, T, Tw = 64, 64, 8, 512, 4
    q, ke, ve, kw, vw = _case(cuda, B, Hq, Hkv, T, Tw, seed=720)
    plan = ops.AttnPlan(q, ke, ve, kw, vw, noalloc=True)     # 2 splits + 2 window pieces: 64 * 64 * 4 * 520 B = 8.1 MiB
    with pytest.raises(ops.PackKVError) as e:
        plan()
    assert e.value.code == _lib.ERR_UNSUPPORTED and "static buffer" in str(e.value)
    assert torch.equal(ops.attn_decode(q, ke, ve, kw, vw), ops.attn_decode(q, ke, ve, kw, vw))   # the allocating one takes it
