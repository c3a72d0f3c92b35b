// The decode step's write into the cache's 16-bit window: rotary embedding of the new K rows and the copy of the
// new K and V rows behind the rows already there, in one launch.
//
// Reference: the cache applies the rotary embedding to the incoming keys itself
// (models/cache/packkv_quant.py:59-60, `apply_rotary_pos_emb_single`, utils/compute.py:35-43:
// (t * cos) + (rotate_half(t) * sin) with rotate_half(t) = cat(-t[64:], t[:64])) and appends keys and values to its
// buffer with torch.cat (packkv_quant.py:62-83).  The three elementwise operations run in the 16-bit storage type --
// each computes in fp32 and rounds its result -- so the kernel rounds both products and the sum, and its rows are
// bit for bit what the reference's chain of kernels produces.
#include "pkv_common.hpp"
#include "pkv_runtime.hpp"

// Every product and sum below is rounded on its own, as separate kernels would round them: no fused multiply-add
// may be formed across them (the compiler narrows the fp32 arithmetic on 16-bit values to 16-bit instructions,
// which is exact, and would then be free to contract them).
#pragma clang fp contract(off)

namespace pkv {

template <int DT> __device__ __forceinline__ float ld16(const uint16_t *p) {
    return DT == PKV_F16 ? __half2float(__ushort_as_half(*p)) : __uint_as_float((uint32_t)*p << 16);
}
template <int DT> __device__ __forceinline__ uint16_t rn16(float x) {
    if (DT == PKV_F16) return __half_as_ushort(__float2half_rn(x));
    uint32_t u = __float_as_uint(x);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x40u);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
template <int DT> __device__ __forceinline__ float rt(float x) {
    const uint16_t b = rn16<DT>(x);
    return ld16<DT>(&b);
}

// grid (n, H, B), 64 threads: thread d owns channels d and d + 64 of one (sequence, head, new token)
template <int DT>
__global__ void __launch_bounds__(64) window_append_kernel(const uint16_t *__restrict__ k_new, const uint16_t *__restrict__ v_new,
                                                           const uint16_t *__restrict__ cos, const uint16_t *__restrict__ sin,
                                                           long sb, long sh, long st, long rot_sb, uint16_t *__restrict__ k_win,
                                                           uint16_t *__restrict__ v_win, int H, int n, int win_pos, int win_stride) {
    const int tok = blockIdx.x, h = blockIdx.y, b = blockIdx.z, d = threadIdx.x;
    const size_t src = (size_t)b * sb + (size_t)h * sh + (size_t)tok * st;
    const size_t dst = (((size_t)b * H + h) * win_stride + win_pos + tok) * kHeadDim;
    v_win[dst + d] = v_new[src + d];
    v_win[dst + d + 64] = v_new[src + d + 64];
    if (cos == nullptr) {
        k_win[dst + d] = k_new[src + d];
        k_win[dst + d + 64] = k_new[src + d + 64];
        return;
    }
    const size_t rot = (size_t)b * rot_sb + (size_t)tok * kHeadDim;
    if (DT == PKV_F16) {     // correctly rounded 16-bit multiplies and adds are exactly the reference's fp32-then-round ops
        const _Float16 *kp = reinterpret_cast<const _Float16 *>(k_new) + src, *cp = reinterpret_cast<const _Float16 *>(cos) + rot,
                       *sp = reinterpret_cast<const _Float16 *>(sin) + rot;
        _Float16 *op = reinterpret_cast<_Float16 *>(k_win) + dst;
        const _Float16 k0 = kp[d], k1 = kp[d + 64];
        const _Float16 a0 = k0 * cp[d], b0 = -k1 * sp[d], a1 = k1 * cp[d + 64], b1 = k0 * sp[d + 64];
        op[d] = a0 + b0;
        op[d + 64] = a1 + b1;
        return;
    }
    const float k0 = ld16<DT>(k_new + src + d), k1 = ld16<DT>(k_new + src + d + 64);
    const float c0 = ld16<DT>(cos + rot + d), c1 = ld16<DT>(cos + rot + d + 64);
    const float s0 = ld16<DT>(sin + rot + d), s1 = ld16<DT>(sin + rot + d + 64);
    k_win[dst + d] = rn16<DT>(rt<DT>(k0 * c0) + rt<DT>(-k1 * s0));
    k_win[dst + d + 64] = rn16<DT>(rt<DT>(k1 * c1) + rt<DT>(k0 * s1));
}

}  // namespace pkv

extern "C" {

int pkv_window_append(const void *k_new, const void *v_new, const void *cos, const void *sin, int dtype, int B, int H,
                      int n, int64_t stride_b, int64_t stride_h, int64_t stride_t, int64_t rot_stride_b, void *k_win,
                      void *v_win, int win_pos, int win_stride, pkv_stream_t s_) {
    using namespace pkv;
    hipStream_t s = (hipStream_t)s_;
    PKV_REQUIRE(k_new && v_new && k_win && v_win, PKV_ERR_INVALID, "null pointer argument");
    PKV_REQUIRE((cos == nullptr) == (sin == nullptr), PKV_ERR_INVALID, "cos and sin go together");
    PKV_REQUIRE(dtype == PKV_F16 || dtype == PKV_BF16, PKV_ERR_UNSUPPORTED, "Unsupported data type");
    PKV_REQUIRE(B > 0 && H > 0 && n > 0 && B <= 65535 && H <= 65535, PKV_ERR_INVALID, "sizes must be positive (batch, heads <= 65535)");
    PKV_REQUIRE(win_pos >= 0 && win_stride > 0 && win_pos + n <= win_stride, PKV_ERR_INVALID,
                "the new rows do not fit the window (%d + %d > %d)", win_pos, n, win_stride);
    PKV_REQUIRE(stride_b >= 0 && stride_h >= 0 && stride_t >= 0 && rot_stride_b >= 0, PKV_ERR_INVALID, "negative stride");
    const dim3 grid((unsigned)n, (unsigned)H, (unsigned)B);
    if (dtype == PKV_F16)
        window_append_kernel<PKV_F16><<<grid, 64, 0, s>>>((const uint16_t *)k_new, (const uint16_t *)v_new, (const uint16_t *)cos,
                                                          (const uint16_t *)sin, (long)stride_b, (long)stride_h, (long)stride_t,
                                                          (long)rot_stride_b, (uint16_t *)k_win, (uint16_t *)v_win, H, n, win_pos,
                                                          win_stride);
    else
        window_append_kernel<PKV_BF16><<<grid, 64, 0, s>>>((const uint16_t *)k_new, (const uint16_t *)v_new, (const uint16_t *)cos,
                                                           (const uint16_t *)sin, (long)stride_b, (long)stride_h, (long)stride_t,
                                                           (long)rot_stride_b, (uint16_t *)k_win, (uint16_t *)v_win, H, n, win_pos,
                                                           win_stride);
    PKV_HIP_CHECK(hipGetLastError());
    return PKV_OK;
}

}  // extern "C"
