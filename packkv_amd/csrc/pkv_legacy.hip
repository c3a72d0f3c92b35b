// The reference's four GPU ops, generalised to any head count and any hidden_dim that is a
// multiple of the block width, with fp32 accumulation (the reference accumulates in 16 bit,
// include/type_traits.h:26-58):
//   kq_mat_vec_mul  packkv_cuda_ext/src/kernels.cu:426-535   (K unpack fused with q . code)
//   wv_mat_vec_mul  packkv_cuda_ext/src/kernels.cu:632-765   (V unpack fused with w . code)
//   fused_kq        packkv_cuda_ext/src/fused_kernels.cu:13-76
//   fused_wv        packkv_cuda_ext/src/fused_kernels.cu:187-261
#include "pkv_block.hpp"
#include "pkv_runtime.hpp"

namespace pkv {

__device__ __forceinline__ float ld16(const uint16_t *p, size_t i, int dtype) {
    const uint32_t u = p[i];
    return dtype == PKV_F16 ? __half2float(__ushort_as_half((unsigned short)u)) : __uint_as_float(u << 16);
}

__device__ __forceinline__ uint16_t st16(float x, int dtype) {
    if (dtype == PKV_F16) return __half_as_ushort(__float2half_rn(x));
    uint32_t u = __float_as_uint(x);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x40u);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

// grid = number of K blocks, threads = 2 * ctx_blk (one half-wavefront per round).  (Padding the tile rows so
// that the dot product's reads spread over the LDS banks changes nothing measurable: the kernel's time is the
// latency chain stage -> decode -> dot of many small workgroups.)
__global__ void kq_kernel(const uint8_t *__restrict__ stream, uint64_t stream_bytes, const uint32_t *__restrict__ info,
                          const uint16_t *__restrict__ q, uint16_t *__restrict__ kq_out, int ctx_len,
                          int hidden_dim, int ctx_blk, int nunits, int W, uint32_t blk_cap, int dtype,
                          int q_interleaved) {
    extern __shared__ __align__(16) uint8_t lds[];
    __shared__ float qs[kHeadDim];
    uint8_t *tile = lds;
    uint8_t *blk = lds + ctx_blk * kHeadDim;
    const int n_hid = hidden_dim / kHeadDim;
    const uint32_t b = blockIdx.x;
    const uint32_t cb = b / n_hid, hb = b % n_hid;
    uint32_t off, size;
    block_span(info, b, blk_cap, stream_bytes, off, size);
    const uint32_t phase = stage_to_lds(stream + off, size, blk, threadIdx.x, blockDim.x);
    for (int c = threadIdx.x; c < kHeadDim; c += blockDim.x) {
        int src = c;
        if (q_interleaved) {   // evaluation/evaluation.py:465-468
            const int l = c >> 2, i = c & 3;
            src = i < 2 ? 2 * l + i : 64 + 2 * l + (i - 2);
        }
        qs[c] = ld16(q, (size_t)hb * kHeadDim + src, dtype);
    }
    __syncthreads();
    block_decode<true>(blk, phase, nunits, W, tile, kHeadDim);
    __syncthreads();
    const int r = threadIdx.x >> 1, half = threadIdx.x & 1;
    float acc = 0.f;
    if (r < ctx_blk) {
        const uint32_t *row = reinterpret_cast<const uint32_t *>(tile + r * kHeadDim + half * 64);
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const uint32_t w = row[i];
            const float *qq = qs + half * 64 + 4 * i;
            acc += qq[0] * (float)(w & 0xFFu) + qq[1] * (float)((w >> 8) & 0xFFu) +
                   qq[2] * (float)((w >> 16) & 0xFFu) + qq[3] * (float)(w >> 24);
        }
    }
    acc += __shfl_xor(acc, 1, 64);
    if (half == 0 && r < ctx_blk)
        kq_out[(size_t)hb * ctx_len + (size_t)cb * ctx_blk + r] = st16(acc, dtype);
}

// grid = number of V blocks, threads = 2 * hid_blk (one half-wavefront per segment; 8 * hid_blk / 4 in the dot product).
__global__ void wv_kernel(const uint8_t *__restrict__ stream, uint64_t stream_bytes, const uint32_t *__restrict__ info,
                          const uint16_t *__restrict__ w, float *__restrict__ wv_out, int ctx_len,
                          int hidden_dim, int hid_blk, int nunits, int W, uint32_t blk_cap, int dtype) {
    extern __shared__ __align__(16) uint8_t lds[];
    __shared__ float ws[128];
    uint8_t *tile = lds;
    uint8_t *blk = lds + 128 * hid_blk;
    const int n_hid = hidden_dim / hid_blk;
    const uint32_t b = blockIdx.x;
    const uint32_t cb = b / n_hid, hb = b % n_hid;
    const uint32_t head = (hb * (uint32_t)hid_blk) / kHeadDim;
    uint32_t off, size;
    block_span(info, b, blk_cap, stream_bytes, off, size);
    const uint32_t phase = stage_to_lds(stream + off, size, blk, threadIdx.x, blockDim.x);
    for (int t = threadIdx.x; t < 128; t += blockDim.x)
        ws[t] = ld16(w, (size_t)head * ctx_len + (size_t)cb * 128 + t, dtype);
    __syncthreads();
    block_decode<false>(blk, phase, nunits, W, tile, hid_blk);
    __syncthreads();
    // thread = 4 adjacent channels x 16 tokens (one dword of the tile per token); the eight token slices meet in
    // LDS, over the staged block, which nobody reads any more (it holds at least 32 * hid_blk bytes at 2 bits)
    const int ncg = hid_blk >> 2;
    const int cg = threadIdx.x % ncg, ts = threadIdx.x / ncg;
    const uint32_t *col = reinterpret_cast<const uint32_t *>(tile) + (ts * 16) * ncg + cg;
    float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
#pragma unroll
    for (int t = 0; t < 16; t++) {
        const uint32_t c = col[t * ncg];
        const float wt = ws[ts * 16 + t];
        a0 += wt * (float)(c & 0xFFu);
        a1 += wt * (float)((c >> 8) & 0xFFu);
        a2 += wt * (float)((c >> 16) & 0xFFu);
        a3 += wt * (float)(c >> 24);
    }
    float *part = reinterpret_cast<float *>(blk);
    *reinterpret_cast<float4 *>(part + ts * hid_blk + 4 * cg) = make_float4(a0, a1, a2, a3);
    __syncthreads();
    if ((int)threadIdx.x < hid_blk) {
        float acc = 0.f;
#pragma unroll
        for (int i = 0; i < 8; i++) acc += part[i * hid_blk + threadIdx.x];
        atomicAdd(wv_out + (size_t)hb * hid_blk + threadIdx.x, acc);
    }
}

__device__ __forceinline__ float wave_sum_f32(float x) {
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) x += __shfl_xor(x, d, 64);
    return x;
}

// grid = (ceil(N / 2048), M), 256 threads: every workgroup forms the row's sum of q itself (K values) and then
// finishes 2048 columns, eight per thread.
__global__ void __launch_bounds__(256) fused_kq_kernel(uint16_t *__restrict__ out, const uint16_t *__restrict__ q,
                                                       const uint16_t *__restrict__ zero, const uint16_t *__restrict__ scale,
                                                       const uint16_t *__restrict__ t, int K, int N, int dtype) {
    __shared__ float red[4];
    const int m = blockIdx.y;
    float s = 0.f;
    for (int d = threadIdx.x; d < K; d += 256) s += ld16(q, (size_t)m * K + d, dtype);
    s = wave_sum_f32(s);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = s;
    __syncthreads();
    const float sm = (red[0] + red[1]) + (red[2] + red[3]);
    const int n0 = blockIdx.x * 2048;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const int n = n0 + threadIdx.x + 256 * i;
        if (n < N) {
            const float u = sm * ld16(zero, n, dtype) + ld16(t, (size_t)m * N + n, dtype);
            out[(size_t)m * N + n] = st16(u * ld16(scale, n, dtype), dtype);
        }
    }
}

// Row sums of w * zero * scale in two steps: grid (ceil(N / 4096), M) partial sums, then one workgroup per row
// adds the partials and finishes the D outputs.
__global__ void __launch_bounds__(256) fused_wv_partial_kernel(const uint16_t *__restrict__ w, const uint16_t *__restrict__ zero,
                                                               const uint16_t *__restrict__ scale, float *__restrict__ part,
                                                               int N, int dtype) {
    __shared__ float red[4];
    const int m = blockIdx.y, n0 = blockIdx.x * 4096;
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 16; i++) {
        const int n = n0 + threadIdx.x + 256 * i;
        if (n < N) s += ld16(w, (size_t)m * N + n, dtype) * ld16(zero, n, dtype) * ld16(scale, n, dtype);
    }
    s = wave_sum_f32(s);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = s;
    __syncthreads();
    if (threadIdx.x == 0) part[(size_t)m * gridDim.x + blockIdx.x] = (red[0] + red[1]) + (red[2] + red[3]);
}

__global__ void __launch_bounds__(256) fused_wv_kernel(uint16_t *__restrict__ out, const float *__restrict__ part, int nparts,
                                                       const uint16_t *__restrict__ term1, int D, int dtype) {
    __shared__ float red[4];
    const int m = blockIdx.x;
    float s = 0.f;
    for (int i = threadIdx.x; i < nparts; i += 256) s += part[(size_t)m * nparts + i];
    s = wave_sum_f32(s);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = s;
    __syncthreads();
    const float c = (red[0] + red[1]) + (red[2] + red[3]);
    for (int d = threadIdx.x; d < D; d += 256)
        out[(size_t)m * D + d] = st16(c + ld16(term1, (size_t)m * D + d, dtype), dtype);
}

static int check_dtype(int dtype) {
    PKV_REQUIRE(dtype == PKV_F16 || dtype == PKV_BF16, PKV_ERR_UNSUPPORTED, "Unsupported data type");
    return PKV_OK;
}

}  // namespace pkv

extern "C" {

int pkv_kq_mat_vec_mul(const uint8_t *stream, uint64_t stream_bytes, const uint32_t *block_info, const void *q, void *kq_out,
                       int ctx_len, int hidden_dim, int ctx_blk, int hid_blk, int bits, int dtype,
                       int q_interleaved, float *ms_out, pkv_stream_t s_) {
    using namespace pkv;
    hipStream_t s = (hipStream_t)s_;
    int rc = check_dtype(dtype);
    if (rc) return rc;
    PKV_REQUIRE(stream && block_info && q && kq_out, PKV_ERR_INVALID, "null pointer argument");
    PKV_REQUIRE(stream_bytes > 0 && stream_bytes < (1ull << 32), PKV_ERR_INVALID, "stream size must be in 1 .. 4 GiB - 1");
    PKV_REQUIRE(bits >= 2 && bits <= 4 && hid_blk == kHeadDim && ctx_blk > 0 && ctx_blk % kPackTok == 0 &&
                    ctx_blk <= 256 && ctx_len > 0 && ctx_len % ctx_blk == 0 && hidden_dim > 0 &&
                    hidden_dim % hid_blk == 0,
                PKV_ERR_UNSUPPORTED, "no such case");
    const int nunits = ctx_blk / kPackTok;
    const uint32_t cap = (uint32_t)k_block_bound(ctx_blk, bits);
    const int nblocks = (ctx_len / ctx_blk) * (hidden_dim / hid_blk);
    const uint32_t lds_bytes = (uint32_t)(ctx_blk * kHeadDim) + ((cap + 15u) & ~15u) + 32u;
    const int threads = ((2 * ctx_blk + 63) / 64) * 64;
    LaunchTimer tm(s, ms_out != nullptr);
    if ((rc = tm.begin())) return rc;
    kq_kernel<<<nblocks, threads, lds_bytes, s>>>(stream, stream_bytes, block_info, (const uint16_t *)q, (uint16_t *)kq_out,
                                                   ctx_len, hidden_dim, ctx_blk, nunits, bits, cap, dtype,
                                                   q_interleaved);
    PKV_HIP_CHECK(hipGetLastError());
    return tm.end(ms_out);
}

int pkv_wv_mat_vec_mul(const uint8_t *stream, uint64_t stream_bytes, const uint32_t *block_info, const void *w, float *wv_out,
                       int ctx_len, int hidden_dim, int ctx_blk, int hid_blk, int bits, int dtype,
                       float *ms_out, pkv_stream_t s_) {
    using namespace pkv;
    hipStream_t s = (hipStream_t)s_;
    int rc = check_dtype(dtype);
    if (rc) return rc;
    PKV_REQUIRE(stream && block_info && w && wv_out, PKV_ERR_INVALID, "null pointer argument");
    PKV_REQUIRE(stream_bytes > 0 && stream_bytes < (1ull << 32), PKV_ERR_INVALID, "stream size must be in 1 .. 4 GiB - 1");
    PKV_REQUIRE(bits >= 2 && bits <= 4 && ctx_blk == 128 && (hid_blk == 32 || hid_blk == 64 || hid_blk == 128) &&
                    ctx_len > 0 && ctx_len % ctx_blk == 0 && hidden_dim > 0 && hidden_dim % kHeadDim == 0,
                PKV_ERR_UNSUPPORTED, "no such case");
    const int nunits = 2 * (hid_blk / kLanes);
    const uint32_t cap = (uint32_t)v_block_bound(hid_blk, bits);
    const int nblocks = (ctx_len / ctx_blk) * (hidden_dim / hid_blk);
    const uint32_t lds_bytes = (uint32_t)(128 * hid_blk) + ((cap + 15u) & ~15u) + 32u;
    LaunchTimer tm(s, ms_out != nullptr);
    if ((rc = tm.begin())) return rc;
    wv_kernel<<<nblocks, 2 * hid_blk, lds_bytes, s>>>(stream, stream_bytes, block_info, (const uint16_t *)w, wv_out, ctx_len,
                                                      hidden_dim, hid_blk, nunits, bits, cap, dtype);
    PKV_HIP_CHECK(hipGetLastError());
    return tm.end(ms_out);
}

int pkv_fused_kq(void *our_kq, const void *q, const void *k_zero, const void *k_scale, const void *t, int M,
                 int K, int N, int dtype, float *ms_out, pkv_stream_t s_) {
    using namespace pkv;
    hipStream_t s = (hipStream_t)s_;
    int rc = check_dtype(dtype);
    if (rc) return rc;
    PKV_REQUIRE(our_kq && q && k_zero && k_scale && t, PKV_ERR_INVALID, "null pointer argument");
    PKV_REQUIRE(M > 0 && K > 0 && N > 0, PKV_ERR_INVALID, "sizes must be positive");
    PKV_REQUIRE(M <= 65535, PKV_ERR_UNSUPPORTED, "more than 65535 rows");
    LaunchTimer tm(s, ms_out != nullptr);
    if ((rc = tm.begin())) return rc;
    fused_kq_kernel<<<dim3((unsigned)((N + 2047) / 2048), (unsigned)M), 256, 0, s>>>(
        (uint16_t *)our_kq, (const uint16_t *)q, (const uint16_t *)k_zero, (const uint16_t *)k_scale,
        (const uint16_t *)t, K, N, dtype);
    PKV_HIP_CHECK(hipGetLastError());
    return tm.end(ms_out);
}

int pkv_fused_wv(void *our_wv, const void *w, const void *v_zero, const void *v_scale, const void *term1,
                 int M, int N, int D, int dtype, float *ms_out, pkv_stream_t s_) {
    using namespace pkv;
    hipStream_t s = (hipStream_t)s_;
    int rc = check_dtype(dtype);
    if (rc) return rc;
    PKV_REQUIRE(our_wv && w && v_zero && v_scale && term1, PKV_ERR_INVALID, "null pointer argument");
    PKV_REQUIRE(M > 0 && N > 0 && D > 0, PKV_ERR_INVALID, "sizes must be positive");
    PKV_REQUIRE(M <= 65535, PKV_ERR_UNSUPPORTED, "more than 65535 rows");
    const int nparts = (N + 4095) / 4096;
    void *scratch = nullptr;
    if ((rc = scratch_get((size_t)M * nparts * sizeof(float), s, &scratch))) return rc;
    LaunchTimer tm(s, ms_out != nullptr);
    if ((rc = tm.begin())) return rc;
    fused_wv_partial_kernel<<<dim3((unsigned)nparts, (unsigned)M), 256, 0, s>>>(
        (const uint16_t *)w, (const uint16_t *)v_zero, (const uint16_t *)v_scale, (float *)scratch, N, dtype);
    fused_wv_kernel<<<M, 256, 0, s>>>((uint16_t *)our_wv, (const float *)scratch, nparts, (const uint16_t *)term1,
                                      D, dtype);
    PKV_HIP_CHECK(hipGetLastError());
    return tm.end(ms_out);
}

}  // extern "C"
