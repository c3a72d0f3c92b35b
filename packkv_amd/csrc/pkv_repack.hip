// Token repacking and the analytic pack-size model on the device.
//
// Reference (utils/compute.py): `median_repacking` (:262-270) reorders the tokens of every quantisation block,
// jointly for K and V across all heads and sequences, by descending median of the token's V codes;
// `bit_pack` (:272-297) prices a code matrix as  sum over packs of pack_len * bit_length(max - min)  payload bits
// plus (W + ceil(log2(W + 1))) metadata bits per pack, W = ceil(log2(#distinct codes)).  Both work on the uint8
// code matrix [ctx_len, hidden] (channel = (b * H + h) * 128 + d), the layout the codecs consume.
//
// Tie order: the reference sorts with torch.sort(descending=True) without stable=True, which leaves the order
// of equal medians to the backend.  Here ties keep their original order (a stable descending sort).
#include "pkv_common.hpp"
#include "pkv_runtime.hpp"

namespace pkv {

// ---- lower median of every token row: one wavefront per token ----
// Rows of up to 16384 codes below 128 stay in registers (16 bytes x 16 per lane) and the median is found by
// bisection on the value: a step counts the bytes above the probe with three word-wide instructions per four codes
// ((x | 0x80) - (probe + 1) keeps bit 7 of a byte exactly when the byte is above the probe; no borrow crosses bytes
// while both are at most 128).  Other rows use a 256-bin histogram in LDS (slow when few values dominate: equal
// addresses serialise the LDS atomics).
__device__ __forceinline__ uint32_t wave_sum_u32(uint32_t x) {
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) x += __shfl_xor(x, d, 64);
    return x;
}

__global__ void __launch_bounds__(256) token_median_kernel(const uint8_t *__restrict__ codes, int ctx_len, int hidden,
                                                           uint8_t *__restrict__ median) {
    __shared__ uint32_t hist[4][256];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int tok = blockIdx.x * 4 + wave;
    if (tok >= ctx_len) return;                                   // whole wavefronts leave; no workgroup barrier below
    const uint4 *row = reinterpret_cast<const uint4 *>(codes + (size_t)tok * hidden);
    const int nchunks = hidden / 16;
    const uint32_t k = (uint32_t)(hidden - 1) / 2u;               // torch.median: the lower of the two middle values
    if (nchunks <= 16 * 64) {
        uint32_t w[64];
        uint32_t high = 0u;
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const int c = lane + 64 * i;
            const uint4 v = c < nchunks ? row[c] : make_uint4(0x7F7F7F7Fu, 0x7F7F7F7Fu, 0x7F7F7F7Fu, 0x7F7F7F7Fu);
            w[4 * i] = v.x; w[4 * i + 1] = v.y; w[4 * i + 2] = v.z; w[4 * i + 3] = v.w;
            high |= v.x | v.y | v.z | v.w;
        }
        if (__ballot((high & 0x80808080u) != 0u) == 0ull) {
            const uint32_t n_pad = (uint32_t)(16 * 64 * 16 - hidden);   // padding bytes hold 127: above every probe
            uint32_t lo = 0u, hi = 127u;
            while (lo < hi) {
                const uint32_t mid = (lo + hi) >> 1;
                const uint32_t cmpw = (mid + 1u) * 0x01010101u;
                uint32_t above = 0u;
#pragma unroll
                for (int i = 0; i < 64; i++)
                    above += (uint32_t)__builtin_popcount(((w[i] | 0x80808080u) - cmpw) & 0x80808080u);
                above = wave_sum_u32(above) - n_pad;
                if ((uint32_t)hidden - above >= k + 1u) hi = mid; else lo = mid + 1u;   // codes <= mid reach rank k
            }
            if (lane == 0) median[tok] = (uint8_t)lo;
            return;
        }
    }
    uint32_t *h = hist[wave];
    for (int i = lane; i < 256; i += 64) h[i] = 0u;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    for (int c = lane; c < nchunks; c += 64) {
        const uint4 v = row[c];
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int kk = 0; kk < 4; kk++) atomicAdd(&h[(w[i] >> (8 * kk)) & 0xFFu], 1u);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    // lane l owns bins 4l..4l+3
    const uint32_t c0 = h[4 * lane], c1 = h[4 * lane + 1], c2 = h[4 * lane + 2], c3 = h[4 * lane + 3];
    const uint32_t mine = c0 + c1 + c2 + c3;
    uint32_t inc = mine;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const uint32_t up = __shfl_up(inc, d, 64);
        if (lane >= d) inc += up;
    }
    const uint32_t before = inc - mine;
    if (before <= k && k < inc) {
        uint32_t bin = 4 * lane, run = before + c0;
        if (k >= run) { bin++; run += c1; }
        if (k >= run) { bin++; run += c2; }
        if (k >= run) bin++;
        median[tok] = (uint8_t)bin;
    }
}

// ---- order of the tokens of every block: descending median, ties in original order ----
// perm[blk * bs + r] = index inside the block of the token that moves to position r.
__global__ void block_order_kernel(const uint8_t *__restrict__ median, int block_size, uint32_t *__restrict__ perm) {
    extern __shared__ uint8_t m_s[];
    const int i = threadIdx.x;
    const size_t base = (size_t)blockIdx.x * block_size;
    if (i < block_size) m_s[i] = median[base + i];
    __syncthreads();
    if (i >= block_size) return;
    const uint32_t mine = m_s[i];
    uint32_t rank = 0;
    for (int j = 0; j < block_size; j++) {
        const uint32_t o = m_s[j];
        rank += (o > mine) || (o == mine && j < i);
    }
    perm[base + rank] = (uint32_t)i;
}

// ---- out row r = in row perm[r], for K and V at once: grid (ctx_len), 256 threads ----
__global__ void __launch_bounds__(256) gather_rows_kernel(const uint8_t *__restrict__ k_in, const uint8_t *__restrict__ v_in,
                                                          uint8_t *__restrict__ k_out, uint8_t *__restrict__ v_out,
                                                          const uint32_t *__restrict__ perm, int block_size, int hidden) {
    const size_t r = blockIdx.x;
    const size_t src = r - r % (size_t)block_size + perm[r];
    const uint4 *ks = reinterpret_cast<const uint4 *>(k_in + src * hidden), *vs = reinterpret_cast<const uint4 *>(v_in + src * hidden);
    uint4 *kd = reinterpret_cast<uint4 *>(k_out + r * hidden), *vd = reinterpret_cast<uint4 *>(v_out + r * hidden);
    for (int c = threadIdx.x; c < hidden / 16; c += 256) {
        kd[c] = ks[c];
        vd[c] = vs[c];
    }
}

// ---- analytic size: sum of bit_length(max - min) over packs, and which code values occur ----
struct PackSizeOut {
    unsigned long long len_sum;
    uint32_t present[256];
};

__global__ void pack_size_zero_kernel(PackSizeOut *out) {
    if (threadIdx.x == 0) out->len_sum = 0ull;
    out->present[threadIdx.x] = 0u;
}

// grid (ceil(hidden / 4096), ctx_len / pack_len), 256 threads; thread = 16 adjacent channels of one pack, four rows
// in flight; minima and maxima as packed 16-bit lanes (even and odd bytes of every dword apart)
typedef unsigned short pk_u16x2 __attribute__((ext_vector_type(2)));

__global__ void __launch_bounds__(256) pack_size_kernel(const uint8_t *__restrict__ codes, int hidden, int pack_len,
                                                        PackSizeOut *out) {
    __shared__ uint32_t seen[256];
    __shared__ uint32_t wsum[4];
    seen[threadIdx.x] = 0u;
    __syncthreads();
    const int ch = (blockIdx.x * 256 + threadIdx.x) * 16;
    uint32_t lens = 0;
    if (ch < hidden) {
        const uint8_t *p = codes + (size_t)blockIdx.y * pack_len * hidden + ch;
        pk_u16x2 mn[8], mx[8];
#pragma unroll
        for (int i = 0; i < 8; i++) { mn[i] = (pk_u16x2){255, 255}; mx[i] = (pk_u16x2){0, 0}; }
        auto take = [&](const uint4 v) {
            const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const pk_u16x2 e = __builtin_bit_cast(pk_u16x2, w[i] & 0x00FF00FFu);
                const pk_u16x2 o = __builtin_bit_cast(pk_u16x2, (w[i] >> 8) & 0x00FF00FFu);
                mn[2 * i] = __builtin_elementwise_min(mn[2 * i], e);
                mx[2 * i] = __builtin_elementwise_max(mx[2 * i], e);
                mn[2 * i + 1] = __builtin_elementwise_min(mn[2 * i + 1], o);
                mx[2 * i + 1] = __builtin_elementwise_max(mx[2 * i + 1], o);
                seen[e[0]] = 1u;              // every writer stores the same value
                seen[e[1]] = 1u;
                seen[o[0]] = 1u;
                seen[o[1]] = 1u;
            }
        };
        int k = 0;
        for (; k + 4 <= pack_len; k += 4) {
            uint4 v[4];
#pragma unroll
            for (int u = 0; u < 4; u++) v[u] = *reinterpret_cast<const uint4 *>(p + (size_t)(k + u) * hidden);
#pragma unroll
            for (int u = 0; u < 4; u++) take(v[u]);
        }
        for (; k < pack_len; k++) take(*reinterpret_cast<const uint4 *>(p + (size_t)k * hidden));
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const pk_u16x2 r = mx[i] - mn[i];
#pragma unroll
            for (int hlf = 0; hlf < 2; hlf++)
                lens += r[hlf] ? 32u - (uint32_t)__builtin_clz((uint32_t)r[hlf]) : 0u;   // bit_length = ceil(log2(range + 1))
        }
    }
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) lens += __shfl_xor(lens, d, 64);
    if ((threadIdx.x & 63) == 0) wsum[threadIdx.x >> 6] = lens;
    __syncthreads();
    if (threadIdx.x == 0) atomicAdd(&out->len_sum, (unsigned long long)(wsum[0] + wsum[1] + wsum[2] + wsum[3]));
    if (seen[threadIdx.x]) out->present[threadIdx.x] = 1u;
}

}  // namespace pkv

extern "C" {

int pkv_bit_pack_size(const uint8_t *codes, int ctx_len, int hidden_dim, int pack_len, uint64_t *len_sum_out,
                      uint32_t *n_unique_out, float *ms_out, pkv_stream_t s_) {
    using namespace pkv;
    hipStream_t s = (hipStream_t)s_;
    PKV_REQUIRE(codes && len_sum_out && n_unique_out, PKV_ERR_INVALID, "null pointer argument");
    PKV_REQUIRE(ctx_len > 0 && hidden_dim > 0 && pack_len > 0, PKV_ERR_INVALID, "sizes must be positive");
    PKV_REQUIRE(hidden_dim % 16 == 0 && (reinterpret_cast<uintptr_t>(codes) & 15u) == 0, PKV_ERR_INVALID,
                "hidden_dim must be a multiple of 16 and the code matrix 16-byte aligned");
    PKV_REQUIRE(ctx_len % pack_len == 0, PKV_ERR_INVALID, "ctx_len must be divisible by the pack length");
    PKV_REQUIRE(ctx_len / pack_len <= 65535, PKV_ERR_UNSUPPORTED, "more than 65535 packs along the context");
    void *scratch = nullptr;
    int rc = scratch_get(sizeof(PackSizeOut), &scratch);
    if (rc) return rc;
    PackSizeOut *out = static_cast<PackSizeOut *>(scratch);
    LaunchTimer tm(s, ms_out != nullptr);
    if ((rc = tm.begin())) return rc;
    pack_size_zero_kernel<<<1, 256, 0, s>>>(out);
    pack_size_kernel<<<dim3((unsigned)((hidden_dim + 4095) / 4096), (unsigned)(ctx_len / pack_len)), 256, 0, s>>>(
        codes, hidden_dim, pack_len, out);
    PKV_HIP_CHECK(hipGetLastError());
    if ((rc = tm.end(ms_out))) return rc;
    PackSizeOut h;
    PKV_HIP_CHECK(hipMemcpyAsync(&h, out, sizeof(h), hipMemcpyDeviceToHost, s));
    PKV_HIP_CHECK(hipStreamSynchronize(s));
    uint32_t n = 0;
    for (int i = 0; i < 256; i++) n += h.present[i];
    *len_sum_out = h.len_sum;
    *n_unique_out = n;
    return PKV_OK;
}

int pkv_median_repack(const uint8_t *k_codes, const uint8_t *v_codes, uint8_t *k_out, uint8_t *v_out, uint32_t *perm,
                      int ctx_len, int hidden_dim, int block_size, float *ms_out, pkv_stream_t s_) {
    using namespace pkv;
    hipStream_t s = (hipStream_t)s_;
    PKV_REQUIRE(k_codes && v_codes && k_out && v_out && perm, PKV_ERR_INVALID, "null pointer argument");
    PKV_REQUIRE(k_codes != k_out && v_codes != v_out, PKV_ERR_INVALID, "repacking cannot run in place");
    PKV_REQUIRE(ctx_len > 0 && hidden_dim > 0 && block_size > 0, PKV_ERR_INVALID, "sizes must be positive");
    PKV_REQUIRE(hidden_dim % 16 == 0 && ((reinterpret_cast<uintptr_t>(k_codes) | reinterpret_cast<uintptr_t>(v_codes) |
                                          reinterpret_cast<uintptr_t>(k_out) | reinterpret_cast<uintptr_t>(v_out)) & 15u) == 0,
                PKV_ERR_INVALID, "hidden_dim must be a multiple of 16 and the code matrices 16-byte aligned");
    PKV_REQUIRE(block_size <= 1024 && ctx_len % block_size == 0, PKV_ERR_INVALID,
                "ctx_len must be divisible by a block size of at most 1024 tokens");
    void *scratch = nullptr;
    int rc = scratch_get((size_t)ctx_len, &scratch);
    if (rc) return rc;
    uint8_t *median = static_cast<uint8_t *>(scratch);
    LaunchTimer tm(s, ms_out != nullptr);
    if ((rc = tm.begin())) return rc;
    token_median_kernel<<<(unsigned)((ctx_len + 3) / 4), 256, 0, s>>>(v_codes, ctx_len, hidden_dim, median);
    const int threads = (block_size + 63) / 64 * 64;
    block_order_kernel<<<(unsigned)(ctx_len / block_size), threads, (size_t)block_size, s>>>(median, block_size, perm);
    gather_rows_kernel<<<(unsigned)ctx_len, 256, 0, s>>>(k_codes, v_codes, k_out, v_out, perm, block_size, hidden_dim);
    PKV_HIP_CHECK(hipGetLastError());
    return tm.end(ms_out);
}

}  // extern "C"
