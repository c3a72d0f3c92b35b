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
#include "pkv_block.hpp"

#include <map>
#include <mutex>

namespace pkv {

typedef unsigned short ushort2v __attribute__((ext_vector_type(2)));

// ---- lower median of every token row: one wavefront per token ----
// Rows of up to 16384 codes below 128 stay in registers (16 bytes x 16 per lane) and the median is found by
// bisection on the value: a step counts the bytes above the probe with three word-wide instructions per four codes
// ((x | 0x80) - (probe + 1) keeps bit 7 of a byte exactly when the byte is above the probe; no borrow crosses bytes
// while both are at most 128).  Other rows use a 256-bin histogram in LDS (slow when few values dominate: equal
// addresses serialise the LDS atomics).
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

int launch_block_order(const uint8_t *median, int ctx_len, int block_size, uint32_t *perm, hipStream_t s) {
    const int threads = (block_size + 63) / 64 * 64;
    block_order_kernel<<<(unsigned)(ctx_len / block_size), threads, (size_t)block_size, s>>>(median, block_size, perm);
    PKV_HIP_CHECK(hipGetLastError());
    return PKV_OK;
}

// ---- greedy order of the tokens of every block: one workgroup of 1024 threads per block ----
// `greedy_repacking` (utils/compute.py:210-260): a block's N tokens are rows of D2 = 2 * hidden codes (K half, then
// V half).  Every pack starts from the remaining token with the largest cosine to the rounded mean of the remaining
// tokens and then takes, pack_len - 1 times, the remaining token whose addition costs the fewest payload bits,
// sum over channels of bit_length(max - min).  All of it is integer work here: the bit counts are exact, the
// bits already spent are common to all candidates (so the new total decides), and the cosines are compared exactly
// (codes are non-negative and the mean is common: cos_a > cos_b  <=>  dot_a^2 |b|^2 > dot_b^2 |a|^2, 128-bit
// products).  Ties go to the earlier token -- the order the reference's argmax / argmin see on a CPU backend;
// the reference itself leaves them, and fp32 near-ties of the cosine, to the backend.
//
// LDS: running minimum and maximum per channel (D2 bytes each; the mean borrows the maximum's array), one cost or
// one (dot, norm) pair per token, and the alive flags.  A wavefront prices whole tokens (tokens wave, wave + 16, ..),
// its lanes stride over the row 16 channels at a time; every wavefront then finds the winner for itself from the
// LDS array, so a pick costs two barriers.
constexpr int kGreedyThreads = 1024;
constexpr int kGreedyMaxTokens = 256;

__device__ __forceinline__ uint32_t bytes_even(uint32_t x) { return x & 0x00FF00FFu; }          // bytes 0, 2 -> 16-bit lanes
__device__ __forceinline__ uint32_t bytes_odd(uint32_t x) { return (x >> 8) & 0x00FF00FFu; }    // bytes 1, 3
__device__ __forceinline__ uint32_t pk_max_u16(uint32_t a, uint32_t b) {
    return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(ushort2v, a), __builtin_bit_cast(ushort2v, b)));
}
__device__ __forceinline__ uint32_t pk_min_u16(uint32_t a, uint32_t b) {
    return __builtin_bit_cast(uint32_t, __builtin_elementwise_min(__builtin_bit_cast(ushort2v, a), __builtin_bit_cast(ushort2v, b)));
}
// bit_length of a value below 256 held in byte `B` of x: the exponent of its float (frexp: 0 -> 0, 1 -> 1, 2..3 -> 2, ..)
template <int B>
__device__ __forceinline__ uint32_t byte_bit_length(uint32_t x) {
    return (uint32_t)__builtin_amdgcn_frexp_expf((float)((x >> (8 * B)) & 0xFFu));
}
// sum over the four bytes of bit_length(max(x, mx) - min(x, mn))
__device__ __forceinline__ uint32_t range_bits4(uint32_t x, uint32_t mn, uint32_t mx) {
    const uint32_t re = pk_max_u16(bytes_even(x), bytes_even(mx)) - pk_min_u16(bytes_even(x), bytes_even(mn));
    const uint32_t ro = pk_max_u16(bytes_odd(x), bytes_odd(mx)) - pk_min_u16(bytes_odd(x), bytes_odd(mn));
    return byte_bit_length<0>(re) + byte_bit_length<2>(re) + byte_bit_length<0>(ro) + byte_bit_length<2>(ro);
}
__device__ __forceinline__ uint32_t bytes_min4(uint32_t a, uint32_t b) {
    return pk_min_u16(bytes_even(a), bytes_even(b)) | (pk_min_u16(bytes_odd(a), bytes_odd(b)) << 8);
}
__device__ __forceinline__ uint32_t bytes_max4(uint32_t a, uint32_t b) {
    return pk_max_u16(bytes_even(a), bytes_even(b)) | (pk_max_u16(bytes_odd(a), bytes_odd(b)) << 8);
}
__device__ __forceinline__ uint32_t dot_bytes4(uint32_t a, uint32_t b) {      // sum of the four byte products
    return (a & 0xFFu) * (b & 0xFFu) + ((a >> 8) & 0xFFu) * ((b >> 8) & 0xFFu) + ((a >> 16) & 0xFFu) * ((b >> 16) & 0xFFu) +
           (a >> 24) * (b >> 24);
}
__device__ __forceinline__ unsigned long long wave_sum_u64(unsigned long long x) {
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) x += __shfl_xor(x, d, 64);
    return x;
}
// cos_a > cos_b for non-negative vectors with a common second operand: (dot, squared norm) pairs, exact
__device__ __forceinline__ bool cos_greater(unsigned long long dot_a, unsigned long long nx_a, unsigned long long dot_b,
                                            unsigned long long nx_b) {
    if (nx_a == 0) return false;                 // a is the zero vector: cosine 0, never above a non-negative cosine
    if (nx_b == 0) return dot_a > 0;
    const unsigned long long pa = dot_a * dot_a, pb = dot_b * dot_b;          // < 2^63 for rows of up to 2^16 bytes
    const unsigned long long lhs_hi = __umul64hi(pa, nx_b), lhs_lo = pa * nx_b;
    const unsigned long long rhs_hi = __umul64hi(pb, nx_a), rhs_lo = pb * nx_a;
    return lhs_hi > rhs_hi || (lhs_hi == rhs_hi && lhs_lo > rhs_lo);
}

__global__ void __launch_bounds__(kGreedyThreads) greedy_order_kernel(const uint8_t *__restrict__ k_codes,
                                                                      const uint8_t *__restrict__ v_codes, int hidden,
                                                                      int block_size, int pack_len,
                                                                      uint32_t *__restrict__ perm) {
    extern __shared__ __attribute__((aligned(16))) uint8_t g_lds[];
    const int D2 = 2 * hidden, n16 = D2 / 16, h16 = hidden / 16;
    uint4 *mn = reinterpret_cast<uint4 *>(g_lds), *mx = mn + n16;                 // [D2] bytes each
    unsigned long long *key_dot = reinterpret_cast<unsigned long long *>(mx + n16);   // [256]
    unsigned long long *key_nx = key_dot + kGreedyMaxTokens;                           // [256]
    uint32_t *cost = reinterpret_cast<uint32_t *>(key_nx + kGreedyMaxTokens);        // [2][256]
    uint8_t *alive = reinterpret_cast<uint8_t *>(cost + 2 * kGreedyMaxTokens);        // [256]

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int N = block_size;
    const size_t row0 = (size_t)blockIdx.x * N;
    // 16 channels `c16` of token `tok`: K half first, then V half
    auto row16 = [&](int tok, int c16) -> uint4 {
        const uint8_t *base = c16 < h16 ? k_codes + (row0 + tok) * (size_t)hidden + 16 * (size_t)c16
                                        : v_codes + (row0 + tok) * (size_t)hidden + 16 * (size_t)(c16 - h16);
        return *reinterpret_cast<const uint4 *>(base);
    };
    if (tid < kGreedyMaxTokens) alive[tid] = tid < N;
    __syncthreads();

    int n_alive = N, picked = 0, flip = 0;
    for (int pk = 0; pk < N / pack_len; pk++) {
        // ---- seed: rounded mean of the remaining tokens (into mx), then the best cosine ----
        for (int c16 = tid; c16 < n16; c16 += kGreedyThreads) {
            uint32_t sum[16];
#pragma unroll
            for (int i = 0; i < 16; i++) sum[i] = 0;
            for (int tok = 0; tok < N; tok++) {
                if (!alive[tok]) continue;
                const uint4 x = row16(tok, c16);
                const uint32_t w[4] = {x.x, x.y, x.z, x.w};
#pragma unroll
                for (int i = 0; i < 16; i++) sum[i] += (w[i >> 2] >> (8 * (i & 3))) & 0xFFu;
            }
            uint32_t m[4] = {0, 0, 0, 0};
#pragma unroll
            for (int i = 0; i < 16; i++)      // mean(dim=1).round(): fp32 quotient, round half to even
                m[i >> 2] |= (uint32_t)rintf((float)sum[i] / (float)n_alive) << (8 * (i & 3));
            mx[c16] = make_uint4(m[0], m[1], m[2], m[3]);
        }
        __syncthreads();
        for (int tok = wave; tok < N; tok += kGreedyThreads / 64) {
            if (!alive[tok]) continue;
            unsigned long long dot = 0, nx = 0;
            for (int c16 = lane; c16 < n16; c16 += 64) {
                const uint4 x = row16(tok, c16), m = mx[c16];
                dot += dot_bytes4(x.x, m.x) + dot_bytes4(x.y, m.y) + dot_bytes4(x.z, m.z) + dot_bytes4(x.w, m.w);
                nx += dot_bytes4(x.x, x.x) + dot_bytes4(x.y, x.y) + dot_bytes4(x.z, x.z) + dot_bytes4(x.w, x.w);
            }
            dot = wave_sum_u64(dot);
            nx = wave_sum_u64(nx);
            if (lane == 0) { key_dot[tok] = dot; key_nx[tok] = nx; }
        }
        __syncthreads();
        int sel = -1;
        {   // every wavefront finds the winner itself: lane-local scan in token order, then a reduction that
            // prefers the earlier token on equal cosines
            unsigned long long bd = 0, bn = 0;
            for (int tok = lane; tok < N; tok += 64) {
                if (!alive[tok]) continue;
                if (sel < 0 || cos_greater(key_dot[tok], key_nx[tok], bd, bn)) { sel = tok; bd = key_dot[tok]; bn = key_nx[tok]; }
            }
#pragma unroll
            for (int d = 32; d >= 1; d >>= 1) {
                const int os = __shfl_xor(sel, d, 64);
                const unsigned long long od = __shfl_xor(bd, d, 64), on = __shfl_xor(bn, d, 64);
                if (os >= 0 && (sel < 0 || cos_greater(od, on, bd, bn) || (!cos_greater(bd, bn, od, on) && os < sel))) {
                    sel = os; bd = od; bn = on;
                }
            }
        }
        __syncthreads();                          // everyone has read the mean and the alive flags
        for (int c16 = tid; c16 < n16; c16 += kGreedyThreads) {
            const uint4 x = row16(sel, c16);
            mn[c16] = x;
            mx[c16] = x;
        }
        if (tid == 0) { alive[sel] = 0; perm[row0 + picked] = (uint32_t)sel; }
        picked++;
        n_alive--;
        __syncthreads();

        // ---- the pack's other tokens: fewest bits after the pick ----
        for (int j = 1; j < pack_len; j++) {
            uint32_t *cst = cost + flip * kGreedyMaxTokens;
            flip ^= 1;
            for (int tok = wave; tok < N; tok += kGreedyThreads / 64) {
                if (!alive[tok]) continue;
                uint32_t bits = 0;
                for (int c16 = lane; c16 < n16; c16 += 64) {
                    const uint4 x = row16(tok, c16), lo = mn[c16], hi = mx[c16];
                    bits += range_bits4(x.x, lo.x, hi.x) + range_bits4(x.y, lo.y, hi.y) + range_bits4(x.z, lo.z, hi.z) +
                            range_bits4(x.w, lo.w, hi.w);
                }
                bits = wave_sum_u32(bits);
                if (lane == 0) cst[tok] = bits;
            }
            __syncthreads();
            uint32_t best = 0xFFFFFFFFu;           // (cost, token) in one word: the minimum is the first cheapest token
            for (int tok = lane; tok < N; tok += 64)
                if (alive[tok]) best = min(best, (cst[tok] << 8) | (uint32_t)tok);
#pragma unroll
            for (int d = 32; d >= 1; d >>= 1) best = min(best, (uint32_t)__shfl_xor(best, d, 64));
            sel = (int)(best & 0xFFu);
            __syncthreads();                      // everyone has read the alive flags
            for (int c16 = tid; c16 < n16; c16 += kGreedyThreads) {
                const uint4 x = row16(sel, c16), lo = mn[c16], hi = mx[c16];
                mn[c16] = make_uint4(bytes_min4(lo.x, x.x), bytes_min4(lo.y, x.y), bytes_min4(lo.z, x.z), bytes_min4(lo.w, x.w));
                mx[c16] = make_uint4(bytes_max4(hi.x, x.x), bytes_max4(hi.y, x.y), bytes_max4(hi.z, x.z), bytes_max4(hi.w, x.w));
            }
            if (tid == 0) { alive[sel] = 0; perm[row0 + picked] = (uint32_t)sel; }
            picked++;
            n_alive--;
            __syncthreads();
        }
    }
}

// ---- greedy order of blocks of up to 64 tokens: the block's rows stay in registers, sliced by channel ----
// A workgroup of 512 threads holds 4096 channels of all the tokens of a block (thread = 8 adjacent channels, one
// dword pair per token, in registers for the whole block), so a pick re-reads nothing from memory; rows of up to
// 2048 channels take workgroups of 256 threads, two per CU.  The workgroups that cover a block form a group: every step (a seed or a pick) each member
// sums its slice per token (every thread leaves its sums in LDS, eight threads per pair of tokens add them up),
// publishes the sums as (step number << 32 | value) words -- a pick: one word per pair of tokens, two 16-bit sums;
// a seed: dot product and squared norm per token -- reads the words of all members and finds the winner for itself.
// The words of two consecutive steps live in two buffers, and a member can be at most one step ahead of another, so
// a word is never overwritten before it was read.  Workgroups take tickets in the order they start and a group is a
// run of consecutive tickets: whenever a member waits, the members it waits for run already or start as soon as a
// complete group ahead of them leaves; the launch never holds more groups than fit the device.  The waits are
// bounded all the same (kGreedySpinLimit, error word of the state).
//
// The remaining tokens occupy register slots 0 .. n_alive - 1 (the winner's slot takes the rows of the last slot;
// lane l of every wavefront knows which token slot l holds), so a step walks a prefix of the slots without a test
// per token and two tokens are priced side by side.
//
// Pricing a token: min and max as packed 16-bit lanes, r = max - min, then bit_length(r) is the exponent of
// (2 r + 1) 2^-10 as a half: one packed fma on r read as a subnormal half (r 2^-24 * 2^15 + 2^-10, exact), the
// exponent fields masked and added by a sum of absolute differences -- 3.7 vector instructions per channel.  The
// constant bias of the exponent (5 per channel) is common to all tokens.  A step of a group of eight wide
// workgroups takes ~6.5 us on an MI355X: 3.8 us of pricing at the full rate of the vector ALUs, the rest the sums,
// the exchange, the winner and the slot move, which nothing overlaps.
constexpr int kSlicedThreadsWide = 512;                 // one workgroup per CU, two wavefronts per SIMD: rows of two or more slices
constexpr int kSlicedThreadsNarrow = 256;               // two workgroups per CU: rows of up to 2048 channels
constexpr int kSlicedTokens = 64;
constexpr int kGreedySpinLimit = 1 << 22;
// words per row of the per-thread sums: runs of 32 threads, each + 4, then + 4

typedef _Float16 half2v __attribute__((ext_vector_type(2)));

// Even / odd bytes of a dword as 16-bit lanes, with the mask and the byte selector as operands: the kernel below
// makes these two constants opaque once per step, so that nothing derived from the packed rows -- which stay in
// registers for a whole block -- is kept in registers of its own from step to step.
__device__ __forceinline__ uint32_t even_bytes(uint32_t x, uint32_t mask_00ff00ff) { return x & mask_00ff00ff; }
__device__ __forceinline__ uint32_t odd_bytes(uint32_t x, uint32_t sel_0c030c01) { return __builtin_amdgcn_perm(0u, x, sel_0c030c01); }

// Two tokens (a, b), 8 channels each: sums of the exponent fields, << 10.  Stage by stage over the eight independent
// chains, so that no instruction waits for the one before it.
__device__ __forceinline__ void price8x2(uint32_t x0a, uint32_t x1a, uint32_t x0b, uint32_t x1b, const uint32_t (&mn)[4],
                                         const uint32_t (&mx)[4], uint32_t k_even, uint32_t k_odd, uint32_t &sum_a, uint32_t &sum_b) {
    const uint32_t v[8] = {even_bytes(x0a, k_even), even_bytes(x0b, k_even), odd_bytes(x0a, k_odd), odd_bytes(x0b, k_odd),
                           even_bytes(x1a, k_even), even_bytes(x1b, k_even), odd_bytes(x1a, k_odd), odd_bytes(x1b, k_odd)};
    ushort2v hi[8], lo[8];
    uint32_t e[8];
#pragma unroll
    for (int i = 0; i < 8; i++) hi[i] = __builtin_elementwise_max(__builtin_bit_cast(ushort2v, v[i]), __builtin_bit_cast(ushort2v, mx[i >> 1]));
#pragma unroll
    for (int i = 0; i < 8; i++) lo[i] = __builtin_elementwise_min(__builtin_bit_cast(ushort2v, v[i]), __builtin_bit_cast(ushort2v, mn[i >> 1]));
#pragma unroll
    for (int i = 0; i < 8; i++) hi[i] -= lo[i];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const half2v f = __builtin_elementwise_fma(__builtin_bit_cast(half2v, hi[i]), (half2v){(_Float16)32768.0f, (_Float16)32768.0f},
                                                   (half2v){(_Float16)0.0009765625f, (_Float16)0.0009765625f});
        e[i] = __builtin_bit_cast(uint32_t, f);
    }
#pragma unroll
    for (int i = 0; i < 8; i++) e[i] &= 0x7C007C00u;
    sum_a = __builtin_amdgcn_sad_u16(e[0], 0u, 0u);
    sum_b = __builtin_amdgcn_sad_u16(e[1], 0u, 0u);
#pragma unroll
    for (int i = 1; i < 4; i++) {
        sum_a = __builtin_amdgcn_sad_u16(e[2 * i], 0u, sum_a);
        sum_b = __builtin_amdgcn_sad_u16(e[2 * i + 1], 0u, sum_b);
    }
}

// data-parallel-primitive moves between the lanes of a row of 16 (0x100 | n: from lane + n, 0x110 | n: from lane - n,
// 0x142 / 0x143: lane 15 / 31 to the following rows, below 0x100: a permutation of every four lanes)
template <int CTRL, int ROW_MASK, bool ZERO_FILL>
__device__ __forceinline__ uint32_t lane_move(uint32_t old, uint32_t src) {
    return (uint32_t)__builtin_amdgcn_update_dpp((int)old, (int)src, CTRL, ROW_MASK, 0xF, ZERO_FILL);
}
__device__ __forceinline__ uint32_t wave_min_u32(uint32_t v) {      // the minimum over the wavefront, uniform
    v = min(v, lane_move<0x111, 0xF, false>(0xFFFFFFFFu, v));
    v = min(v, lane_move<0x112, 0xF, false>(0xFFFFFFFFu, v));
    v = min(v, lane_move<0x114, 0xF, false>(0xFFFFFFFFu, v));
    v = min(v, lane_move<0x118, 0xF, false>(0xFFFFFFFFu, v));
    v = min(v, lane_move<0x142, 0xA, false>(0xFFFFFFFFu, v));
    v = min(v, lane_move<0x143, 0xC, false>(0xFFFFFFFFu, v));
    return (uint32_t)__builtin_amdgcn_readlane((int)v, 63);
}
__device__ __forceinline__ uint32_t quad_sum(uint32_t v) {          // every lane: the sum over its four lanes
    v += lane_move<0xB1, 0xF, false>(0u, v);
    return v + lane_move<0x4E, 0xF, false>(0u, v);
}
__device__ __forceinline__ uint32_t sum8_down(uint32_t v) {         // lanes 0, 8, ..: the sum over lanes l .. l + 7
    v += lane_move<0x101, 0xF, true>(0u, v);
    v += lane_move<0x102, 0xF, true>(0u, v);
    return v + lane_move<0x104, 0xF, true>(0u, v);
}

// Word `idx` of the 128 published words of the members first, first + stride, ..: up to four loads in flight, all of
// them repeated until every word carries the step number.  `take(w)` gets the low halves.
template <typename F>
__device__ __forceinline__ void gather_words(const uint64_t *words, uint32_t idx, uint32_t first, uint32_t stride, uint32_t members,
                                             uint32_t seq, ScanState *st, F &&take) {
    for (uint32_t m0 = first; m0 < members; m0 += 4 * stride) {
        const uint64_t *p = words + (size_t)m0 * 128 + idx;
        const bool on1 = m0 + stride < members, on2 = m0 + 2 * stride < members, on3 = m0 + 3 * stride < members;
        const uint64_t *p1 = on1 ? p + (size_t)stride * 128 : p, *p2 = on2 ? p + (size_t)2 * stride * 128 : p,
                       *p3 = on3 ? p + (size_t)3 * stride * 128 : p;
        uint64_t w0, w1, w2, w3;
        int spins = 0;
        do {
            w0 = __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            w1 = __hip_atomic_load(p1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            w2 = __hip_atomic_load(p2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            w3 = __hip_atomic_load(p3, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        } while (((uint32_t)(w0 >> 32) != seq || (uint32_t)(w1 >> 32) != seq || (uint32_t)(w2 >> 32) != seq ||
                  (uint32_t)(w3 >> 32) != seq) && ++spins < kGreedySpinLimit);
        if (spins >= kGreedySpinLimit) st->error = (uint32_t)PKV_ERR_INTERNAL;
        take((uint32_t)w0);
        if (on1) take((uint32_t)w1);
        if (on2) take((uint32_t)w2);
        if (on3) take((uint32_t)w3);
    }
}

// The rows of a thread: 64 slots as two vectors of 32 registers, which the slot move indexes with a uniform run-time
// index (register-indexed moves); every other access is by constant.
typedef uint32_t u32x32 __attribute__((ext_vector_type(32)));

template <int THREADS>
__global__ void __launch_bounds__(THREADS, 2)
greedy_order_sliced_kernel(const uint8_t *__restrict__ k_codes, const uint8_t *__restrict__ v_codes, int hidden, int N,
                           int pack_len, uint32_t nblocks, uint32_t members, uint32_t groups,
                           uint32_t *__restrict__ perm, ScanState *st) {
    constexpr int kRuns = THREADS / 32, kPartStride = kRuns * 36 + 4, kSeedParts = THREADS / 128;
    __shared__ __attribute__((aligned(16))) uint32_t s_part[32 * kPartStride];   // picks: [pair of slots][thread], padded
    __shared__ uint32_t s_seed[128 * 32];            // seeds: [2 * slot + (0: dot, 1: squared norm)][adder]
    __shared__ uint32_t s_tot[kRuns][64];            // picks: sums over the members q, q + kRuns, ..
    __shared__ unsigned long long s_tot64[kSeedParts][128];   // seeds: sums over the members q, q + kSeedParts, ..
    __shared__ uint32_t s_ticket;
    const int tid = threadIdx.x, lane = tid & 63;
    if (tid == 0) s_ticket = atomicAdd(&st->ticket, 1u);
    __syncthreads();
    const uint32_t ticket = s_ticket;
    const uint32_t grp = ticket / members, mem = ticket - grp * members;
    if (grp >= groups) return;
    uint64_t *xw = st->status + (size_t)grp * 2 * members * 128;      // [buffer][member][128]
    const int D2 = 2 * hidden;
    const int ch = ((int)mem * THREADS + tid) * 8;                    // first of the thread's 8 channels
    const uint8_t *col = ch < hidden ? k_codes + ch : v_codes + (ch - hidden);
    const bool have = ch < D2;
    const int adder = (tid >> 2) & 31;               // the LDS word that takes the sums of the thread's four lanes
    const bool quad_first = (tid & 3) == 0;
    uint32_t seq = 0;
    int flip = 0;
    // a thread's word in a row of s_part and, as a reader, where the 32 words it adds start: rows and runs of 32 are
    // padded so that the 16-byte reads of a wavefront spread over all banks
    const int part_word = (tid >> 5) * 36 + (tid & 31), part_read = (tid / kRuns) * kPartStride + (tid % kRuns) * 36;

    for (uint32_t blk = grp; blk < nblocks; blk += groups) {
        const size_t row0 = (size_t)blk * N;
        u32x32 x0v[2], x1v[2];
#define x0(t) x0v[(t) >> 5][(t) & 31]
#define x1(t) x1v[(t) >> 5][(t) & 31]
#pragma unroll
        for (int t = 0; t < kSlicedTokens; t++) {
            uint2 v = make_uint2(0u, 0u);
            if (t < N && have) v = *reinterpret_cast<const uint2 *>(col + (row0 + t) * (size_t)hidden);
            x0(t) = v.x;
            x1(t) = v.y;
        }
        uint32_t orig = (uint32_t)lane;          // the token in slot `lane`
        int n_alive = N, picked = 0;
        uint32_t mn[4], mx[4];       // even / odd bytes of dword 0, even / odd bytes of dword 1, as 16-bit lanes

        for (int step = 0; step < N / pack_len * pack_len; step++) {
            const bool seed = step % pack_len == 0;
            int sel = -1;
            uint32_t k_even = 0x00FF00FFu, k_odd = 0x0C030C01u, k_zero = 0u;     // opaque from here on: see even_bytes
            asm volatile("" : "+s"(k_even), "+s"(k_odd), "+v"(k_zero));
            if (seed) {
            // ---- seed: rounded mean of the remaining tokens, then the best cosine ----
            uint32_t sum[4] = {0u, 0u, 0u, 0u};
#pragma unroll
            for (int t8 = 0; t8 < kSlicedTokens; t8 += 8) {
                if (t8 < n_alive) {
#pragma unroll
                    for (int t = t8; t < t8 + 8; t++)
                        if (t < n_alive) {
                            sum[0] += even_bytes(x0(t), k_even); sum[1] += odd_bytes(x0(t), k_odd);
                            sum[2] += even_bytes(x1(t), k_even); sum[3] += odd_bytes(x1(t), k_odd);
                        }
                }
            }
            uint32_t mean[2];
#pragma unroll
            for (int d = 0; d < 2; d++) {      // mean(dim=1).round(): fp32 quotient, round half to even
                const float na = (float)n_alive;
                const uint32_t e_lo = (uint32_t)rintf((float)(sum[2 * d] & 0xFFFFu) / na), e_hi = (uint32_t)rintf((float)(sum[2 * d] >> 16) / na);
                const uint32_t o_lo = (uint32_t)rintf((float)(sum[2 * d + 1] & 0xFFFFu) / na), o_hi = (uint32_t)rintf((float)(sum[2 * d + 1] >> 16) / na);
                mean[d] = e_lo | (o_lo << 8) | (e_hi << 16) | (o_hi << 24);
            }
            for (int i = tid; i < 128 * 32; i += THREADS) s_seed[i] = 0u;
            __syncthreads();
#pragma unroll
            for (int t8 = 0; t8 < kSlicedTokens; t8 += 8) {
                if (t8 < n_alive) {
#pragma unroll
                    for (int t = t8; t < t8 + 8; t++)
                        if (t < n_alive) {
                            const uint32_t dot = quad_sum(__builtin_amdgcn_udot4(x0(t), mean[0], __builtin_amdgcn_udot4(x1(t), mean[1], 0u, false), false));
                            const uint32_t nx = quad_sum(__builtin_amdgcn_udot4(x0(t), x0(t), __builtin_amdgcn_udot4(x1(t), x1(t), k_zero, false), false));
                            if (quad_first) {
                                atomicAdd(&s_seed[(2 * t) * 32 + adder], dot);
                                atomicAdd(&s_seed[(2 * t + 1) * 32 + adder], nx);
                            }
                        }
                }
            }
            __syncthreads();
            seq++;
            {   // value v: two or four adjacent threads add 16 or 8 adders each
                const int v = tid / kSeedParts, part = tid % kSeedParts;
                uint32_t a = 0u;
#pragma unroll
                for (int i = 0; i < 32 / kSeedParts; i++) a += s_seed[v * 32 + part * (32 / kSeedParts) + i];
                a += lane_move<0xB1, 0xF, false>(0u, a);
                if (kSeedParts == 4) a += lane_move<0x4E, 0xF, false>(0u, a);
                if (part == 0 && v < 2 * n_alive) {
                    if (members > 1)
                        __hip_atomic_store(xw + ((size_t)flip * members + mem) * 128 + v, ((uint64_t)seq << 32) | a,
                                           __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    else
                        s_tot64[0][v] = a;
                }
            }
            if (members > 1) {
                const int v = tid & 127, q = tid >> 7;
                unsigned long long a = 0ull;
                if (v < 2 * n_alive)
                    gather_words(xw + (size_t)flip * members * 128, (uint32_t)v, (uint32_t)q, (uint32_t)kSeedParts, members, seq, st,
                                 [&](uint32_t w) { a += w; });
                s_tot64[q][v] = a;
                flip ^= 1;
            }
            __syncthreads();
            {
                unsigned long long bd = 0, bn = 0;
                uint32_t bo = orig;
                if (lane < n_alive) {
                    sel = lane;
                    bd = s_tot64[0][2 * lane];
                    bn = s_tot64[0][2 * lane + 1];
                    if (members > 1) {
#pragma unroll
                        for (int q = 1; q < kSeedParts; q++) { bd += s_tot64[q][2 * lane]; bn += s_tot64[q][2 * lane + 1]; }
                    }
                }
#pragma unroll
                for (int d = 32; d >= 1; d >>= 1) {      // equal cosines: the earlier token
                    const int os = __shfl_xor(sel, d, 64);
                    const uint32_t oo = __shfl_xor(bo, d, 64);
                    const unsigned long long od = __shfl_xor(bd, d, 64), on = __shfl_xor(bn, d, 64);
                    if (os >= 0 && (sel < 0 || cos_greater(od, on, bd, bn) || (!cos_greater(bd, bn, od, on) && oo < bo))) {
                        sel = os; bo = oo; bd = od; bn = on;
                    }
                }
                sel = __builtin_amdgcn_readfirstlane(sel);
            }
            } else {
            // ---- the pack's other tokens: fewest bits after the pick ----
#pragma unroll
                for (int k4 = 0; k4 < kSlicedTokens / 2; k4 += 4) {
                    if (2 * k4 < n_alive) {
#pragma unroll
                        for (int k = k4; k < k4 + 4; k++)
                            if (2 * k < n_alive) {
                                // (with an odd count the slot past the last one is priced as well: a bounded sum nobody reads)
                                uint32_t a0, a1;
                                price8x2(x0(2 * k), x1(2 * k), x0(2 * k + 1), x1(2 * k + 1), mn, mx, k_even, k_odd, a0, a1);
                                s_part[k * kPartStride + part_word] = (a0 >> 10) | (a1 << 6);   // sums of fields at bit 10: a 16-bit lane per slot
                            }
                    }
                }
                __syncthreads();
                seq++;
                {   // pair k: kRuns adjacent threads add 32 words each
                    const int k = tid / kRuns, part = tid % kRuns;
                    const uint4 *src = reinterpret_cast<const uint4 *>(s_part + part_read);
                    uint32_t a = 0u;
#pragma unroll
                    for (int i = 0; i < 8; i++) {
                        const uint4 w = src[i];
                        a += w.x + w.y + w.z + w.w;
                    }
                    a = sum8_down(a);
                    if (kRuns == 16) a += lane_move<0x108, 0xF, true>(0u, a);
                    if (part == 0 && 2 * k < n_alive) {
                        if (members > 1) {      // both slots of the pair in one word
                            __hip_atomic_store(xw + ((size_t)flip * members + mem) * 128 + k, ((uint64_t)seq << 32) | a, __ATOMIC_RELAXED,
                                               __HIP_MEMORY_SCOPE_AGENT);
                        } else {
                            s_tot[0][2 * k] = a & 0xFFFFu;
                            s_tot[0][2 * k + 1] = a >> 16;
                        }
                    }
                }
                if (members > 1) {       // pair k = tid & 31 of the members q, q + kRuns, ..
                    const int k = tid & 31, q = tid >> 5;
                    uint32_t a_lo = 0u, a_hi = 0u;
                    if (2 * k < n_alive)
                        gather_words(xw + (size_t)flip * members * 128, (uint32_t)k, (uint32_t)q, (uint32_t)kRuns, members, seq, st,
                                     [&](uint32_t w) { a_lo += w & 0xFFFFu; a_hi += w >> 16; });
                    s_tot[q][2 * k] = a_lo;
                    s_tot[q][2 * k + 1] = a_hi;
                    flip ^= 1;
                }
                __syncthreads();
                uint32_t key = 0xFFFFFFFFu;            // (cost, token) in one word: the minimum is the first cheapest token
                if (lane < n_alive) {
                    uint32_t a = s_tot[0][lane];
                    if (members > 1) {
#pragma unroll
                        for (int q = 1; q < kRuns; q++) a += s_tot[q][lane];
                    }
                    key = (a << 8) | orig;
                }
                const uint32_t best = wave_min_u32(key);
                sel = (int)__builtin_ctzll(__ballot(key == best));
            }
            // the winner in slot `sel` leaves: its rows widen the pack's ranges and the last slot moves into `sel`
            const int last = n_alive - 1;
            const uint32_t tok = (uint32_t)__builtin_amdgcn_readlane((int)orig, sel);
            const uint32_t moved = (uint32_t)__builtin_amdgcn_readlane((int)orig, last);
            if (lane == sel) orig = moved;
            // (both halves of the slot arrays are read and written at the index modulo 32, with what they hold unless
            // the slot lies in them: no branch, so the arrays stay where they are)
            const int li = last & 31, si = sel & 31;
            const uint32_t la0 = x0v[0][li], la1 = x1v[0][li], lb0 = x0v[1][li], lb1 = x1v[1][li];
            const uint32_t l0 = last < 32 ? la0 : lb0, l1 = last < 32 ? la1 : lb1;
            const uint32_t sa0 = x0v[0][si], sa1 = x1v[0][si], sb0 = x0v[1][si], sb1 = x1v[1][si];
            const uint32_t w0 = sel < 32 ? sa0 : sb0, w1 = sel < 32 ? sa1 : sb1;
            x0v[0][si] = sel < 32 ? l0 : sa0;
            x1v[0][si] = sel < 32 ? l1 : sa1;
            x0v[1][si] = sel < 32 ? sb0 : l0;
            x1v[1][si] = sel < 32 ? sb1 : l1;
            if (mem == 0 && tid == 0) perm[row0 + picked] = tok;
            picked++;
            n_alive--;
            if (seed) {
                mn[0] = mx[0] = even_bytes(w0, k_even); mn[1] = mx[1] = odd_bytes(w0, k_odd);
                mn[2] = mx[2] = even_bytes(w1, k_even); mn[3] = mx[3] = odd_bytes(w1, k_odd);
            } else {
                mn[0] = pk_min_u16(mn[0], even_bytes(w0, k_even)); mx[0] = pk_max_u16(mx[0], even_bytes(w0, k_even));
                mn[1] = pk_min_u16(mn[1], odd_bytes(w0, k_odd)); mx[1] = pk_max_u16(mx[1], odd_bytes(w0, k_odd));
                mn[2] = pk_min_u16(mn[2], even_bytes(w1, k_even)); mx[2] = pk_max_u16(mx[2], even_bytes(w1, k_even));
                mn[3] = pk_min_u16(mn[3], odd_bytes(w1, k_odd)); mx[3] = pk_max_u16(mx[3], odd_bytes(w1, k_odd));
            }
        }
    }
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

// 256 threads per workgroup, a grid-stride walk over the items (pack, 16 adjacent channels), the channel chunk
// running fastest so that a wavefront reads whole rows; four rows in flight per thread; minima and maxima as packed
// 16-bit lanes (even and odd bytes of every dword apart).  One atomic per workgroup: same-address atomics retire
// one after the other, so their number, not the bytes, would set the time of a grid with a workgroup per pack.
// Bound by instruction issue: 7 vector instructions per dword for the ranges and 8 for the presence flags (a
// register bit mask for values below 32 instead of the LDS flags costs the same).
typedef unsigned short pk_u16x2 __attribute__((ext_vector_type(2)));

__global__ void __launch_bounds__(256) pack_size_kernel(const uint8_t *__restrict__ codes, int hidden, int pack_len,
                                                        size_t n_items, PackSizeOut *out) {
    // a presence word per (code value, lane % 32): a lane marks its own column, so the marks of a wavefront never
    // share a bank however few values the matrix holds (one word per value made every mark a same-address conflict)
    __shared__ uint32_t seen[256 * 32];
    __shared__ unsigned long long wsum[4];
    for (int i = threadIdx.x; i < 256 * 32; i += 256) seen[i] = 0u;
    __syncthreads();
    uint32_t *col = seen + (threadIdx.x & 31);
    const uint32_t chunks = (uint32_t)hidden / 16u;
    unsigned long long lens = 0;
    for (size_t item = (size_t)blockIdx.x * 256 + threadIdx.x; item < n_items; item += (size_t)gridDim.x * 256) {
        const size_t pack = item / chunks;
        const uint32_t chunk = (uint32_t)(item - pack * chunks);
        const uint8_t *p = codes + pack * (size_t)pack_len * hidden + (size_t)chunk * 16;
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
                col[32u * e[0]] = 1u;
                col[32u * e[1]] = 1u;
                col[32u * o[0]] = 1u;
                col[32u * o[1]] = 1u;
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
        uint32_t l = 0;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const pk_u16x2 r = mx[i] - mn[i];
#pragma unroll
            for (int hlf = 0; hlf < 2; hlf++)
                l += r[hlf] ? 32u - (uint32_t)__builtin_clz((uint32_t)r[hlf]) : 0u;   // bit_length = ceil(log2(range + 1))
        }
        lens += l;
    }
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) lens += __shfl_xor(lens, d, 64);
    if ((threadIdx.x & 63) == 0) wsum[threadIdx.x >> 6] = lens;
    __syncthreads();
    if (threadIdx.x == 0) atomicAdd(&out->len_sum, wsum[0] + wsum[1] + wsum[2] + wsum[3]);
    {   // value threadIdx.x: any of its 32 columns (read rotated, so that the threads of a wavefront spread over the banks)
        uint32_t any = 0u;
#pragma unroll 8
        for (int c = 0; c < 32; c++) any |= seen[32 * threadIdx.x + ((c + threadIdx.x) & 31)];
        if (any) out->present[threadIdx.x] = 1u;
    }
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
    void *scratch = nullptr;
    int rc = scratch_get(sizeof(PackSizeOut), s, &scratch);
    if (rc) return rc;
    PackSizeOut *out = static_cast<PackSizeOut *>(scratch);
    LaunchTimer tm(s, ms_out != nullptr);
    if ((rc = tm.begin())) return rc;
    pack_size_zero_kernel<<<1, 256, 0, s>>>(out);
    const size_t n_items = (size_t)(ctx_len / pack_len) * (size_t)(hidden_dim / 16);
    const size_t wanted = (n_items + 255) / 256;
    pack_size_kernel<<<(unsigned)(wanted < 2048 ? wanted : 2048), 256, 0, s>>>(codes, hidden_dim, pack_len, n_items, out);
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
    int rc = scratch_get((size_t)ctx_len, s, &scratch);
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

int pkv_greedy_repack(const uint8_t *k_codes, const uint8_t *v_codes, uint8_t *k_out, uint8_t *v_out, uint32_t *perm,
                      int ctx_len, int hidden_dim, int block_size, int pack_len, float *ms_out, pkv_stream_t s_) {
    using namespace pkv;
    hipStream_t s = (hipStream_t)s_;
    PKV_REQUIRE(k_codes && v_codes && perm && (k_out != nullptr) == (v_out != nullptr), PKV_ERR_INVALID, "null pointer argument");
    PKV_REQUIRE(k_codes != k_out && v_codes != v_out, PKV_ERR_INVALID, "repacking cannot run in place");
    const bool rows = k_out != nullptr;               // without outputs: the order only
    PKV_REQUIRE(ctx_len > 0 && hidden_dim > 0 && block_size > 0 && pack_len > 0, PKV_ERR_INVALID, "sizes must be positive");
    PKV_REQUIRE(hidden_dim % 16 == 0 && ((reinterpret_cast<uintptr_t>(k_codes) | reinterpret_cast<uintptr_t>(v_codes) |
                                          reinterpret_cast<uintptr_t>(k_out) | reinterpret_cast<uintptr_t>(v_out)) & 15u) == 0,
                PKV_ERR_INVALID, "hidden_dim must be a multiple of 16 and the code matrices 16-byte aligned");
    PKV_REQUIRE(block_size <= kGreedyMaxTokens && ctx_len % block_size == 0, PKV_ERR_INVALID,
                "ctx_len must be divisible by a block size of at most 256 tokens");
    PKV_REQUIRE(block_size % pack_len == 0, PKV_ERR_INVALID,
                "block_size must be a multiple of pack_len (the reference drops the tokens of an incomplete pack)");
    const uint32_t nblocks = (uint32_t)(ctx_len / block_size);
    // blocks of up to 64 tokens: register-resident channel slices, as many groups of workgroups as fit the device;
    // rows of more than one narrow slice go to the wide workgroups, which have a CU to themselves: two members of a
    // group on one CU, or another group's member in the same phase, would price at half speed and hold up their group
    const bool wide = 2 * (size_t)hidden_dim > 8u * kSlicedThreadsNarrow;
    const uint32_t slice = 8u * (wide ? kSlicedThreadsWide : kSlicedThreadsNarrow);
    uint32_t members = (uint32_t)((2 * (size_t)hidden_dim + slice - 1) / slice), groups = 0;
    if (block_size <= kSlicedTokens) {
        int dev = 0;
        PKV_HIP_CHECK(hipGetDevice(&dev));
        static std::mutex mu;
        static std::map<std::pair<int, bool>, uint32_t> resident;      // workgroups of the sliced kernel that fit the device at once
        std::lock_guard<std::mutex> lock(mu);
        auto it = resident.find({dev, wide});
        if (it == resident.end()) {
            int cus = 0, per_cu = 0;
            PKV_HIP_CHECK(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
            if (wide)
                PKV_HIP_CHECK(hipOccupancyMaxActiveBlocksPerMultiprocessor(
                    &per_cu, reinterpret_cast<const void *>(greedy_order_sliced_kernel<kSlicedThreadsWide>), kSlicedThreadsWide, 0));
            else
                PKV_HIP_CHECK(hipOccupancyMaxActiveBlocksPerMultiprocessor(
                    &per_cu, reinterpret_cast<const void *>(greedy_order_sliced_kernel<kSlicedThreadsNarrow>), kSlicedThreadsNarrow, 0));
            it = resident.emplace(std::make_pair(dev, wide), (uint32_t)(cus > 0 && per_cu > 0 ? cus * per_cu : 0)).first;
        }
        groups = it->second / members;
        if (groups > nblocks) groups = nblocks;
    }
    int rc;
    if (groups > 0) {
        ScanState *st = nullptr;
        if ((rc = prepare_scan_state(groups * 2u * members * 128u, &st, s))) return rc;
        LaunchTimer tm(s, ms_out != nullptr);
        if ((rc = tm.begin())) return rc;
        if (wide)
            greedy_order_sliced_kernel<kSlicedThreadsWide><<<groups * members, kSlicedThreadsWide, 0, s>>>(
                k_codes, v_codes, hidden_dim, block_size, pack_len, nblocks, members, groups, perm, st);
        else
            greedy_order_sliced_kernel<kSlicedThreadsNarrow><<<groups * members, kSlicedThreadsNarrow, 0, s>>>(
                k_codes, v_codes, hidden_dim, block_size, pack_len, nblocks, members, groups, perm, st);
        if (rows) gather_rows_kernel<<<(unsigned)ctx_len, 256, 0, s>>>(k_codes, v_codes, k_out, v_out, perm, block_size, hidden_dim);
        PKV_HIP_CHECK(hipGetLastError());
        if ((rc = tm.end(ms_out))) return rc;
        if (ms_out) {                                  // a timed call has waited for the kernels: look at the error word
            uint32_t head[2] = {0u, 0u};
            PKV_HIP_CHECK(hipMemcpyAsync(head, st, sizeof(head), hipMemcpyDeviceToHost, s));
            PKV_HIP_CHECK(hipStreamSynchronize(s));
            PKV_REQUIRE(head[1] == 0u, PKV_ERR_INTERNAL, "greedy order: a workgroup waited too long for the sums of its group");
        }
        return PKV_OK;
    }
    // longer blocks: the cost word holds (bits << 8 | token): bits <= 8 * 2 * hidden_dim must stay below 2^24
    const size_t lds = 4 * (size_t)hidden_dim + kGreedyMaxTokens * (8 + 8 + 8 + 1);
    PKV_REQUIRE(hidden_dim <= 32768 && lds <= 160 * 1024, PKV_ERR_UNSUPPORTED,
                "not supported: the greedy order of blocks of more than 64 tokens keeps 4 * hidden_dim bytes in LDS (hidden_dim <= 32768)");
    if (lds > 48 * 1024)
        PKV_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(greedy_order_kernel),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    LaunchTimer tm(s, ms_out != nullptr);
    if ((rc = tm.begin())) return rc;
    greedy_order_kernel<<<nblocks, kGreedyThreads, lds, s>>>(k_codes, v_codes, hidden_dim, block_size, pack_len, perm);
    if (rows) gather_rows_kernel<<<(unsigned)ctx_len, 256, 0, s>>>(k_codes, v_codes, k_out, v_out, perm, block_size, hidden_dim);
    PKV_HIP_CHECK(hipGetLastError());
    return tm.end(ms_out);
}

}  // extern "C"
