// Fused decompress-attention decode: one query token per sequence attends over a compressed
// K/V cache (plus an optional 16-bit tail window) without materialising K or V.
//
// Fuses the reference's chain  kq_mat_vec_mul -> fused_kq -> softmax -> w * v_scale ->
// wv_mat_vec_mul -> fused_wv  (packkv_cuda_ext/src/kernels.cu:426-535, :632-765,
// src/fused_kernels.cu:13-76, :187-261, models/llama.py:202-209,
// evaluation/evaluation.py:661) and adds batch and GQA-group dimensions.
//
// Work decomposition (flash-decoding): grid (split, kv_head, batch).  A workgroup walks
// 128-token super-tiles = 2 K blocks (64 x 128) + 2 V blocks (128 x 64) of its head and keeps
// an online-softmax state; each split writes (m, l, acc[128]) per query head, a small merge
// kernel combines the splits and the tail window.
#include "pkv_block.hpp"
#include "pkv_runtime.hpp"

#include <mutex>

#ifndef PKV_DYNAMIC_TILES
#define PKV_DYNAMIC_TILES 1
#endif
#ifndef PKV_SPLIT_TARGET
#define PKV_SPLIT_TARGET 1024
#endif

namespace pkv {

constexpr int kTile = 128;              // tokens per super-tile
constexpr int kPartStride = 2 + kHeadDim;  // floats per partial: m, l, acc[128]
typedef float float2v __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float a_ld16(const uint16_t *p, size_t i, int dtype) {
    const uint32_t u = p[i];
    return dtype == PKV_F16 ? __half2float(__ushort_as_half((unsigned short)u)) : __uint_as_float(u << 16);
}

__device__ __forceinline__ uint16_t a_st16(float x, int dtype) {
    if (dtype == PKV_F16) return __half_as_ushort(__float2half_rn(x));
    uint32_t u = __float_as_uint(x);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x40u);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

struct AttnParams {
    const uint8_t *k_stream;
    const uint32_t *k_info;
    const uint8_t *v_stream;
    const uint32_t *v_info;
    const uint16_t *k_scale, *k_zero, *v_scale, *v_zero;
    const uint16_t *q;
    const uint16_t *k_win, *v_win;
    float *part;          // [B, Hq, nparts, kPartStride]
    uint16_t *out;        // [B, Hq, 128]: written directly by the attention kernel when there is a single partial
    int B, Hq, Hkv, T_c, T_w;
    int Gq;               // query heads per KV head; the kernels are built for the next of 1, 2, 4, 8 and leave the rest idle
    int par_stride;       // tokens per sequence row of the scale / zero arrays (>= T_c)
    int win_stride;       // tokens per (sequence, KV head) row of k_win / v_win (>= T_w)
    int k_bits, v_bits, dtype;
    float sm_scale;
    int tiles_per_split, nsplit, nparts;
    int win_piece;        // > 0: split i of the compressed part also takes window tokens [i * win_piece, ...) and
                          // writes partial nsplit + i; 0: the window has a kernel of its own (partial nparts - 1)
    uint32_t k_cap, v_cap, blk_stride;
    uint32_t k_bytes, v_bytes;   // valid bytes of the streams
    int out_f32;          // `out` holds fp32 instead of the 16-bit storage type
    int direct_out;       // a single partial and a 16-bit result: the async-copy kernel writes `out` itself
    int dynamic;          // async-copy kernel: the members of a (sequence, KV head) take tiles from a common counter
    int batch_shift;      // ... in batches of (tiles left >> batch_shift), at least 1 and at most 4
    uint32_t *counters;   // [B Hkv] tile counters, then [B Hkv] counts of members that are done; zero between launches
};

// x rounded to the 16-bit storage type (nearest even), as fp32.
__device__ __forceinline__ float round16(float x, int dtype) {
    const uint32_t u = a_st16(x, dtype);
    return dtype == PKV_F16 ? __half2float(__ushort_as_half((unsigned short)u)) : __uint_as_float(u << 16);
}

// ---- variant 1: decode tiles into LDS, then plain VALU attention --------------------------
// Straightforward and easy to audit; kept as the cross-check for the tuned kernel.
// REF: decompress-then-attend to the letter -- every element is formed as the reference stores it,
// T(T(code + zero) * scale) (utils/compute.py:178), and the dot products run on those values.
template <int G, bool REF>
__global__ void __launch_bounds__(256) attn_tiles_kernel(const AttnParams p) {
    extern __shared__ __align__(16) uint8_t lds[];
    uint8_t *ktile = lds;                                   // [128 tok][128 ch]
    uint8_t *vtile = ktile + kTile * kHeadDim;              // [128 tok][128 ch]
    uint8_t *blkbuf = vtile + kTile * kHeadDim;             // 4 x blk_stride
    float *fl = reinterpret_cast<float *>(blkbuf + 4 * p.blk_stride);
    float *qf = fl;                       // [G][128]
    float *S = qf + G * kHeadDim;         // [G][128]
    float *P = S + G * kTile;             // [G][128]
    float *ks = P + G * kTile;            // [128] x4
    float *kz = ks + kTile, *vs = kz + kTile, *vz = vs + kTile;
    float *st_m = vz + kTile;             // [G] each
    float *st_l = st_m + G, *st_a = st_l + G, *st_z = st_a + G, *qsum = st_z + G;
    __shared__ uint32_t s_phase[4], s_off[4];

    const int split = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const int tid = threadIdx.x;
    const int lane32 = tid & 31, hw = tid >> 5;
    const int bh = b * p.Hkv + h;
    const int n_hid_k = p.B * p.Hkv, n_hid_v = 2 * p.B * p.Hkv;
    const UnitGeom gk = unit_geom(p.k_bits), gv = unit_geom(p.v_bits);

    for (int i = tid; i < G * kHeadDim; i += 256)
        qf[i] = i < p.Gq * kHeadDim ? a_ld16(p.q, ((size_t)b * p.Hq + (size_t)h * p.Gq) * kHeadDim + i, p.dtype) : 0.f;
    if (tid < G) { st_m[tid] = -INFINITY; st_l[tid] = 0.f; st_z[tid] = 0.f; }
    __syncthreads();
    if (tid < G) {
        float s = 0.f;
        for (int d = 0; d < kHeadDim; d++) s += qf[tid * kHeadDim + d];
        qsum[tid] = s;
    }
    float acc[G];
#pragma unroll
    for (int g = 0; g < G; g++) acc[g] = 0.f;

    const int n_tiles = p.T_c / kTile;
    const int tile0 = split * p.tiles_per_split;
    const int tile1 = min(n_tiles, tile0 + p.tiles_per_split);
    for (int tau = tile0; tau < tile1; tau++) {
        // 1. stage the four blocks and the per-token quantizer parameters
        for (int j = 0; j < 4; j++) {
            const bool is_k = j < 2;
            const uint32_t bidx = is_k ? (uint32_t)((2 * tau + j) * n_hid_k + bh)
                                       : (uint32_t)(tau * n_hid_v + 2 * bh + (j - 2));
            const uint32_t *info = is_k ? p.k_info : p.v_info;
            const uint8_t *stream = is_k ? p.k_stream : p.v_stream;
            uint32_t off, size;
            block_span(info, bidx, is_k ? p.k_cap : p.v_cap, is_k ? p.k_bytes : p.v_bytes, off, size);
            const uint32_t ph = stage_to_lds(stream + off, size, blkbuf + j * p.blk_stride, tid, 256);
            if (tid == 0) s_phase[j] = ph;
        }
        if (tid < kTile) {
            const size_t ti = (size_t)b * p.par_stride + (size_t)tau * kTile + tid;
            ks[tid] = a_ld16(p.k_scale, ti, p.dtype);
            kz[tid] = a_ld16(p.k_zero, ti, p.dtype);
            vs[tid] = a_ld16(p.v_scale, ti, p.dtype);
            vz[tid] = a_ld16(p.v_zero, ti, p.dtype);
        }
        __syncthreads();
        // 2. unpack: half-wave hw handles K unit (block hw/4, round hw%4) and V unit
        //    (block hw/4 = channel half, segment hw%4)
        {
            const int j = hw >> 2, unit = hw & 3;
            const uint8_t *kb = blkbuf + j * p.blk_stride;
            const uint32_t kph = s_phase[j];
            const uint16_t *kcum = reinterpret_cast<const uint16_t *>(kb + kph);
            const uint32_t kstart = kph + 8u + (unit ? (uint32_t)kcum[unit - 1] : 0u);
            unit_decode<true>(kb, kstart, unit, lane32, gk, ktile + j * 64 * kHeadDim, kHeadDim);
            const uint8_t *vb = blkbuf + (2 + j) * p.blk_stride;
            const uint32_t vph = s_phase[2 + j];
            const uint16_t *vcum = reinterpret_cast<const uint16_t *>(vb + vph);
            const uint32_t vstart = vph + 8u + (unit ? (uint32_t)vcum[unit - 1] : 0u);
            unit_decode<false>(vb, vstart, unit, lane32, gv, vtile + j * 64, kHeadDim);
        }
        __syncthreads();
        // 3. scores: two threads per token, 64 channels each
        {
            const int tok = tid >> 1, half = tid & 1;
            const uint32_t *row = reinterpret_cast<const uint32_t *>(ktile + tok * kHeadDim + half * 64);
            float dot[G];
#pragma unroll
            for (int g = 0; g < G; g++) dot[g] = 0.f;
            const float s_tok = ks[tok], z_tok = kz[tok];
#pragma unroll 4
            for (int i = 0; i < 16; i++) {
                const uint32_t w = row[i];
                float c0 = (float)(w & 0xFFu), c1 = (float)((w >> 8) & 0xFFu),
                      c2 = (float)((w >> 16) & 0xFFu), c3 = (float)(w >> 24);
                if (REF) {
                    c0 = round16(round16(c0 + z_tok, p.dtype) * s_tok, p.dtype);
                    c1 = round16(round16(c1 + z_tok, p.dtype) * s_tok, p.dtype);
                    c2 = round16(round16(c2 + z_tok, p.dtype) * s_tok, p.dtype);
                    c3 = round16(round16(c3 + z_tok, p.dtype) * s_tok, p.dtype);
                }
#pragma unroll
                for (int g = 0; g < G; g++) {
                    const float *qq = qf + g * kHeadDim + half * 64 + 4 * i;
                    dot[g] += qq[0] * c0 + qq[1] * c1 + qq[2] * c2 + qq[3] * c3;
                }
            }
#pragma unroll
            for (int g = 0; g < G; g++) {
                const float d = dot[g] + __shfl_xor(dot[g], 1, 64);
                if (half == 0) S[g * kTile + tok] = REF ? d * p.sm_scale : p.sm_scale * s_tok * (d + z_tok * qsum[g]);
            }
        }
        __syncthreads();
        // 4. online softmax: wavefront w owns query heads w, w+4, ...
        for (int g = tid >> 6; g < G; g += 4) {
            const int lane = tid & 63;
            const float s0 = S[g * kTile + lane], s1 = S[g * kTile + 64 + lane];
            float mx = fmaxf(s0, s1);
#pragma unroll
            for (int d = 32; d >= 1; d >>= 1) mx = fmaxf(mx, __shfl_xor(mx, d, 64));
            const float m_old = st_m[g];
            const float m_new = fmaxf(m_old, mx);
            const float p0 = __expf(s0 - m_new), p1 = __expf(s1 - m_new);
            const float w0 = REF ? p0 : p0 * vs[lane], w1 = REF ? p1 : p1 * vs[64 + lane];
            P[g * kTile + lane] = w0;
            P[g * kTile + 64 + lane] = w1;
            float sum = p0 + p1;
            float zs = REF ? 0.f : w0 * vz[lane] + w1 * vz[64 + lane];
#pragma unroll
            for (int d = 32; d >= 1; d >>= 1) {
                sum += __shfl_xor(sum, d, 64);
                zs += __shfl_xor(zs, d, 64);
            }
            if (lane == 0) {
                const float alpha = __expf(m_old - m_new);   // exp(-inf) = 0 on the first tile
                st_a[g] = alpha;
                st_m[g] = m_new;
                st_l[g] = st_l[g] * alpha + sum;
                st_z[g] = st_z[g] * alpha + zs;
            }
        }
        __syncthreads();
        // 5. PV: thread = (channel, token half)
        {
            const int ch = tid & 127, half = tid >> 7;
            float part[G];
#pragma unroll
            for (int g = 0; g < G; g++) part[g] = 0.f;
#pragma unroll 8
            for (int t = 0; t < 64; t++) {
                float c = (float)vtile[(half * 64 + t) * kHeadDim + ch];
                if (REF) c = round16(round16(c + vz[half * 64 + t], p.dtype) * vs[half * 64 + t], p.dtype);
#pragma unroll
                for (int g = 0; g < G; g++) part[g] += P[g * kTile + half * 64 + t] * c;
            }
#pragma unroll
            for (int g = 0; g < G; g++) acc[g] = acc[g] * st_a[g] + part[g];
        }
        __syncthreads();
    }
    // combine the two token halves and write the partial
    {
        const int ch = tid & 127, half = tid >> 7;
        float *red = S;   // reuse: [G][128]
        if (half == 1)
            for (int g = 0; g < G; g++) red[g * kTile + ch] = acc[g];
        __syncthreads();
        if (half == 0) {
            for (int g = 0; g < p.Gq; g++) {
                const size_t hq = (size_t)b * p.Hq + (size_t)h * p.Gq + g;
                float *dst = p.part + (hq * p.nparts + split) * kPartStride;
                dst[2 + ch] = acc[g] + red[g * kTile + ch] + st_z[g];
                if (ch == 0) { dst[0] = st_m[g]; dst[1] = st_l[g]; }
            }
        }
    }
}

// ---- matrix-core kernels (variants 0 and 2): shared arithmetic ----------------------------
// K side: every half-wavefront unpacks one round (16 tokens x 128 channels, lane t = channels
// 4t..4t+3) into an int8 tile in LDS laid out [token][channel]; the tile is read back in the
// operand layout of the 16x16 int8 MFMAs (lane = token, 8 consecutive channels per 8-byte read;
// the staged kernel pairs two reads into one v_mfma_i32_16x16x64_i8 operand, the gather kernel
// issues v_mfma_i32_16x16x32_i8 per read) and contracted against q, which is split per query head into three signed 7-bit digits
// (q = qs * (d0 * 2^14 + d1 * 2^7 + d2)), one MFMA row per (digit, head).  Integer arithmetic
// is exact, so the scores carry only the 2^-21 relative rounding of that split.
// V side: lane = channel as in the stream, nothing is transposed.  MFMA number k of a segment
// takes token k of each of the lane's four packs (rounds) as its four contraction slots, so a
// register pair of 16-bit fields is an operand as it stands: the masked field bits are the fp16
// SUBNORMAL delta * 2^-24 (the matrix cores take subnormal inputs exactly), no conversion.  The A
// operand holds the softmax weights (times v_scale) of the 4 query heads, so the per-lane
// accumulators are out[g][channel] and need no cross-lane reduction; pack minima enter through
// one more MFMA against the per-round weight sums (split hi/lo).
typedef int int4v __attribute__((ext_vector_type(4)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef _Float16 half4v __attribute__((ext_vector_type(4)));
typedef unsigned short ushort2v __attribute__((ext_vector_type(2)));

constexpr int kKtStride = 136;         // bytes per token row of the int8 K tile (128 + 8 pad)
constexpr int kKtDw = kKtStride / 4;

__device__ __forceinline__ uint32_t pk_shr16(uint32_t v, uint32_t sh) {
    ushort2v a = __builtin_bit_cast(ushort2v, v), b = __builtin_bit_cast(ushort2v, sh);
    return __builtin_bit_cast(uint32_t, (ushort2v)(a >> b));
}

template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_keep(float x) {   // lanes without a valid source keep x
    const int v = __builtin_bit_cast(int, x);
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(v, v, CTRL, ROW_MASK, 0xF, false));
}

__device__ __forceinline__ float wave_max(float x) {
    x = fmaxf(x, dpp_keep<0xB1, 0xF>(x));    // quad_perm [1,0,3,2]
    x = fmaxf(x, dpp_keep<0x4E, 0xF>(x));    // quad_perm [2,3,0,1]
    x = fmaxf(x, dpp_keep<0x141, 0xF>(x));   // row_half_mirror
    x = fmaxf(x, dpp_keep<0x140, 0xF>(x));   // row_mirror
    x = fmaxf(x, dpp_keep<0x142, 0xA>(x));   // row_bcast:15 into rows 1 and 3
    x = fmaxf(x, dpp_keep<0x143, 0xC>(x));   // row_bcast:31 into rows 2 and 3
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), 63));
}

__device__ __forceinline__ float row16_sum(float x) {  // every lane gets the sum of its 16-lane row
    x += dpp_keep<0xB1, 0xF>(x);
    x += dpp_keep<0x4E, 0xF>(x);
    x += dpp_keep<0x141, 0xF>(x);
    x += dpp_keep<0x140, 0xF>(x);
    return x;
}

__device__ __forceinline__ float wave_sum(float x) {
    x = row16_sum(x);
    const int v = __builtin_bit_cast(int, x);
    float s = 0.f;
#pragma unroll
    for (int r = 0; r < 4; r++) s += __builtin_bit_cast(float, __builtin_amdgcn_readlane(v, 16 * r));
    return s;
}

// ---- 16-bit tail window: dense attention over T_w tokens, one workgroup per (kv head, batch)
// Attention of the G query heads of KV head (h, b) over tokens [t0, t1) of the uncompressed tail window, written
// as partial `part_idx` (an empty range writes a partial of weight zero).  `lds` provides G * (128 + t1 - t0)
// floats.  Called by all 256 threads of a workgroup.
constexpr int kWinPieceLds = 36864;   // LDS every instance of the async-copy kernel has in its two slots

template <int G>
__device__ __forceinline__ void window_body(const AttnParams &p, uint8_t *lds, int h, int b, int t0, int t1,
                                            int part_idx) {
    float *qf = reinterpret_cast<float *>(lds);   // [G][128]
    float *S = qf + G * kHeadDim;                 // [G][Tw]
    __shared__ float st_m[G], st_l[G];
    const int tid = threadIdx.x;
    const int Tw = t1 > t0 ? t1 - t0 : 0;
    for (int i = tid; i < G * kHeadDim; i += 256)
        qf[i] = i < p.Gq * kHeadDim ? a_ld16(p.q, ((size_t)b * p.Hq + (size_t)h * p.Gq) * kHeadDim + i, p.dtype) : 0.f;
    __syncthreads();
    const uint16_t *kbase = p.k_win + (((size_t)b * p.Hkv + h) * p.win_stride + t0) * kHeadDim;
    const uint16_t *vbase = p.v_win + (((size_t)b * p.Hkv + h) * p.win_stride + t0) * kHeadDim;
    {   // scores: 16 tokens per pass, 16 threads per token, each with 8 channels of the row
        const int c = tid & 15;
        float qr[G][8];
#pragma unroll
        for (int g = 0; g < G; g++)
#pragma unroll
            for (int j = 0; j < 8; j++) qr[g][j] = qf[g * kHeadDim + 8 * c + j];
        for (int base = 0; base < Tw; base += 16) {
            const int t = base + (tid >> 4);
            float dot[G];
#pragma unroll
            for (int g = 0; g < G; g++) dot[g] = 0.f;
            if (t < Tw) {
                const uint4 v = reinterpret_cast<const uint4 *>(kbase + (size_t)t * kHeadDim)[c];
                const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const float k0 = p.dtype == PKV_F16 ? __half2float(__ushort_as_half((unsigned short)(w[i] & 0xFFFFu)))
                                                        : __uint_as_float(w[i] << 16);
                    const float k1 = p.dtype == PKV_F16 ? __half2float(__ushort_as_half((unsigned short)(w[i] >> 16)))
                                                        : __uint_as_float(w[i] & 0xFFFF0000u);
#pragma unroll
                    for (int g = 0; g < G; g++) dot[g] += qr[g][2 * i] * k0 + qr[g][2 * i + 1] * k1;
                }
            }
#pragma unroll
            for (int g = 0; g < G; g++) {
                const float d = row16_sum(dot[g]);
                if (c == 0 && t < Tw) S[g * Tw + t] = d * p.sm_scale;
            }
        }
    }
    __syncthreads();
    for (int g = tid >> 6; g < G; g += 4) {
        const int lane = tid & 63;
        float mx = -INFINITY;
        for (int t = lane; t < Tw; t += 64) mx = fmaxf(mx, S[g * Tw + t]);
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) mx = fmaxf(mx, __shfl_xor(mx, d, 64));
        float sum = 0.f;
        for (int t = lane; t < Tw; t += 64) {
            const float e = __expf(S[g * Tw + t] - mx);
            S[g * Tw + t] = e;
            sum += e;
        }
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) sum += __shfl_xor(sum, d, 64);
        if (lane == 0) { st_m[g] = mx; st_l[g] = sum; }
    }
    __syncthreads();
    {   // weighted V sum: thread = (token parity, channel); the odd half hands its sums over through qf
        const int half = tid >> 7, ch = tid & (kHeadDim - 1);
        float acc[G];
#pragma unroll
        for (int g = 0; g < G; g++) acc[g] = 0.f;
        int t = half;
        for (; t + 6 < Tw; t += 8) {
            float v[4];
#pragma unroll
            for (int u = 0; u < 4; u++) v[u] = a_ld16(vbase, (size_t)(t + 2 * u) * kHeadDim + ch, p.dtype);
#pragma unroll
            for (int u = 0; u < 4; u++)
#pragma unroll
                for (int g = 0; g < G; g++) acc[g] += S[g * Tw + t + 2 * u] * v[u];
        }
        for (; t < Tw; t += 2) {
            const float v = a_ld16(vbase, (size_t)t * kHeadDim + ch, p.dtype);
#pragma unroll
            for (int g = 0; g < G; g++) acc[g] += S[g * Tw + t] * v;
        }
        if (half) {
#pragma unroll
            for (int g = 0; g < G; g++) qf[g * kHeadDim + ch] = acc[g];
        }
        __syncthreads();
        if (!half) {
#pragma unroll
            for (int g = 0; g < G; g++) {
                if (g >= p.Gq) break;
                const size_t hq = (size_t)b * p.Hq + (size_t)h * p.Gq + g;
                float *dst = p.part + (hq * p.nparts + part_idx) * kPartStride;
                dst[2 + ch] = acc[g] + qf[g * kHeadDim + ch];
                if (ch == 0) { dst[0] = st_m[g]; dst[1] = st_l[g]; }
            }
        }
    }
}

template <int G>
__global__ void __launch_bounds__(256) attn_window_kernel(const AttnParams p) {
    extern __shared__ __align__(16) uint8_t lds[];
    window_body<G>(p, lds, blockIdx.x, blockIdx.y, 0, p.T_w, p.nparts - 1);
}

// ---- merge of the per-split partials: grid (Hq, B), 256 threads, nparts floats of dynamic LDS ----
// Partials are read in parallel: thread <-> partial for the maxima and weights, then thread <-> (parity of the
// partial, channel) for the weighted sum, four rows in flight.
__global__ void __launch_bounds__(256) attn_merge_kernel(const float *__restrict__ part, uint16_t *__restrict__ out,
                                                         int Hq, int nparts, int dtype, int out_f32) {
    extern __shared__ float w_s[];                   // weight of every partial
    __shared__ float red[8];
    __shared__ __attribute__((aligned(8))) float part_num[3 * kHeadDim];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const size_t hq = (size_t)blockIdx.y * Hq + blockIdx.x;
    const float *base = part + hq * nparts * kPartStride;
    float mx = -INFINITY;
    for (int s = tid; s < nparts; s += 256) mx = fmaxf(mx, base[(size_t)s * kPartStride]);
    mx = wave_max(mx);
    if (lane == 0) red[wave] = mx;
    __syncthreads();
    const float M = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    float den = 0.f;
    for (int s = tid; s < nparts; s += 256) {
        const float w = __expf(base[(size_t)s * kPartStride] - M);
        w_s[s] = w;
        den += w * base[(size_t)s * kPartStride + 1];
    }
    den = wave_sum(den);
    if (lane == 0) red[4 + wave] = den;
    __syncthreads();
    den = (red[4] + red[5]) + (red[6] + red[7]);
    // weighted sum: wavefront = every fourth partial, lane = two adjacent channels (rows are 8-byte aligned), eight
    // loads in flight per lane -- a long list of partials (small batches spread one head over many splits) is a
    // chain of dependent round trips otherwise
    const float2v *col = reinterpret_cast<const float2v *>(base + 2) + lane;
    float2v num = {0.f, 0.f};
    int s = wave;
    for (; s + 28 < nparts; s += 32) {
        float2v v[8];
#pragma unroll
        for (int u = 0; u < 8; u++) v[u] = col[(size_t)(s + 4 * u) * (kPartStride / 2)];
#pragma unroll
        for (int u = 0; u < 8; u++) num += w_s[s + 4 * u] * v[u];
    }
    if (s < nparts) {                                  // the last, partial batch: still one round trip
        float2v v[8];
        float w[8];
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const int idx = min(s + 4 * u, nparts - 1);
            v[u] = col[(size_t)idx * (kPartStride / 2)];
            w[u] = s + 4 * u < nparts ? w_s[idx] : 0.f;
        }
#pragma unroll
        for (int u = 0; u < 8; u++) num += w[u] * v[u];
    }
    if (wave) reinterpret_cast<float2v *>(part_num + (wave - 1) * kHeadDim)[lane] = num;
    __syncthreads();
    if (wave == 0) {
#pragma unroll
        for (int w = 0; w < 3; w++) num += reinterpret_cast<const float2v *>(part_num + w * kHeadDim)[lane];
        if (out_f32) {
            reinterpret_cast<float2v *>(reinterpret_cast<float *>(out) + hq * kHeadDim)[lane] = num / den;
        } else {
            const uint32_t lo = a_st16(num[0] / den, dtype), hi = a_st16(num[1] / den, dtype);
            reinterpret_cast<uint32_t *>(out + hq * kHeadDim)[lane] = lo | (hi << 16);
        }
    }
}

}  // namespace pkv
#include "pkv_attn_direct.hpp"
namespace pkv {

template <int G, int KW, int VW>
static int launch_direct(const AttnParams &p, hipStream_t s) {
    constexpr int GP = ((G + 3) / 4) * 4;
    const uint32_t lds_bytes = 8u * 16u * kKtStride + kRing * 16u * 4u + GP * kTile * 2u + 2u * GP * 8u * 2u + 6u * 8u * 4u;
    const dim3 grid((unsigned)p.nsplit, (unsigned)p.Hkv, (unsigned)p.B);
    if (p.dtype == PKV_BF16)
        attn_direct_kernel<G, KW, VW, true><<<grid, 256, lds_bytes, s>>>(p);
    else
        attn_direct_kernel<G, KW, VW, false><<<grid, 256, lds_bytes, s>>>(p);
    PKV_HIP_CHECK(hipGetLastError());
    return PKV_OK;
}

}  // namespace pkv
#include "pkv_attn_dma.hpp"
namespace pkv {

template <int G, int KW, int VW>
static int launch_dma(const AttnParams &p, hipStream_t s) {
    static_assert(dma_lds_bytes<G, KW, VW>() >= kWinPieceLds, "window pieces borrow the slots");
    const dim3 grid((unsigned)p.nsplit * (unsigned)p.Hkv * (unsigned)p.B);
    if (p.dtype == PKV_BF16)
        attn_dma_kernel<G, KW, VW, true><<<grid, 256, 0, s>>>(p);
    else
        attn_dma_kernel<G, KW, VW, false><<<grid, 256, 0, s>>>(p);
    PKV_HIP_CHECK(hipGetLastError());
    return PKV_OK;
}

// PKV_ATTN_MINIMAL (kernel development only): instantiate the 4-bit kernels for groups of 4 and 1 alone; every other
// shape is refused.  Cuts the compile of this file from minutes to seconds.
template <int G>
static int launch_dma_bits(const AttnParams &p, hipStream_t s) {
#ifdef PKV_ATTN_MINIMAL
#if PKV_ATTN_MINIMAL == 55     // (-DPKV_ATTN_MINIMAL=55: the 5-bit kernel instead, =33: the 3-bit kernel)
    if constexpr (G == 4) { if (p.k_bits == 5 && p.v_bits == 5) return launch_dma<G, 5, 5>(p, s); }
#elif PKV_ATTN_MINIMAL == 33
    if constexpr (G == 4) { if (p.k_bits == 3 && p.v_bits == 3) return launch_dma<G, 3, 3>(p, s); }
#else
    if constexpr (G == 4 || G == 1) { if (p.k_bits == 4 && p.v_bits == 4) return launch_dma<G, 4, 4>(p, s); }
#endif
    PKV_REQUIRE(false, PKV_ERR_UNSUPPORTED, "minimal build: 4-bit codes and groups of 4 only");
#else
    switch (p.k_bits * 8 + p.v_bits) {
        case 2 * 8 + 2: return launch_dma<G, 2, 2>(p, s);
        case 2 * 8 + 3: return launch_dma<G, 2, 3>(p, s);
        case 2 * 8 + 4: return launch_dma<G, 2, 4>(p, s);
        case 3 * 8 + 2: return launch_dma<G, 3, 2>(p, s);
        case 3 * 8 + 3: return launch_dma<G, 3, 3>(p, s);
        case 3 * 8 + 4: return launch_dma<G, 3, 4>(p, s);
        case 4 * 8 + 2: return launch_dma<G, 4, 2>(p, s);
        case 4 * 8 + 3: return launch_dma<G, 4, 3>(p, s);
        case 5 * 8 + 5: return launch_dma<G, 5, 5>(p, s);       // the extension widths 5 and 6, for K, V or both
        case 6 * 8 + 6: return launch_dma<G, 6, 6>(p, s);
        case 5 * 8 + 4: return launch_dma<G, 5, 4>(p, s);
        case 4 * 8 + 5: return launch_dma<G, 4, 5>(p, s);
        case 6 * 8 + 5: return launch_dma<G, 6, 5>(p, s);
        case 5 * 8 + 6: return launch_dma<G, 5, 6>(p, s);
        case 6 * 8 + 4: return launch_dma<G, 6, 4>(p, s);
        case 4 * 8 + 6: return launch_dma<G, 4, 6>(p, s);
        default: return launch_dma<G, 4, 4>(p, s);
    }
#endif
}

template <int G>
static int launch_direct_bits(const AttnParams &p, hipStream_t s) {
#ifdef PKV_ATTN_MINIMAL
    PKV_REQUIRE(false, PKV_ERR_UNSUPPORTED, "minimal build: the asynchronous-copy kernel only");
#else
    switch (p.k_bits * 8 + p.v_bits) {
        case 2 * 8 + 2: return launch_direct<G, 2, 2>(p, s);
        case 2 * 8 + 3: return launch_direct<G, 2, 3>(p, s);
        case 2 * 8 + 4: return launch_direct<G, 2, 4>(p, s);
        case 3 * 8 + 2: return launch_direct<G, 3, 2>(p, s);
        case 3 * 8 + 3: return launch_direct<G, 3, 3>(p, s);
        case 3 * 8 + 4: return launch_direct<G, 3, 4>(p, s);
        case 4 * 8 + 2: return launch_direct<G, 4, 2>(p, s);
        case 4 * 8 + 3: return launch_direct<G, 4, 3>(p, s);
        default: return launch_direct<G, 4, 4>(p, s);
    }
#endif
}

template <int G>
static int launch_attn(const AttnParams &p, int variant, bool aligned16, bool ref_rounding, uint16_t *out, hipStream_t s) {
    PKV_REQUIRE(variant >= 0 && variant <= 2, PKV_ERR_INVALID, "variant must be 0, 1 or 2");
    // variant 0: asynchronous-copy kernel (needs 16-byte aligned streams; otherwise, and as
    // variant 2, the kernel that gathers straight from global memory); variant 1: plain VALU kernel
    if (p.T_c > 0 && variant == 0 && aligned16) {
        const int rc = launch_dma_bits<G>(p, s);
        if (rc) return rc;
    } else if (p.T_c > 0 && (variant == 0 || variant == 2)) {
        const int rc = launch_direct_bits<G>(p, s);
        if (rc) return rc;
    } else if (p.T_c > 0) {
        const uint32_t lds_bytes = 2u * kTile * kHeadDim + 4u * p.blk_stride +
                                   (uint32_t)sizeof(float) * (G * kHeadDim + 2 * G * kTile + 4 * kTile + 5 * G);
        const dim3 grid((unsigned)p.nsplit, (unsigned)p.Hkv, (unsigned)p.B);
        const void *fn = ref_rounding ? reinterpret_cast<const void *>(attn_tiles_kernel<G, true>)
                                      : reinterpret_cast<const void *>(attn_tiles_kernel<G, false>);
        PKV_HIP_CHECK(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
        if (ref_rounding)
            attn_tiles_kernel<G, true><<<grid, 256, lds_bytes, s>>>(p);
        else
            attn_tiles_kernel<G, false><<<grid, 256, lds_bytes, s>>>(p);
        PKV_HIP_CHECK(hipGetLastError());
    }
    if (p.T_w > 0 && p.win_piece == 0) {
        const uint32_t lds_bytes = (uint32_t)sizeof(float) * (G * kHeadDim + G * p.T_w);
        PKV_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(attn_window_kernel<G>),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
        attn_window_kernel<G><<<dim3((unsigned)p.Hkv, (unsigned)p.B), 256, lds_bytes, s>>>(p);
        PKV_HIP_CHECK(hipGetLastError());
    }
    const bool dma_path = p.T_c > 0 && variant == 0 && aligned16;
    if (!(dma_path && p.direct_out)) {       // a single partial is the result: the async-copy kernel wrote it out itself
        attn_merge_kernel<<<dim3((unsigned)p.Hq, (unsigned)p.B), 256, (size_t)p.nparts * sizeof(float), s>>>(
            p.part, out, p.Hq, p.nparts, p.dtype, p.out_f32);
        PKV_HIP_CHECK(hipGetLastError());
    }
    return PKV_OK;
}

}  // namespace pkv

// ---- partials without an allocation --------------------------------------------------------------
// pkv_attn_decode_noalloc keeps the per-split partials in this array instead of library-allocated memory.  Every
// GPU the library runs on holds its own copy, at its own address, until the process ends.  In host code the name
// below is only a handle for hipGetSymbolAddress: the device address it yields (per device) is what kernels get.
#define PKV_ATTN_STATIC_SCRATCH_BYTES (8u << 20)
static __device__ __align__(256) unsigned char scratch[PKV_ATTN_STATIC_SCRATCH_BYTES];
// layout: partials, then the tile counters of the async-copy kernel (zero at load, left at zero by every launch)
static constexpr size_t kStaticPartBytes = (size_t)PKV_ATTN_STATIC_SCRATCH_BYTES - (size_t)pkv::kAttnCounters * sizeof(uint32_t);

namespace pkv {
namespace {
constexpr int kStaticMaxDevices = 16;
void *g_static_part[kStaticMaxDevices];          // device address of `scratch` on each device, once looked up
std::mutex g_static_mu;

// Device address of this device's copy of `scratch` (looked up once per device, with that device current).
int static_scratch_ptr(void **out) {
    int dev = 0;
    PKV_HIP_CHECK(hipGetDevice(&dev));
    PKV_REQUIRE(dev >= 0 && dev < kStaticMaxDevices, PKV_ERR_INVALID, "device index %d out of range", dev);
    std::lock_guard<std::mutex> lock(g_static_mu);
    if (!g_static_part[dev]) {
        void *ptr = nullptr;
        PKV_HIP_CHECK(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        PKV_REQUIRE(ptr != nullptr, PKV_ERR_HIP, "hipGetSymbolAddress returned a null address");
        g_static_part[dev] = ptr;
    }
    *out = g_static_part[dev];
    return PKV_OK;
}

}  // namespace
static int attn_decode_impl(const pkv_attn_args *a, float *ms_out, hipStream_t s, bool static_partials);
}  // namespace pkv

extern "C" int pkv_attn_decode(const pkv_attn_args *a, float *ms_out, pkv_stream_t s_) {
    return pkv::attn_decode_impl(a, ms_out, (hipStream_t)s_, false);
}

extern "C" int pkv_attn_decode_noalloc(const pkv_attn_args *a, pkv_stream_t s_) {
    return pkv::attn_decode_impl(a, nullptr, (hipStream_t)s_, true);
}

int pkv::attn_decode_impl(const pkv_attn_args *a, float *ms_out, hipStream_t s, bool static_partials) {
    PKV_REQUIRE(a != nullptr, PKV_ERR_INVALID, "null pointer argument");
    PKV_REQUIRE(a->dtype == PKV_F16 || a->dtype == PKV_BF16, PKV_ERR_UNSUPPORTED, "Unsupported data type");
    PKV_REQUIRE(a->B > 0 && a->Hq > 0 && a->Hkv > 0 && a->Hq % a->Hkv == 0, PKV_ERR_INVALID,
                "need B, Hq, Hkv > 0 and Hq divisible by Hkv");
    PKV_REQUIRE(a->B <= 65535 && a->Hkv <= 65535, PKV_ERR_UNSUPPORTED, "batch / head count above 65535");
    PKV_REQUIRE(a->T_c >= 0 && a->T_w >= 0 && a->T_c + a->T_w > 0, PKV_ERR_INVALID, "empty cache");
    PKV_REQUIRE(a->T_c % kTile == 0, PKV_ERR_INVALID, "compressed length must be a multiple of 128 tokens");
    PKV_REQUIRE(a->T_w <= 2048, PKV_ERR_UNSUPPORTED, "tail window longer than 2048 tokens");
    PKV_REQUIRE(a->q && a->out, PKV_ERR_INVALID, "null pointer argument");
    PKV_REQUIRE((a->flags & ~(PKV_ATTN_REF_ROUNDING | PKV_ATTN_OUT_F32)) == 0, PKV_ERR_INVALID, "unknown flag bits");
    const bool ref_rounding = (a->flags & PKV_ATTN_REF_ROUNDING) != 0;
    PKV_REQUIRE(!ref_rounding || a->variant == 1, PKV_ERR_INVALID,
                "PKV_ATTN_REF_ROUNDING is a mode of the plain kernel (variant 1)");
    if (a->T_c > 0) {
        PKV_REQUIRE(a->k_stream && a->k_info && a->v_stream && a->v_info && a->k_scale && a->k_zero &&
                        a->v_scale && a->v_zero,
                    PKV_ERR_INVALID, "null pointer argument");
        PKV_REQUIRE(a->k_bits >= 2 && a->k_bits <= kMaxBits && a->v_bits >= 2 && a->v_bits <= kMaxBits, PKV_ERR_UNSUPPORTED,
                    "not supported: bits_len outside 2..8");
        PKV_REQUIRE(a->k_bytes > 0 && a->v_bytes > 0 && a->k_bytes < (1ull << 32) && a->v_bytes < (1ull << 32),
                    PKV_ERR_INVALID, "stream sizes must be in 1 .. 4 GiB - 1");
    }
    const int par_stride = a->par_stride ? a->par_stride : a->T_c, win_stride = a->win_stride ? a->win_stride : a->T_w;
    PKV_REQUIRE(par_stride >= a->T_c && win_stride >= a->T_w, PKV_ERR_INVALID, "row stride shorter than the row");
    PKV_REQUIRE((uint64_t)a->B * (uint64_t)par_stride < (1ull << 28), PKV_ERR_UNSUPPORTED,
                "batch x compressed tokens above 2^28");
    PKV_REQUIRE((uint64_t)(a->T_c / 64) * (uint64_t)a->B * (uint64_t)a->Hkv < (1ull << 27), PKV_ERR_UNSUPPORTED,
                "more than 2^27 blocks per stream");
    if (a->T_w > 0) {
        PKV_REQUIRE(a->k_win && a->v_win, PKV_ERR_INVALID, "null pointer argument");
        PKV_REQUIRE((reinterpret_cast<uintptr_t>(a->k_win) & 15u) == 0, PKV_ERR_INVALID,
                    "k_win must be 16-byte aligned");
    }
    const int Gq = a->Hq / a->Hkv;
    PKV_REQUIRE(Gq <= 8, PKV_ERR_UNSUPPORTED, "not supported: more than 8 query heads per KV head");
    const int G = Gq <= 2 ? Gq : Gq <= 4 ? 4 : 8;      // groups of 3 and of 5..7 run the kernels of 4 and 8 with idle head slots

    AttnParams p;
    p.k_stream = a->k_stream; p.k_info = a->k_info; p.v_stream = a->v_stream; p.v_info = a->v_info;
    p.k_scale = (const uint16_t *)a->k_scale; p.k_zero = (const uint16_t *)a->k_zero;
    p.v_scale = (const uint16_t *)a->v_scale; p.v_zero = (const uint16_t *)a->v_zero;
    p.q = (const uint16_t *)a->q;
    p.k_win = (const uint16_t *)a->k_win; p.v_win = (const uint16_t *)a->v_win;
    p.B = a->B; p.Hq = a->Hq; p.Hkv = a->Hkv; p.T_c = a->T_c; p.T_w = a->T_w;
    p.Gq = Gq;
    p.par_stride = par_stride; p.win_stride = win_stride;
    p.k_bits = a->k_bits; p.v_bits = a->v_bits; p.dtype = a->dtype; p.sm_scale = a->sm_scale;
    const int n_tiles = a->T_c / kTile;
    int nsplit = 0, tps = 0;
    if (n_tiles > 0) {
        // Members per (sequence, KV head): about PKV_SPLIT_TARGET workgroups in all for the reference's widths -- four resident on each of 256
        // CUs.  When the heads do not divide that number, rounding the members up leaves a few workgroups over that
        // only start once others have finished, each with a full share of tiles (12 sequences x 8 heads: 11 members,
        // 1056 workgroups, 115 us per step against 99 us with 10 members); so both roundings are priced as
        // generations x tiles per member and the cheaper one is taken, the finer cut on a tie.
        const int pairs = a->B * a->Hkv;
        // (as many members as are resident at once: widths 5 and 6 run two workgroups per CU -- 193 us per step with
        // 512 members against 199 us with 1024 in two generations, 6 bits 201 against 218 us -- and groups of eight
        // query heads three: 156 against 165 us)
        const int target = PKV_SPLIT_TARGET / 4 * PKV_DMA_WAVES((a->k_bits > a->v_bits ? a->k_bits : a->v_bits), G);
        long best_cost = -1;
        for (int up = 1; up >= 0; up--) {
            int want = up ? (target + pairs - 1) / pairs : target / pairs;
            if (want < 1) want = 1;
            if (want > n_tiles) want = n_tiles;
            const int t = (n_tiles + want - 1) / want, n = (n_tiles + t - 1) / t;
            const long cost = (((long)pairs * n + target - 1) / target) * (long)t;
            if (best_cost < 0 || cost < best_cost) { best_cost = cost; tps = t; nsplit = n; }
        }
    }
    p.tiles_per_split = tps; p.nsplit = nsplit;
    // The async-copy kernel spreads the tail window over its splits (each takes win_piece tokens after its
    // tiles and writes one more partial), so the window costs no launch and no idle tail; other paths
    // give the window a kernel of its own.
    // the matrix-core kernels take the reference's widths and, in the asynchronous-copy kernel, the extension widths
    // 5 and 6 (the other side then 4, 5 or 6); any other combination with an extension width runs the plain kernel
    const bool narrow = a->T_c == 0 || (a->k_bits <= 4 && a->v_bits <= 4);
    const bool wide_fast = !narrow && a->k_bits >= 4 && a->v_bits >= 4 && a->k_bits <= 6 && a->v_bits <= 6 && a->variant == 0;
    const bool aligned16 = (narrow || wide_fast) &&
                           ((reinterpret_cast<uintptr_t>(a->k_stream) | reinterpret_cast<uintptr_t>(a->v_stream)) & 15u) == 0;
    p.win_piece = 0;
    if (a->T_w > 0 && nsplit > 0 && a->variant == 0 && aligned16) {
        const int piece = (a->T_w + nsplit - 1) / nsplit;
        if ((size_t)G * (kHeadDim + piece) * sizeof(float) <= (size_t)kWinPieceLds) p.win_piece = piece;
    }
    p.nparts = nsplit + (a->T_w > 0 ? (p.win_piece ? nsplit : 1) : 0);
    p.k_cap = a->T_c > 0 ? (uint32_t)k_block_bound(64, a->k_bits) : 0;
    p.v_cap = a->T_c > 0 ? (uint32_t)v_block_bound(64, a->v_bits) : 0;
    const uint32_t cap = p.k_cap > p.v_cap ? p.k_cap : p.v_cap;
    p.blk_stride = ((cap + 14u + 15u) & ~15u) + 32u;
    p.k_bytes = (uint32_t)a->k_bytes; p.v_bytes = (uint32_t)a->v_bytes;   // up to 14 bytes of phase in front, slack behind
    p.out = (uint16_t *)a->out;
    p.out_f32 = (a->flags & PKV_ATTN_OUT_F32) ? 1 : 0;
    p.direct_out = p.nparts == 1 && !p.out_f32;
    // The async-copy kernel balances the members of a head through two counters per head (with one member there is
    // nothing to balance).
    const bool dma_path = a->T_c > 0 && a->variant == 0 && aligned16 && (narrow || wide_fast);
    // Tiles by counter pay when a member has many tiles (the first five are its own anyway): short launches -- a few
    // tiles per member, the small-batch decode steps -- only get the counters' atomic round trips on top (batch 1,
    // 32768 tokens: 46 us against 19 us with fixed shares).  And only up to eight members per head: every member asks
    // its head's counter once per tile, and atomics on one address retire one after the other -- with 16 members a
    // step of batch 8 x 65536 tokens takes 172 us against 126 us with fixed shares, with 64 (batch 2 x 131072) 206
    // against 67 us; at 4 and 8 members the counters are worth 1-2 %.
    p.dynamic = PKV_DYNAMIC_TILES && dma_path && nsplit > 1 && nsplit <= 8 && tps >= 12 && 2 * a->B * a->Hkv <= kAttnCounters;
    p.batch_shift = 1;                     // a member asks for 1 / (2 nsplit) of what is left: ceil(log2(2 nsplit))
    while ((1 << p.batch_shift) < 2 * nsplit) p.batch_shift++;
    p.counters = nullptr;
    // Partials and counters: the stream's own scratch, or the static array -- for pkv_attn_decode_noalloc, and for a
    // stream that is capturing a graph before it has scratch of its own.
    void *part = nullptr, *static_part = nullptr;
    const size_t part_bytes = (size_t)a->B * a->Hq * p.nparts * kPartStride * sizeof(float);
    int rc = static_scratch_ptr(&static_part);     // looked up on the first call on a device, while nothing is capturing
    if (rc) return rc;
    bool use_static = static_partials;
    if (!use_static) {
        rc = scratch_get(part_bytes, s, &part);
        if (rc == PKV_OK && p.dynamic) rc = attn_counters_get(s, &p.counters);
        if (rc == PKV_ERR_CAPTURING && part_bytes <= kStaticPartBytes) use_static = true;
        else if (rc) return rc == PKV_ERR_CAPTURING ? PKV_ERR_HIP : rc;
    }
    if (use_static) {
        PKV_REQUIRE(part_bytes <= kStaticPartBytes, PKV_ERR_UNSUPPORTED,
                    "pkv_attn_decode_noalloc: %zu bytes of partials (batch %d x %d query heads x %d partials) exceed the "
                    "%zu bytes the static buffer has for them; use pkv_attn_decode", part_bytes, a->B, a->Hq, p.nparts,
                    kStaticPartBytes);
        part = static_part;
        p.counters = reinterpret_cast<uint32_t *>(static_cast<unsigned char *>(part) + kStaticPartBytes);
    }
    p.part = (float *)part;

    LaunchTimer tm(s, ms_out != nullptr);
    if ((rc = tm.begin())) return rc;
    const int variant = narrow || (wide_fast && aligned16) ? a->variant : 1;
    switch (G) {
        case 1: rc = launch_attn<1>(p, variant, aligned16, ref_rounding, (uint16_t *)a->out, s); break;
        case 2: rc = launch_attn<2>(p, variant, aligned16, ref_rounding, (uint16_t *)a->out, s); break;
        case 4: rc = launch_attn<4>(p, variant, aligned16, ref_rounding, (uint16_t *)a->out, s); break;
        default: rc = launch_attn<8>(p, variant, aligned16, ref_rounding, (uint16_t *)a->out, s); break;
    }
    if (rc) return rc;
    return tm.end(ms_out);
}
