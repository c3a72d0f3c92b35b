// Per-token affine quantizer and the fused quantize + bit-pack encoders.
//
// Restates on the device the reference's TokenQuant chain (utils/compute.py:84-112):
//   scale = T((max - min) * rel),  zero = T(round(T(min / scale))),
//   code  = T(round(T(x / scale))) - zero,     dequant = T(T(code + zero) * scale)
// where T is the 16-bit storage type and every op computes in fp32 and rounds to T, as the
// PyTorch kernels do.  min / max run over all heads and channels of one (batch, token).
#include "pkv_block.hpp"
#include "pkv_runtime.hpp"

namespace pkv {

template <int DT> struct T16;

template <> struct T16<PKV_F16> {
    static __device__ __forceinline__ float from_bits(uint32_t u16) {
        return __half2float(__ushort_as_half((unsigned short)u16));
    }
    static __device__ __forceinline__ uint32_t to_bits(float x) {
        return (uint32_t)__half_as_ushort(__float2half_rn(x));
    }
};

template <> struct T16<PKV_BF16> {
    static __device__ __forceinline__ float from_bits(uint32_t u16) { return __uint_as_float(u16 << 16); }
    static __device__ __forceinline__ uint32_t to_bits(float x) {   // round to nearest even
        uint32_t u = __float_as_uint(x);
        if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (u >> 16) | 0x40u;   // NaN stays NaN
        u += 0x7FFFu + ((u >> 16) & 1u);
        return u >> 16;
    }
};

template <int DT> __device__ __forceinline__ float round_t(float x) {
    return T16<DT>::from_bits(T16<DT>::to_bits(x));
}

// code of x given the token's (scale, zero); all values are T-representable floats.
template <int DT> __device__ __forceinline__ float quant_code(float x, float scale, float zero) {
    const float qv = rintf(round_t<DT>(__fdiv_rn(x, scale)));
    return round_t<DT>(round_t<DT>(qv) - zero);
}

template <int DT> __device__ __forceinline__ void unpack8(const uint4 v, float out[8]) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; i++) {
        out[2 * i] = T16<DT>::from_bits(w[i] & 0xFFFFu);
        out[2 * i + 1] = T16<DT>::from_bits(w[i] >> 16);
    }
}

// ---- per-token scale / zero ------------------------------------------------------------
// grid (T/16, B), 256 threads: 16 lanes per token, 8 channels per lane, loop over heads.
template <int DT>
__global__ void quant_params_kernel(const uint16_t *__restrict__ x, int H, int T, float rel,
                                    uint16_t *__restrict__ scale, uint16_t *__restrict__ zero) {
    const int b = blockIdx.y;
    const int tok = blockIdx.x * 16 + (threadIdx.x >> 4);
    const int l16 = threadIdx.x & 15;
    float mn = INFINITY, mx = -INFINITY;
    if (tok < T) {
        for (int h = 0; h < H; h++) {
            const uint4 v = *reinterpret_cast<const uint4 *>(
                x + (((size_t)b * H + h) * T + tok) * kHeadDim + l16 * 8);
            float f[8];
            unpack8<DT>(v, f);
#pragma unroll
            for (int i = 0; i < 8; i++) {
                mn = fminf(mn, f[i]);
                mx = fmaxf(mx, f[i]);
            }
        }
    }
#pragma unroll
    for (int d = 8; d >= 1; d >>= 1) {
        mn = fminf(mn, __shfl_xor(mn, d, 16));
        mx = fmaxf(mx, __shfl_xor(mx, d, 16));
    }
    if (l16 == 0 && tok < T) {
        const float range = round_t<DT>(mx - mn);
        const float sc = round_t<DT>(range * rel);
        const float z = round_t<DT>(rintf(round_t<DT>(__fdiv_rn(mn, sc))));
        scale[(size_t)b * T + tok] = (uint16_t)T16<DT>::to_bits(sc);
        zero[(size_t)b * T + tok] = (uint16_t)T16<DT>::to_bits(z);
    }
}

// ---- fused quantize + encode: the cell ---------------------------------------------------
// 128 threads work on one block.  Thread = "cell": 16 tokens (one round) x 4 adjacent channels,
// i.e. four packs.  The cell is loaded straight from x (8 bytes per token row, rows of a
// half-wavefront contiguous), quantized and analysed in registers with packed 16-bit arithmetic;
// no code tile is ever formed.
//   K block (64 x 128):  cell (round r = tid / 32, channels 4t..4t+3, t = tid % 32) IS lane t of
//                        unit r, so the packs are emitted where they were computed.
//   V block (128 x 64):  cell (round r = tid / 16, channels 4g..4g+3, g = tid % 16); V units want
//                        lane = channel with the packs of four consecutive rounds, so the pack
//                        records change hands once through LDS.
//
// Exact division without the division sequence.  code = rint(T(x / scale)) - zero needs
// h = RN16(RN32(x / scale)), which equals RN16(x / scale) (24 >= 2 * 11 + 2 bits: double rounding
// is innocuous).  With r = 1 / scale refined to half an ulp once per token,
//   q0 = x * r;  e = fma(-scale, q0, x);  q1 = fma(e, r, q0)
// is within 2^-24 (1 + 2^-20) of the quotient, while a quotient of two 11-bit significands is
// either exactly an fp16 rounding midpoint (then e is exact and q1 hits it exactly, so the tie is
// broken as in the reference) or at least 2^-23 away from every midpoint; so RN16(q1) is the
// reference's value.  bf16 inputs take the plain path (quant_code).
typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

// Per-token constants: scale, 1 / scale, and for fp16 either
//   sub2 != 0 (zero in [-500, 3000], the usual case): add2 = (c, c) with c = 1536 + (zero & 1) - zero as fp16 and
//             sub2 = (0x6600 + (zero & 1)) in both halves.  h + c is then one correctly rounded fp16 addition whose
//             result lies in [1535.5, 2048), where the spacing is 1: it rounds h - zero to an integer, and because
//             c - zero is even a tie goes to the same side as in rint(h).  The code is the result's bit pattern
//             minus sub2 -- no separate rounding instruction;
//   sub2 == 0: add2 = (-zero, -zero) for the general sequence rint(h) + (-zero).
// bf16: sub2 != 0 (|zero| <= 2^20): add2 = 2^23 - zero as fp32 bits; sub2 == 0: add2 = zero as fp32 bits.
struct TokPar { float s, r; uint32_t add2, sub2; };
template <int DT> __device__ __forceinline__ TokPar token_par(float sc, uint32_t zero_bits, bool general_form = false);

__device__ __forceinline__ uint32_t pk_u16(u16x2 v) { return __builtin_bit_cast(uint32_t, v); }
__device__ __forceinline__ u16x2 as_u16x2(uint32_t v) { return __builtin_bit_cast(u16x2, v); }

// codes of four adjacent channels of one token as two pairs of 16-bit integers
// (UNIFORM: every lane of the wavefront holds the same token constants, so the choice of the sequence is a uniform
// branch; otherwise each lane chooses for itself)
template <int DT, bool UNIFORM = true>
__device__ __forceinline__ void quant4(uint2 xw, const TokPar tp, uint32_t &c01, uint32_t &c23) {
    if (DT == PKV_F16) {
        const f16x2 x01 = __builtin_bit_cast(f16x2, xw.x), x23 = __builtin_bit_cast(f16x2, xw.y);
        auto quot = [&](_Float16 xh) -> _Float16 {
            const float f = (float)xh;
            const float q0 = __fmul_rn(f, tp.r);
            const float e = __fmaf_rn(-tp.s, q0, f);
            return (_Float16)__fmaf_rn(e, tp.r, q0);
        };
        const f16x2 h01 = {quot(x01[0]), quot(x01[1])}, h23 = {quot(x23[0]), quot(x23[1])};
        const f16x2 add = __builtin_bit_cast(f16x2, tp.add2);
        if ((UNIFORM ? (uint32_t)__builtin_amdgcn_readfirstlane(tp.sub2) : tp.sub2) != 0u) {
            const u16x2 sub = as_u16x2(tp.sub2);
            c01 = pk_u16((u16x2)(__builtin_bit_cast(u16x2, (f16x2)(h01 + add)) - sub));
            c23 = pk_u16((u16x2)(__builtin_bit_cast(u16x2, (f16x2)(h23 + add)) - sub));
        } else {
            const f16x2 magic = {(_Float16)1024.f, (_Float16)1024.f};    // 1024 + c has c in its low mantissa bits
            const f16x2 d01 = __builtin_elementwise_roundeven(h01) + add, d23 = __builtin_elementwise_roundeven(h23) + add;
            c01 = __builtin_bit_cast(uint32_t, (f16x2)(d01 + magic)) & 0x00FF00FFu;
            c23 = __builtin_bit_cast(uint32_t, (f16x2)(d23 + magic)) & 0x00FF00FFu;
        }
    } else if ((UNIFORM ? (uint32_t)__builtin_amdgcn_readfirstlane(tp.sub2) : tp.sub2) != 0u) {
        // bf16, zero point of moderate size: the same three-instruction quotient (a quotient of two 8-bit
        // significands is either exactly a bf16 rounding midpoint or at least 2^-17 away from every one), rounded to
        // bf16 by the hardware conversion; rint(h) and rint(h) - zero are then exact in fp32 (bf16 values of 256 and
        // above are integers already), so adding 2^23 - zero leaves the code in the low mantissa bits.
        typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
        typedef float f32x2 __attribute__((ext_vector_type(2)));
        auto quot = [&](float f) -> float {
            const float q0 = __fmul_rn(f, tp.r);
            const float e = __fmaf_rn(-tp.s, q0, f);
            return __fmaf_rn(e, tp.r, q0);
        };
        const f32x2 q01 = {quot(__uint_as_float(xw.x << 16)), quot(__uint_as_float(xw.x & 0xFFFF0000u))};
        const f32x2 q23 = {quot(__uint_as_float(xw.y << 16)), quot(__uint_as_float(xw.y & 0xFFFF0000u))};
        const uint32_t h01 = __builtin_bit_cast(uint32_t, __builtin_convertvector(q01, bf16x2));
        const uint32_t h23 = __builtin_bit_cast(uint32_t, __builtin_convertvector(q23, bf16x2));
        const float mz = __uint_as_float(tp.add2);                        // 2^23 - zero
        const uint32_t a = __float_as_uint(rintf(__uint_as_float(h01 << 16)) + mz) & 0xFFu;
        const uint32_t b = __float_as_uint(rintf(__uint_as_float(h01 & 0xFFFF0000u)) + mz) & 0xFFu;
        const uint32_t c = __float_as_uint(rintf(__uint_as_float(h23 << 16)) + mz) & 0xFFu;
        const uint32_t d = __float_as_uint(rintf(__uint_as_float(h23 & 0xFFFF0000u)) + mz) & 0xFFu;
        c01 = a | (b << 16);
        c23 = c | (d << 16);
    } else {
        const float z = __uint_as_float(tp.add2);
        const uint32_t a = (uint32_t)(int)quant_code<DT>(T16<DT>::from_bits(xw.x & 0xFFFFu), tp.s, z) & 0xFFu;
        const uint32_t b = (uint32_t)(int)quant_code<DT>(T16<DT>::from_bits(xw.x >> 16), tp.s, z) & 0xFFu;
        const uint32_t c = (uint32_t)(int)quant_code<DT>(T16<DT>::from_bits(xw.y & 0xFFFFu), tp.s, z) & 0xFFu;
        const uint32_t d = (uint32_t)(int)quant_code<DT>(T16<DT>::from_bits(xw.y >> 16), tp.s, z) & 0xFFu;
        c01 = a | (b << 16);
        c23 = c | (d << 16);
    }
}

// The usual case of quant4 for fp16 (sub2 != 0) on its own, for rounds whose 16 tokens all take it (one test per
// round instead of one branch per token).  The first product x * r reads the fp16 x directly (v_fma_mix_f32 with
// -0 as the addend: x * r + (-0) is the product, sign of zero included), which saves the conversion of x.
__device__ __forceinline__ void quant4_f16_fast(uint2 xw, const TokPar tp, uint32_t &c01, uint32_t &c23) {
    const uint32_t negzero = 0x80000000u;
    float q0[4];
    asm("v_fma_mix_f32 %0, %1, %2, %3 op_sel_hi:[1,0,0]" : "=v"(q0[0]) : "v"(xw.x), "v"(tp.r), "s"(negzero));
    asm("v_fma_mix_f32 %0, %1, %2, %3 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "=v"(q0[1]) : "v"(xw.x), "v"(tp.r), "s"(negzero));
    asm("v_fma_mix_f32 %0, %1, %2, %3 op_sel_hi:[1,0,0]" : "=v"(q0[2]) : "v"(xw.y), "v"(tp.r), "s"(negzero));
    asm("v_fma_mix_f32 %0, %1, %2, %3 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "=v"(q0[3]) : "v"(xw.y), "v"(tp.r), "s"(negzero));
    const f16x2 x01 = __builtin_bit_cast(f16x2, xw.x), x23 = __builtin_bit_cast(f16x2, xw.y);
    const float f[4] = {(float)x01[0], (float)x01[1], (float)x23[0], (float)x23[1]};
    _Float16 h[4];
#pragma unroll
    for (int i = 0; i < 4; i++) h[i] = (_Float16)__fmaf_rn(__fmaf_rn(-tp.s, q0[i], f[i]), tp.r, q0[i]);
    const f16x2 h01 = {h[0], h[1]}, h23 = {h[2], h[3]};
    const f16x2 add = __builtin_bit_cast(f16x2, tp.add2);
    const u16x2 sub = as_u16x2(tp.sub2);
    c01 = pk_u16((u16x2)(__builtin_bit_cast(u16x2, (f16x2)(h01 + add)) - sub));
    c23 = pk_u16((u16x2)(__builtin_bit_cast(u16x2, (f16x2)(h23 + add)) - sub));
}

// ---- x -> uint8 code matrix [T, B*H*128] -----------------------------------------------
// grid (T/16, ceil(H / 4), B), 256 threads: 16 lanes per token, 8 channels per lane, up to four heads per thread with
// all of their rows requested before the first is used; the quotient as in the fused encoders (quant4: the lanes of a
// wavefront hold four different tokens, so each chooses its sequence for itself).
constexpr int kQuantHeads = 4;
template <int DT>
__global__ void __launch_bounds__(256) quantize_kernel(const uint16_t *__restrict__ x, int H, int T,
                                                       const uint16_t *__restrict__ scale, const uint16_t *__restrict__ zero,
                                                       uint8_t *__restrict__ codes, uint32_t *max_code_out) {
    const int b = blockIdx.z, h0 = blockIdx.y * kQuantHeads;
    const int B = gridDim.z;
    const int tok = blockIdx.x * 16 + (threadIdx.x >> 4);
    const int l16 = threadIdx.x & 15;
    const int nh = min(kQuantHeads, H - h0);               // uniform
    uint32_t cmax = 0;
    if (tok < T) {
        uint4 v[kQuantHeads];
#pragma unroll
        for (int i = 0; i < kQuantHeads; i++)
            if (i < nh) v[i] = *reinterpret_cast<const uint4 *>(x + (((size_t)b * H + h0 + i) * T + tok) * kHeadDim + l16 * 8);
        const TokPar tp = token_par<DT>(T16<DT>::from_bits(scale[(size_t)b * T + tok]), zero[(size_t)b * T + tok], false);
        const size_t hidden = (size_t)B * H * kHeadDim;
        uint8_t *row = codes + (size_t)tok * hidden + ((size_t)b * H + h0) * kHeadDim + l16 * 8;
#pragma unroll
        for (int i = 0; i < kQuantHeads; i++) {
            if (i < nh) {
                uint32_t a01, a23, b01, b23;
                quant4<DT, false>(make_uint2(v[i].x, v[i].y), tp, a01, a23);
                quant4<DT, false>(make_uint2(v[i].z, v[i].w), tp, b01, b23);
                const uint32_t lo = __builtin_amdgcn_perm(a23, a01, 0x06040200u), hi = __builtin_amdgcn_perm(b23, b01, 0x06040200u);
                const u16x2 m = __builtin_elementwise_max(__builtin_elementwise_max(as_u16x2(a01 & 0x00FF00FFu), as_u16x2(a23 & 0x00FF00FFu)),
                                                          __builtin_elementwise_max(as_u16x2(b01 & 0x00FF00FFu), as_u16x2(b23 & 0x00FF00FFu)));
                cmax = max(cmax, max((uint32_t)m[0], (uint32_t)m[1]));
                *reinterpret_cast<uint2 *>(row + (size_t)i * kHeadDim) = make_uint2(lo, hi);
            }
        }
    }
    if (max_code_out) {
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) cmax = max(cmax, __shfl_xor(cmax, d, 64));
        // a read first: once the largest code has been seen nobody writes any more (a million atomics on one
        // address would cost milliseconds)
        if ((threadIdx.x & 63) == 0 && cmax > __hip_atomic_load(max_code_out, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))
            atomicMax(max_code_out, cmax);
    }
}

// ---- uint8 code matrix -> x_hat [B, H, T, 128] -----------------------------------------
// the same grid and thread roles
template <int DT>
__global__ void __launch_bounds__(256) dequantize_kernel(const uint8_t *__restrict__ codes, int H, int T,
                                                         const uint16_t *__restrict__ scale, const uint16_t *__restrict__ zero,
                                                         uint16_t *__restrict__ x) {
    const int b = blockIdx.z, h0 = blockIdx.y * kQuantHeads;
    const int B = gridDim.z;
    const int tok = blockIdx.x * 16 + (threadIdx.x >> 4);
    const int l16 = threadIdx.x & 15;
    const int nh = min(kQuantHeads, H - h0);               // uniform
    if (tok >= T) return;
    const size_t hidden = (size_t)B * H * kHeadDim;
    const uint8_t *row = codes + (size_t)tok * hidden + ((size_t)b * H + h0) * kHeadDim + l16 * 8;
    uint2 c[kQuantHeads];
#pragma unroll
    for (int i = 0; i < kQuantHeads; i++)
        if (i < nh) c[i] = *reinterpret_cast<const uint2 *>(row + (size_t)i * kHeadDim);
    const float sc = T16<DT>::from_bits(scale[(size_t)b * T + tok]);
    const float z = T16<DT>::from_bits(zero[(size_t)b * T + tok]);
#pragma unroll
    for (int i = 0; i < kQuantHeads; i++) {
        if (i < nh) {
            uint32_t out[4];
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const uint32_t w = q < 2 ? c[i].x : c[i].y;
                const float a0 = (float)((w >> (16 * (q & 1))) & 0xFFu);
                const float a1 = (float)((w >> (16 * (q & 1) + 8)) & 0xFFu);
                const uint32_t r0 = T16<DT>::to_bits(round_t<DT>(a0 + z) * sc);
                const uint32_t r1 = T16<DT>::to_bits(round_t<DT>(a1 + z) * sc);
                out[q] = r0 | (r1 << 16);
            }
            *reinterpret_cast<uint4 *>(x + (((size_t)b * H + h0 + i) * T + tok) * kHeadDim + l16 * 8) =
                make_uint4(out[0], out[1], out[2], out[3]);
        }
    }
}

// bit_length of both 16-bit halves, clamped to 4 (values above 15 mean the codes overflow the
// format; the launch reports that through max_code)
__device__ __forceinline__ uint32_t pk_bitlen4(uint32_t d) {
    const u16x2 v = as_u16x2(d), one = {1, 1};
    const u16x2 l = __builtin_elementwise_min(v, one) + __builtin_elementwise_min((u16x2)(v >> 1), one) +
                    __builtin_elementwise_min((u16x2)(v >> 2), one) + __builtin_elementwise_min((u16x2)(v >> 3), one);
    return pk_u16(l);
}

// The two packs held in one register pair column: codes c[k] (k = token, two channels per word)
// -> minima, widths and the two 64-bit pack words  sum (c_k - min) << ((15 - k) * len).
__device__ __forceinline__ void build_pair(const uint32_t c[16], uint32_t &mn2, uint32_t &len2, uint32_t &mx2,
                                           uint64_t &w_lo, uint64_t &w_hi) {
    u16x2 mn = as_u16x2(c[0]), mx = as_u16x2(c[0]);
#pragma unroll
    for (int k = 1; k < 16; k++) {
        mn = __builtin_elementwise_min(mn, as_u16x2(c[k]));
        mx = __builtin_elementwise_max(mx, as_u16x2(c[k]));
    }
    mn2 = pk_u16(mn);
    mx2 = pk_u16(mx);
    len2 = pk_bitlen4(pk_u16((u16x2)(mx - mn)));
    const u16x2 one = {1, 1};
    const u16x2 p = one << as_u16x2(len2);                       // 2^len per half
    // quarter windows (4 tokens, 4 * len <= 16 bits), all arithmetic modulo 2^16 per half:
    //   sum c_k p^(3-k) - min (1 + p + p^2 + p^3)
    const u16x2 rep = ((p + one) * p + one) * p + one;
    const u16x2 mnrep = mn * rep;
    uint32_t qw[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        u16x2 w = as_u16x2(c[4 * j]);
        w = w * p + as_u16x2(c[4 * j + 1]);
        w = w * p + as_u16x2(c[4 * j + 2]);
        w = w * p + as_u16x2(c[4 * j + 3]);
        qw[j] = pk_u16((u16x2)(w - mnrep));
    }
    // 64-bit words: tokens 0..7 above tokens 8..15
    const uint32_t l0 = len2 & 0xFFFFu, l1 = len2 >> 16;
    const uint32_t a0 = ((qw[0] & 0xFFFFu) << (4u * l0)) | (qw[1] & 0xFFFFu), b0 = ((qw[2] & 0xFFFFu) << (4u * l0)) | (qw[3] & 0xFFFFu);
    const uint32_t a1 = ((qw[0] >> 16) << (4u * l1)) | (qw[1] >> 16), b1 = ((qw[2] >> 16) << (4u * l1)) | (qw[3] >> 16);
    w_lo = ((uint64_t)a0 << (8u * l0)) | b0;
    w_hi = ((uint64_t)a1 << (8u * l1)) | b1;
}

// running (min, max) of the 8 values of one 16-byte row chunk
template <int DT>
__device__ __forceinline__ void minmax8(const uint4 v, float &mn, float &mx) {
    if (DT == PKV_F16) {   // packed fp16 comparisons, converted once
        const f16x2 a = __builtin_bit_cast(f16x2, v.x), b = __builtin_bit_cast(f16x2, v.y), c = __builtin_bit_cast(f16x2, v.z),
                    d = __builtin_bit_cast(f16x2, v.w);
        const f16x2 lo = __builtin_elementwise_min(__builtin_elementwise_min(a, b), __builtin_elementwise_min(c, d));
        const f16x2 hi = __builtin_elementwise_max(__builtin_elementwise_max(a, b), __builtin_elementwise_max(c, d));
        mn = fminf(mn, fminf((float)lo[0], (float)lo[1]));
        mx = fmaxf(mx, fmaxf((float)hi[0], (float)hi[1]));
    } else {
        float f[8];
        unpack8<DT>(v, f);
#pragma unroll
        for (int i = 0; i < 8; i++) {
            mn = fminf(mn, f[i]);
            mx = fmaxf(mx, f[i]);
        }
    }
}


// min and max over the 16 lanes of a row of the wavefront (every lane gets the results): the exchanges are DPP
// operands of the min / max instructions themselves (quad permutes, then the half-row and row mirrors).
__device__ __forceinline__ void row16_minmax(float &mn, float &mx) {
    // (written out: the compiler keeps the exchanges as separate moves; a VGPR written by a VALU instruction must be
    // two instructions old before a DPP operand reads it, which the interleaving and the s_nop provide)
    asm("s_nop 1\n\t"
        "v_min_f32_dpp %0, %0, %0 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t"
        "v_max_f32_dpp %1, %1, %1 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 0\n\t"
        "v_min_f32_dpp %0, %0, %0 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"
        "v_max_f32_dpp %1, %1, %1 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 0\n\t"
        "v_min_f32_dpp %0, %0, %0 row_half_mirror row_mask:0xf bank_mask:0xf\n\t"
        "v_max_f32_dpp %1, %1, %1 row_half_mirror row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 0\n\t"
        "v_min_f32_dpp %0, %0, %0 row_mirror row_mask:0xf bank_mask:0xf\n\t"
        "v_max_f32_dpp %1, %1, %1 row_mirror row_mask:0xf bank_mask:0xf"
        : "+v"(mn), "+v"(mx));
}
// packed fp16 min / max as the instructions themselves (the builtins first quieten every operand with an extra
// instruction; the instructions ignore quiet NaNs as the builtins do)
__device__ __forceinline__ f16x2 pk_min_h(f16x2 a, f16x2 b) {
    f16x2 r;
    asm("v_pk_min_f16 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}
__device__ __forceinline__ f16x2 pk_max_h(f16x2 a, f16x2 b) {
    f16x2 r;
    asm("v_pk_max_f16 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}

// Token parameters of one round of the round-major encoders for a group of up to four heads (several of which share
// a workgroup).  256 threads per 16 tokens: thread (tt = token, l16) reads 8 channels of every head; lane l16 == 0
// writes the token's scale and zero and its constants for quant4.  `rows` is x at (sequence, head 0, the round's first
// token) and uniform, so the loads are one 32-bit lane offset on scalar bases; only the rows that exist are
// fetched and compared.
template <int DT>
__device__ __forceinline__ void round_token_params_few(const uint16_t *rows, size_t head_stride, int H, int tt, int l16, float rel,
                                                       uint16_t *scale_out, uint16_t *zero_out, TokPar *par_out) {
    const uint32_t lane_off = (uint32_t)(tt * kHeadDim + l16 * 8) * 2u;          // bytes
    uint4 v[4];
    v[0] = *reinterpret_cast<const uint4 *>(reinterpret_cast<const char *>(rows) + lane_off);
#pragma unroll
    for (int i = 1; i < 4; i++)
        if (i < H) v[i] = *reinterpret_cast<const uint4 *>(reinterpret_cast<const char *>(rows + (size_t)i * head_stride) + lane_off);
    float mn, mx;
    if (DT == PKV_F16) {
        f16x2 lo, hi;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            if (i < H) {
                const f16x2 a = __builtin_bit_cast(f16x2, v[i].x), b = __builtin_bit_cast(f16x2, v[i].y),
                            c = __builtin_bit_cast(f16x2, v[i].z), d = __builtin_bit_cast(f16x2, v[i].w);
                const f16x2 l = pk_min_h(pk_min_h(a, b), pk_min_h(c, d)), h = pk_max_h(pk_max_h(a, b), pk_max_h(c, d));
                lo = i ? pk_min_h(lo, l) : l;
                hi = i ? pk_max_h(hi, h) : h;
            }
        }
        mn = fminf((float)lo[0], (float)lo[1]);
        mx = fmaxf((float)hi[0], (float)hi[1]);
    } else {
        mn = INFINITY, mx = -INFINITY;
#pragma unroll
        for (int i = 0; i < 4; i++)
            if (i < H) minmax8<DT>(v[i], mn, mx);
    }
    row16_minmax(mn, mx);
    if (l16 == 0) {
        const float range = round_t<DT>(mx - mn);
        const float sc = round_t<DT>(range * rel);
        const uint32_t zb = T16<DT>::to_bits(rintf(round_t<DT>(__fdiv_rn(mn, sc))));
        *scale_out = (uint16_t)T16<DT>::to_bits(sc);
        *zero_out = (uint16_t)zb;
        *par_out = token_par<DT>(sc, zb, false);
    }
}

__device__ __forceinline__ void cell_load(const uint16_t *xc, uint2 xr[16]) {
#pragma unroll
    for (int k = 0; k < 16; k++) xr[k] = *reinterpret_cast<const uint2 *>(xc + (size_t)k * kHeadDim);
}

// The same cell from permuted rows: row k is token rows[k] (uniform: the indices come from scalar loads) of the
// tokens that start at `seq`, which is uniform too; `lane_off` is the lane's byte offset inside a token's rows.
__device__ __forceinline__ void cell_load_rows(const uint16_t *seq, const uint32_t *rows, uint32_t last_row, uint32_t lane_off, uint2 xr[16]) {
#pragma unroll
    for (int k = 0; k < 16; k++)                          // (row indices clamped: a damaged order cannot read outside the block)
        xr[k] = *reinterpret_cast<const uint2 *>(reinterpret_cast<const char *>(seq + (size_t)min(rows[k], last_row) * kHeadDim) + lane_off);
}

// The same when the lanes of a wavefront do not share their rows (`rows` differs between lanes; 64-byte aligned): the
// 16 indices are loaded by the lane itself and the row offsets are per-lane 32-bit offsets on the uniform base.
__device__ __forceinline__ void cell_load_rows_lanes(const uint16_t *seq, const uint32_t *rows, uint32_t last_row, uint32_t lane_off, uint2 xr[16]) {
    uint4 idx[4];
#pragma unroll
    for (int q = 0; q < 4; q++) idx[q] = reinterpret_cast<const uint4 *>(rows)[q];
#pragma unroll
    for (int k = 0; k < 16; k++) {
        const uint4 v = idx[k >> 2];
        const uint32_t row = min((k & 3) == 0 ? v.x : (k & 3) == 1 ? v.y : (k & 3) == 2 ? v.z : v.w, last_row);
        xr[k] = *reinterpret_cast<const uint2 *>(reinterpret_cast<const char *>(seq) + (row * (uint32_t)(kHeadDim * 2) + lane_off));
    }
}

// (general_form: the constants of the general sequence whatever the zero point -- for callers whose wavefronts hold
// several tokens and must take one path for all of them)
template <int DT>
__device__ __forceinline__ TokPar token_par(float sc, uint32_t zero_bits, bool general_form) {
    float r = __builtin_amdgcn_rcpf(sc);
    r = __fmaf_rn(__fmaf_rn(-sc, r, 1.f), r, r);
    TokPar tp;
    tp.s = sc;
    tp.r = r;
    tp.sub2 = 0;
    if (DT == PKV_F16) {
        const float z = T16<DT>::from_bits(zero_bits);        // an integer (or inf / nan for degenerate tokens)
        if (!general_form && z >= -500.f && z <= 3000.f) {
            const int zi = (int)z, odd = zi & 1;
            tp.add2 = (uint32_t)__half_as_ushort(__float2half_rn((float)(1536 + odd - zi))) * 0x00010001u;   // exact: |c| < 2048
            tp.sub2 = (uint32_t)(0x6600 + odd) * 0x00010001u;
        } else {
            tp.add2 = (zero_bits ^ 0x8000u) * 0x00010001u;
        }
    } else {
        const float z = T16<DT>::from_bits(zero_bits);        // an integer (or inf / nan for degenerate tokens)
        if (!general_form && fabsf(z) <= 1048576.f) {       // 2^23 - zero and the sums below stay exact
            tp.add2 = __float_as_uint(8388608.f - z);
            tp.sub2 = 1u;
        } else {
            tp.add2 = __float_as_uint(z);
        }
    }
    return tp;
}

// True (uniformly) when all 16 tokens of the round at `par` (LDS) take the usual case of quant4.
__device__ __forceinline__ bool round_all_fast(const TokPar *par) {
    const uint32_t sub2 = par[threadIdx.x & 15].sub2;
    return !__any(sub2 == 0u);
}

// The codes of a loaded cell (rows xr, the 16 tokens' constants at par) as pairs of 16-bit integers.
template <int DT, bool UNIFORM = true>
__device__ __forceinline__ void cell_quant(const uint2 xr[16], const TokPar *par, uint32_t c01[16], uint32_t c23[16]) {
    if (DT == PKV_F16 && round_all_fast(par)) {
#pragma unroll
        for (int k = 0; k < 16; k++) quant4_f16_fast(xr[k], par[k], c01[k], c23[k]);
    } else {
#pragma unroll
        for (int k = 0; k < 16; k++) quant4<DT, UNIFORM>(xr[k], par[k], c01[k], c23[k]);
    }
}

// The four packs of a cell's codes: words, minima, widths.
__device__ __forceinline__ void cell_build(const uint32_t c01[16], const uint32_t c23[16], UnitPacks &u, uint32_t &cmax) {
    uint32_t mn01, mn23, len01, len23, mx01, mx23;
    build_pair(c01, mn01, len01, mx01, u.word[0], u.word[1]);
    build_pair(c23, mn23, len23, mx23, u.word[2], u.word[3]);
    const u16x2 m = __builtin_elementwise_max(as_u16x2(mx01), as_u16x2(mx23));
    cmax = max((uint32_t)m[0], (uint32_t)m[1]);
    u.mn[0] = mn01 & 0xFFFFu; u.mn[1] = mn01 >> 16; u.mn[2] = mn23 & 0xFFFFu; u.mn[3] = mn23 >> 16;
    u.len[0] = len01 & 0xFFFFu; u.len[1] = len01 >> 16; u.len[2] = len23 & 0xFFFFu; u.len[3] = len23 >> 16;
}

// The four packs of a loaded cell (rows xr, the 16 tokens' constants at par): words, minima, widths.
template <int DT>
__device__ __forceinline__ void cell_packs(const uint2 xr[16], const TokPar *par, UnitPacks &u, uint32_t &cmax) {
    uint32_t c01[16], c23[16];
    if (DT == PKV_F16 && round_all_fast(par)) {
#pragma unroll
        for (int k = 0; k < 16; k++) quant4_f16_fast(xr[k], par[k], c01[k], c23[k]);
    } else {
#pragma unroll
        for (int k = 0; k < 16; k++) quant4<DT>(xr[k], par[k], c01[k], c23[k]);
    }
    uint32_t mn01, mn23, len01, len23, mx01, mx23;
    build_pair(c01, mn01, len01, mx01, u.word[0], u.word[1]);
    build_pair(c23, mn23, len23, mx23, u.word[2], u.word[3]);
    const u16x2 m = __builtin_elementwise_max(as_u16x2(mx01), as_u16x2(mx23));
    cmax = max((uint32_t)m[0], (uint32_t)m[1]);
    u.mn[0] = mn01 & 0xFFFFu; u.mn[1] = mn01 >> 16; u.mn[2] = mn23 & 0xFFFFu; u.mn[3] = mn23 >> 16;
    u.len[0] = len01 & 0xFFFFu; u.len[1] = len01 >> 16; u.len[2] = len23 & 0xFFFFu; u.len[3] = len23 >> 16;
}

// ---- widths 5 and 6 (extension of the format) in the round-major encoders ------------------------------------
// A pack word grows to 16 * len <= 96 bits.  It is kept as two halves of 8 * len bits -- `hi` tokens 0..7, `lo`
// tokens 8..15 -- and since 8 * len bits are len whole bytes, the word's 2 * len bytes in the stream are simply the
// bytes of `lo` followed by the bytes of `hi`.  The halves are assembled from windows of TWO tokens (2 * len <= 12
// bits fit the packed 16-bit arithmetic the quarter windows of the reference's widths use).
struct UnitPacksW {
    uint64_t lo[4], hi[4];
    uint32_t len[4];
    uint32_t mn[4];
    uint32_t off[4];
    uint32_t payload;
};

// bit_length of both 16-bit halves, clamped to 6
__device__ __forceinline__ uint32_t pk_bitlen6(uint32_t d) {
    const u16x2 v = as_u16x2(d), one = {1, 1};
    u16x2 l = __builtin_elementwise_min(v, one);
#pragma unroll
    for (int k = 1; k < 6; k++) l += __builtin_elementwise_min((u16x2)(v >> (uint16_t)k), one);
    return pk_u16(l);
}

__device__ __forceinline__ uint64_t join4(uint32_t e0, uint32_t e1, uint32_t e2, uint32_t e3, uint32_t l2) {
    return ((((((uint64_t)e0 << l2) | e1) << l2) | e2) << l2) | e3;      // l2 = 2 * len
}

__device__ __forceinline__ void build_pair_wide(const uint32_t c[16], uint32_t &mn2, uint32_t &len2, uint32_t &mx2,
                                                uint64_t &lo_a, uint64_t &hi_a, uint64_t &lo_b, uint64_t &hi_b) {
    u16x2 mn = as_u16x2(c[0]), mx = as_u16x2(c[0]);
#pragma unroll
    for (int k = 1; k < 16; k++) {
        mn = __builtin_elementwise_min(mn, as_u16x2(c[k]));
        mx = __builtin_elementwise_max(mx, as_u16x2(c[k]));
    }
    mn2 = pk_u16(mn);
    mx2 = pk_u16(mx);
    len2 = pk_bitlen6(pk_u16((u16x2)(mx - mn)));
    const u16x2 one = {1, 1};
    const u16x2 p = one << as_u16x2(len2);                       // 2^len per half
    const u16x2 mnrep = mn * (p + one);
    uint32_t ew[8];                                              // tokens 2j, 2j+1: (c - min) p + (c' - min) < 2^12
#pragma unroll
    for (int j = 0; j < 8; j++) ew[j] = pk_u16((u16x2)(as_u16x2(c[2 * j]) * p + as_u16x2(c[2 * j + 1]) - mnrep));
    const uint32_t l0 = 2u * (len2 & 0xFFFFu), l1 = 2u * (len2 >> 16);
    hi_a = join4(ew[0] & 0xFFFFu, ew[1] & 0xFFFFu, ew[2] & 0xFFFFu, ew[3] & 0xFFFFu, l0);
    lo_a = join4(ew[4] & 0xFFFFu, ew[5] & 0xFFFFu, ew[6] & 0xFFFFu, ew[7] & 0xFFFFu, l0);
    hi_b = join4(ew[0] >> 16, ew[1] >> 16, ew[2] >> 16, ew[3] >> 16, l1);
    lo_b = join4(ew[4] >> 16, ew[5] >> 16, ew[6] >> 16, ew[7] >> 16, l1);
}

__device__ __forceinline__ void cell_build(const uint32_t c01[16], const uint32_t c23[16], UnitPacksW &u, uint32_t &cmax) {
    uint32_t mn01, mn23, len01, len23, mx01, mx23;
    build_pair_wide(c01, mn01, len01, mx01, u.lo[0], u.hi[0], u.lo[1], u.hi[1]);
    build_pair_wide(c23, mn23, len23, mx23, u.lo[2], u.hi[2], u.lo[3], u.hi[3]);
    const u16x2 m = __builtin_elementwise_max(as_u16x2(mx01), as_u16x2(mx23));
    cmax = max((uint32_t)m[0], (uint32_t)m[1]);
    u.mn[0] = mn01 & 0xFFFFu; u.mn[1] = mn01 >> 16; u.mn[2] = mn23 & 0xFFFFu; u.mn[3] = mn23 >> 16;
    u.len[0] = len01 & 0xFFFFu; u.len[1] = len01 >> 16; u.len[2] = len23 & 0xFFFFu; u.len[3] = len23 >> 16;
}

template <int DT>
__device__ __forceinline__ void cell_packs(const uint2 xr[16], const TokPar *par, UnitPacksW &u, uint32_t &cmax) {
    uint32_t c01[16], c23[16];
    if (DT == PKV_F16 && round_all_fast(par)) {
#pragma unroll
        for (int k = 0; k < 16; k++) quant4_f16_fast(xr[k], par[k], c01[k], c23[k]);
    } else {
#pragma unroll
        for (int k = 0; k < 16; k++) quant4<DT>(xr[k], par[k], c01[k], c23[k]);
    }
    uint32_t mn01, mn23, len01, len23, mx01, mx23;
    build_pair_wide(c01, mn01, len01, mx01, u.lo[0], u.hi[0], u.lo[1], u.hi[1]);
    build_pair_wide(c23, mn23, len23, mx23, u.lo[2], u.hi[2], u.lo[3], u.hi[3]);
    const u16x2 m = __builtin_elementwise_max(as_u16x2(mx01), as_u16x2(mx23));
    cmax = max((uint32_t)m[0], (uint32_t)m[1]);
    u.mn[0] = mn01 & 0xFFFFu; u.mn[1] = mn01 >> 16; u.mn[2] = mn23 & 0xFFFFu; u.mn[3] = mn23 >> 16;
    u.len[0] = len01 & 0xFFFFu; u.len[1] = len01 >> 16; u.len[2] = len23 & 0xFFFFu; u.len[3] = len23 >> 16;
}

template <bool WIDE> struct PacksOf { typedef UnitPacks type; };
template <> struct PacksOf<true> { typedef UnitPacksW type; };

// the 2 * len bytes of pack k at dst (2-byte aligned): one predicated 16-bit store per piece, written out (a loop
// over the lane's own length costs a shift, a compare and the loop's control flow per piece)
__device__ __forceinline__ void put_pack(uint16_t *dst, const UnitPacks &u, int k) {
    const uint32_t lo = (uint32_t)u.word[k], hi = (uint32_t)(u.word[k] >> 32), len = u.len[k];
    if (len > 0u) dst[0] = (uint16_t)lo;
    if (len > 1u) dst[1] = (uint16_t)(lo >> 16);
    if (len > 2u) dst[2] = (uint16_t)hi;
    if (len > 3u) dst[3] = (uint16_t)(hi >> 16);
}
__device__ __forceinline__ void put_pack(uint16_t *dst, const UnitPacksW &u, int k) {
    const unsigned __int128 wd = ((unsigned __int128)u.hi[k] << (8u * u.len[k])) | u.lo[k];
    const uint32_t d0 = (uint32_t)wd, d1 = (uint32_t)(wd >> 32), d2 = (uint32_t)(wd >> 64), len = u.len[k];
    if (len > 0u) dst[0] = (uint16_t)d0;
    if (len > 1u) dst[1] = (uint16_t)(d0 >> 16);
    if (len > 2u) dst[2] = (uint16_t)d1;
    if (len > 3u) dst[3] = (uint16_t)(d1 >> 16);
    if (len > 4u) dst[4] = (uint16_t)d2;
    if (len > 5u) dst[5] = (uint16_t)(d2 >> 16);
}

// Emit one analysed unit at blk[unit_off] (the K layout: lane t's packs sit where they were computed).
template <class U>
__device__ __forceinline__ void unit_emit_any(uint8_t *blk, uint32_t unit_off, int t, const UnitGeom g, const U &u) {
    uint32_t minsw = 0, lensw = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        minsw |= u.mn[i] << (i * g.W);
        lensw |= u.len[i] << (i * g.LB);
    }
    lds_put_meta(blk + unit_off, t, g.W, minsw);
    lds_put_meta(blk + unit_off + g.mins_bytes, t, g.LB, lensw);
    uint8_t *pay = blk + unit_off + g.mins_bytes + g.lens_bytes;
#pragma unroll
    for (int i = 0; i < 4; i++) put_pack(reinterpret_cast<uint16_t *>(pay + u.off[i]), u, i);
}

// A group is the run of blocks that share one (context block, sequence): H blocks for K, 2 H for V, consecutive in
// stream order.  The encoders below give a workgroup the blocks of up to eight heads of a group.
constexpr int kSubBlocks = 8;

// Wave priorities (s_setprio) of the round-major encoders' phases: the parameter pass goes first, so that its rows
// are requested from HBM as early as possible; forming the packs, the long arithmetic phase, yields to everything
// else.  Worth 3-4 % (0.392 -> 0.377 ms for K, 0.431 -> 0.414 ms for V on 1 GiB of input).
#ifndef PKV_EPRIO_STAT
#define PKV_EPRIO_STAT 3
#define PKV_EPRIO_PACK 0
#define PKV_EPRIO_EMIT 2
#endif

// Copy n bytes (even) from LDS (src 4-byte aligned, readable up to 20 bytes past n) to global memory (dst 2-byte
// aligned) with the 32 lanes of a half-wavefront: head to the first 16-byte boundary and tail in 2-byte pieces, the
// body as aligned 16-byte stores fed by aligned LDS reads and byte funnel shifts.
__device__ __forceinline__ void copy_out32(uint8_t *dst, const uint8_t *src, uint32_t n, int t) {
    const uint32_t head = min(n, (uint32_t)((16u - (uint32_t)(reinterpret_cast<uintptr_t>(dst) & 15u)) & 15u));
    const uint32_t nq = (n - head) >> 4;
    for (uint32_t i = t; i < (head >> 1); i += 32)
        reinterpret_cast<uint16_t *>(dst)[i] = reinterpret_cast<const uint16_t *>(src)[i];
    const uint32_t *src32 = reinterpret_cast<const uint32_t *>(src + (head & ~3u));
    for (uint32_t i = t; i < nq; i += 32) {
        const uint32_t *q = src32 + 4 * i;
        const uint32_t d0 = q[0], d1 = q[1], d2 = q[2], d3 = q[3], d4 = q[4];
        uint4 v;
        v.x = __builtin_amdgcn_alignbyte(d1, d0, head);
        v.y = __builtin_amdgcn_alignbyte(d2, d1, head);
        v.z = __builtin_amdgcn_alignbyte(d3, d2, head);
        v.w = __builtin_amdgcn_alignbyte(d4, d3, head);
        *reinterpret_cast<uint4 *>(dst + head + 16 * (size_t)i) = v;
    }
    const uint32_t done = head + 16u * nq;
    for (uint32_t i = t; i < ((n - done) >> 1); i += 32)
        reinterpret_cast<uint16_t *>(dst + done)[i] = reinterpret_cast<const uint16_t *>(src + done)[i];
}

// Minimum and maximum of every token of a round over a wavefront's cells.  Lane's cell: rows xr[k] = token
// k, four channels.  The 16 per-token values of a lane are reduced and transposed at once: each step exchanges half
// of the registers with the lane 32, 16, 8, 4 positions away and keeps the other half, so the register count halves
// while the lanes behind a value double -- v_permlane32_swap / v_permlane16_swap trade whole half-wavefronts and
// rows between two registers, the two steps inside a row are DPP moves under bank masks.  Afterwards lane l holds
// token l / 4 (all four lanes of a quad the same): ~120 vector instructions instead of a second pass over the rows.
// (The packed min / max are written as instructions, see pk_min_h; a lane exchange must not read a register that a
// vector instruction wrote less than two instructions earlier, and the compiler does not see into the assembly, so
// these carry their own two wait states.)
// KEYS: the operands are order keys of bf16 values (bf16_keys), compared as signed 16-bit integers.
template <bool MAX, bool KEYS>
__device__ __forceinline__ uint32_t pk_sel_x(uint32_t a, uint32_t b) {
    uint32_t r;
    if (KEYS) {
        if (MAX) asm("v_pk_max_i16 %0, %1, %2\n\ts_nop 1" : "=v"(r) : "v"(a), "v"(b));
        else asm("v_pk_min_i16 %0, %1, %2\n\ts_nop 1" : "=v"(r) : "v"(a), "v"(b));
    } else {
        if (MAX) asm("v_pk_max_f16 %0, %1, %2\n\ts_nop 1" : "=v"(r) : "v"(a), "v"(b));
        else asm("v_pk_min_f16 %0, %1, %2\n\ts_nop 1" : "=v"(r) : "v"(a), "v"(b));
    }
    return r;
}
// bf16 has no packed min / max: both halves of a word become 16-bit integers that order like the values (negative
// values have their magnitude bits flipped); the map is its own inverse.
__device__ __forceinline__ uint32_t bf16_keys(uint32_t w) {
    typedef short i16x2 __attribute__((ext_vector_type(2)));
    const i16x2 v = __builtin_bit_cast(i16x2, w);
    const i16x2 m = (v >> (short)15) & (short)0x7FFF;
    return __builtin_bit_cast(uint32_t, (i16x2)(v ^ m));
}
// A token's (minimum, maximum) as one word that a packed MINIMUM combines: the minimum in the low half, the negated
// maximum in the high half (fp16: sign bit flipped; bf16: both as order keys, the maximum's complemented).
template <int DT>
__device__ __forceinline__ uint32_t minmax_word(float mn, float mx) {
    if (DT == PKV_F16) return T16<DT>::to_bits(mn) | ((T16<DT>::to_bits(mx) ^ 0x8000u) << 16);
    return bf16_keys(T16<DT>::to_bits(mn) | (T16<DT>::to_bits(mx) << 16)) ^ 0xFFFF0000u;
}
template <int DT>
__device__ __forceinline__ void minmax_unword(uint32_t w, float &mn, float &mx) {
    if (DT != PKV_F16) w = bf16_keys(w ^ 0xFFFF0000u);
    else w ^= 0x80000000u;
    mn = T16<DT>::from_bits(w & 0xFFFFu);
    mx = T16<DT>::from_bits(w >> 16);
}
template <bool MAX, bool KEYS>
__device__ __forceinline__ uint32_t swap32_sel(uint32_t a, uint32_t b) {
    const auto r = __builtin_amdgcn_permlane32_swap(a, b, false, false);
    return pk_sel_x<MAX, KEYS>((uint32_t)r[0], (uint32_t)r[1]);
}
template <bool MAX, bool KEYS>
__device__ __forceinline__ uint32_t swap16_sel(uint32_t a, uint32_t b) {
    const auto r = __builtin_amdgcn_permlane16_swap(a, b, false, false);
    return pk_sel_x<MAX, KEYS>((uint32_t)r[0], (uint32_t)r[1]);
}
// lanes whose bank is in HI_BANKS keep b and meet the partner's b, the others keep a and meet the partner's a;
// CTRL_LO / CTRL_HI: how the low / high banks read their partner
template <bool MAX, bool KEYS, int CTRL_LO, int CTRL_HI, int HI_BANKS>
__device__ __forceinline__ uint32_t row_step_sel(uint32_t a, uint32_t b) {
    const int mine = __builtin_amdgcn_update_dpp((int)a, (int)b, 0xE4, 0xF, HI_BANKS, false);
    int theirs = __builtin_amdgcn_update_dpp(0, (int)a, CTRL_LO, 0xF, 0xF ^ HI_BANKS, false);
    theirs = __builtin_amdgcn_update_dpp(theirs, (int)b, CTRL_HI, 0xF, HI_BANKS, false);
    return pk_sel_x<MAX, KEYS>((uint32_t)mine, (uint32_t)theirs);
}
// one side (minimum or maximum) of cell_token_minmax as packed halves: lane l holds token l / 4, two channel parities
template <int DT, bool MAX>
__device__ __forceinline__ uint32_t cell_token_side(const uint2 xr[16]) {
    constexpr bool KEYS = DT != PKV_F16;
    uint32_t v[16];
#pragma unroll
    for (int k = 0; k < 16; k++)
        v[k] = KEYS ? pk_sel_x<MAX, true>(bf16_keys(xr[k].x), bf16_keys(xr[k].y)) : pk_sel_x<MAX, false>(xr[k].x, xr[k].y);
#pragma unroll
    for (int k = 0; k < 8; k++) v[k] = swap32_sel<MAX, KEYS>(v[k], v[k + 8]);          // lanes 0..31: token k, lanes 32..63: token k + 8
#pragma unroll
    for (int k = 0; k < 4; k++) v[k] = swap16_sel<MAX, KEYS>(v[k], v[k + 4]);          // row rho: token k + 4 rho
#pragma unroll
    for (int k = 0; k < 2; k++) v[k] = row_step_sel<MAX, KEYS, 0x128, 0x128, 0xC>(v[k], v[k + 2]);   // lanes 8..15 of a row: token k + 2 + 4 rho
    const uint32_t r = row_step_sel<MAX, KEYS, 0x104, 0x114, 0xA>(v[0], v[1]);         // banks 1, 3: the odd token; token = lane / 4
    return KEYS ? bf16_keys(r) : r;
}
template <int DT>
__device__ __forceinline__ void cell_token_minmax(const uint2 xr[16], float &mn, float &mx) {
    const uint32_t lo = cell_token_side<DT, false>(xr);
    __builtin_amdgcn_sched_barrier(0);                     // (one side after the other: 16 registers in flight, not 32)
    const uint32_t hi = cell_token_side<DT, true>(xr);
    mn = fminf(T16<DT>::from_bits(lo & 0xFFFFu), T16<DT>::from_bits(lo >> 16));
    mx = fmaxf(T16<DT>::from_bits(hi & 0xFFFFu), T16<DT>::from_bits(hi >> 16));
    asm("s_nop 1\n\t"
        "v_min_f32_dpp %0, %0, %0 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t"
        "v_max_f32_dpp %1, %1, %1 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 0\n\t"
        "v_min_f32_dpp %0, %0, %0 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"
        "v_max_f32_dpp %1, %1, %1 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf"
        : "+v"(mn), "+v"(mx));
}

// The same for a wavefront whose two halves hold different rounds (lanes 0..31 the tokens of one round, lanes 32..63
// those of the next): the reduction stays inside the halves -- rows, then 8, 4 and 2 lanes -- and lane l ends up
// with token l / 2 of the 32.
template <int DT, bool MAX>
__device__ __forceinline__ uint32_t cell_token_side_halves(const uint2 xr[16], bool odd_pair) {
    constexpr bool KEYS = DT != PKV_F16;
    uint32_t v[16];
#pragma unroll
    for (int k = 0; k < 16; k++)
        v[k] = KEYS ? pk_sel_x<MAX, true>(bf16_keys(xr[k].x), bf16_keys(xr[k].y)) : pk_sel_x<MAX, false>(xr[k].x, xr[k].y);
#pragma unroll
    for (int k = 0; k < 8; k++) v[k] = swap16_sel<MAX, KEYS>(v[k], v[k + 8]);          // odd rows: token k + 8
#pragma unroll
    for (int k = 0; k < 4; k++) v[k] = row_step_sel<MAX, KEYS, 0x128, 0x128, 0xC>(v[k], v[k + 4]);   // lanes 8..15 of a row: + 4
#pragma unroll
    for (int k = 0; k < 2; k++) v[k] = row_step_sel<MAX, KEYS, 0x104, 0x114, 0xA>(v[k], v[k + 2]);   // banks 1, 3: + 2
    // lanes 2, 3 of a quad: + 1 (no bank mask reaches inside a quad: selects, and the exchange as a quad permute)
    const uint32_t mine = odd_pair ? v[1] : v[0], send = odd_pair ? v[0] : v[1];
    const uint32_t theirs = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)send, 0x4E, 0xF, 0xF, false);
    const uint32_t r = pk_sel_x<MAX, KEYS>(mine, theirs);
    return KEYS ? bf16_keys(r) : r;
}
template <int DT>
__device__ __forceinline__ void cell_token_minmax_halves(const uint2 xr[16], float &mn, float &mx) {
    const bool odd_pair = (threadIdx.x & 2) != 0;
    const uint32_t lo = cell_token_side_halves<DT, false>(xr, odd_pair);
    __builtin_amdgcn_sched_barrier(0);
    const uint32_t hi = cell_token_side_halves<DT, true>(xr, odd_pair);
    mn = fminf(T16<DT>::from_bits(lo & 0xFFFFu), T16<DT>::from_bits(lo >> 16));
    mx = fmaxf(T16<DT>::from_bits(hi & 0xFFFFu), T16<DT>::from_bits(hi >> 16));
    asm("s_nop 1\n\t"
        "v_min_f32_dpp %0, %0, %0 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t"
        "v_max_f32_dpp %1, %1, %1 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf"
        : "+v"(mn), "+v"(mx));
}

// ---- K, all heads in one workgroup, x read ONCE as cells ----------------------------------------
// The round-major encoder above reads a round's rows twice: once row-wise for the token parameters (the trip that
// goes to HBM and whose latency every round waits out) and again as cells.  Here a round is read as cells only; the
// token minima and maxima come from the cell registers (cell_token_minmax: per wavefront, then four partial
// results per token through LDS, from which every wavefront forms the round's parameters for itself, so a round
// has one barrier), and the next round's cells are requested as soon as this round's are quantized -- into the same
// registers -- so that they travel while the packs are formed and emitted.  For 5..8 heads (one group per
// workgroup); PERM as in the round-major kernel.  Same stream, parameters and block_info as that kernel.
template <int DT, bool WIDE, bool PERM, bool XCH = false>
__global__ void __launch_bounds__(256) k_quant_encode_cells_kernel(
    const uint16_t *__restrict__ x, int B, int H, int T, float rel, uint16_t *__restrict__ scale,
    uint16_t *__restrict__ zero, uint8_t *__restrict__ stream, uint64_t capacity, uint32_t *__restrict__ info,
    ScanState *st, int W, uint32_t ngroups, uint32_t bound, uint64_t base, int par_stride,
    const uint32_t *__restrict__ perm, int perm_block, const Stagger stagger, int nsg = 1, uint64_t *xw = nullptr) {
    extern __shared__ __align__(16) uint8_t gbuf[];        // H block slots of `bound` bytes
    __shared__ uint32_t s_idx;
    __shared__ uint64_t s_off;
    __shared__ uint32_t blk_off[kSubBlocks + 1];
    __shared__ __attribute__((aligned(16))) TokPar s_par[4 * 16];       // [wavefront][token of the round]
    __shared__ float2 s_mm[2][4][16];                                    // [round parity][wavefront][token]: (min, max)
    const int tid = threadIdx.x;
    stagger_first_generation(stagger);
    if (tid == 0) s_idx = atomicAdd(&st->ticket, 1u);
    __syncthreads();
    const uint32_t gidx = (uint32_t)__builtin_amdgcn_readfirstlane((int)s_idx);
    if (gidx >= ngroups) return;
    // XCH (more than eight heads): runs of eight heads, one workgroup and one ticket each, as in the round-major
    // kernel: a run forms the minima and maxima over its own heads, publishes them per token and collects the others'.
    const int H_all = H;
    const uint32_t sgi = XCH ? gidx % (uint32_t)nsg : 0u;
    const int hbase = XCH ? 8 * (int)sgi : 0;
    if (XCH) H = min(8, H_all - hbase);
    const int j = tid >> 5, t = tid & 31, wave = tid >> 6, lane = tid & 63;
    const uint32_t grp = XCH ? gidx / (uint32_t)nsg : gidx;
    const uint32_t cb = grp / (uint32_t)B, b = grp % (uint32_t)B;
    const size_t tok0 = (size_t)cb * 64;
    const UnitGeom g = unit_geom(W);
    const bool active = j < H;
    const int jc = min(j, H - 1);                          // (a repeated head changes no minimum or maximum)
    const TokPar *my_par = XCH ? s_par : s_par + 16 * wave;
    uint8_t *blk = gbuf + (size_t)j * bound;
    uint32_t my_off = 8u;
    uint32_t cmax_all = 0;
    const uint16_t *cells = x + (((size_t)b * H_all + hbase + jc) * T + tok0) * kHeadDim + 4 * t;
    // PERM: the rows of a round are tokens perm[...] of the repacking block that holds this context block
    const uint16_t *pseq = x + (((size_t)b * H) * T + (tok0 / (size_t)(PERM ? perm_block : 1)) * (size_t)(PERM ? perm_block : 1)) * kHeadDim;
    const uint32_t plane = (uint32_t)(((size_t)jc * T * kHeadDim + 4 * t) * 2);
    // (bf16 with the wide packs or with the exchange between runs would need more than 128 registers to keep a round
    // in flight: it asks at the top)
    constexpr bool AHEAD = !((WIDE || XCH) && DT != PKV_F16);
    uint2 xr[16];
    if (AHEAD) {
        if (PERM) cell_load_rows(pseq, perm + tok0, (uint32_t)perm_block - 1u, plane, xr);
        else cell_load(cells, xr);
    }
#pragma unroll 1
    for (int r = 0; r < 4; r++) {
        if (!AHEAD) {
            if (PERM) cell_load_rows(pseq, perm + tok0 + 16 * r, (uint32_t)perm_block - 1u, plane, xr);
            else cell_load(cells + (size_t)r * 16 * kHeadDim, xr);
        }
        __builtin_amdgcn_s_setprio(PKV_EPRIO_STAT);
        {
            float mn, mx;
            cell_token_minmax<DT>(xr, mn, mx);
            if ((lane & 3) == 0) s_mm[r & 1][wave][lane >> 2] = make_float2(mn, mx);
        }
        __syncthreads();
        if (XCH) {
            if (wave == 0) {
                const int tk = lane & 15;
                const float2 p0 = s_mm[r & 1][0][tk], p1 = s_mm[r & 1][1][tk], p2 = s_mm[r & 1][2][tk], p3 = s_mm[r & 1][3][tk];
                const float rmn = fminf(fminf(p0.x, p1.x), fminf(p2.x, p3.x)), rmx = fmaxf(fmaxf(p0.y, p1.y), fmaxf(p2.y, p3.y));
                uint64_t *words = xw + ((size_t)(gidx - sgi) * 4 + r) * 16;       // [run][round][token] of this group
                if (lane < 16)
                    __hip_atomic_store(words + (size_t)sgi * 64 + lane, (1ull << 63) | ((uint64_t)T16<DT>::to_bits(rmn) << 16) | (uint64_t)T16<DT>::to_bits(rmx),
                                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                // lane = (run, token) for up to four runs at a time
                float amn = INFINITY, amx = -INFINITY;
                for (int s0 = 0; s0 < nsg; s0 += 4) {
                    const int run = s0 + (lane >> 4);
                    if (run < nsg) {
                        const uint64_t *wp = words + (size_t)run * 64 + tk;
                        uint64_t w = __hip_atomic_load(wp, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        int spins = 0;
                        while ((w >> 63) == 0 && spins < kSpinLimit) {
                            __builtin_amdgcn_s_sleep(8);
                            w = __hip_atomic_load(wp, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                            spins++;
                        }
                        if ((w >> 63) == 0) atomicExch(&st->error, (uint32_t)PKV_ERR_INTERNAL);     // (bounded wait: the host reports it)
                        amn = fminf(amn, T16<DT>::from_bits((uint32_t)(w >> 16) & 0xFFFFu));
                        amx = fmaxf(amx, T16<DT>::from_bits((uint32_t)w & 0xFFFFu));
                    }
                }
                amn = fminf(amn, __shfl_xor(amn, 16, 64)); amx = fmaxf(amx, __shfl_xor(amx, 16, 64));
                amn = fminf(amn, __shfl_xor(amn, 32, 64)); amx = fmaxf(amx, __shfl_xor(amx, 32, 64));
                if (lane < 16) {
                    const float range = round_t<DT>(amx - amn);
                    const float sc = round_t<DT>(range * rel);
                    const uint32_t zb = T16<DT>::to_bits(rintf(round_t<DT>(__fdiv_rn(amn, sc))));
                    if (sgi == 0) {
                        const size_t tok = (size_t)b * par_stride + tok0 + 16 * r + lane;
                        scale[tok] = (uint16_t)T16<DT>::to_bits(sc);
                        zero[tok] = (uint16_t)zb;
                    }
                    s_par[lane] = token_par<DT>(sc, zb, false);
                }
            }
            __syncthreads();
        } else if (lane < 16) {
            const float2 p0 = s_mm[r & 1][0][lane], p1 = s_mm[r & 1][1][lane], p2 = s_mm[r & 1][2][lane], p3 = s_mm[r & 1][3][lane];
            const float mn = fminf(fminf(p0.x, p1.x), fminf(p2.x, p3.x)), mx = fmaxf(fmaxf(p0.y, p1.y), fmaxf(p2.y, p3.y));
            const float range = round_t<DT>(mx - mn);
            const float sc = round_t<DT>(range * rel);
            const uint32_t zb = T16<DT>::to_bits(rintf(round_t<DT>(__fdiv_rn(mn, sc))));
            if (wave == 0) {
                const size_t tok = (size_t)b * par_stride + tok0 + 16 * r + lane;
                scale[tok] = (uint16_t)T16<DT>::to_bits(sc);
                zero[tok] = (uint16_t)zb;
            }
            s_par[16 * wave + lane] = token_par<DT>(sc, zb, false);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        __builtin_amdgcn_s_setprio(PKV_EPRIO_PACK);
        uint32_t c01[16], c23[16];
        cell_quant<DT>(xr, my_par, c01, c23);
        if (AHEAD && r < 3) {                              // travels while the packs are formed
            if (PERM) cell_load_rows(pseq, perm + tok0 + 16 * (r + 1), (uint32_t)perm_block - 1u, plane, xr);
            else cell_load(cells + (size_t)(r + 1) * 16 * kHeadDim, xr);
        }
        typename PacksOf<WIDE>::type u;
        uint32_t cmax;
        cell_build(c01, c23, u, cmax);
        __builtin_amdgcn_s_setprio(PKV_EPRIO_EMIT);
        pack_offsets(u.len, u.off, u.payload);
        const uint32_t usz = (uint32_t)(g.mins_bytes + g.lens_bytes) + u.payload;
        if (r == 3) {
            // every block's final size is known before its last unit is written: the group's size is published now
            if (active && t == 0) blk_off[j + 1] = my_off + usz;
            if (tid == 0) blk_off[0] = 0;
            __syncthreads();
            if (tid == 0) {
                for (int q = 1; q <= H; q++) blk_off[q] += blk_off[q - 1];
                lookback_publish(st, gidx, blk_off[H]);
            }
        }
        if (active) {
            cmax_all = max(cmax_all, cmax);
            if (t == 0) reinterpret_cast<uint16_t *>(blk)[r] = (uint16_t)(my_off - 8u + usz);
            unit_emit_any(blk, my_off, t, g, u);
            my_off += usz;
        }
    }
    if (__any(cmax_all >= (1u << W))) {   // codes that do not fit W bits are an error the host reports
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) cmax_all = max(cmax_all, __shfl_xor(cmax_all, d, 64));
        if ((tid & 63) == 0) atomicMax(&st->max_code, cmax_all);
    }
    __syncthreads();
    const uint32_t bytes = blk_off[H];
    if (tid < 64) {
        const uint64_t off = base + lookback_offset(st, gidx, bytes, true);
        if (tid == 0) {
            s_off = off;
            if (gidx == ngroups - 1) st->total = off + bytes;
            if (off + bytes > capacity) atomicExch(&st->error, (uint32_t)PKV_ERR_CAPACITY);
        }
    }
    __syncthreads();
    const uint64_t off = s_off;
    if (off + bytes > capacity) return;
    if (tid < H) {
        const uint32_t first = XCH ? grp * (uint32_t)H_all + (uint32_t)hbase : gidx * (uint32_t)H;      // block index = group * heads + head
        info[2 * (size_t)(first + tid)] = (uint32_t)(off + blk_off[tid]);
        info[2 * (size_t)(first + tid) + 1] = blk_off[tid + 1] - blk_off[tid];
    }
    if (active) copy_out32(stream + off + blk_off[j], blk, my_off, t);
}

// ---- K, up to four heads: round-major, several groups to a workgroup ---------------------------
// The eight blocks a workgroup of 256 threads owns (block j = tid / 32, lane t = tid % 32) are here the H <= 4 heads
// of gpw = 8 / H (rounded down) consecutive (context block, sequence) groups -- consecutive in the stream too -- so
// that all eight half-wavefronts have a block.  The workgroup goes through its groups ROUND BY ROUND (16 tokens):
// it reads the round's rows row-wise for the token parameters (round_token_params_few, one group after the other),
// then at once re-reads them as cells -- the lines are still in L2 -- quantizes, and emits unit `round` of every
// block behind the units already there.  x crosses HBM once.  Blocks sit in worst-case slots in LDS and are
// compacted by the final copy.  (Five to eight heads, more than eight, and every token order take the cells
// kernel above, which reads a round once.)  `ngroups` counts workgroups, `ngroups_all` groups.
template <int DT, bool WIDE>
__global__ void __launch_bounds__(256) k_quant_encode_rounds_kernel(
    const uint16_t *__restrict__ x, int B, int H, int T, float rel, uint16_t *__restrict__ scale,
    uint16_t *__restrict__ zero, uint8_t *__restrict__ stream, uint64_t capacity, uint32_t *__restrict__ info,
    ScanState *st, int W, uint32_t ngroups, uint32_t bound, uint64_t base, int par_stride, const Stagger stagger,
    int gpw, uint32_t ngroups_all) {
    extern __shared__ __align__(16) uint8_t gbuf[];        // gpw * H block slots of `bound` bytes
    __shared__ uint32_t s_idx;
    __shared__ uint64_t s_off;
    __shared__ uint32_t blk_off[kSubBlocks + 1];           // byte offset of each block inside the workgroup's bytes
    __shared__ __attribute__((aligned(16))) TokPar s_par[kSubBlocks * 16];      // [group of the workgroup][token of the round]
    const int tid = threadIdx.x;
    stagger_first_generation(stagger);
    if (tid == 0) s_idx = atomicAdd(&st->ticket, 1u);
    __syncthreads();
    const uint32_t gidx = (uint32_t)__builtin_amdgcn_readfirstlane((int)s_idx);   // uniform: the rows' addresses become scalar
    if (gidx >= ngroups) return;
    // half-wavefront j serves head j % H of group gidx * gpw + j / H
    const int j = tid >> 5, t = tid & 31;                 // block and lane of the unit
    const int jg = j / H, jh = j % H;
    const uint32_t grp_first = gidx * (uint32_t)gpw;
    const int ng = (int)min((uint32_t)gpw, ngroups_all - grp_first);          // groups of this workgroup
    const int nblk = ng * H;                              // blocks of this workgroup
    const uint32_t grp = grp_first + (uint32_t)min(jg, ng - 1);
    const uint32_t cb = grp / (uint32_t)B, b = grp % (uint32_t)B;
    const size_t tok0 = (size_t)cb * 64;
    const UnitGeom g = unit_geom(W);
    const bool active = jg < ng && j < gpw * H;
    const TokPar *my_par = s_par + 16 * min(jg, ng - 1);
    uint8_t *blk = gbuf + (size_t)j * bound;
    uint32_t my_off = 8u;                                 // bytes of this block so far (uniform per half-wavefront)
    uint32_t cmax_all = 0;
#pragma unroll 1
    for (int r = 0; r < 4; r++) {
        // token parameters of the round: 16 lanes x 8 channels per token, the heads of one group after the other
        __builtin_amdgcn_s_setprio(PKV_EPRIO_STAT);
        {
            const int tt = tid >> 4, l16 = tid & 15;
            for (int q = 0; q < ng; q++) {
                const uint32_t gq = grp_first + (uint32_t)q;
                const uint32_t cq = gq / (uint32_t)B, bq = gq % (uint32_t)B;
                const size_t tq = (size_t)bq * par_stride + (size_t)cq * 64 + 16 * r + tt;
                round_token_params_few<DT>(x + (((size_t)bq * H) * T + (size_t)cq * 64 + 16 * r) * kHeadDim, (size_t)T * kHeadDim, H,
                                           tt, l16, rel, scale + tq, zero + tq, s_par + 16 * q + tt);
            }
        }
        // the same rows again, as cells (issued before the barrier; they hit the lines just fetched)
        uint2 xr[16];
        cell_load(x + (((size_t)b * H + jh) * T + tok0 + 16 * r) * kHeadDim + 4 * t, xr);
        __syncthreads();
        __builtin_amdgcn_s_setprio(PKV_EPRIO_PACK);
        typename PacksOf<WIDE>::type u;
        uint32_t cmax;
        cell_packs<DT>(xr, my_par, u, cmax);
        __syncthreads();                                  // s_par is rewritten by the next round
        __builtin_amdgcn_s_setprio(PKV_EPRIO_EMIT);
        pack_offsets(u.len, u.off, u.payload);            // (all lanes: the scan runs on whole wavefronts)
        const uint32_t usz = (uint32_t)(g.mins_bytes + g.lens_bytes) + u.payload;
        if (r == 3) {
            // every block's final size is known before its last unit is written: the workgroup's size is published
            // now, so that the workgroups behind it in the stream wait that much less for it
            if (active && t == 0) blk_off[j + 1] = my_off + usz;          // sizes first ...
            if (tid == 0) blk_off[0] = 0;
            __syncthreads();
            if (tid == 0) {                                               // ... then their running sum
                for (int q = 1; q <= nblk; q++) blk_off[q] += blk_off[q - 1];
                lookback_publish(st, gidx, blk_off[nblk]);
            }
        }
        if (active) {
            cmax_all = max(cmax_all, cmax);
            if (t == 0) reinterpret_cast<uint16_t *>(blk)[r] = (uint16_t)(my_off - 8u + usz);
            unit_emit_any(blk, my_off, t, g, u);
            my_off += usz;
        }
    }
    if (__any(cmax_all >= (1u << W))) {   // codes that do not fit W bits are an error the host reports
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) cmax_all = max(cmax_all, __shfl_xor(cmax_all, d, 64));
        if ((tid & 63) == 0) atomicMax(&st->max_code, cmax_all);
    }
    __syncthreads();
    const uint32_t bytes = blk_off[nblk];
    if (tid < 64) {
        const uint64_t off = base + lookback_offset(st, gidx, bytes, true);
        if (tid == 0) {
            s_off = off;
            if (gidx == ngroups - 1) st->total = off + bytes;
            if (off + bytes > capacity) atomicExch(&st->error, (uint32_t)PKV_ERR_CAPACITY);
        }
    }
    __syncthreads();
    const uint64_t off = s_off;
    if (off + bytes > capacity) return;
    if (tid < nblk) {
        const uint32_t first = grp_first * (uint32_t)H;                   // block index = group * H + head
        info[2 * (size_t)(first + tid)] = (uint32_t)(off + blk_off[tid]);
        info[2 * (size_t)(first + tid) + 1] = blk_off[tid + 1] - blk_off[tid];
    }
    if (active) copy_out32(stream + off + blk_off[j], blk, my_off, t);     // each half-wavefront copies its own block
}

// OR the FB-bit fields f[0..3] of four adjacent lanes 4m..4m+3, slot i, into a unit's LSB-first metadata array
// (field of lane c, slot i at bit (4c + i) * FB).  The 16 * FB bits of the four lanes start at byte 2 * FB * m.
__device__ __forceinline__ void meta_or4(uint8_t *arr, int m, int FB, int i, const uint32_t f[4]) {
    if (FB > 4) {                                 // widths 5, 6: 80 / 96 bits of four lanes, plus up to 16 bits of phase
        unsigned __int128 v = 0;
#pragma unroll
        for (int k = 0; k < 4; k++) v |= (unsigned __int128)f[k] << (4 * FB * k + FB * i);
        const uint32_t byte = 2u * (uint32_t)FB * (uint32_t)m;
        uint32_t *w = reinterpret_cast<uint32_t *>(arr + (byte & ~3u));
        v <<= 8u * (byte & 3u);
#pragma unroll
        for (int d = 0; d < 4; d++) {
            const uint32_t piece = (uint32_t)(v >> (32 * d));
            if (piece) atomicOr(w + d, piece);
        }
        return;
    }
    if (FB == 4) {                                // fields on 16-bit lanes: two aligned words, 32-bit arithmetic only
        uint32_t *w = reinterpret_cast<uint32_t *>(arr + 8u * (uint32_t)m);
        atomicOr(w, (f[0] | (f[1] << 16)) << (4 * i));
        atomicOr(w + 1, (f[2] | (f[3] << 16)) << (4 * i));
        return;
    }
    if (FB == 2) {                                // fields on byte lanes: one aligned word
        uint32_t *w = reinterpret_cast<uint32_t *>(arr + 4u * (uint32_t)m);
        atomicOr(w, (f[0] | (f[1] << 8) | (f[2] << 16) | (f[3] << 24)) << (2 * i));
        return;
    }
    // FB == 3: 48 bits at byte 6 m (odd m: two bytes into the word; 48 + 16 bits still fit two words)
    const uint32_t lo = (f[0] | (f[1] << 12)) << (3 * i), hi = (f[2] | (f[3] << 12)) << (3 * i);     // 27 bits each
    uint64_t v = (uint64_t)lo | ((uint64_t)hi << 24);
    const uint32_t byte = 6u * (uint32_t)m;
    uint32_t *w = reinterpret_cast<uint32_t *>(arr + (byte & ~3u));
    v <<= 8u * (byte & 3u);
    atomicOr(w, (uint32_t)v);
    atomicOr(w + 1, (uint32_t)(v >> 32));
}

// Inclusive prefix sum over each run of eight lanes (m = lane % 8) on the DPP data path; `total` receives the run's
// sum in all eight lanes.
__device__ __forceinline__ uint32_t oct_incl_scan(uint32_t v, int m, uint32_t &total) {
    uint32_t x = v;
    const uint32_t u1 = __builtin_amdgcn_update_dpp(0u, x, 0x111, 0xF, 0xF, true);      // row_shr:1
    x += m >= 1 ? u1 : 0u;
    const uint32_t u2 = __builtin_amdgcn_update_dpp(0u, x, 0x112, 0xF, 0xF, true);      // row_shr:2
    x += m >= 2 ? u2 : 0u;
    x += __builtin_amdgcn_update_dpp(0u, x, 0x114, 0xF, 0xA, false);                    // row_shr:4 into lanes 4..7 of a run
    const uint32_t last = __builtin_amdgcn_update_dpp(0u, x, 0xFF, 0xF, 0xF, false);    // every quad: its lane 3
    total = __builtin_amdgcn_update_dpp(last, last, 0x104, 0xF, 0x5, false);            // first quad of a run: the second quad's
    return x;
}

// ---- V, up to four heads: round-major, several groups to a workgroup ---------------------------
// One workgroup of 512 threads owns the 2 H blocks of each of gpw = 8 / H (rounded down) consecutive (128-token
// context block, sequence) groups, H <= 4, and goes through them 32 tokens (two rounds) at a time: read the rows
// row-wise for the token parameters, then at once re-read them as cells -- still in L2 -- quantize and append.
// Thread = (round parity rp, head slot j, cell lane t); head slot j serves head j % H of group gidx * gpw + j / H.
// Its cell (round 2 it + rp, channels 4t..4t+3) holds slot (2 it + rp) % 4 of lanes 4m..4m+3, m = t % 8, of unit
// (warp (t / 8) % 2, segment it / 2) of block 2 j + t / 16.  A unit's payload is slot-major, so the eight threads of
// a (unit, slot) append their packs behind the slots already there; the metadata bit-fields are OR-ed in with LDS
// atomics.  Units sit in worst-case slots in LDS; the final copy compacts them into the stream.  (Five to eight
// heads, more than eight, and every token order take the cells kernel below.)  `ngroups` counts workgroups,
// `ngroups_total` groups.
template <int DT, bool WIDE>
__global__ void __launch_bounds__(512) v_quant_encode_rounds_kernel(
    const uint16_t *__restrict__ x, int B, int H, int T, float rel, uint16_t *__restrict__ scale,
    uint16_t *__restrict__ zero, uint8_t *__restrict__ stream, uint64_t capacity, uint32_t *__restrict__ info,
    ScanState *st, int W, uint32_t ngroups, uint32_t unit_slot, uint64_t base, int par_stride, const Stagger stagger,
    int gpw, uint32_t ngroups_total) {
    extern __shared__ __align__(16) uint8_t gbuf[];        // 16 blocks x 4 units x unit_slot bytes
    __shared__ uint32_t s_idx;
    __shared__ uint64_t s_off;
    __shared__ uint32_t blk_off[17];                       // byte offset of each block inside the workgroup's bytes
    __shared__ uint32_t s_tot[2][8][4];                    // payload bytes the two rounds of an iteration append per unit
    __shared__ uint16_t s_usz[16][4];                      // bytes of every unit (block, unit index 2 w + sg)
    __shared__ __attribute__((aligned(16))) TokPar s_par[kSubBlocks * 32];      // [group of the workgroup][token of the iteration]
    const int tid = threadIdx.x;
    stagger_first_generation(stagger);
    if (tid == 0) s_idx = atomicAdd(&st->ticket, 1u);
    __syncthreads();
    const uint32_t gidx = s_idx;
    if (gidx >= ngroups) return;
    const int rp = tid >> 8, j = (tid >> 5) & 7, t = tid & 31;
    const int jg = j / H, jh = j % H;
    const uint32_t grp_first = gidx * (uint32_t)gpw;
    const int ng = (int)min((uint32_t)gpw, ngroups_total - grp_first);        // groups of this workgroup
    const int nheads = ng * H;                            // head slots in use
    const uint32_t grp = grp_first + (uint32_t)min(jg, ng - 1);
    const uint32_t cb = grp / (uint32_t)B, b = grp % (uint32_t)B;
    const size_t tok0 = (size_t)cb * 128;
    const UnitGeom g = unit_geom(W);
    const uint32_t meta = (uint32_t)(g.mins_bytes + g.lens_bytes);
    const bool active = jg < ng;
    const TokPar *my_par = s_par + 32 * min(jg, ng - 1) + 16 * rp;
    const int blkid = 2 * j + (t >> 4), w = (t >> 3) & 1, m = t & 7;
    // metadata areas start as zeros (fields are OR-ed in)
    for (uint32_t i = tid; i < 64u * (meta / 4u); i += 512)
        reinterpret_cast<uint32_t *>(gbuf + (size_t)(i / (meta / 4u)) * unit_slot)[i % (meta / 4u)] = 0u;
    uint32_t run_off = 0;                                  // payload bytes of the thread's current unit so far
    uint32_t cmax_all = 0;
#pragma unroll 1
    for (int it = 0; it < 4; it++) {
        // token parameters of the 32 tokens: 16 lanes x 8 channels per token, the heads of one group after the other
        __builtin_amdgcn_s_setprio(PKV_EPRIO_STAT);
        {
            const int tt = tid >> 4, l16 = tid & 15;
            for (int q = 0; q < ng; q++) {
                const uint32_t gq = grp_first + (uint32_t)q;
                const uint32_t cq = gq / (uint32_t)B, bq = gq % (uint32_t)B;
                const size_t tq = (size_t)bq * par_stride + (size_t)cq * 128 + 32 * it + tt;
                round_token_params_few<DT>(x + (((size_t)bq * H) * T + (size_t)cq * 128 + 32 * it) * kHeadDim, (size_t)T * kHeadDim,
                                           H, tt, l16, rel, scale + tq, zero + tq, s_par + 32 * q + tt);
            }
        }
        // the same rows again, as cells (issued before the barrier; they hit the lines just fetched)
        uint2 xr[16];
        cell_load(x + (((size_t)b * H + jh) * T + tok0 + 32 * it + 16 * rp) * kHeadDim + 4 * t, xr);
        __syncthreads();
        __builtin_amdgcn_s_setprio(PKV_EPRIO_PACK);
        typename PacksOf<WIDE>::type u;
        uint32_t cmax;
        cell_packs<DT>(xr, my_par, u, cmax);
        // bytes of the thread's four packs, their offsets inside the (unit, slot) and the slot's total
        const uint32_t pb = 2u * (u.len[0] + u.len[1] + u.len[2] + u.len[3]);
        uint32_t tot;
        const uint32_t inc = oct_incl_scan(pb, m, tot);
        if (m == 0) s_tot[rp][j][t >> 3] = tot;
        __syncthreads();                                  // s_par is rewritten by the next iteration; s_tot is published
        __builtin_amdgcn_s_setprio(PKV_EPRIO_EMIT);
        const uint32_t tot_even = s_tot[0][j][t >> 3], tot_odd = s_tot[1][j][t >> 3];
        if (it == 3) {
            // the last units' sizes are known before their packs are written: the workgroup's size is published now,
            // so that the workgroups behind it in the stream wait that much less for it
            if (active && rp == 0 && m == 0) s_usz[blkid][2 * w + 1] = (uint16_t)(meta + run_off + tot_even + tot_odd);
            __syncthreads();
            if (tid == 0) {
                uint32_t run = 0;
                for (int q = 0; q < 2 * nheads; q++) {
                    blk_off[q] = run;
                    run += 8u + s_usz[q][0] + s_usz[q][1] + s_usz[q][2] + s_usz[q][3];
                }
                blk_off[2 * nheads] = run;
                lookback_publish(st, gidx, run);
            }
        }
        if (active) {
            cmax_all = max(cmax_all, cmax);
            const int sg = it >> 1, slot = 2 * (it & 1) + rp;
            uint8_t *unit = gbuf + (size_t)(blkid * 4 + 2 * w + sg) * unit_slot;
            meta_or4(unit, m, g.W, slot, u.mn);
            meta_or4(unit + g.mins_bytes, m, g.LB, slot, u.len);
            uint32_t o = meta + run_off + (rp ? tot_even : 0u) + (inc - pb);
#pragma unroll
            for (int k = 0; k < 4; k++) {
                put_pack(reinterpret_cast<uint16_t *>(unit + o), u, k);
                o += 2u * u.len[k];
            }
        }
        run_off += tot_even + tot_odd;                    // both rounds of the iteration are behind the unit now
        if (it & 1) {                                     // the unit (w, it / 2) is complete
            if (it == 1 && active && rp == 0 && m == 0) s_usz[blkid][2 * w] = (uint16_t)(meta + run_off);
            run_off = 0;
        }
    }
    if (__any(cmax_all >= (1u << W))) {   // codes that do not fit W bits are an error the host reports
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) cmax_all = max(cmax_all, __shfl_xor(cmax_all, d, 64));
        if ((tid & 63) == 0) atomicMax(&st->max_code, cmax_all);
    }
    __syncthreads();
    const int nblk = 2 * nheads;
    const uint32_t bytes = blk_off[nblk];
    if (tid < 64) {
        const uint64_t off = base + lookback_offset(st, gidx, bytes, true);
        if (tid == 0) {
            s_off = off;
            if (gidx == ngroups - 1) st->total = off + bytes;
            if (off + bytes > capacity) atomicExch(&st->error, (uint32_t)PKV_ERR_CAPACITY);
        }
    }
    __syncthreads();
    const uint64_t off = s_off;
    if (off + bytes > capacity) return;
    if (tid < nblk) {
        const uint32_t first = grp_first * (uint32_t)(2 * H);             // block index = group * 2 H + 2 head + half
        info[2 * (size_t)(first + tid)] = (uint32_t)(off + blk_off[tid]);
        info[2 * (size_t)(first + tid) + 1] = blk_off[tid + 1] - blk_off[tid];
    }
    // half-wavefront q copies block q: the header of cumulative unit sizes, then its four units one after another
    const int q = tid >> 5;
    if (q < nblk) {
        uint8_t *dst = stream + off + blk_off[q];
        uint32_t cum = 0;
#pragma unroll
        for (int un = 0; un < 4; un++) {
            const uint32_t n = s_usz[q][un];
            copy_out32(dst + 8 + cum, gbuf + (size_t)(q * 4 + un) * unit_slot, n, t);
            cum += n;
            if (t == un) reinterpret_cast<uint16_t *>(dst)[un] = (uint16_t)cum;
        }
    }
}

// ---- V, all heads in one workgroup, x read ONCE as cells ----------------------------------------
// The V counterpart of k_quant_encode_cells_kernel: the threads keep the roles of the round-major V encoder (round
// parity rp, head j, cell lane t), but an iteration's 32 tokens are read as cells only, and a wavefront is ONE head
// with both rounds of the iteration (lanes 0..31 the even round, lanes 32..63 the odd one).  Everything a head's
// blocks need from each other -- the payload bytes the even round puts in front of the odd one -- is then an
// exchange between the halves of a wavefront, and the only thing wavefronts share is the token minima and maxima:
// each forms those of its head from the cell registers, the eight partial results per token go through LDS, and
// every wavefront forms the 32 tokens' parameters for itself.  One barrier per iteration.  For 5..8 heads, tokens
// in their own order; same stream, parameters and block_info as the round-major kernel.
// PERM: the tokens in the order of a repacking, as in the round-major kernel; with scale_in / zero_in (the tokens'
// parameters in the order of x, known from the pass that made the order) nothing is left to exchange and an
// iteration has no barrier at all.
template <int DT, bool WIDE, bool PERM, bool XCH = false>
__global__ void __launch_bounds__(512) v_quant_encode_cells_kernel(
    const uint16_t *__restrict__ x, int B, int H, int T, float rel, uint16_t *__restrict__ scale,
    uint16_t *__restrict__ zero, uint8_t *__restrict__ stream, uint64_t capacity, uint32_t *__restrict__ info,
    ScanState *st, int W, uint32_t ngroups, uint32_t unit_slot, uint64_t base, int par_stride,
    const uint32_t *__restrict__ perm, int perm_block, const uint16_t *__restrict__ scale_in,
    const uint16_t *__restrict__ zero_in, const Stagger stagger, int nsg = 1, uint64_t *xw = nullptr) {
    extern __shared__ __align__(16) uint8_t gbuf[];        // 16 blocks x 4 units x unit_slot bytes
    __shared__ uint32_t s_idx;
    __shared__ uint64_t s_off;
    __shared__ uint32_t blk_off[17];
    __shared__ uint16_t s_usz[16][4];
    __shared__ __attribute__((aligned(16))) TokPar s_par[8 * 32];       // [wavefront][token of the iteration]
    __shared__ uint32_t s_mm[2][8][32];                                  // [iteration parity][wavefront][token]: minmax_word
    const int tid = threadIdx.x;
    stagger_first_generation(stagger);
    if (tid == 0) s_idx = atomicAdd(&st->ticket, 1u);
    __syncthreads();
    const uint32_t gidx = PERM ? (uint32_t)__builtin_amdgcn_readfirstlane((int)s_idx) : s_idx;
    if (gidx >= ngroups) return;
    // XCH (more than eight heads): runs of eight heads that exchange the minima and maxima of their heads per token,
    // as in the K kernel; a run's words are [iteration][token of the iteration]
    const int H_all = H;
    const uint32_t sgi = XCH ? gidx % (uint32_t)nsg : 0u;
    const int hbase = XCH ? 8 * (int)sgi : 0;
    if (XCH) H = min(8, H_all - hbase);
    const int j = tid >> 6, rp = (tid >> 5) & 1, t = tid & 31, wave = j, lane = tid & 63;
    const uint32_t grp = XCH ? gidx / (uint32_t)nsg : gidx;
    const uint32_t cb = grp / (uint32_t)B, b = grp % (uint32_t)B;
    const size_t tok0 = (size_t)cb * 128;
    const UnitGeom g = unit_geom(W);
    const uint32_t meta = (uint32_t)(g.mins_bytes + g.lens_bytes);
    const bool active = j < H;
    const int jc = min(j, H - 1);
    const TokPar *my_par = (XCH ? s_par : s_par + 32 * wave) + 16 * rp;
    const int blkid = 2 * j + (t >> 4), w = (t >> 3) & 1, m = t & 7;
    for (uint32_t i = tid; i < 64u * (meta / 4u); i += 512)                 // metadata areas start as zeros
        reinterpret_cast<uint32_t *>(gbuf + (size_t)(i / (meta / 4u)) * unit_slot)[i % (meta / 4u)] = 0u;
    uint32_t run_off = 0;
    uint32_t cmax_all = 0;
    const uint16_t *cells = x + (((size_t)b * H_all + hbase + jc) * T + tok0 + 16 * rp) * kHeadDim + 4 * t;
    const uint32_t plane = (uint32_t)(((size_t)jc * T * kHeadDim + 4 * t) * 2);
    const bool known = PERM && scale_in != nullptr;              // uniform
    if (known) __syncthreads();                                  // the metadata zeros are in place before the first OR (no barrier below)
#pragma unroll 1
    for (int it = 0; it < 4; it++) {
        // (no request ahead as in the K kernel: placing the packs holds too many registers to keep 16 rows in flight)
        uint2 xr[16];
        // PERM: (the 32 tokens of an iteration lie in one repacking block: perm_block is a multiple of 64)
        const size_t rb = PERM ? ((tok0 + 32 * it) / (size_t)perm_block) * (size_t)perm_block : 0;
        if (PERM) cell_load_rows_lanes(x + (((size_t)b * H) * T + rb) * kHeadDim, perm + tok0 + 32 * it + 16 * rp, (uint32_t)perm_block - 1u, plane, xr);
        else cell_load(cells + (size_t)it * 32 * kHeadDim, xr);
        __builtin_amdgcn_s_setprio(PKV_EPRIO_STAT);
        if (known) {
            if (lane < 32) {
                const uint32_t src = min(perm[tok0 + 32 * it + lane], (uint32_t)perm_block - 1u);
                const uint32_t sb = scale_in[(size_t)b * T + rb + src], zb = zero_in[(size_t)b * T + rb + src];
                if (wave == 0) {
                    const size_t tok = (size_t)b * par_stride + tok0 + 32 * it + lane;
                    scale[tok] = (uint16_t)sb;
                    zero[tok] = (uint16_t)zb;
                }
                s_par[32 * wave + lane] = token_par<DT>(T16<DT>::from_bits(sb), zb, false);
            }
        } else {
        {
            float mn, mx;
            cell_token_minmax_halves<DT>(xr, mn, mx);
            if ((lane & 1) == 0) s_mm[it & 1][wave][lane >> 1] = minmax_word<DT>(mn, mx);
        }
        __syncthreads();
        if (XCH) {
            if (wave == 0) {
                const int tk = lane & 31;
                uint32_t pw = s_mm[it & 1][0][tk];
#pragma unroll
                for (int q = 1; q < 8; q++) pw = pk_sel_x<false, DT != PKV_F16>(pw, s_mm[it & 1][q][tk]);
                float rmn, rmx;
                minmax_unword<DT>(pw, rmn, rmx);
                uint64_t *words = xw + (size_t)(gidx - sgi) * 128 + 32 * it;      // [run][iteration][token] of this group
                if (lane < 32)
                    __hip_atomic_store(words + (size_t)sgi * 128 + lane, (1ull << 63) | ((uint64_t)T16<DT>::to_bits(rmn) << 16) | (uint64_t)T16<DT>::to_bits(rmx),
                                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                // lane = (parity of the run, token)
                float amn = INFINITY, amx = -INFINITY;
                for (int run = lane >> 5; run < nsg; run += 2) {
                    const uint64_t *wp = words + (size_t)run * 128 + tk;
                    uint64_t w = __hip_atomic_load(wp, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    int spins = 0;
                    while ((w >> 63) == 0 && spins < kSpinLimit) {
                        __builtin_amdgcn_s_sleep(8);
                        w = __hip_atomic_load(wp, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        spins++;
                    }
                    if ((w >> 63) == 0) atomicExch(&st->error, (uint32_t)PKV_ERR_INTERNAL);     // (bounded wait: the host reports it)
                    amn = fminf(amn, T16<DT>::from_bits((uint32_t)(w >> 16) & 0xFFFFu));
                    amx = fmaxf(amx, T16<DT>::from_bits((uint32_t)w & 0xFFFFu));
                }
                amn = fminf(amn, __shfl_xor(amn, 32, 64)); amx = fmaxf(amx, __shfl_xor(amx, 32, 64));
                if (lane < 32) {
                    const float range = round_t<DT>(amx - amn);
                    const float sc = round_t<DT>(range * rel);
                    const uint32_t zb = T16<DT>::to_bits(rintf(round_t<DT>(__fdiv_rn(amn, sc))));
                    if (sgi == 0) {
                        const size_t tok = (size_t)b * par_stride + tok0 + 32 * it + lane;
                        scale[tok] = (uint16_t)T16<DT>::to_bits(sc);
                        zero[tok] = (uint16_t)zb;
                    }
                    s_par[lane] = token_par<DT>(sc, zb, false);
                }
            }
            __syncthreads();
        } else
        if (lane < 32) {
            uint32_t pw = s_mm[it & 1][0][lane];             // the eight heads' words, combined by packed minima
#pragma unroll
            for (int q = 1; q < 8; q++) pw = pk_sel_x<false, DT != PKV_F16>(pw, s_mm[it & 1][q][lane]);
            float mn, mx;
            minmax_unword<DT>(pw, mn, mx);
            const float range = round_t<DT>(mx - mn);
            const float sc = round_t<DT>(range * rel);
            const uint32_t zb = T16<DT>::to_bits(rintf(round_t<DT>(__fdiv_rn(mn, sc))));
            if (wave == 0) {
                const size_t tok = (size_t)b * par_stride + tok0 + 32 * it + lane;
                scale[tok] = (uint16_t)T16<DT>::to_bits(sc);
                zero[tok] = (uint16_t)zb;
            }
            s_par[32 * wave + lane] = token_par<DT>(sc, zb, false);
        }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        __builtin_amdgcn_s_setprio(PKV_EPRIO_PACK);
        uint32_t c01[16], c23[16];
        cell_quant<DT, false>(xr, my_par, c01, c23);          // (the halves of the wavefront hold different tokens)
        typename PacksOf<WIDE>::type u;
        uint32_t cmax;
        cell_build(c01, c23, u, cmax);
        const uint32_t pb = 2u * (u.len[0] + u.len[1] + u.len[2] + u.len[3]);
        uint32_t tot;
        const uint32_t inc = oct_incl_scan(pb, m, tot);
        __builtin_amdgcn_s_setprio(PKV_EPRIO_EMIT);
        const auto halves = __builtin_amdgcn_permlane32_swap(tot, tot, false, false);      // the even round's total, the odd round's
        const uint32_t tot_even = halves[0], tot_odd = halves[1];
        if (it == 3) {
            if (active && rp == 0 && m == 0) s_usz[blkid][2 * w + 1] = (uint16_t)(meta + run_off + tot_even + tot_odd);
            __syncthreads();
            if (tid == 0) {
                uint32_t run = 0;
                for (int q = 0; q < 2 * H; q++) {
                    blk_off[q] = run;
                    run += 8u + s_usz[q][0] + s_usz[q][1] + s_usz[q][2] + s_usz[q][3];
                }
                blk_off[2 * H] = run;
                lookback_publish(st, gidx, run);
            }
        }
        if (active) {
            cmax_all = max(cmax_all, cmax);
            const int sg = it >> 1, slot = 2 * (it & 1) + rp;
            uint8_t *unit = gbuf + (size_t)(blkid * 4 + 2 * w + sg) * unit_slot;
            meta_or4(unit, m, g.W, slot, u.mn);
            meta_or4(unit + g.mins_bytes, m, g.LB, slot, u.len);
            uint32_t o = meta + run_off + (rp ? tot_even : 0u) + (inc - pb);
#pragma unroll
            for (int k = 0; k < 4; k++) {
                put_pack(reinterpret_cast<uint16_t *>(unit + o), u, k);
                o += 2u * u.len[k];
            }
        }
        run_off += tot_even + tot_odd;
        if (it & 1) {
            if (it == 1 && active && rp == 0 && m == 0) s_usz[blkid][2 * w] = (uint16_t)(meta + run_off);
            run_off = 0;
        }
    }
    if (__any(cmax_all >= (1u << W))) {
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) cmax_all = max(cmax_all, __shfl_xor(cmax_all, d, 64));
        if ((tid & 63) == 0) atomicMax(&st->max_code, cmax_all);
    }
    __syncthreads();
    const int nblk = 2 * H;
    const uint32_t bytes = blk_off[nblk];
    if (tid < 64) {
        const uint64_t off = base + lookback_offset(st, gidx, bytes, true);
        if (tid == 0) {
            s_off = off;
            if (gidx == ngroups - 1) st->total = off + bytes;
            if (off + bytes > capacity) atomicExch(&st->error, (uint32_t)PKV_ERR_CAPACITY);
        }
    }
    __syncthreads();
    const uint64_t off = s_off;
    if (off + bytes > capacity) return;
    if (tid < nblk) {
        const uint32_t first = XCH ? grp * (uint32_t)(2 * H_all) + (uint32_t)(2 * hbase) : gidx * (uint32_t)nblk;    // block index = group * 2 heads + 2 head + half
        info[2 * (size_t)(first + tid)] = (uint32_t)(off + blk_off[tid]);
        info[2 * (size_t)(first + tid) + 1] = blk_off[tid + 1] - blk_off[tid];
    }
    const int q = tid >> 5;
    if (q < nblk) {
        uint8_t *dst = stream + off + blk_off[q];
        uint32_t cum = 0;
#pragma unroll
        for (int un = 0; un < 4; un++) {
            const uint32_t n = s_usz[q][un];
            copy_out32(dst + 8 + cum, gbuf + (size_t)(q * 4 + un) * unit_slot, n, t);
            cum += n;
            if (t == un) reinterpret_cast<uint16_t *>(dst)[un] = (uint16_t)cum;
        }
    }
}

// ---- the block codec from a code matrix, as cells --------------------------------------------------------------
// The cells encoders with nothing to quantize: the input is the uint8 code matrix [ctx_len, hidden] of pkv_k_encode /
// pkv_v_encode.  Eight consecutive K blocks (64 x 128) or sixteen consecutive V blocks (128 x 64) of the stream are
// 1024 adjacent channels of one context block, i.e. exactly the group a cells workgroup owns, with the "heads" being
// 128-channel slices of the matrix.  A thread reads its cell as sixteen dwords (four codes of one token each; the 32
// lanes of a half-wavefront one 128-byte line per token), asks for the next round's while it forms and emits this
// round's packs, and no code tile is staged in LDS.  For hidden a multiple of 1024, the reference's block shapes and
// widths up to 6; pack_group_kernel takes everything else.
// `rows` (uniform: scalar registers) is the first of the 16 token rows, `lane_off` the lane's byte offset inside a
// row, so that a load is one 32-bit lane offset on a scalar base
__device__ __forceinline__ void code_cell_load(const uint8_t *rows, size_t row_bytes, uint32_t lane_off, uint32_t w[16]) {
#pragma unroll
    for (int k = 0; k < 16; k++) w[k] = *reinterpret_cast<const uint32_t *>(rows + (size_t)k * row_bytes + lane_off);
}
// four codes of a dword as two pairs of 16-bit integers (codes 0, 1 and codes 2, 3)
__device__ __forceinline__ void code_cell_pairs(const uint32_t w[16], uint32_t c01[16], uint32_t c23[16]) {
#pragma unroll
    for (int k = 0; k < 16; k++) {
        c01[k] = __builtin_amdgcn_perm(0u, w[k], 0x0C010C00u);
        c23[k] = __builtin_amdgcn_perm(0u, w[k], 0x0C030C02u);
    }
}

template <bool WIDE>
__global__ void __launch_bounds__(256) k_code_cells_kernel(
    const uint8_t *__restrict__ codes, int hidden, uint8_t *__restrict__ stream, uint64_t capacity,
    uint32_t *__restrict__ info, ScanState *st, int W, uint32_t ngroups, uint32_t bound, const Stagger stagger) {
    extern __shared__ __align__(16) uint8_t gbuf[];        // 8 block slots of `bound` bytes
    __shared__ uint32_t s_idx;
    __shared__ uint64_t s_off;
    __shared__ uint32_t blk_off[kSubBlocks + 1];
    const int tid = threadIdx.x;
    stagger_first_generation(stagger);
    if (tid == 0) s_idx = atomicAdd(&st->ticket, 1u);
    __syncthreads();
    const uint32_t gidx = (uint32_t)__builtin_amdgcn_readfirstlane((int)s_idx);
    if (gidx >= ngroups) return;
    const int j = tid >> 5, t = tid & 31;                 // block of the group, lane of the unit
    const uint32_t per_row = (uint32_t)hidden / 1024u;    // groups per context block
    const uint32_t cb = gidx / per_row, hg = gidx % per_row;
    const UnitGeom g = unit_geom(W);
    uint8_t *blk = gbuf + (size_t)j * bound;
    uint32_t my_off = 8u;
    const uint8_t *rows = codes + (size_t)cb * 64 * (size_t)hidden + (size_t)hg * 1024;      // uniform
    const uint32_t lane_off = (uint32_t)(j * 128 + 4 * t);
    uint32_t w[16];
    code_cell_load(rows, (size_t)hidden, lane_off, w);
#pragma unroll 1
    for (int r = 0; r < 4; r++) {
        __builtin_amdgcn_s_setprio(PKV_EPRIO_PACK);
        uint32_t c01[16], c23[16];
        code_cell_pairs(w, c01, c23);
        if (r < 3) code_cell_load(rows + (size_t)(r + 1) * 16 * (size_t)hidden, (size_t)hidden, lane_off, w);     // travels while the packs are formed
        typename PacksOf<WIDE>::type u;
        uint32_t cmax;
        cell_build(c01, c23, u, cmax);
        __builtin_amdgcn_s_setprio(PKV_EPRIO_EMIT);
        pack_offsets(u.len, u.off, u.payload);
        const uint32_t usz = (uint32_t)(g.mins_bytes + g.lens_bytes) + u.payload;
        if (r == 3) {                                     // the group's size is known before its last units are written
            if (t == 0) blk_off[j + 1] = my_off + usz;
            if (tid == 0) blk_off[0] = 0;
            __syncthreads();
            if (tid == 0) {
                for (int q = 1; q <= kSubBlocks; q++) blk_off[q] += blk_off[q - 1];
                lookback_publish(st, gidx, blk_off[kSubBlocks]);
            }
        }
        if (t == 0) reinterpret_cast<uint16_t *>(blk)[r] = (uint16_t)(my_off - 8u + usz);
        unit_emit_any(blk, my_off, t, g, u);
        my_off += usz;
    }
    __syncthreads();
    const uint32_t bytes = blk_off[kSubBlocks];
    if (tid < 64) {
        const uint64_t off = lookback_offset(st, gidx, bytes, true);
        if (tid == 0) {
            s_off = off;
            if (gidx == ngroups - 1) st->total = off + bytes;
            if (off + bytes > capacity) atomicExch(&st->error, (uint32_t)PKV_ERR_CAPACITY);
        }
    }
    __syncthreads();
    const uint64_t off = s_off;
    if (off + bytes > capacity) return;
    if (tid < kSubBlocks) {
        info[2 * (size_t)(gidx * (uint32_t)kSubBlocks + tid)] = (uint32_t)(off + blk_off[tid]);
        info[2 * (size_t)(gidx * (uint32_t)kSubBlocks + tid) + 1] = blk_off[tid + 1] - blk_off[tid];
    }
    copy_out32(stream + off + blk_off[j], blk, my_off, t);
}

// V: the thread roles of v_quant_encode_cells_kernel (a wavefront = one 128-channel slice with both rounds of an
// iteration in its halves), no barrier inside an iteration.
template <bool WIDE>
__global__ void __launch_bounds__(512) v_code_cells_kernel(
    const uint8_t *__restrict__ codes, int hidden, uint8_t *__restrict__ stream, uint64_t capacity,
    uint32_t *__restrict__ info, ScanState *st, int W, uint32_t ngroups, uint32_t unit_slot, const Stagger stagger) {
    extern __shared__ __align__(16) uint8_t gbuf[];        // 16 blocks x 4 units x unit_slot bytes
    __shared__ uint32_t s_idx;
    __shared__ uint64_t s_off;
    __shared__ uint32_t blk_off[17];
    __shared__ uint16_t s_usz[16][4];
    const int tid = threadIdx.x;
    stagger_first_generation(stagger);
    if (tid == 0) s_idx = atomicAdd(&st->ticket, 1u);
    __syncthreads();
    const uint32_t gidx = (uint32_t)__builtin_amdgcn_readfirstlane((int)s_idx);      // uniform: the rows' addresses become scalar
    if (gidx >= ngroups) return;
    const int j = tid >> 6, rp = (tid >> 5) & 1, t = tid & 31;
    const uint32_t per_row = (uint32_t)hidden / 1024u;
    const uint32_t cb = gidx / per_row, hg = gidx % per_row;
    const UnitGeom g = unit_geom(W);
    const uint32_t meta = (uint32_t)(g.mins_bytes + g.lens_bytes);
    const int blkid = 2 * j + (t >> 4), wq = (t >> 3) & 1, m = t & 7;
    for (uint32_t i = tid; i < 64u * (meta / 4u); i += 512)                 // metadata areas start as zeros
        reinterpret_cast<uint32_t *>(gbuf + (size_t)(i / (meta / 4u)) * unit_slot)[i % (meta / 4u)] = 0u;
    uint32_t run_off = 0;
    const uint8_t *rows = codes + (size_t)cb * 128 * (size_t)hidden + (size_t)hg * 1024;      // uniform
    const uint32_t lane_off = (uint32_t)(16 * rp) * (uint32_t)hidden + (uint32_t)(j * 128 + 4 * t);
    __syncthreads();                                       // the metadata zeros are in place before the first OR
#pragma unroll 1
    for (int it = 0; it < 4; it++) {
        // (no request ahead: with sixteen more registers in flight while the packs are placed the kernel needs 142
        // and a CU holds one workgroup instead of two)
        uint32_t w[16];
        code_cell_load(rows + (size_t)it * 32 * (size_t)hidden, (size_t)hidden, lane_off, w);
        __builtin_amdgcn_s_setprio(PKV_EPRIO_PACK);
        uint32_t c01[16], c23[16];
        code_cell_pairs(w, c01, c23);
        typename PacksOf<WIDE>::type u;
        uint32_t cmax;
        cell_build(c01, c23, u, cmax);
        const uint32_t pb = 2u * (u.len[0] + u.len[1] + u.len[2] + u.len[3]);
        uint32_t tot;
        const uint32_t inc = oct_incl_scan(pb, m, tot);
        __builtin_amdgcn_s_setprio(PKV_EPRIO_EMIT);
        const auto halves = __builtin_amdgcn_permlane32_swap(tot, tot, false, false);      // the even round's total, the odd round's
        const uint32_t tot_even = halves[0], tot_odd = halves[1];
        if (it == 3) {
            if (rp == 0 && m == 0) s_usz[blkid][2 * wq + 1] = (uint16_t)(meta + run_off + tot_even + tot_odd);
            __syncthreads();
            if (tid == 0) {
                uint32_t run = 0;
                for (int q = 0; q < 16; q++) {
                    blk_off[q] = run;
                    run += 8u + s_usz[q][0] + s_usz[q][1] + s_usz[q][2] + s_usz[q][3];
                }
                blk_off[16] = run;
                lookback_publish(st, gidx, run);
            }
        }
        {
            const int sg = it >> 1, slot = 2 * (it & 1) + rp;
            uint8_t *unit = gbuf + (size_t)(blkid * 4 + 2 * wq + sg) * unit_slot;
            meta_or4(unit, m, g.W, slot, u.mn);
            meta_or4(unit + g.mins_bytes, m, g.LB, slot, u.len);
            uint32_t o = meta + run_off + (rp ? tot_even : 0u) + (inc - pb);
#pragma unroll
            for (int k = 0; k < 4; k++) {
                put_pack(reinterpret_cast<uint16_t *>(unit + o), u, k);
                o += 2u * u.len[k];
            }
        }
        run_off += tot_even + tot_odd;
        if (it & 1) {
            if (it == 1 && rp == 0 && m == 0) s_usz[blkid][2 * wq] = (uint16_t)(meta + run_off);
            run_off = 0;
        }
    }
    __syncthreads();
    const uint32_t bytes = blk_off[16];
    if (tid < 64) {
        const uint64_t off = lookback_offset(st, gidx, bytes, true);
        if (tid == 0) {
            s_off = off;
            if (gidx == ngroups - 1) st->total = off + bytes;
            if (off + bytes > capacity) atomicExch(&st->error, (uint32_t)PKV_ERR_CAPACITY);
        }
    }
    __syncthreads();
    const uint64_t off = s_off;
    if (off + bytes > capacity) return;
    if (tid < 16) {
        info[2 * (size_t)(gidx * 16u + tid)] = (uint32_t)(off + blk_off[tid]);
        info[2 * (size_t)(gidx * 16u + tid) + 1] = blk_off[tid + 1] - blk_off[tid];
    }
    const int q = tid >> 5;                                // half-wavefront q copies block q
    uint8_t *dst = stream + off + blk_off[q];
    uint32_t cum = 0;
#pragma unroll
    for (int un = 0; un < 4; un++) {
        const uint32_t n = s_usz[q][un];
        copy_out32(dst + 8 + cum, gbuf + (size_t)(q * 4 + un) * unit_slot, n, t);
        cum += n;
        if (t == un) reinterpret_cast<uint16_t *>(dst)[un] = (uint16_t)cum;
    }
}

// Launch of the two kernels above (pkv_codec.hip decides when they apply): `st` is a prepared scan state with one
// status word per group, `bound` the worst-case bytes of a block.
int launch_code_cells(bool is_k, const uint8_t *codes, int ctx_len, int hidden, int bits, uint32_t bound, uint8_t *stream,
                      uint64_t capacity, uint32_t *info, ScanState *st, uint32_t ngroups, hipStream_t s) {
    int rc;
    Stagger sg;
    if (is_k) {
        const uint32_t slot = (bound + 15u) & ~15u;
        const uint32_t lds = (uint32_t)kSubBlocks * slot + 32u;
        auto kern = bits > 4 ? k_code_cells_kernel<true> : k_code_cells_kernel<false>;
        if ((rc = stagger_for(reinterpret_cast<const void *>(kern), 256, lds, ngroups, &sg))) return rc;
        kern<<<ngroups, 256, lds, s>>>(codes, hidden, stream, capacity, info, st, bits, ngroups, slot, sg);
    } else {
        const uint32_t unit_slot = (uint32_t)(((bound - 8u) / 4u + 15u) & ~15u);
        const uint32_t lds = 64u * unit_slot + 64u;
        auto kern = bits > 4 ? v_code_cells_kernel<true> : v_code_cells_kernel<false>;
        PKV_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        if ((rc = stagger_for(reinterpret_cast<const void *>(kern), 512, lds, ngroups, &sg))) return rc;
        kern<<<ngroups, 512, lds, s>>>(codes, hidden, stream, capacity, info, st, bits, ngroups, unit_slot, sg);
    }
    (void)ctx_len;
    PKV_HIP_CHECK(hipGetLastError());
    return PKV_OK;
}

// ---- per-token median of the V codes, straight from V -----------------------------------------------------------
// `median_repacking` (utils/compute.py:262-270) orders the tokens of a block by the lower median of each token's
// V codes over ALL channels of all sequences and heads.  This kernel gets those medians without a code matrix: a
// workgroup of 256 threads owns 16 tokens and walks the sequences; thread (token tt, l16) reads 8 channels of every
// head (the parameter pass of the round-major encoders), every lane of a token's row computes the token's scale and
// zero for itself, quantises its 64 values and counts them into a histogram column of its own in LDS
// (hist[level][thread]: one LDS add per value, no two threads on one word).  At the end the columns of a token are
// summed per level and the level that reaches rank (n - 1) / 2 is the median.  H <= 8, code width <= 6 bits.
template <int DT>
__global__ void __launch_bounds__(256, DT == PKV_F16 ? 8 : 4) token_median_from_x_kernel(const uint16_t *__restrict__ x, int B, int H, int T, float rel,
                                                                  int W, uint8_t *__restrict__ median,
                                                                  uint16_t *__restrict__ scale_out, uint16_t *__restrict__ zero_out) {
    extern __shared__ uint32_t hist[];                     // [1 << W][256]
    const int tid = threadIdx.x, tt = tid >> 4, l16 = tid & 15;
    const int levels = 1 << W;
    // workgroups go round-robin over the 8 XCDs: each XCD takes a contiguous eighth of the tokens
    const uint32_t wg = (gridDim.x & 7u) == 0u ? (blockIdx.x & 7u) * (gridDim.x >> 3) + (blockIdx.x >> 3) : blockIdx.x;
    const size_t tok0 = (size_t)wg * 16;
    const uint32_t tok_idx = (uint32_t)tok0 + (uint32_t)tt;
    for (int l = 0; l < levels; l++) hist[l * 256 + tid] = 0u;       // the thread's own column: no barrier needed
    const uint32_t lane_off = (uint32_t)(tt * kHeadDim + l16 * 8) * 2u;
    typedef __attribute__((address_space(3))) uint32_t *lds_u32_ptr;
    const uint32_t col = (uint32_t)reinterpret_cast<uintptr_t>((lds_u32_ptr)hist) + 4u * (uint32_t)tid;    // LDS byte address of the thread's column
    // the rows of sequence b + 1 are requested head by head as soon as the head's values of sequence b have been
    // quantised (into the registers they leave), so the next round trip to memory runs under this sequence's work
    auto load_row = [&](int b, int i) {
        const uint16_t *rows = x + (((size_t)b * H) * T + tok0) * kHeadDim;
        return *reinterpret_cast<const uint4 *>(reinterpret_cast<const char *>(rows + (size_t)min(i, H - 1) * T * kHeadDim) + lane_off);
    };
    uint4 v[8];
    // groups of 16 neighbouring workgroups start at different sequences: with every workgroup on the same sequence
    // at the same time the requests of the whole grid lie 8 MiB-strided rows apart in one 64 MiB range and pile up
    // on a part of the memory channels (0.251 -> 0.233 ms on 16 x 8 x 32768 tokens, with the mapping above)
    const int b_rot = (int)(wg >> 4) % B;
#pragma unroll
    for (int i = 0; i < 8; i++) v[i] = load_row(b_rot, i);
    for (int bb = 0; bb < B; bb++) {
        const int b = bb + b_rot < B ? bb + b_rot : bb + b_rot - B;
        const int bn1 = bb + 1 + b_rot;                    // the next sequence (requested while there is one)
        const int bn = bn1 < B ? bn1 : bn1 - B;
        const bool more = bb + 1 < B;
        float mn, mx;
        if (DT == PKV_F16) {
            f16x2 lo[8], hi[8];
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const f16x2 a = __builtin_bit_cast(f16x2, v[i].x), b2 = __builtin_bit_cast(f16x2, v[i].y),
                            c = __builtin_bit_cast(f16x2, v[i].z), d = __builtin_bit_cast(f16x2, v[i].w);
                lo[i] = pk_min_h(pk_min_h(a, b2), pk_min_h(c, d));
                hi[i] = pk_max_h(pk_max_h(a, b2), pk_max_h(c, d));
            }
#pragma unroll
            for (int w = 4; w >= 1; w >>= 1)
#pragma unroll
                for (int i = 0; i < w; i++) {
                    lo[i] = pk_min_h(lo[i], lo[i + w]);
                    hi[i] = pk_max_h(hi[i], hi[i + w]);
                }
            mn = fminf((float)lo[0][0], (float)lo[0][1]);
            mx = fmaxf((float)hi[0][0], (float)hi[0][1]);
        } else {
            mn = INFINITY, mx = -INFINITY;
#pragma unroll
            for (int i = 0; i < 8; i++) minmax8<DT>(v[i], mn, mx);
        }
        row16_minmax(mn, mx);
        const float range = round_t<DT>(mx - mn);
        const float sc = round_t<DT>(range * rel);
        const uint32_t zb = T16<DT>::to_bits(rintf(round_t<DT>(__fdiv_rn(mn, sc))));
        // a wavefront holds four tokens: it takes the usual quantisation sequence when all four can, else the general
        // one for all (quant4 branches on the first lane's constants)
        if (scale_out && l16 == 0) {                       // the parameters pkv_quant_params would write, for the encoder
            // (a uniform row pointer and a 32-bit offset, written out as the store itself: the compiler kept 64-bit
            // per-lane addresses across the loop and spilled them, with a reload and a full wait in every sequence)
            uint16_t *srow = scale_out + (size_t)b * T, *zrow = zero_out + (size_t)b * T;
            const uint32_t boff = 2u * tok_idx, sbits = T16<DT>::to_bits(sc);
            asm volatile("global_store_short %0, %1, %2" : : "v"(boff), "v"(sbits), "s"(srow) : "memory");
            asm volatile("global_store_short %0, %1, %2" : : "v"(boff), "v"(zb), "s"(zrow) : "memory");
        }
        TokPar tp = token_par<DT>(sc, zb, false);
        const bool wave_usual = !__any(tp.sub2 == 0u);
        if (!wave_usual) tp = token_par<DT>(sc, zb, true);
        // count one head's eight codes (four 16-bit pairs): both halves clamped to the top level with one packed
        // operation, then one multiply-add per code forms the byte address of the level's row in the thread's column
        // (v_mad_u32_u16: 16-bit half selected by op_sel, times the row pitch, plus the column's offset)
        auto count = [&](const uint32_t c[4], int i) {
            const uint32_t one = i < H ? 1u : 0u;          // heads beyond H - 1 repeat the last one: counted as nothing
            const u16x2 top = {(unsigned short)(levels - 1), (unsigned short)(levels - 1)};
            const uint32_t pitch = 1024u;
#pragma unroll
            for (int q = 0; q < 4; q++) {
                // (a code that does not fit W bits is counted at the top level; the encoders report it)
                const uint32_t cc = pk_u16(__builtin_elementwise_min(as_u16x2(c[q]), top));
                uint32_t a_lo, a_hi;
                asm("v_mad_u32_u16 %0, %1, %2, %3" : "=v"(a_lo) : "v"(cc), "s"(pitch), "v"(col));
                asm("v_mad_u32_u16 %0, %1, %2, %3 op_sel:[1,0,0,0]" : "=v"(a_hi) : "v"(cc), "s"(pitch), "v"(col));
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Wint-to-pointer-cast"      // the host pass sees a 64-bit pointer here; LDS pointers are 32 bits wide
                __hip_atomic_fetch_add((lds_u32_ptr)a_lo, one, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                __hip_atomic_fetch_add((lds_u32_ptr)a_hi, one, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
#pragma clang diagnostic pop
            }
        };
        // (the branch is per head and uniform, so that the request of the next sequence's row is common code: with
        // one loop per case the rows came back in different registers and were copied at the join)
#pragma unroll
        for (int i = 0; i < 8; i++) {
            uint32_t c[4];
            if (DT == PKV_F16 && wave_usual) {
                quant4_f16_fast(make_uint2(v[i].x, v[i].y), tp, c[0], c[1]);
                quant4_f16_fast(make_uint2(v[i].z, v[i].w), tp, c[2], c[3]);
            } else {
                quant4<DT>(make_uint2(v[i].x, v[i].y), tp, c[0], c[1]);
                quant4<DT>(make_uint2(v[i].z, v[i].w), tp, c[2], c[3]);
            }
            if (more) v[i] = load_row(bn, i);
            count(c, i);
        }
    }
    __syncthreads();
    // thread (tt, l16) sums the columns of token tt for its levels l16 * nper .. (a level per lane up to 16 levels)
    const int nper = levels > 16 ? levels / 16 : 1;
    uint32_t cnt[4] = {0u, 0u, 0u, 0u}, tot = 0;
    for (int sl = 0; sl < nper; sl++) {
        const int l = l16 * nper + sl;
        if (l < levels)
            for (int q = 0; q < 16; q++) cnt[sl] += hist[l * 256 + tt * 16 + ((q + l16) & 15)];
        tot += cnt[sl];
    }
    uint32_t incl = tot;                                   // inclusive scan over the 16 lanes of the token's row
    incl += __builtin_amdgcn_update_dpp(0u, incl, 0x111, 0xF, 0xF, true);
    incl += __builtin_amdgcn_update_dpp(0u, incl, 0x112, 0xF, 0xF, true);
    incl += __builtin_amdgcn_update_dpp(0u, incl, 0x114, 0xF, 0xF, true);
    incl += __builtin_amdgcn_update_dpp(0u, incl, 0x118, 0xF, 0xF, true);
    const uint32_t need = (uint32_t)((size_t)B * H * kHeadDim - 1) / 2u + 1u;      // values at or below the lower median
    uint32_t run = incl - tot;
    int found = -1;
    for (int sl = 0; sl < nper; sl++) {
        run += cnt[sl];
        if (found < 0 && run >= need) found = l16 * nper + sl;
    }
    const uint64_t has = __ballot(found >= 0);
    const uint32_t mine = (uint32_t)(has >> (16 * (tt & 3))) & 0xFFFFu;            // the token's row of the wavefront
    if (found >= 0 && (mine & ((1u << l16) - 1u)) == 0u) median[tok0 + tt] = (uint8_t)found;
}

// medians of the V codes of every token (device array of T bytes) from V itself
static int launch_token_median_from_x(const void *x, int dtype, int B, int H, int T, float rel, int bits, uint8_t *median,
                                      void *scale_out, void *zero_out, hipStream_t s) {
    const size_t lds = (size_t)(1 << bits) * 256 * sizeof(uint32_t);
    auto kern = dtype == PKV_F16 ? token_median_from_x_kernel<PKV_F16> : token_median_from_x_kernel<PKV_BF16>;
    if (lds > 48 * 1024)
        PKV_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    kern<<<(unsigned)(T / 16), 256, lds, s>>>((const uint16_t *)x, B, H, T, rel, bits, median, (uint16_t *)scale_out, (uint16_t *)zero_out);
    PKV_HIP_CHECK(hipGetLastError());
    return PKV_OK;
}

static int check_xshape(const void *x, int dtype, int B, int H, int T) {
    PKV_REQUIRE(x != nullptr, PKV_ERR_INVALID, "null pointer argument");
    PKV_REQUIRE(dtype == PKV_F16 || dtype == PKV_BF16, PKV_ERR_UNSUPPORTED, "Unsupported data type");
    PKV_REQUIRE(B > 0 && H > 0 && T > 0, PKV_ERR_INVALID, "sizes must be positive");
    PKV_REQUIRE(B <= 65535 && H <= 65535, PKV_ERR_UNSUPPORTED, "batch / head count above 65535");
    return PKV_OK;
}

template <bool IS_K>
static int run_quant_encode(const void *x, int dtype, int B, int H, int T, float rel, int bits,
                            uint8_t *stream, uint64_t capacity, uint64_t base, uint32_t *info, void *scale,
                            void *zero, int par_stride, uint64_t *size_out, float *ms_out, hipStream_t s,
                            const uint32_t *perm = nullptr, int perm_block = 0, const void *scale_in = nullptr,
                            const void *zero_in = nullptr) {
    int rc = check_xshape(x, dtype, B, H, T);
    if (rc) return rc;
    PKV_REQUIRE(stream && info && scale && zero, PKV_ERR_INVALID, "null pointer argument");
    PKV_REQUIRE((reinterpret_cast<uintptr_t>(stream) & 1u) == 0, PKV_ERR_INVALID,
                "compressed_buffer must start at an even address (blocks are written in 2-byte units)");
    PKV_REQUIRE(capacity > 0, PKV_ERR_INVALID, "compressed_buffer must be a non-empty tensor");
    PKV_REQUIRE(bits >= 2 && bits <= 6, PKV_ERR_UNSUPPORTED,
                "not supported: bits_len %d (the fused encoders take 2..6; wider codes go through pkv_quant_params, "
                "pkv_quantize and pkv_{k,v}_encode)", bits);
    PKV_REQUIRE(rel > 0.f, PKV_ERR_INVALID, "quant_scale_rel must be positive");
    const int ctx_blk = IS_K ? 64 : 128, hid_blk = IS_K ? 128 : 64;
    PKV_REQUIRE(T % ctx_blk == 0, PKV_ERR_INVALID, "ctx_len must be divisible by ctx_len_block_size");
    PKV_REQUIRE(par_stride >= T, PKV_ERR_INVALID, "parameter row stride shorter than the token count");
    if (perm) {
        PKV_REQUIRE(H <= kSubBlocks, PKV_ERR_UNSUPPORTED, "not supported: a token order with more than 8 KV heads");
        PKV_REQUIRE(perm_block >= 64 && perm_block % 64 == 0 && T % perm_block == 0, PKV_ERR_INVALID,
                    "the repacking block must be a multiple of 64 tokens that divides ctx_len");
        PKV_REQUIRE((uint64_t)H * (uint64_t)T * 256ull < (1ull << 32), PKV_ERR_UNSUPPORTED,
                    "not supported: a token order on more than 4 GiB of rows per sequence");
    }
    PKV_REQUIRE(base <= capacity, PKV_ERR_INVALID, "stream offset beyond the buffer");
    // block_info holds 32-bit byte offsets (uint32 in the reference too, evaluation/evaluation.py:420-426): a stream
    // that would grow past 4 GiB is reported as a full buffer instead of wrapping its offsets
    if (capacity > (1ull << 32)) capacity = 1ull << 32;
    PKV_REQUIRE(base <= capacity, PKV_ERR_CAPACITY, "stream offset beyond 4 GiB: block_info offsets are 32 bits");
    ScanState *st = nullptr;
    // One workgroup per run of up to eight heads of a (context block, sequence) group -- K: its up to eight blocks;
    // V: its up to sixteen -- or, with fewer than five heads, per 8 / H groups.
    {
        const int HB = IS_K ? H : 2 * H;
        const uint32_t bound = IS_K ? (uint32_t)k_block_bound(ctx_blk, bits) : (uint32_t)v_block_bound(hid_blk, bits);
        const uint32_t nsub = (uint32_t)(T / ctx_blk) * (uint32_t)B * (uint32_t)((HB + kSubBlocks - 1) / kSubBlocks);
        // status words (one per ticket; nsub bounds the tickets of every kernel below), then, with more than eight
        // heads, the words the runs of a group exchange: one per (run, token)
        const int nruns = (H + kSubBlocks - 1) / kSubBlocks;                // runs of eight heads per group
        const uint32_t nruns_all = (uint32_t)(T / ctx_blk) * (uint32_t)B * (uint32_t)nruns;
        PKV_REQUIRE((uint64_t)nsub + (uint64_t)nruns_all * (uint64_t)ctx_blk < (1ull << 31), PKV_ERR_UNSUPPORTED, "batch x tokens too large");
        const uint32_t xwords = H <= kSubBlocks ? 0u : nruns_all * (uint32_t)ctx_blk;
        if ((rc = prepare_scan_state(nsub + xwords, &st, s))) return rc;
        LaunchTimer tm(s, ms_out != nullptr);
        if ((rc = tm.begin())) return rc;
        if (!IS_K && H <= 8) {               // one workgroup per group of 2 H blocks
            const uint32_t unit_slot = (uint32_t)(((bound - 8u) / 4u + 15u) & ~15u);
            const uint32_t lds = 64u * unit_slot + 64u;
            const uint32_t ngroups_all = (uint32_t)(T / ctx_blk) * (uint32_t)B;
            // up to four heads: 8 / H groups to a workgroup, so that all eight head slots have blocks
            const int gpw = (H <= 4 && !perm) ? kSubBlocks / H : 1;
            const uint32_t ngroups = (ngroups_all + (uint32_t)gpw - 1u) / (uint32_t)gpw;
            // (a token order always comes with gpw == 1, i.e. the cells kernel)
            auto kern = bits > 4 ? (dtype == PKV_F16 ? v_quant_encode_rounds_kernel<PKV_F16, true>
                                                      : v_quant_encode_rounds_kernel<PKV_BF16, true>)
                                 : (dtype == PKV_F16 ? v_quant_encode_rounds_kernel<PKV_F16, false>
                                                      : v_quant_encode_rounds_kernel<PKV_BF16, false>);
            PKV_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
            Stagger sg;
            if (gpw == 1) {                         // five to eight heads, or any token order: x read once, as cells
                auto cells = perm ? (bits > 4 ? (dtype == PKV_F16 ? v_quant_encode_cells_kernel<PKV_F16, true, true>
                                                                  : v_quant_encode_cells_kernel<PKV_BF16, true, true>)
                                              : (dtype == PKV_F16 ? v_quant_encode_cells_kernel<PKV_F16, false, true>
                                                                  : v_quant_encode_cells_kernel<PKV_BF16, false, true>))
                                  : (bits > 4 ? (dtype == PKV_F16 ? v_quant_encode_cells_kernel<PKV_F16, true, false>
                                                                  : v_quant_encode_cells_kernel<PKV_BF16, true, false>)
                                              : (dtype == PKV_F16 ? v_quant_encode_cells_kernel<PKV_F16, false, false>
                                                                  : v_quant_encode_cells_kernel<PKV_BF16, false, false>));
                PKV_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(cells),
                                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
                if ((rc = stagger_for(reinterpret_cast<const void *>(cells), 512, lds, ngroups, &sg))) return rc;
                cells<<<ngroups, 512, lds, s>>>((const uint16_t *)x, B, H, T, rel, (uint16_t *)scale, (uint16_t *)zero,
                                                stream, capacity, info, st, bits, ngroups, unit_slot, base, par_stride, perm, perm_block,
                                                (const uint16_t *)scale_in, (const uint16_t *)zero_in, sg, 1, nullptr);
            } else {
                if ((rc = stagger_for(reinterpret_cast<const void *>(kern), 512, lds, ngroups, &sg))) return rc;
                kern<<<ngroups, 512, lds, s>>>((const uint16_t *)x, B, H, T, rel, (uint16_t *)scale, (uint16_t *)zero,
                                               stream, capacity, info, st, bits, ngroups, unit_slot, base, par_stride, sg, gpw,
                                               ngroups_all);
            }
        } else if (IS_K && H <= kSubBlocks) {       // nsub == number of groups
            const uint32_t slot = (bound + 15u) & ~15u;
            // up to four heads: 8 / H groups to a workgroup, so that all eight half-wavefronts have a block
            const int gpw = (H <= 4 && !perm) ? kSubBlocks / H : 1;
            const uint32_t nwg = (nsub + (uint32_t)gpw - 1u) / (uint32_t)gpw;
            const uint32_t lds = (uint32_t)(gpw * H) * slot + 32u;
            // (a token order always comes with gpw == 1, i.e. the cells kernel: the round-major kernel serves groups of
            // up to four heads in their own order)
            auto kern = bits > 4 ? (dtype == PKV_F16 ? k_quant_encode_rounds_kernel<PKV_F16, true>
                                                      : k_quant_encode_rounds_kernel<PKV_BF16, true>)
                                 : (dtype == PKV_F16 ? k_quant_encode_rounds_kernel<PKV_F16, false>
                                                      : k_quant_encode_rounds_kernel<PKV_BF16, false>);
            Stagger sg;
            if (gpw == 1) {                         // five to eight heads: x read once, as cells
                auto cells = perm ? (bits > 4 ? (dtype == PKV_F16 ? k_quant_encode_cells_kernel<PKV_F16, true, true>
                                                                  : k_quant_encode_cells_kernel<PKV_BF16, true, true>)
                                              : (dtype == PKV_F16 ? k_quant_encode_cells_kernel<PKV_F16, false, true>
                                                                  : k_quant_encode_cells_kernel<PKV_BF16, false, true>))
                                  : (bits > 4 ? (dtype == PKV_F16 ? k_quant_encode_cells_kernel<PKV_F16, true, false>
                                                                  : k_quant_encode_cells_kernel<PKV_BF16, true, false>)
                                              : (dtype == PKV_F16 ? k_quant_encode_cells_kernel<PKV_F16, false, false>
                                                                  : k_quant_encode_cells_kernel<PKV_BF16, false, false>));
                if ((rc = stagger_for(reinterpret_cast<const void *>(cells), 256, lds, nwg, &sg))) return rc;
                cells<<<nwg, 256, lds, s>>>((const uint16_t *)x, B, H, T, rel, (uint16_t *)scale, (uint16_t *)zero, stream,
                                            capacity, info, st, bits, nwg, slot, base, par_stride, perm, perm_block, sg, 1, nullptr);
            } else {
                if ((rc = stagger_for(reinterpret_cast<const void *>(kern), 256, lds, nwg, &sg))) return rc;
                kern<<<nwg, 256, lds, s>>>((const uint16_t *)x, B, H, T, rel, (uint16_t *)scale, (uint16_t *)zero, stream,
                                           capacity, info, st, bits, nwg, slot, base, par_stride, sg, gpw, nsub);
            }
        } else if (IS_K) {                           // more than eight heads: runs of eight, one workgroup each, that exchange their minima and maxima
            const uint32_t slot = (bound + 15u) & ~15u;
            const uint32_t lds = (uint32_t)kSubBlocks * slot + 32u;
            const int nsg = (H + kSubBlocks - 1) / kSubBlocks;
            auto kern = bits > 4 ? (dtype == PKV_F16 ? k_quant_encode_cells_kernel<PKV_F16, true, false, true>
                                                      : k_quant_encode_cells_kernel<PKV_BF16, true, false, true>)
                                 : (dtype == PKV_F16 ? k_quant_encode_cells_kernel<PKV_F16, false, false, true>
                                                      : k_quant_encode_cells_kernel<PKV_BF16, false, false, true>);
            Stagger sg;
            if ((rc = stagger_for(reinterpret_cast<const void *>(kern), 256, lds, nsub, &sg))) return rc;
            kern<<<nsub, 256, lds, s>>>((const uint16_t *)x, B, H, T, rel, (uint16_t *)scale, (uint16_t *)zero, stream,
                                        capacity, info, st, bits, nsub, slot, base, par_stride, nullptr, 0, sg, nsg,
                                        st->status + nsub);
        } else {                                     // V, more than eight heads: the same runs of eight
            const uint32_t unit_slot = (uint32_t)(((bound - 8u) / 4u + 15u) & ~15u);
            const uint32_t lds = 64u * unit_slot + 64u;
            auto kern = bits > 4 ? (dtype == PKV_F16 ? v_quant_encode_cells_kernel<PKV_F16, true, false, true>
                                                      : v_quant_encode_cells_kernel<PKV_BF16, true, false, true>)
                                 : (dtype == PKV_F16 ? v_quant_encode_cells_kernel<PKV_F16, false, false, true>
                                                      : v_quant_encode_cells_kernel<PKV_BF16, false, false, true>);
            PKV_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
            Stagger sg;
            if ((rc = stagger_for(reinterpret_cast<const void *>(kern), 512, lds, nruns_all, &sg))) return rc;
            kern<<<nruns_all, 512, lds, s>>>((const uint16_t *)x, B, H, T, rel, (uint16_t *)scale, (uint16_t *)zero,
                                             stream, capacity, info, st, bits, nruns_all, unit_slot, base, par_stride, nullptr, 0,
                                             nullptr, nullptr, sg, nruns, st->status + nruns_all);
        }
        PKV_HIP_CHECK(hipGetLastError());
        if ((rc = tm.end(ms_out))) return rc;
        return finish_encode(st, size_out, bits, s);
    }
}

}  // namespace pkv

extern "C" {

int pkv_median_order(const void *v, int dtype, int B, int H, int T, float rel, int bits, int block_size, uint32_t *perm,
                     void *scale_out, void *zero_out, float *ms_out, pkv_stream_t s_) {
    using namespace pkv;
    hipStream_t s = (hipStream_t)s_;
    int rc = check_xshape(v, dtype, B, H, T);
    if (rc) return rc;
    PKV_REQUIRE(perm != nullptr, PKV_ERR_INVALID, "null pointer argument");
    PKV_REQUIRE((scale_out == nullptr) == (zero_out == nullptr), PKV_ERR_INVALID, "scale_out and zero_out go together");
    PKV_REQUIRE(rel > 0.f, PKV_ERR_INVALID, "quant_scale_rel must be positive");
    PKV_REQUIRE(H <= kSubBlocks, PKV_ERR_UNSUPPORTED, "not supported: more than 8 KV heads (order the code matrix with pkv_median_repack)");
    PKV_REQUIRE(bits >= 2 && bits <= 6, PKV_ERR_UNSUPPORTED, "not supported: bits_len %d (2..6)", bits);
    PKV_REQUIRE(block_size > 0 && block_size <= 1024 && T % block_size == 0 && T % 16 == 0, PKV_ERR_INVALID,
                "ctx_len must be divisible by 16 and by a block size of at most 1024 tokens");
    void *scratch = nullptr;
    if ((rc = scratch_get((size_t)T, s, &scratch))) return rc;
    uint8_t *median = static_cast<uint8_t *>(scratch);
    LaunchTimer tm(s, ms_out != nullptr);
    if ((rc = tm.begin())) return rc;
    if ((rc = launch_token_median_from_x(v, dtype, B, H, T, rel, bits, median, scale_out, zero_out, s))) return rc;
    if ((rc = launch_block_order(median, T, block_size, perm, s))) return rc;
    return tm.end(ms_out);
}

int pkv_k_quant_encode_perm(const void *x, int dtype, int B, int H, int T, float rel, int bits, const uint32_t *perm,
                            int perm_block, uint8_t *stream, uint64_t capacity, uint32_t *block_info, void *scale,
                            void *zero, uint64_t *size_out, float *ms_out, pkv_stream_t s) {
    PKV_REQUIRE(perm != nullptr, PKV_ERR_INVALID, "null pointer argument");
    return pkv::run_quant_encode<true>(x, dtype, B, H, T, rel, bits, stream, capacity, 0, block_info, scale, zero, T,
                                       size_out, ms_out, (hipStream_t)s, perm, perm_block);
}

int pkv_v_quant_encode_perm(const void *x, int dtype, int B, int H, int T, float rel, int bits, const uint32_t *perm,
                            int perm_block, const void *scale_in, const void *zero_in, uint8_t *stream, uint64_t capacity,
                            uint32_t *block_info, void *scale, void *zero, uint64_t *size_out, float *ms_out, pkv_stream_t s) {
    PKV_REQUIRE(perm != nullptr, PKV_ERR_INVALID, "null pointer argument");
    PKV_REQUIRE((scale_in == nullptr) == (zero_in == nullptr), PKV_ERR_INVALID, "scale_in and zero_in go together");
    PKV_REQUIRE(scale_in == nullptr || (scale_in != scale && zero_in != zero), PKV_ERR_INVALID,
                "the known parameters (order of x) and the written ones (order of the stream) are different arrays");
    return pkv::run_quant_encode<false>(x, dtype, B, H, T, rel, bits, stream, capacity, 0, block_info, scale, zero, T,
                                        size_out, ms_out, (hipStream_t)s, perm, perm_block, scale_in, zero_in);
}

int pkv_quant_params(const void *x, int dtype, int B, int H, int T, float rel, void *scale, void *zero,
                     float *ms_out, pkv_stream_t s_) {
    using namespace pkv;
    hipStream_t s = (hipStream_t)s_;
    int rc = check_xshape(x, dtype, B, H, T);
    if (rc) return rc;
    PKV_REQUIRE(scale && zero, PKV_ERR_INVALID, "null pointer argument");
    PKV_REQUIRE(rel > 0.f, PKV_ERR_INVALID, "quant_scale_rel must be positive");
    LaunchTimer tm(s, ms_out != nullptr);
    if ((rc = tm.begin())) return rc;
    const dim3 grid((unsigned)((T + 15) / 16), (unsigned)B);
    if (dtype == PKV_F16)
        quant_params_kernel<PKV_F16><<<grid, 256, 0, s>>>((const uint16_t *)x, H, T, rel, (uint16_t *)scale,
                                                          (uint16_t *)zero);
    else
        quant_params_kernel<PKV_BF16><<<grid, 256, 0, s>>>((const uint16_t *)x, H, T, rel, (uint16_t *)scale,
                                                           (uint16_t *)zero);
    PKV_HIP_CHECK(hipGetLastError());
    return tm.end(ms_out);
}

int pkv_quantize(const void *x, int dtype, int B, int H, int T, const void *scale, const void *zero,
                 uint8_t *codes, uint32_t *max_code_out, float *ms_out, pkv_stream_t s_) {
    using namespace pkv;
    hipStream_t s = (hipStream_t)s_;
    int rc = check_xshape(x, dtype, B, H, T);
    if (rc) return rc;
    PKV_REQUIRE(scale && zero && codes, PKV_ERR_INVALID, "null pointer argument");
    LaunchTimer tm(s, ms_out != nullptr);
    if ((rc = tm.begin())) return rc;
    const dim3 grid((unsigned)((T + 15) / 16), (unsigned)((H + kQuantHeads - 1) / kQuantHeads), (unsigned)B);
    if (dtype == PKV_F16)
        quantize_kernel<PKV_F16><<<grid, 256, 0, s>>>((const uint16_t *)x, H, T, (const uint16_t *)scale,
                                                      (const uint16_t *)zero, codes, max_code_out);
    else
        quantize_kernel<PKV_BF16><<<grid, 256, 0, s>>>((const uint16_t *)x, H, T, (const uint16_t *)scale,
                                                       (const uint16_t *)zero, codes, max_code_out);
    PKV_HIP_CHECK(hipGetLastError());
    return tm.end(ms_out);
}

int pkv_dequantize(const uint8_t *codes, int dtype, int B, int H, int T, const void *scale,
                   const void *zero, void *x_out, float *ms_out, pkv_stream_t s_) {
    using namespace pkv;
    hipStream_t s = (hipStream_t)s_;
    int rc = check_xshape(x_out, dtype, B, H, T);
    if (rc) return rc;
    PKV_REQUIRE(scale && zero && codes, PKV_ERR_INVALID, "null pointer argument");
    LaunchTimer tm(s, ms_out != nullptr);
    if ((rc = tm.begin())) return rc;
    const dim3 grid((unsigned)((T + 15) / 16), (unsigned)((H + kQuantHeads - 1) / kQuantHeads), (unsigned)B);
    if (dtype == PKV_F16)
        dequantize_kernel<PKV_F16><<<grid, 256, 0, s>>>(codes, H, T, (const uint16_t *)scale,
                                                        (const uint16_t *)zero, (uint16_t *)x_out);
    else
        dequantize_kernel<PKV_BF16><<<grid, 256, 0, s>>>(codes, H, T, (const uint16_t *)scale,
                                                         (const uint16_t *)zero, (uint16_t *)x_out);
    PKV_HIP_CHECK(hipGetLastError());
    return tm.end(ms_out);
}

int pkv_k_quant_encode(const void *x, int dtype, int B, int H, int T, float rel, int bits, uint8_t *stream,
                       uint64_t capacity, uint32_t *block_info, void *scale, void *zero,
                       uint64_t *size_out, float *ms_out, pkv_stream_t s) {
    return pkv::run_quant_encode<true>(x, dtype, B, H, T, rel, bits, stream, capacity, 0, block_info, scale,
                                       zero, T, size_out, ms_out, (hipStream_t)s);
}

int pkv_v_quant_encode(const void *x, int dtype, int B, int H, int T, float rel, int bits, uint8_t *stream,
                       uint64_t capacity, uint32_t *block_info, void *scale, void *zero,
                       uint64_t *size_out, float *ms_out, pkv_stream_t s) {
    return pkv::run_quant_encode<false>(x, dtype, B, H, T, rel, bits, stream, capacity, 0, block_info, scale,
                                        zero, T, size_out, ms_out, (hipStream_t)s);
}

int pkv_k_quant_encode_append(const void *x, int dtype, int B, int H, int T_new, float rel, int bits,
                               uint8_t *stream, uint64_t capacity, uint64_t stream_used, uint32_t *block_info_tail,
                               void *scale_tail, void *zero_tail, int par_stride, uint64_t *size_out,
                               float *ms_out, pkv_stream_t s) {
    return pkv::run_quant_encode<true>(x, dtype, B, H, T_new, rel, bits, stream, capacity, stream_used,
                                       block_info_tail, scale_tail, zero_tail, par_stride, size_out, ms_out,
                                       (hipStream_t)s);
}

int pkv_v_quant_encode_append(const void *x, int dtype, int B, int H, int T_new, float rel, int bits,
                               uint8_t *stream, uint64_t capacity, uint64_t stream_used, uint32_t *block_info_tail,
                               void *scale_tail, void *zero_tail, int par_stride, uint64_t *size_out,
                               float *ms_out, pkv_stream_t s) {
    return pkv::run_quant_encode<false>(x, dtype, B, H, T_new, rel, bits, stream, capacity, stream_used,
                                        block_info_tail, scale_tail, zero_tail, par_stride, size_out, ms_out,
                                        (hipStream_t)s);
}

}  // extern "C"
