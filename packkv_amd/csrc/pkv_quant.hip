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

// ---- x -> uint8 code matrix [T, B*H*128] -----------------------------------------------
// grid (T/16, H, B), 256 threads.
template <int DT>
__global__ void quantize_kernel(const uint16_t *__restrict__ x, int H, int T,
                                const uint16_t *__restrict__ scale, const uint16_t *__restrict__ zero,
                                uint8_t *__restrict__ codes, uint32_t *max_code_out) {
    const int b = blockIdx.z, h = blockIdx.y;
    const int B = gridDim.z;
    const int tok = blockIdx.x * 16 + (threadIdx.x >> 4);
    const int l16 = threadIdx.x & 15;
    uint32_t cmax = 0;
    if (tok < T) {
        const float sc = T16<DT>::from_bits(scale[(size_t)b * T + tok]);
        const float z = T16<DT>::from_bits(zero[(size_t)b * T + tok]);
        const uint4 v = *reinterpret_cast<const uint4 *>(
            x + (((size_t)b * H + h) * T + tok) * kHeadDim + l16 * 8);
        float f[8];
        unpack8<DT>(v, f);
        uint32_t lo = 0, hi = 0;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t c0 = (uint32_t)(int)quant_code<DT>(f[i], sc, z) & 0xFFu;
            const uint32_t c1 = (uint32_t)(int)quant_code<DT>(f[4 + i], sc, z) & 0xFFu;
            lo |= c0 << (8 * i);
            hi |= c1 << (8 * i);
            cmax = max(cmax, max(c0, c1));
        }
        const size_t hidden = (size_t)B * H * kHeadDim;
        uint2 *dst = reinterpret_cast<uint2 *>(codes + (size_t)tok * hidden +
                                               ((size_t)b * H + h) * kHeadDim + l16 * 8);
        *dst = make_uint2(lo, hi);
    }
    if (max_code_out) {
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) cmax = max(cmax, __shfl_xor(cmax, d, 64));
        if ((threadIdx.x & 63) == 0 && cmax) atomicMax(max_code_out, cmax);
    }
}

// ---- uint8 code matrix -> x_hat [B, H, T, 128] -----------------------------------------
template <int DT>
__global__ void dequantize_kernel(const uint8_t *__restrict__ codes, int H, int T,
                                  const uint16_t *__restrict__ scale, const uint16_t *__restrict__ zero,
                                  uint16_t *__restrict__ x) {
    const int b = blockIdx.z, h = blockIdx.y;
    const int B = gridDim.z;
    const int tok = blockIdx.x * 16 + (threadIdx.x >> 4);
    const int l16 = threadIdx.x & 15;
    if (tok >= T) return;
    const float sc = T16<DT>::from_bits(scale[(size_t)b * T + tok]);
    const float z = T16<DT>::from_bits(zero[(size_t)b * T + tok]);
    const size_t hidden = (size_t)B * H * kHeadDim;
    const uint2 c = *reinterpret_cast<const uint2 *>(codes + (size_t)tok * hidden +
                                                    ((size_t)b * H + h) * kHeadDim + l16 * 8);
    uint32_t out[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const uint32_t w = i < 2 ? c.x : c.y;
        const float a0 = (float)((w >> (16 * (i & 1))) & 0xFFu);
        const float a1 = (float)((w >> (16 * (i & 1) + 8)) & 0xFFu);
        const uint32_t r0 = T16<DT>::to_bits(round_t<DT>(a0 + z) * sc);
        const uint32_t r1 = T16<DT>::to_bits(round_t<DT>(a1 + z) * sc);
        out[i] = r0 | (r1 << 16);
    }
    *reinterpret_cast<uint4 *>(x + (((size_t)b * H + h) * T + tok) * kHeadDim + l16 * 8) =
        make_uint4(out[0], out[1], out[2], out[3]);
}

// ---- fused quantize + encode -------------------------------------------------------------
// One workgroup per block, in ticket order.  The workgroup quantizes its tile of x straight
// into the LDS code tile and then runs the same block encoder as the codes->stream kernel.
template <bool IS_K, int DT>
__global__ void quant_pack_kernel(const uint16_t *__restrict__ x, int H, int T,
                                  const uint16_t *__restrict__ scale, const uint16_t *__restrict__ zero,
                                  uint8_t *__restrict__ stream, uint64_t capacity,
                                  uint32_t *__restrict__ info, ScanState *st, int hidden_dim, int ctx_blk,
                                  int hid_blk, int nunits, int W, uint32_t nblocks) {
    extern __shared__ __align__(16) uint8_t lds[];
    __shared__ uint32_t s_idx;
    __shared__ uint64_t s_off;
    __shared__ uint32_t unit_bytes[16];
    uint8_t *tile = lds;
    uint8_t *blk = lds + ((uint32_t)(ctx_blk * hid_blk + 15) & ~15u);
    if (threadIdx.x == 0) s_idx = atomicAdd(&st->ticket, 1u);
    __syncthreads();
    const uint32_t bidx = s_idx;
    if (bidx >= nblocks) return;
    const int n_hid = hidden_dim / hid_blk;
    const uint32_t cb = bidx / n_hid, hb = bidx % n_hid;
    const uint32_t ch0 = hb * hid_blk;              // first channel of the block in [0, B*H*128)
    const uint32_t bh = ch0 / kHeadDim;             // b * H + h
    const uint32_t b = bh / H;
    const uint32_t d0 = ch0 % kHeadDim;
    const int lanes_per_row = hid_blk / 8;          // 8 channels per thread
    const int rows_per_pass = blockDim.x / lanes_per_row;
    const int lr = threadIdx.x % lanes_per_row;
    uint32_t cmax = 0;
    for (int r = threadIdx.x / lanes_per_row; r < ctx_blk; r += rows_per_pass) {
        const size_t tok = (size_t)cb * ctx_blk + r;
        const float sc = T16<DT>::from_bits(scale[(size_t)b * T + tok]);
        const float z = T16<DT>::from_bits(zero[(size_t)b * T + tok]);
        const uint4 v = *reinterpret_cast<const uint4 *>(
            x + ((size_t)bh * T + tok) * kHeadDim + d0 + lr * 8);
        float f[8];
        unpack8<DT>(v, f);
        uint32_t lo = 0, hi = 0;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t c0 = (uint32_t)(int)quant_code<DT>(f[i], sc, z) & 0xFFu;
            const uint32_t c1 = (uint32_t)(int)quant_code<DT>(f[4 + i], sc, z) & 0xFFu;
            lo |= c0 << (8 * i);
            hi |= c1 << (8 * i);
            cmax = max(cmax, max(c0, c1));
        }
        *reinterpret_cast<uint2 *>(tile + r * hid_blk + lr * 8) = make_uint2(lo, hi);
    }
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) cmax = max(cmax, __shfl_xor(cmax, d, 64));
    if ((threadIdx.x & 63) == 0 && cmax >= (1u << W)) atomicMax(&st->max_code, cmax);
    __syncthreads();
    block_finish<IS_K>(tile, blk, unit_bytes, &s_off, st, bidx, nblocks, stream, capacity, info, hid_blk,
                       nunits, W);
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
                            uint8_t *stream, uint64_t capacity, uint32_t *info, void *scale, void *zero,
                            uint64_t *size_out, float *ms_out, hipStream_t s) {
    int rc = check_xshape(x, dtype, B, H, T);
    if (rc) return rc;
    PKV_REQUIRE(stream && info && scale && zero, PKV_ERR_INVALID, "null pointer argument");
    PKV_REQUIRE(capacity > 0, PKV_ERR_INVALID, "compressed_buffer must be a non-empty tensor");
    PKV_REQUIRE(bits >= 2 && bits <= 4, PKV_ERR_UNSUPPORTED, "not supported: bits_len %d (need 2..4)", bits);
    PKV_REQUIRE(rel > 0.f, PKV_ERR_INVALID, "quant_scale_rel must be positive");
    const int ctx_blk = IS_K ? 64 : 128, hid_blk = IS_K ? 128 : 64;
    PKV_REQUIRE(T % ctx_blk == 0, PKV_ERR_INVALID, "ctx_len must be divisible by ctx_len_block_size");
    const int hidden = B * H * kHeadDim;
    const int nunits = 4;
    const uint32_t nblocks = (uint32_t)(T / ctx_blk) * (uint32_t)(hidden / hid_blk);
    const uint32_t cap = IS_K ? (uint32_t)k_block_bound(ctx_blk, bits) : (uint32_t)v_block_bound(hid_blk, bits);
    const uint32_t lds_bytes = (uint32_t)(ctx_blk * hid_blk) + ((cap + 15u) & ~15u) + 32u;
    ScanState *st = nullptr;
    if ((rc = prepare_scan_state(nblocks, &st, s))) return rc;
    LaunchTimer tm(s, ms_out != nullptr);
    if ((rc = tm.begin())) return rc;
    const dim3 pgrid((unsigned)((T + 15) / 16), (unsigned)B);
    if (dtype == PKV_F16) {
        quant_params_kernel<PKV_F16><<<pgrid, 256, 0, s>>>((const uint16_t *)x, H, T, rel, (uint16_t *)scale,
                                                           (uint16_t *)zero);
        quant_pack_kernel<IS_K, PKV_F16><<<nblocks, 128, lds_bytes, s>>>(
            (const uint16_t *)x, H, T, (const uint16_t *)scale, (const uint16_t *)zero, stream, capacity, info,
            st, hidden, ctx_blk, hid_blk, nunits, bits, nblocks);
    } else {
        quant_params_kernel<PKV_BF16><<<pgrid, 256, 0, s>>>((const uint16_t *)x, H, T, rel, (uint16_t *)scale,
                                                            (uint16_t *)zero);
        quant_pack_kernel<IS_K, PKV_BF16><<<nblocks, 128, lds_bytes, s>>>(
            (const uint16_t *)x, H, T, (const uint16_t *)scale, (const uint16_t *)zero, stream, capacity, info,
            st, hidden, ctx_blk, hid_blk, nunits, bits, nblocks);
    }
    PKV_HIP_CHECK(hipGetLastError());
    if ((rc = tm.end(ms_out))) return rc;
    return finish_encode(st, size_out, bits, s);
}

}  // namespace pkv

extern "C" {

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
    const dim3 grid((unsigned)((T + 15) / 16), (unsigned)H, (unsigned)B);
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
    const dim3 grid((unsigned)((T + 15) / 16), (unsigned)H, (unsigned)B);
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
    return pkv::run_quant_encode<true>(x, dtype, B, H, T, rel, bits, stream, capacity, block_info, scale,
                                       zero, size_out, ms_out, (hipStream_t)s);
}

int pkv_v_quant_encode(const void *x, int dtype, int B, int H, int T, float rel, int bits, uint8_t *stream,
                       uint64_t capacity, uint32_t *block_info, void *scale, void *zero,
                       uint64_t *size_out, float *ms_out, pkv_stream_t s) {
    return pkv::run_quant_encode<false>(x, dtype, B, H, T, rel, bits, stream, capacity, block_info, scale,
                                        zero, size_out, ms_out, (hipStream_t)s);
}

}  // extern "C"
