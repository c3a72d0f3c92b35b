// Shared definitions for the PackKV gfx950 kernels: stream-format constants, error
// plumbing, and the small wavefront-level helpers every kernel uses.
//
// Stream format (restated from packkv_cuda_ext/src/{k,v}_encode_cpu.cpp of the reference):
//   pack    16 consecutive tokens of one channel; min, len = bit_length(max - min),
//           word = sum_k (code_k - min) << ((15 - k) * len), stored as 2*len bytes LE
//   K block ctx_blk tokens x 128 channels: u16 cumulative round sizes, then per round
//           (16 tokens): mins (W bits/pack) | lens (LB bits/pack) | payload in the order
//           slot-major, lane-minor, lane t owning channels 4t..4t+3 (slot i = channel 4t+i)
//   V block 128 tokens x 32*warps channels: u16 cumulative segment sizes in (warp, seg)
//           order, then per segment (64 tokens x 32 channels): mins | lens | payload,
//           lane t owning channel 32*warp + t, slot i = round 4*seg + i
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include "../../include/packkv.h"   // PKV_* status codes and the exported prototypes

namespace pkv {

constexpr int kPackTok = 16;    // tokens per pack        (static_def.h:6)
constexpr int kLanes = 32;      // format lanes per round (static_def.h:4)
constexpr int kHeadDim = 128;   // K block width          (static_def.h:5)

__host__ __device__ constexpr int len_field_bits(int W) {  // include/utils.h:24-36: bits that hold 0..W
    return W >= 8 ? 4 : (W >= 4 ? 3 : (W >= 2 ? 2 : 1));
}
constexpr int kMaxBits = 8;     // widths 5..8 are this library's extension of the format (pack words up to 128 bits)
__host__ __device__ constexpr int k_block_bound(int ctx_blk, int W) {
    return 2 * (ctx_blk / kPackTok) +
           (ctx_blk / kPackTok) * kHeadDim * (W + len_field_bits(W)) / 8 +
           (ctx_blk / kPackTok) * kHeadDim * 2 * W;
}
__host__ __device__ constexpr int v_block_bound(int hid_blk, int W) {
    return 4 * (hid_blk / kLanes) + 8 * hid_blk * (W + len_field_bits(W)) / 8 + 8 * hid_blk * 2 * W;
}

void set_error(const char *fmt, ...);

#define PKV_HIP_CHECK(expr)                                                              \
    do {                                                                                 \
        hipError_t e__ = (expr);                                                         \
        if (e__ != hipSuccess) {                                                         \
            ::pkv::set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(e__),     \
                             __FILE__, __LINE__);                                        \
            return PKV_ERR_HIP;                                                   \
        }                                                                                \
    } while (0)

#define PKV_REQUIRE(cond, code, ...)                                                     \
    do {                                                                                 \
        if (!(cond)) {                                                                   \
            ::pkv::set_error(__VA_ARGS__);                                               \
            return (code);                                                               \
        }                                                                                \
    } while (0)

// ---- device helpers ---------------------------------------------------------
#ifdef __HIPCC__

__device__ __forceinline__ int bit_length_u32(uint32_t v) { return 32 - __clz((int)v); }

// Inclusive prefix sum inside each 32-lane half of the wavefront, on the DPP data path
// (row_shr 1/2/4/8 inside 16-lane rows, then row_bcast:15 into rows 1 and 3).
__device__ __forceinline__ uint32_t half_incl_scan(uint32_t v) {
    uint32_t x = v;
    x += __builtin_amdgcn_update_dpp(0u, x, 0x111, 0xF, 0xF, true);
    x += __builtin_amdgcn_update_dpp(0u, x, 0x112, 0xF, 0xF, true);
    x += __builtin_amdgcn_update_dpp(0u, x, 0x114, 0xF, 0xF, true);
    x += __builtin_amdgcn_update_dpp(0u, x, 0x118, 0xF, 0xF, true);
    x += __builtin_amdgcn_update_dpp(0u, x, 0x142, 0xA, 0xF, true);
    return x;
}

// Value held by the last lane of the caller's 32-lane half.
__device__ __forceinline__ uint32_t half_last(uint32_t x) {
    const uint32_t a = __builtin_amdgcn_readlane(x, 31), b = __builtin_amdgcn_readlane(x, 63);
    return (threadIdx.x & 32) ? b : a;
}

// Exclusive prefix sum over the 32 lanes of a half-wavefront; `total` receives the sum.
__device__ __forceinline__ uint32_t half_excl_scan(uint32_t v, uint32_t &total) {
    const uint32_t incl = half_incl_scan(v);
    total = half_last(incl);
    return incl - v;
}

// Payload byte offsets of a lane's four packs (stream order: slot-major, lane-minor) from
// their bit widths: two packed 16-bit scans instead of four.
__device__ __forceinline__ void pack_offsets(const uint32_t len[4], uint32_t off[4], uint32_t &payload) {
    const uint32_t a = (2u * len[0]) | ((2u * len[1]) << 16);
    const uint32_t b = (2u * len[2]) | ((2u * len[3]) << 16);
    const uint32_t ia = half_incl_scan(a), ib = half_incl_scan(b);
    const uint32_t ta = half_last(ia), tb = half_last(ib);
    const uint32_t ea = ia - a, eb = ib - b;
    const uint32_t t0 = ta & 0xFFFFu, t01 = t0 + (ta >> 16), t012 = t01 + (tb & 0xFFFFu);
    off[0] = ea & 0xFFFFu;
    off[1] = t0 + (ea >> 16);
    off[2] = t01 + (eb & 0xFFFFu);
    off[3] = t012 + (eb >> 16);
    payload = t012 + (tb >> 16);
}

// 64 bits starting at byte offset `off` (2-byte aligned) of an LDS byte array whose base is
// 4-byte aligned.  gfx950 does execute DS reads at any alignment, but a misaligned 64-bit read
// stalls the LDS pipeline (SQ_LDS_UNALIGNED_STALL), so this reads the three aligned dwords that
// cover the range and funnel-shifts them.
__device__ __forceinline__ uint64_t lds_load64(const uint8_t *lds, uint32_t off) {
    const uint32_t *p = reinterpret_cast<const uint32_t *>(lds + (off & ~3u));
    const uint32_t d0 = p[0], d1 = p[1], d2 = p[2];
    const uint32_t sh = (off & 2u) * 8u;
    const uint32_t lo = __builtin_amdgcn_alignbit(d1, d0, sh);
    const uint32_t hi = __builtin_amdgcn_alignbit(d2, d1, sh);
    return ((uint64_t)hi << 32) | lo;
}

// The 4*nbits-bit metadata word of format lane t from an LSB-first bit array in LDS (4 fields
// of nbits each; nbits in 2..8; `arr` 2-byte aligned).  Reads the two aligned dwords around
// the field and funnel-shifts: adjacent byte reads would be merged into misaligned 16-bit DS
// reads, which stall the LDS pipeline.
__device__ __forceinline__ uint32_t lds_meta_word(const uint8_t *arr, int t, int nbits) {
    const uint32_t addr = (uint32_t)reinterpret_cast<uintptr_t>(arr);      // LDS byte address
    const uint32_t bit = (addr & 3u) * 8u + (uint32_t)t * 4u * (uint32_t)nbits;
    const uint32_t *p = reinterpret_cast<const uint32_t *>(arr - (addr & 3u)) + (bit >> 5);
    const uint32_t v = __builtin_amdgcn_alignbit(p[1], p[0], bit & 31u);
    return nbits >= 8 ? v : v & ((1u << (4 * nbits)) - 1u);
}

// Where block b of a stream of `stream_bytes` bytes lies according to block_info, made safe to read: never more
// than `cap` bytes, never outside the stream.  (block_info is device data the library does not own: a damaged entry
// yields garbage codes, not an access outside the buffer.)
__device__ __forceinline__ void block_span(const uint32_t *__restrict__ info, uint32_t b, uint32_t cap, uint64_t stream_bytes,
                                           uint32_t &off, uint32_t &size) {
    off = info[2 * (size_t)b];
    size = min(info[2 * (size_t)b + 1], cap);
    if ((uint64_t)off > stream_bytes) off = (uint32_t)stream_bytes;       // (streams are below 4 GiB)
    size = (uint32_t)min((uint64_t)size, stream_bytes - (uint64_t)off);
}

// Copy `nbytes` from global `src` (any alignment) into LDS `dst` (16-byte aligned, room for nbytes + 30) so that
// dst[(src & 15) + i] == src[i]; touches only the aligned 16-byte chunks that overlap the range (a chunk never
// straddles a page, so the bytes around the range that come along are always mapped).  Returns the phase (src & 15).
__device__ __forceinline__ uint32_t stage_to_lds(const uint8_t *src, uint32_t nbytes, uint8_t *dst,
                                                 int tid, int nthreads) {
    const uint32_t phase = (uint32_t)(reinterpret_cast<uintptr_t>(src) & 15u);
    const uint4 *s16 = reinterpret_cast<const uint4 *>(src - phase);
    uint4 *d16 = reinterpret_cast<uint4 *>(dst);
    const uint32_t n16 = (phase + nbytes + 15u) >> 4;
    // four loads in flight per thread before the first LDS store: the copy is latency-bound otherwise
    for (uint32_t i = tid; i < n16; i += 4u * (uint32_t)nthreads) {
        uint4 v[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const uint32_t idx = i + (uint32_t)u * (uint32_t)nthreads;
            v[u] = idx < n16 ? s16[idx] : make_uint4(0u, 0u, 0u, 0u);
        }
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const uint32_t idx = i + (uint32_t)u * (uint32_t)nthreads;
            if (idx < n16) d16[idx] = v[u];
        }
    }
    return phase;
}

#endif  // __HIPCC__

}  // namespace pkv
