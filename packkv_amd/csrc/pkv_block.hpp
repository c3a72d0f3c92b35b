// Block-level codec building blocks shared by the unpack, encode and fused
// quantize+encode kernels.  A "unit" is what one 32-lane half-wavefront handles:
//   K: one round  (16 tokens x 128 channels), lane t <-> channels 4t..4t+3, slot i = channel 4t+i
//   V: one segment (64 tokens x 32 channels), lane t <-> channel 32*warp+t, slot i = round 4*seg+i
// In both cases the unit's bytes are  mins | lens | payload  with payload ordered slot-major,
// lane-minor, so parsing and emitting are the same code; only the tile scatter differs.
#pragma once
#include "pkv_common.hpp"

namespace pkv {

struct UnitGeom {
    int mins_bytes;   // W * 128 / 8
    int lens_bytes;   // LB * 128 / 8
    int W, LB;
};

__host__ __device__ inline UnitGeom unit_geom(int W) {
    UnitGeom g;
    g.W = W;
    g.LB = len_field_bits(W);
    g.mins_bytes = W * 16;
    g.lens_bytes = g.LB * 16;
    return g;
}

#ifdef __HIPCC__

// Tile addressing: the uint8 code tile in LDS is row-major [tokens][hid_blk].
template <bool IS_K>
__device__ __forceinline__ int tile_index(int unit, int slot, int k, int t, int hid_blk) {
    if (IS_K) return (unit * kPackTok + k) * hid_blk + 4 * t + slot;
    const int warp = unit >> 1, seg = unit & 1;
    return ((seg * 4 + slot) * kPackTok + k) * hid_blk + warp * kLanes + t;
}

struct UnitPacks {
    uint64_t word[4];
    uint32_t len[4];
    uint32_t mn[4];
    uint32_t off[4];     // byte offset of each pack inside the unit's payload
    uint32_t payload;    // payload bytes of the whole unit
};

// Read lane t's four packs (min, len, word) of the unit whose bytes start at blk[unit_off].
__device__ __forceinline__ void unit_parse(const uint8_t *blk, uint32_t unit_off, int t, const UnitGeom g,
                                           UnitPacks &u) {
    const uint32_t minsw = lds_meta_word(blk + unit_off, t, g.W);
    const uint32_t lensw = lds_meta_word(blk + unit_off + g.mins_bytes, t, g.LB);
    const uint32_t pay0 = unit_off + g.mins_bytes + g.lens_bytes;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        u.len[i] = (lensw >> (i * g.LB)) & ((1u << g.LB) - 1u);
        u.mn[i] = (minsw >> (i * g.W)) & ((1u << g.W) - 1u);
    }
    pack_offsets(u.len, u.off, u.payload);
    // bits above 16*len belong to the next pack; every consumer masks per field
#pragma unroll
    for (int i = 0; i < 4; i++) u.word[i] = lds_load64(blk, pay0 + u.off[i]);
}

// Parse two independent units at once (same lane t in both), batching the LDS round trips:
// all metadata reads first, then both offset scans, then all eight pack words.
__device__ __forceinline__ void unit_parse2(const uint8_t *blk_a, uint32_t off_a, const UnitGeom ga, UnitPacks &ua,
                                            const uint8_t *blk_b, uint32_t off_b, const UnitGeom gb, UnitPacks &ub,
                                            int t) {
    const uint32_t mins_a = lds_meta_word(blk_a + off_a, t, ga.W);
    const uint32_t lens_a = lds_meta_word(blk_a + off_a + ga.mins_bytes, t, ga.LB);
    const uint32_t mins_b = lds_meta_word(blk_b + off_b, t, gb.W);
    const uint32_t lens_b = lds_meta_word(blk_b + off_b + gb.mins_bytes, t, gb.LB);
#pragma unroll
    for (int i = 0; i < 4; i++) {
        ua.len[i] = (lens_a >> (i * ga.LB)) & ((1u << ga.LB) - 1u);
        ua.mn[i] = (mins_a >> (i * ga.W)) & ((1u << ga.W) - 1u);
        ub.len[i] = (lens_b >> (i * gb.LB)) & ((1u << gb.LB) - 1u);
        ub.mn[i] = (mins_b >> (i * gb.W)) & ((1u << gb.W) - 1u);
    }
    pack_offsets(ua.len, ua.off, ua.payload);
    pack_offsets(ub.len, ub.off, ub.payload);
    const uint32_t pay_a = off_a + ga.mins_bytes + ga.lens_bytes, pay_b = off_b + gb.mins_bytes + gb.lens_bytes;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        ua.word[i] = lds_load64(blk_a, pay_a + ua.off[i]);
        ub.word[i] = lds_load64(blk_b, pay_b + ub.off[i]);
    }
}

// ---- widths 5..8 (format extension): pack words of up to 128 bits, plain field-by-field code ----
typedef unsigned __int128 word128;

template <bool IS_K>
__device__ __forceinline__ void unit_decode_wide(const uint8_t *blk, uint32_t unit_off, int unit, int t,
                                                 const UnitGeom g, uint8_t *tile, int hid_blk) {
    const uint32_t minsw = lds_meta_word(blk + unit_off, t, g.W);
    const uint32_t lensw = lds_meta_word(blk + unit_off + g.mins_bytes, t, g.LB);
    const uint32_t pay0 = unit_off + g.mins_bytes + g.lens_bytes;
    uint32_t len[4], mn[4], off[4], payload;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        len[i] = (lensw >> (i * g.LB)) & ((1u << g.LB) - 1u);
        mn[i] = (minsw >> (i * g.W)) & ((1u << g.W) - 1u);
    }
    pack_offsets(len, off, payload);
#pragma unroll
    for (int i = 0; i < 4; i++) {
        // the word as four dwords, shifted down one field at a time (token 15 sits in the lowest field)
        const uint64_t lo = lds_load64(blk, pay0 + off[i]), hi = lds_load64(blk, pay0 + off[i] + 8u);
        uint32_t d0 = (uint32_t)lo, d1 = (uint32_t)(lo >> 32), d2 = (uint32_t)hi, d3 = (uint32_t)(hi >> 32);
        const uint32_t mask = (1u << len[i]) - 1u, sh = len[i];
#pragma unroll
        for (int k = kPackTok - 1; k >= 0; k--) {
            tile[tile_index<IS_K>(unit, i, k, t, hid_blk)] = (uint8_t)((d0 & mask) + mn[i]);
            d0 = __builtin_amdgcn_alignbit(d1, d0, sh);
            d1 = __builtin_amdgcn_alignbit(d2, d1, sh);
            d2 = __builtin_amdgcn_alignbit(d3, d2, sh);
            d3 >>= sh;
        }
    }
}

// Decode one unit whose bytes start at blk[unit_off] into the LDS tile.
// The four pack words are cut into 16-bit windows of four tokens (packs 0|1 and 2|3 share a
// register), so one packed 16-bit shift moves two packs at a time and a byte permute gathers the
// four codes of a token: 5 instructions per four codes instead of a 64-bit shift per code.
template <bool IS_K>
__device__ __forceinline__ void unit_decode(const uint8_t *blk, uint32_t unit_off, int unit, int t,
                                            const UnitGeom g, uint8_t *tile, int hid_blk) {
    typedef unsigned short u16pair __attribute__((ext_vector_type(2)));
    if (g.W > 4) {      // uniform
        unit_decode_wide<IS_K>(blk, unit_off, unit, t, g, tile, hid_blk);
        return;
    }
    UnitPacks u;
    unit_parse(blk, unit_off, t, g, u);
    uint32_t hlf[4][2];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        hlf[i][0] = (uint32_t)(u.word[i] >> (8u * u.len[i]));   // tokens 0..7
        hlf[i][1] = (uint32_t)u.word[i];                        // tokens 8..15
    }
    const uint32_t len01 = u.len[0] | (u.len[1] << 16), len23 = u.len[2] | (u.len[3] << 16);
    const uint32_t mq = ((1u << u.len[0]) - 1u) | (((1u << u.len[1]) - 1u) << 8) | (((1u << u.len[2]) - 1u) << 16) |
                        (((1u << u.len[3]) - 1u) << 24);
    const uint32_t minq = u.mn[0] | (u.mn[1] << 8) | (u.mn[2] << 16) | (u.mn[3] << 24);
#pragma unroll
    for (int q = 0; q < 4; q++) {
        uint32_t qd[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t src = hlf[i][q >> 1];
            qd[i] = (q & 1) ? src : (src >> (4u * u.len[i]));
        }
        const uint32_t w01 = __builtin_amdgcn_perm(qd[1], qd[0], 0x05040100u);   // tokens 4q..4q+3 of packs 0 | 1
        const uint32_t w23 = __builtin_amdgcn_perm(qd[3], qd[2], 0x05040100u);
#pragma unroll
        for (int pp = 0; pp < 4; pp++) {
            const int k = 4 * q + pp;
            const u16pair s01 = __builtin_bit_cast(u16pair, len01 * (uint32_t)(3 - pp));
            const u16pair s23 = __builtin_bit_cast(u16pair, len23 * (uint32_t)(3 - pp));
            const uint32_t x01 = __builtin_bit_cast(uint32_t, (u16pair)(__builtin_bit_cast(u16pair, w01) >> s01));
            const uint32_t x23 = __builtin_bit_cast(uint32_t, (u16pair)(__builtin_bit_cast(u16pair, w23) >> s23));
            const uint32_t c4 = (__builtin_amdgcn_perm(x23, x01, 0x06040200u) & mq) + minq;   // codes of slots 0..3
            if (IS_K) {   // slots are the four adjacent channels 4t..4t+3 of token k
                *reinterpret_cast<uint32_t *>(tile + tile_index<true>(unit, 0, k, t, hid_blk)) = c4;
            } else {      // slots are four rounds of channel t
#pragma unroll
                for (int i = 0; i < 4; i++) tile[tile_index<false>(unit, i, k, t, hid_blk)] = (uint8_t)(c4 >> (8 * i));
            }
        }
    }
}

// Gather lane t's four packs of `unit` from the LDS code tile and compute min / len / word
// and the payload offsets (one 32-lane exclusive scan per slot).
template <bool IS_K>
__device__ __forceinline__ void unit_analyse(const uint8_t *tile, int hid_blk, int unit, int t,
                                             UnitPacks &u) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
        uint32_t c[kPackTok];
        uint32_t mn = 255u, mx = 0u;
#pragma unroll
        for (int k = 0; k < kPackTok; k++) {
            c[k] = tile[tile_index<IS_K>(unit, i, k, t, hid_blk)];
            mn = min(mn, c[k]);
            mx = max(mx, c[k]);
        }
        const uint32_t len = (uint32_t)bit_length_u32(mx - mn);
        uint64_t w = 0;
#pragma unroll
        for (int k = 0; k < kPackTok; k++) w = (w << len) | (uint64_t)(c[k] - mn);
        u.word[i] = w;
        u.len[i] = len;
        u.mn[i] = mn;
    }
    pack_offsets(u.len, u.off, u.payload);
}

// Write lane t's 4*nbits-bit metadata word into an LSB-first bit array (nbits in {2,3,4}).
__device__ __forceinline__ void lds_put_meta(uint8_t *arr, int t, int nbits, uint32_t w) {
    if (nbits == 4) {
        reinterpret_cast<uint16_t *>(arr)[t] = (uint16_t)w;
    } else if (nbits == 2) {
        arr[t] = (uint8_t)w;
    } else if (nbits == 3) {  // 12 bits per lane: an even/odd lane pair shares three bytes
        const uint32_t hi = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)w, 0xF5, 0xF, 0xF, false);    // the odd neighbour's word (quad_perm [1,1,3,3])
        if ((t & 1) == 0) {
            const uint32_t v = w | (hi << 12);
            uint8_t *p = arr + (t >> 1) * 3;
            p[0] = (uint8_t)v;
            p[1] = (uint8_t)(v >> 8);
            p[2] = (uint8_t)(v >> 16);
        }
    } else if (nbits == 6) {  // 24 bits per lane: three bytes of its own
        uint8_t *p = arr + t * 3;
        p[0] = (uint8_t)w;
        p[1] = (uint8_t)(w >> 8);
        p[2] = (uint8_t)(w >> 16);
    } else {                  // nbits == 5: 20 bits per lane, an even/odd lane pair shares five bytes
        const uint32_t hi = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)w, 0xF5, 0xF, 0xF, false);    // the odd neighbour's word (quad_perm [1,1,3,3])
        if ((t & 1) == 0) {
            const uint64_t v = (uint64_t)w | ((uint64_t)hi << 20);
            uint8_t *p = arr + (t >> 1) * 5;
#pragma unroll
            for (int i = 0; i < 5; i++) p[i] = (uint8_t)(v >> (8 * i));
        }
    }
}

// Emit one analysed unit at blk[unit_off] (unit_off even, blk 4-byte aligned).
__device__ __forceinline__ void unit_emit(uint8_t *blk, uint32_t unit_off, int t, const UnitGeom g,
                                          const UnitPacks &u) {
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
    for (int i = 0; i < 4; i++) {
        // one predicated 16-bit store per piece, written out (a loop over the lane's own length costs a shift, a
        // compare and the loop's control flow per piece)
        uint16_t *dst = reinterpret_cast<uint16_t *>(pay + u.off[i]);
        const uint32_t lo = (uint32_t)u.word[i], hi = (uint32_t)(u.word[i] >> 32), len = u.len[i];
        if (len > 0u) dst[0] = (uint16_t)lo;
        if (len > 1u) dst[1] = (uint16_t)(lo >> 16);
        if (len > 2u) dst[2] = (uint16_t)hi;
        if (len > 3u) dst[3] = (uint16_t)(hi >> 16);
    }
}

// Widths 5..8: analyse lane t's four packs of `unit` and write them at blk[unit_off] (the unit's size is
// known from a first call with blk == nullptr, which only returns it).  The metadata fields do not fall on byte
// boundaries for every width, so the unit's metadata area is cleared and the fields are OR-ed in.
template <bool IS_K>
__device__ __forceinline__ uint32_t unit_encode_wide(const uint8_t *tile, int hid_blk, int unit, int t,
                                                     const UnitGeom g, uint8_t *blk, uint32_t unit_off) {
    word128 word[4];
    uint32_t len[4], mn[4], off[4], payload;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        uint32_t lo = 255u, hi = 0u;
        for (int k = 0; k < kPackTok; k++) {
            const uint32_t c = tile[tile_index<IS_K>(unit, i, k, t, hid_blk)];
            lo = min(lo, c);
            hi = max(hi, c);
        }
        len[i] = (uint32_t)bit_length_u32(hi - lo);
        mn[i] = lo;
        word128 w = 0;
        for (int k = 0; k < kPackTok; k++)
            w = (w << len[i]) | (word128)(tile[tile_index<IS_K>(unit, i, k, t, hid_blk)] - lo);
        word[i] = w;
    }
    pack_offsets(len, off, payload);
    const uint32_t meta = (uint32_t)(g.mins_bytes + g.lens_bytes);
    if (blk == nullptr) return meta + payload;
    uint16_t *m16 = reinterpret_cast<uint16_t *>(blk + unit_off);
    for (uint32_t i = t; i < meta / 2u; i += 32) m16[i] = 0;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");      // LDS serves a wavefront's accesses in order
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    uint32_t minsw = 0, lensw = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        minsw |= mn[i] << (i * g.W);
        lensw |= len[i] << (i * g.LB);
    }
    auto or_field = [&](uint8_t *arr, int nbits, uint32_t v) {       // 4 * nbits bits at bit 4 * t * nbits of arr
        const uint32_t addr = (uint32_t)reinterpret_cast<uintptr_t>(arr);
        const uint32_t bit = (addr & 3u) * 8u + (uint32_t)t * 4u * (uint32_t)nbits;
        uint32_t *p = reinterpret_cast<uint32_t *>(arr - (addr & 3u)) + (bit >> 5);
        const uint64_t wide = (uint64_t)v << (bit & 31u);
        atomicOr(p, (uint32_t)wide);
        if ((uint32_t)(wide >> 32)) atomicOr(p + 1, (uint32_t)(wide >> 32));
    };
    or_field(blk + unit_off, g.W, minsw);
    or_field(blk + unit_off + g.mins_bytes, g.LB, lensw);
    uint8_t *pay = blk + unit_off + meta;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        uint16_t *dst = reinterpret_cast<uint16_t *>(pay + off[i]);
        const word128 w = word[i];
        const uint32_t d[4] = {(uint32_t)w, (uint32_t)(w >> 32), (uint32_t)(w >> 64), (uint32_t)(w >> 96)};
#pragma unroll
        for (uint32_t b = 0; b < 8; b++)                  // (written out: one predicated 16-bit store per piece)
            if (b < len[i]) dst[b] = (uint16_t)(d[b >> 1] >> (16u * (b & 1u)));
    }
    return meta + payload;
}

// Encode the LDS code tile of one block into the LDS buffer `blk`; every thread of the
// workgroup must call it, and the workgroup must hold at least one half-wavefront per unit
// (blockDim.x >= 32 * nunits).  `unit_bytes` is an LDS array of >= nunits uint32.  Returns
// the block size in bytes (uniform).  Contains __syncthreads().
struct ScanState;
__device__ __forceinline__ void lookback_publish(ScanState *st, uint32_t idx, uint32_t my_bytes);

// With `st`, the block's size is published for the look-backs of its successors as soon as it is known, before the
// units are written (the caller then tells lookback_offset that it is published).
template <bool IS_K>
__device__ __forceinline__ uint32_t block_encode(const uint8_t *tile, int hid_blk, int nunits, int W,
                                                 uint8_t *blk, uint32_t *unit_bytes, ScanState *st = nullptr,
                                                 uint32_t idx = 0) {
    const UnitGeom g = unit_geom(W);
    const int t = threadIdx.x & 31;
    const int unit = threadIdx.x >> 5;
    const bool active = unit < nunits;
    const uint32_t hdr = 2u * (uint32_t)nunits;
    UnitPacks u;
    const bool wide = W > 4;
    if (active) {
        if (wide) {
            const uint32_t usz = unit_encode_wide<IS_K>(tile, hid_blk, unit, t, g, nullptr, 0u);
            if (t == 0) unit_bytes[unit] = usz;
        } else {
            unit_analyse<IS_K>(tile, hid_blk, unit, t, u);
            if (t == 0) unit_bytes[unit] = (uint32_t)(g.mins_bytes + g.lens_bytes) + u.payload;
        }
    }
    __syncthreads();
    uint32_t total = hdr;
    for (int q = 0; q < nunits; q++) total += unit_bytes[q];
    if (st && threadIdx.x == 0) lookback_publish(st, idx, total);
    if (active) {
        uint32_t base = hdr;
        for (int q = 0; q < unit; q++) base += unit_bytes[q];
        if (t == 0) reinterpret_cast<uint16_t *>(blk)[unit] = (uint16_t)(base - hdr + unit_bytes[unit]);
        if (wide) unit_encode_wide<IS_K>(tile, hid_blk, unit, t, g, blk, base);
        else unit_emit(blk, base, t, g, u);
    }
    __syncthreads();
    return total;
}

// Decode a staged block (bytes at blk[phase..]) into the LDS code tile; needs one
// half-wavefront per unit like block_encode.
template <bool IS_K>
__device__ __forceinline__ void block_decode(const uint8_t *blk, uint32_t phase, int nunits, int W,
                                             uint8_t *tile, int hid_blk) {
    const UnitGeom g = unit_geom(W);
    const int t = threadIdx.x & 31;
    const int unit = threadIdx.x >> 5;
    const uint32_t hdr = 2u * (uint32_t)nunits;
    const uint16_t *cum = reinterpret_cast<const uint16_t *>(blk + phase);  // phase is even
    if (unit < nunits) {
        const uint32_t start = phase + hdr + (unit ? (uint32_t)cum[unit - 1] : 0u);
        unit_decode<IS_K>(blk, start, unit, t, g, tile, hid_blk);
    }
}

// ---- first generation of a large launch, out of phase -----------------------------------------------------------
// The workgroups that are resident first all start within a few microseconds of each other and go through their
// phases together: the memory system sees every parameter pass at once, the vector ALUs every pack phase at once,
// and the whole generation reaches its look-back together and retires in a convoy -- a pattern that repeats, damped,
// for two or three generations (measured per workgroup: three quarters of the resident workgroups waiting in the
// look-back at the same time).  So the workgroups that fill the second, third, ... residency slot of the CUs wait
// kStaggerTicks each per slot before they take their ticket; tickets are handed out in the order of arrival, so the
// stream order follows the new start order and the generations after the first inherit the spread.  Worth 4 % on the
// K and 6 % on the V encoder for 1 GiB of input; launches of fewer than four generations start as they are.
constexpr uint32_t kStaggerTicks = 400;                    // of the 100 MHz wall clock: 4 us per residency slot
struct Stagger {
    uint32_t cus;       // workgroups that make up one residency slot over the whole device (0: no stagger)
    uint32_t slots;     // resident workgroups per CU
};
__device__ __forceinline__ void stagger_first_generation(const Stagger sg) {
    if (sg.cus != 0u && blockIdx.x < sg.cus * sg.slots) {
        const uint64_t wait = (uint64_t)(blockIdx.x / sg.cus) * kStaggerTicks;
        const uint64_t t0 = wall_clock64();
        while (wall_clock64() - t0 < wait) __builtin_amdgcn_s_sleep(32);
    }
}
// ---- single-pass global offsets: decoupled look-back over block order -------------------
// status word: bits 63..62 = flag (0 empty, 1 aggregate, 2 inclusive), bits 61..0 = bytes.
constexpr uint64_t kFlagAgg = 1ull << 62;
constexpr uint64_t kFlagIncl = 2ull << 62;
constexpr uint64_t kValueMask = (1ull << 62) - 1ull;
constexpr int kSpinLimit = 1 << 18;          // polls before a wait gives up with PKV_ERR_INTERNAL: well under a second at the look-back's back-off

struct ScanState {
    uint32_t ticket;      // next block index to hand out
    uint32_t error;       // non-zero: PKV_ERR_* raised on the device
    uint64_t total;       // stream bytes (written by the last block)
    uint32_t max_code;    // largest code seen by a fused quantize+encode launch
    uint32_t pad_;
    uint64_t status[1];   // one per block
};

// Called by every lane of the FIRST wavefront of the workgroup that owns block `idx`.
// Returns the byte offset of the block in the stream.
// Back-off between two polls of a status word that is still empty, in units of 64 cycles.  Hundreds of workgroups
// poll at the end of their work; with a short back-off their atomic loads slow the memory traffic of the workgroups
// still encoding (K encode of 1 GiB: 0.377 ms at 1, 0.357 ms at 100).
#ifndef PKV_LOOKBACK_SLEEP
#define PKV_LOOKBACK_SLEEP 100
#endif
// One thread may publish the size ahead of the look-back, as soon as it is known (the successors then wait less);
// the look-back is told so and does not store it again.
__device__ __forceinline__ void lookback_publish(ScanState *st, uint32_t idx, uint32_t my_bytes) {
    __hip_atomic_store(&st->status[idx], (idx == 0 ? kFlagIncl : kFlagAgg) | (uint64_t)my_bytes, __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
}

// Sum of a 32-bit value over the 64 lanes (uniform result), on the DPP data path.
__device__ __forceinline__ uint32_t wave_sum_u32(uint32_t v) {
    uint32_t x = v;
    x += __builtin_amdgcn_update_dpp(0u, x, 0x111, 0xF, 0xF, true);
    x += __builtin_amdgcn_update_dpp(0u, x, 0x112, 0xF, 0xF, true);
    x += __builtin_amdgcn_update_dpp(0u, x, 0x114, 0xF, 0xF, true);
    x += __builtin_amdgcn_update_dpp(0u, x, 0x118, 0xF, 0xF, true);
    x += __builtin_amdgcn_update_dpp(0u, x, 0x142, 0xA, 0xF, true);      // row_bcast:15 into rows 1 and 3
    x += __builtin_amdgcn_update_dpp(0u, x, 0x143, 0xC, 0xF, true);      // row_bcast:31 into rows 2 and 3
    return (uint32_t)__builtin_amdgcn_readlane((int)x, 63);
}

// The walk goes back kLookWindows windows of 64 status words per trip.  The nearest window is the one that may still
// be empty (its groups run in step with this one); the older ones are there already and cost one memory round trip
// each, but requesting four windows at once was measured slower (fused K encode of 1 GiB 0.285 -> 0.298 ms, block
// codec 0.213 -> 0.233 ms): every group then reads four times as many status words, and those reads compete with the
// stores that publish them.  A window's aggregates (sizes of single tickets, far below 2^32) are summed in 32 bits
// on the DPP path; the one inclusive prefix that ends the walk is read from its lane.
constexpr int kLookWindows = 1;
__device__ __forceinline__ uint64_t lookback_offset(ScanState *st, uint32_t idx, uint32_t my_bytes, bool published = false) {
    const int lane = threadIdx.x & 63;
    uint64_t *status = st->status;
    if (idx == 0) {
        if (lane == 0 && !published)
            __hip_atomic_store(&status[0], kFlagIncl | (uint64_t)my_bytes, __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
        return 0;
    }
    if (lane == 0 && !published)
        __hip_atomic_store(&status[idx], kFlagAgg | (uint64_t)my_bytes, __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
    uint64_t prefix = 0;
    int64_t base = (int64_t)idx - 1;
    bool failed = false, done = false;
    while (!done && !failed) {
        uint64_t s[kLookWindows];
#pragma unroll
        for (int w = 0; w < kLookWindows; w++) {
            const int64_t j = base - 64 * w - lane;
            s[w] = kFlagIncl;      // the virtual block before block 0: inclusive sum 0
            if (j >= 0) s[w] = __hip_atomic_load(&status[j], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
#pragma unroll
        for (int w = 0; w < kLookWindows; w++) {
            if (done || failed) break;
            const int64_t j = base - 64 * w - lane;
            int spins = 0;
            while ((s[w] >> 62) == 0 && spins < kSpinLimit) {
                __builtin_amdgcn_s_sleep(PKV_LOOKBACK_SLEEP);
                s[w] = __hip_atomic_load(&status[j], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                spins++;
            }
            if (__any((s[w] >> 62) == 0)) { failed = true; break; }
            const uint64_t incl_mask = __ballot((s[w] >> 62) == 2);
            const int first_incl = incl_mask ? (__ffsll((unsigned long long)incl_mask) - 1) : 64;
            prefix += wave_sum_u32(lane < first_incl ? (uint32_t)s[w] : 0u);
            if (incl_mask) {
                const uint64_t v = s[w] & kValueMask;
                const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)v, first_incl);
                const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(v >> 32), first_incl);
                prefix += ((uint64_t)hi << 32) | lo;
                done = true;
            }
        }
        base -= 64 * kLookWindows;
    }
    if (failed) {
        if (lane == 0) atomicExch(&st->error, (uint32_t)PKV_ERR_INTERNAL);
        prefix = 0;
    }
    if (lane == 0)
        __hip_atomic_store(&status[idx], kFlagIncl | (prefix + (uint64_t)my_bytes), __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
    return prefix;
}

// Everything after the code tile is in LDS: encode the block, obtain its stream offset by
// look-back, record block_info and copy the bytes out.  Every thread of the workgroup calls
// it; `s_off` is an LDS uint64, `unit_bytes` an LDS array of 16 uint32.
template <bool IS_K>
__device__ __forceinline__ void block_finish(const uint8_t *tile, uint8_t *blk, uint32_t *unit_bytes,
                                             uint64_t *s_off, ScanState *st, uint32_t b, uint32_t nblocks,
                                             uint8_t *__restrict__ stream, uint64_t capacity,
                                             uint32_t *__restrict__ info, int hid_blk, int nunits, int W) {
    const uint32_t bytes = block_encode<IS_K>(tile, hid_blk, nunits, W, blk, unit_bytes, st, b);
    if (threadIdx.x < 64) {
        const uint64_t off = lookback_offset(st, b, bytes, true);
        if (threadIdx.x == 0) {
            *s_off = off;
            info[2 * b] = (uint32_t)off;
            info[2 * b + 1] = bytes;
            if (b == nblocks - 1) st->total = off + bytes;
            if (off + bytes > capacity) atomicExch(&st->error, (uint32_t)PKV_ERR_CAPACITY);
        }
    }
    __syncthreads();
    const uint64_t off = *s_off;
    if (off + bytes > capacity) return;
    uint16_t *dst = reinterpret_cast<uint16_t *>(stream + off);   // block offsets are even
    const uint16_t *src = reinterpret_cast<const uint16_t *>(blk);
    for (uint32_t i = threadIdx.x; i < (bytes >> 1); i += blockDim.x) dst[i] = src[i];
}

#endif  // __HIPCC__

}  // namespace pkv
