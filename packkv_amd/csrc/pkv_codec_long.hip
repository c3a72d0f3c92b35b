// Block codec for packs LONGER than 16 tokens (32, 64, 128, 256): an extension of the stream format with no
// counterpart in the reference, whose codec fixes PACK_ELE_NUM = 16 (packkv_cuda_ext/include/static_def.h:6) while
// its analytic size model prices any pack length (utils/compute.py:272-297).  These kernels make that model's
// numbers real: stream bytes - 8 per block equal the model's bytes for the same codes, pack length and width.
//
// The format scales the reference's with the pack length P:
//   pack     P consecutive tokens of one channel; min, len = bit_length(max - min) over the P tokens;
//            word = sum_k (code_k - min) << ((P - 1 - k) * len), stored as its low P * len / 8 bytes, little-endian
//            -- i.e. P / 16 sub-words of the reference's shape, the LAST 16 tokens first;
//   K block  4 P tokens x 128 channels: four units (rounds of P tokens); V block 8 P tokens x 64 channels: four
//            units (warp, segment) of 4 slots of P tokens x 32 channels; unit = mins | lens | payload with the
//            metadata bit arrays and the slot-major, lane-minor payload order of the reference's format;
//   header   four u16 cumulative unit sizes, counted in 4-byte words for P >= 32 (every unit size is then a
//            multiple of 4; in bytes a unit of 256-token packs would not fit 16 bits).
// Encoders: K keeps the thread layout of the 16-token codec (half-wavefront per unit, lane <-> 4 channels) times the
// CHUNKS a pack is cut into (P / 16 of them, at most 8: a long pack is a row of independent 16-token sub-words), V
// gives a wavefront to each of a block's eight (segment, slot) token ranges; both read the codes once, keep them in
// registers, build the block in LDS as it will lie in the stream, take its offset from the same ticket + look-back
// as the 16-token codec and copy it out in aligned 16-byte stores.  Decoders stage the stream through LDS and write
// whole 128-byte rows (V: two adjacent blocks per workgroup).  The two *_plain kernels serve V code matrices whose
// rows are no multiple of 128 channels or that do not start at a 16-byte boundary: a workgroup per block, the lane
// layout of the format itself, byte loads and 2-byte stores.
#include "pkv_block.hpp"
#include "pkv_runtime.hpp"

namespace pkv {

// (first token, channel) of pack (unit u, lane t, slot i) relative to the block's first token and channel
template <bool IS_K>
__device__ __forceinline__ void long_pack_at(int u, int t, int i, int P, int &tok0, int &ch) {
    if (IS_K) { tok0 = u * P; ch = 4 * t + i; }
    else { tok0 = ((u & 1) * 4 + i) * P; ch = (u >> 1) * kLanes + t; }
}

// the 2 * len bytes of one 16-token sub-word: codes c[0..15] (min already subtracted)
__device__ __forceinline__ void long_put_sub(uint16_t *dst, const uint32_t c[16], uint32_t len) {
    uint64_t hi = 0, lo = 0;
#pragma unroll
    for (int k = 0; k < 8; k++) {
        hi = (hi << len) | c[k];
        lo = (lo << len) | c[8 + k];
    }
    const unsigned __int128 wd = ((unsigned __int128)hi << (8u * len)) | lo;       // 8 * len bits are len whole bytes
    // one predicated 16-bit store per piece, written out (a loop over the lane's own length costs a 128-bit shift, a
    // compare and the loop's control flow per piece)
    const uint32_t d[4] = {(uint32_t)wd, (uint32_t)(wd >> 32), (uint32_t)(wd >> 64), (uint32_t)(wd >> 96)};
#pragma unroll
    for (uint32_t q = 0; q < 8; q++)
        if (q < len) dst[q] = (uint16_t)(d[q >> 1] >> (16u * (q & 1u)));
}

__device__ __forceinline__ void long_get_sub(const uint16_t *src, uint32_t c[16], uint32_t len) {
    unsigned __int128 wd = 0;
    for (uint32_t q = 0; q < len; q++) wd |= (unsigned __int128)src[q] << (16u * q);
    const uint64_t lo = (uint64_t)(wd & (((unsigned __int128)1 << (8u * len)) - 1));
    const uint64_t hi = (uint64_t)(wd >> (8u * len));
    const uint32_t mask = (1u << len) - 1u;
#pragma unroll
    for (int k = 0; k < 8; k++) {
        c[k] = (uint32_t)(hi >> ((7 - k) * len)) & mask;
        c[8 + k] = (uint32_t)(lo >> ((7 - k) * len)) & mask;
    }
}

// OR lane t's 4 * nbits-bit metadata word into the LSB-first bit array `arr` (dword-aligned LDS, zeroed)
__device__ __forceinline__ void long_put_meta(uint32_t *arr, int t, int nbits, uint32_t w) {
    const uint32_t bit = (uint32_t)t * 4u * (uint32_t)nbits;
    const uint32_t sh = bit & 31u;
    atomicOr(arr + (bit >> 5), w << sh);
    if (sh + 4u * (uint32_t)nbits > 32u) atomicOr(arr + (bit >> 5) + 1, w >> (32u - sh));
}

constexpr int kLongMetaWords = 52;      // 16 * (8 + 4) bytes of metadata at most, and a dword of slack for reads

constexpr int kLongMaxChunks = 8;
__host__ __device__ inline int long_chunks(int P) { return P / 16 < kLongMaxChunks ? P / 16 : kLongMaxChunks; }

__global__ void __launch_bounds__(1024) pack_long_v_plain_kernel(const uint8_t *__restrict__ codes, uint8_t *__restrict__ stream,
                                                        uint64_t capacity, uint32_t *__restrict__ info, ScanState *st,
                                                        int hidden_dim, int P, int W, uint32_t nblocks) {
    __shared__ uint32_t s_idx;
    __shared__ uint64_t s_off;
    __shared__ uint32_t s_unit[4];
    __shared__ uint32_t s_meta[4][kLongMetaWords];
    __shared__ uint4 s_mm[kLongMaxChunks][128];            // minima and maxima of a thread's four packs over its chunk
    const int tid = threadIdx.x, u = (tid >> 5) & 3, t = tid & 31;
    const int chunk = tid >> 7, nch = (int)blockDim.x >> 7;       // this thread's chunk of every pack; chunks per pack
    const uint32_t nsub = (uint32_t)P / 16u;
    const uint32_t s0 = nsub * (uint32_t)chunk / (uint32_t)nch, s1 = nsub * (uint32_t)(chunk + 1) / (uint32_t)nch;   // its sub-words
    const int k0 = P - 16 * (int)s1, k1 = P - 16 * (int)s0;      // ... hold tokens k0 .. k1 - 1 of the pack
    if (tid == 0) s_idx = atomicAdd(&st->ticket, 1u);
    __syncthreads();
    const uint32_t b = s_idx;
    if (b >= nblocks) return;
    const int hid_blk = 64, ctx_blk = 8 * P;
    const int n_hid = hidden_dim / hid_blk;
    const uint32_t cb = b / (uint32_t)n_hid, hb = b % (uint32_t)n_hid;
    const uint8_t *tile = codes + (size_t)cb * ctx_blk * hidden_dim + (size_t)hb * hid_blk;
    const UnitGeom g = unit_geom(W);
    const uint32_t meta = (uint32_t)(g.mins_bytes + g.lens_bytes);

    // ---- minima and widths of the lane's four packs ----
    uint32_t mn[4], len[4];
    {
        uint32_t lohi[4];                                  // minimum | maximum << 16 of each pack over the chunk
#pragma unroll
        for (int i = 0; i < 4; i++) {
            int tok0, ch;
            long_pack_at<false>(u, t, i, P, tok0, ch);
            const uint8_t *col = tile + (size_t)tok0 * hidden_dim + ch;
            uint32_t lo = 255u, hi = 0u;
            for (int k = k0; k < k1; k += 8) {
                uint32_t c[8];
#pragma unroll
                for (int q = 0; q < 8; q++) c[q] = col[(size_t)(k + q) * hidden_dim];
#pragma unroll
                for (int q = 0; q < 8; q++) { lo = min(lo, c[q]); hi = max(hi, c[q]); }
            }
            lohi[i] = lo | (hi << 16);
        }
        s_mm[chunk][tid & 127] = make_uint4(lohi[0], lohi[1], lohi[2], lohi[3]);
        __syncthreads();
#pragma unroll
        for (int i = 0; i < 4; i++) { mn[i] = 255u; len[i] = 0u; }    // (len holds the maximum for the moment)
        for (int c = 0; c < nch; c++) {
            const uint4 o = s_mm[c][tid & 127];
            const uint32_t w[4] = {o.x, o.y, o.z, o.w};
#pragma unroll
            for (int i = 0; i < 4; i++) { mn[i] = min(mn[i], w[i] & 0xFFFFu); len[i] = max(len[i], w[i] >> 16); }
        }
#pragma unroll
        for (int i = 0; i < 4; i++) len[i] = (uint32_t)bit_length_u32(len[i] - mn[i]);
    }
    // byte offsets of the packs inside the unit's payload: those of 16-token packs times P / 16
    uint32_t off[4], payload;
    pack_offsets(len, off, payload);
    payload *= nsub;
    if (t == 0 && chunk == 0) s_unit[u] = meta + payload;
    // metadata bit arrays, assembled in LDS (each half-wavefront of chunk 0 its own area)
    uint32_t *area = s_meta[u];
    if (chunk == 0) {
        area[t] = 0u;
        if (t < kLongMetaWords - 32) area[32 + t] = 0u;
        uint32_t minsw = 0, lensw = 0;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            minsw |= (mn[i] & ((1u << W) - 1u)) << (i * W);
            lensw |= len[i] << (i * g.LB);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        long_put_meta(area, t, W, minsw);
        long_put_meta(area + g.mins_bytes / 4, t, g.LB, lensw);
    }
    __syncthreads();
    const uint32_t bytes = 8u + s_unit[0] + s_unit[1] + s_unit[2] + s_unit[3];
    if (tid == 0) lookback_publish(st, b, bytes);
    if (tid < 64) {
        const uint64_t o = lookback_offset(st, b, bytes, true);
        if (tid == 0) {
            s_off = o;
            info[2 * (size_t)b] = (uint32_t)o;
            info[2 * (size_t)b + 1] = bytes;
            if (b == nblocks - 1) st->total = o + bytes;
            if (o + bytes > capacity) atomicExch(&st->error, (uint32_t)PKV_ERR_CAPACITY);
        }
    }
    __syncthreads();
    const uint64_t o = s_off;
    if (o + bytes > capacity) return;
    uint8_t *dst_blk = stream + o;
    if (tid < 4) {
        uint32_t cum = 0;
        for (int q = 0; q <= tid; q++) cum += s_unit[q];
        reinterpret_cast<uint16_t *>(dst_blk)[tid] = (uint16_t)(P == 16 ? cum : cum >> 2);
    }
    uint32_t ustart = 8u;
    for (int q = 0; q < u; q++) ustart += s_unit[q];
    uint8_t *dst_u = dst_blk + ustart;
    if (chunk == 0)
        for (uint32_t q = (uint32_t)t; q < meta / 2u; q += 32u)
            reinterpret_cast<uint16_t *>(dst_u)[q] = reinterpret_cast<const uint16_t *>(area)[q];
    // ---- the words: sub-word s of a pack holds its tokens P - 16 (s + 1) .. P - 16 s - 1 ----
    uint8_t *pay = dst_u + meta;
    {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            int tok0, ch;
            long_pack_at<false>(u, t, i, P, tok0, ch);
            for (uint32_t s = s0; s < s1; s++) {
                const uint8_t *col = tile + (size_t)(tok0 + P - 16 * (int)(s + 1)) * hidden_dim + ch;
                uint32_t c[16];
#pragma unroll
                for (int k = 0; k < 16; k++) c[k] = (uint32_t)col[(size_t)k * hidden_dim] - mn[i];
                long_put_sub(reinterpret_cast<uint16_t *>(pay + off[i] * nsub + s * 2u * len[i]), c, len[i]);
            }
        }
    }
}

// ---- encoders that keep the codes in registers and build the block in LDS ------------------------------------------
// The kernel above reads a block's codes twice (V: byte by byte, 64 bytes per wavefront load) and writes every
// sub-word to the stream in 2-byte stores.  These two read the codes once with whole-row loads, keep them in
// registers between the pass that finds minima and widths and the pass that forms the words, put the block together
// in LDS byte for byte as it will lie in the stream (bank-swizzled, below), and copy it out in aligned 16-byte stores while the look-back of the
// first wavefront runs beside the second pass.

// The block image in LDS is bank-swizzled: byte a of the block lies at a ^ (((a >> 7) & 31) << 2), i.e. the dword's
// bank is XOR-ed with the number of its 128-byte row.  A lane's pack is a run of 2 len P / 16 bytes, so with 4-bit
// widths and packs of 128 or 256 tokens the lanes' runs start 64 or 128 bytes apart and their 2-byte stores of one
// instruction would all land on one or two banks (123 M conflict cycles per launch at 256 tokens, more than half
// of the kernel's time); rows that differ now take different banks.
__device__ __forceinline__ uint32_t long_swz(uint32_t a) { return a ^ (((a >> 7) & 31u) << 2); }

// the 2 * len bytes of one 16-token sub-word into the swizzled image at byte offset `off` (even)
__device__ __forceinline__ void long_put_sub_swz(uint8_t *image, uint32_t off, const uint32_t c[16], uint32_t len) {
    uint64_t hi = 0, lo = 0;
#pragma unroll
    for (int k = 0; k < 8; k++) {
        hi = (hi << len) | c[k];
        lo = (lo << len) | c[8 + k];
    }
    const unsigned __int128 wd = ((unsigned __int128)hi << (8u * len)) | lo;       // 8 * len bits are len whole bytes
    const uint32_t d[4] = {(uint32_t)wd, (uint32_t)(wd >> 32), (uint32_t)(wd >> 64), (uint32_t)(wd >> 96)};
#pragma unroll
    for (uint32_t q = 0; q < 8; q++)                      // (written out, as in long_put_sub)
        if (q < len) *reinterpret_cast<uint16_t *>(image + long_swz(off + 2u * q)) = (uint16_t)(d[q >> 1] >> (16u * (q & 1u)));
}

// n bytes (even) of the swizzled image -> global memory (dst 2-byte aligned) by the whole workgroup: head to the first
// 16-byte boundary and tail in 2-byte pieces, the body as aligned 16-byte stores fed by dword LDS reads and byte
// funnel shifts (the image is readable 20 bytes past n)
__device__ __forceinline__ void long_copy_out(uint8_t *dst, const uint8_t *image, uint32_t n, int tid, int nthreads) {
    const uint32_t head = min(n, (uint32_t)((16u - (uint32_t)(reinterpret_cast<uintptr_t>(dst) & 15u)) & 15u));
    const uint32_t nq = (n - head) >> 4;
    for (uint32_t i = (uint32_t)tid; i < (head >> 1); i += (uint32_t)nthreads)
        reinterpret_cast<uint16_t *>(dst)[i] = *reinterpret_cast<const uint16_t *>(image + long_swz(2u * i));
    const uint32_t a0 = head & ~3u;
    for (uint32_t i = (uint32_t)tid; i < nq; i += (uint32_t)nthreads) {
        uint32_t d[5];
#pragma unroll
        for (int k = 0; k < 5; k++) d[k] = *reinterpret_cast<const uint32_t *>(image + long_swz(a0 + 16u * i + 4u * (uint32_t)k));
        uint4 v;
        v.x = __builtin_amdgcn_alignbyte(d[1], d[0], head);
        v.y = __builtin_amdgcn_alignbyte(d[2], d[1], head);
        v.z = __builtin_amdgcn_alignbyte(d[3], d[2], head);
        v.w = __builtin_amdgcn_alignbyte(d[4], d[3], head);
        *reinterpret_cast<uint4 *>(dst + head + 16 * (size_t)i) = v;
    }
    const uint32_t done = head + 16u * nq;
    for (uint32_t i = (uint32_t)tid; i < ((n - done) >> 1); i += (uint32_t)nthreads)
        reinterpret_cast<uint16_t *>(dst + done)[i] = *reinterpret_cast<const uint16_t *>(image + long_swz(done + 2u * i));
}

// K: the thread layout of pack_long_kernel (half-wavefront per unit, lane <-> 4 channels, times the chunks of a
// pack); a thread holds the NT = P / chunks tokens of its chunk as one dword (four channels) per token.
template <int NT, int NB>
__global__ void __launch_bounds__(1024) pack_long_k_kernel(const uint8_t *__restrict__ codes, uint8_t *__restrict__ stream,
                                                          uint64_t capacity, uint32_t *__restrict__ info, ScanState *st,
                                                          int hidden_dim, int P, int W, uint32_t ntickets) {
    extern __shared__ __align__(16) uint8_t image[];       // the block as it will lie in the stream (+ 32 bytes of slack)
    __shared__ uint32_t s_idx;
    __shared__ uint64_t s_off;
    __shared__ uint32_t s_unit[NB][4];
    __shared__ uint32_t s_meta[NB][4][kLongMetaWords];
    __shared__ uint4 s_mm[kLongMaxChunks][128];            // minima and maxima of a thread's four packs over its chunk
    // NB consecutive blocks per workgroup and ticket (short packs: a block is small and the tickets, which retire
    // one after the other, would set the pace): block bw is served by threads [bw, bw + 1) * blockDim / NB
    const int tid = threadIdx.x, nthr = (int)blockDim.x / NB, bw = tid / nthr, ltid = tid % nthr;
    const int u = (ltid >> 5) & 3, t = ltid & 31;
    const int chunk = ltid >> 7, nch = nthr >> 7;
    const uint32_t nsub = (uint32_t)P / 16u;
    const uint32_t s1 = nsub * (uint32_t)(chunk + 1) / (uint32_t)nch;     // its sub-words end here; NT / 16 of them
    const int k0 = P - 16 * (int)s1;                                     // ... and hold tokens k0 .. k0 + NT - 1 of the pack
    if (tid == 0) s_idx = atomicAdd(&st->ticket, 1u);
    if (chunk == 0) {
        s_meta[bw][u][t] = 0u;
        if (t < kLongMetaWords - 32) s_meta[bw][u][32 + t] = 0u;
    }
    __syncthreads();
    const uint32_t tk = s_idx;
    if (tk >= ntickets) return;
    const uint32_t b = tk * (uint32_t)NB + (uint32_t)bw;     // (the launcher sees to NB dividing the number of blocks)
    const int n_hid = hidden_dim / 128;
    const uint32_t cb = b / (uint32_t)n_hid, hb = b % (uint32_t)n_hid;
    const uint8_t *tile = codes + (size_t)cb * (4 * P) * hidden_dim + (size_t)hb * 128;
    const UnitGeom g = unit_geom(W);
    const uint32_t meta = (uint32_t)(g.mins_bytes + g.lens_bytes);
    // ---- the codes, minima and widths ----
    uint32_t d[NT];
    const uint8_t *col = tile + (size_t)(u * P + k0) * hidden_dim + 4 * t;
#pragma unroll
    for (int q = 0; q < NT; q++) d[q] = *reinterpret_cast<const uint32_t *>(col + (size_t)q * hidden_dim);
    typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
    u16x2 amn2 = {255, 255}, amx2 = {0, 0}, bmn2 = {255, 255}, bmx2 = {0, 0};   // channels (0, 2) and (1, 3) as 16-bit pairs
#pragma unroll
    for (int q = 0; q < NT; q++) {
        const u16x2 a = __builtin_bit_cast(u16x2, d[q] & 0x00FF00FFu), c = __builtin_bit_cast(u16x2, (d[q] >> 8) & 0x00FF00FFu);
        amn2 = __builtin_elementwise_min(amn2, a);
        amx2 = __builtin_elementwise_max(amx2, a);
        bmn2 = __builtin_elementwise_min(bmn2, c);
        bmx2 = __builtin_elementwise_max(bmx2, c);
    }
    s_mm[bw * nch + chunk][ltid & 127] = make_uint4(__builtin_bit_cast(uint32_t, amn2), __builtin_bit_cast(uint32_t, amx2),
                                        __builtin_bit_cast(uint32_t, bmn2), __builtin_bit_cast(uint32_t, bmx2));
    __syncthreads();
    for (int c = 0; c < nch; c++) {
        const uint4 o = s_mm[bw * nch + c][ltid & 127];
        amn2 = __builtin_elementwise_min(amn2, __builtin_bit_cast(u16x2, o.x));
        amx2 = __builtin_elementwise_max(amx2, __builtin_bit_cast(u16x2, o.y));
        bmn2 = __builtin_elementwise_min(bmn2, __builtin_bit_cast(u16x2, o.z));
        bmx2 = __builtin_elementwise_max(bmx2, __builtin_bit_cast(u16x2, o.w));
    }
    const uint32_t amn = __builtin_bit_cast(uint32_t, amn2), amx = __builtin_bit_cast(uint32_t, amx2),
                   bmn = __builtin_bit_cast(uint32_t, bmn2), bmx = __builtin_bit_cast(uint32_t, bmx2);
    uint32_t mn[4], len[4];
    mn[0] = amn & 0xFFFFu; mn[2] = amn >> 16; mn[1] = bmn & 0xFFFFu; mn[3] = bmn >> 16;
    len[0] = (uint32_t)bit_length_u32((amx & 0xFFFFu) - mn[0]);
    len[2] = (uint32_t)bit_length_u32((amx >> 16) - mn[2]);
    len[1] = (uint32_t)bit_length_u32((bmx & 0xFFFFu) - mn[1]);
    len[3] = (uint32_t)bit_length_u32((bmx >> 16) - mn[3]);
    uint32_t off[4], payload;
    pack_offsets(len, off, payload);
    payload *= nsub;
    if (t == 0 && chunk == 0) s_unit[bw][u] = meta + payload;
    if (chunk == 0) {
        uint32_t minsw = 0, lensw = 0;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            minsw |= (mn[i] & ((1u << W) - 1u)) << (i * W);
            lensw |= len[i] << (i * g.LB);
        }
        long_put_meta(s_meta[bw][u], t, W, minsw);
        long_put_meta(s_meta[bw][u] + g.mins_bytes / 4, t, g.LB, lensw);
    }
    __syncthreads();
    // the blocks lie one behind the other in the image, as in the stream
    uint32_t blk_bytes[NB], bytes = 0, blk0 = 0;
#pragma unroll
    for (int j = 0; j < NB; j++) {
        blk_bytes[j] = 8u + s_unit[j][0] + s_unit[j][1] + s_unit[j][2] + s_unit[j][3];
        if (j < bw) blk0 += blk_bytes[j];
        bytes += blk_bytes[j];
    }
    if (tid == 0) lookback_publish(st, tk, bytes);
    // ---- the block in LDS: header, metadata, words ----
    if (ltid < 4) {
        uint32_t cum = 0;
        for (int q = 0; q <= ltid; q++) cum += s_unit[bw][q];
        *reinterpret_cast<uint16_t *>(image + long_swz(blk0 + 2u * (uint32_t)ltid)) = (uint16_t)(cum >> 2);
    }
    uint32_t ustart = blk0 + 8u;
    for (int q = 0; q < u; q++) ustart += s_unit[bw][q];
    if (chunk == 0)
        for (uint32_t q = (uint32_t)t; q < meta / 4u; q += 32u)
            *reinterpret_cast<uint32_t *>(image + long_swz(ustart + 4u * q)) = s_meta[bw][u][q];
    const uint32_t pay = ustart + meta;                   // byte offset of the unit's payload inside the block
#pragma unroll
    for (int j = 0; j < NT / 16; j++) {
        const uint32_t s = s1 - 1u - (uint32_t)j;           // tokens k0 + 16 j .. + 15 are sub-word s1 - 1 - j
#pragma unroll
        for (int i = 0; i < 4; i++) {
            uint32_t c[16];
#pragma unroll
            for (int k = 0; k < 16; k++) c[k] = ((d[16 * j + k] >> (8 * i)) & 0xFFu) - mn[i];
            long_put_sub_swz(image, pay + off[i] * nsub + s * 2u * len[i], c, len[i]);
        }
    }
    if (tid < 64) {
        const uint64_t o = lookback_offset(st, tk, bytes, true);
        if (tid == 0) {
            s_off = o;
            uint32_t run = 0;
#pragma unroll
            for (int j = 0; j < NB; j++) {
                info[2 * (size_t)(tk * NB + j)] = (uint32_t)(o + run);
                info[2 * (size_t)(tk * NB + j) + 1] = blk_bytes[j];
                run += blk_bytes[j];
            }
            if (tk == ntickets - 1) st->total = o + bytes;
            if (o + bytes > capacity) atomicExch(&st->error, (uint32_t)PKV_ERR_CAPACITY);
        }
    }
    __syncthreads();
    const uint64_t o = s_off;
    if (o + bytes > capacity) return;
    long_copy_out(stream + o, image, bytes, tid, (int)blockDim.x);
}

// V: a workgroup of eight wavefronts per block, wavefront r <-> the P tokens of slot r % 4 of segment r / 4, lane <->
// channel (the lower half-wavefront belongs to the unit of channels 0..31, the upper to that of channels 32..63).  A
// 16-token x 64-channel tile is one 16-byte load per lane (four lanes per 64-byte row piece) and goes through LDS
// to turn rows into the lane's column; the lane keeps its P codes four to a register.
template <int P, int NB>
__global__ void __launch_bounds__(512 * NB) pack_long_v_kernel(const uint8_t *__restrict__ codes, uint8_t *__restrict__ stream,
                                                              uint64_t capacity, uint32_t *__restrict__ info, ScanState *st,
                                                              int hidden_dim, int W, uint32_t ntickets) {
    // NB = 2: two adjacent blocks (consecutive in the stream as well) per workgroup and ticket, eight wavefronts each --
    // together their rows are whole 128-byte lines, and the tickets, which retire one after the other, are half as many
    constexpr int NSUB = P / 16;
    constexpr int kRow = 80;                               // tile rows padded: 16-byte aligned, spread over the banks
    extern __shared__ __align__(16) uint8_t image[];
    __shared__ uint32_t s_idx;
    __shared__ uint64_t s_off;
    __shared__ uint32_t s_unit[NB][4];
    __shared__ uint32_t s_meta[NB][4][kLongMetaWords];
    __shared__ uint8_t s_len[NB][8][64];
    __shared__ __align__(16) uint8_t s_tile[NB * 8][16 * kRow];
    const int tid = threadIdx.x, bw = tid >> 9, r = (tid >> 6) & 7, c = tid & 63;
    const int seg = r >> 2, slot = r & 3, u = (c >> 5) * 2 + seg, t = c & 31;
    if (tid == 0) s_idx = atomicAdd(&st->ticket, 1u);
    if (tid < NB * 4 * kLongMetaWords) (&s_meta[0][0][0])[tid] = 0u;
    __syncthreads();
    const uint32_t tk = s_idx;
    if (tk >= ntickets) return;
    const uint32_t b = tk * (uint32_t)NB + (uint32_t)bw;   // (the launcher pairs blocks only when every row of blocks is even)
    const int n_hid = hidden_dim / 64;
    const uint32_t cb = b / (uint32_t)n_hid, hb = b % (uint32_t)n_hid;
    const UnitGeom g = unit_geom(W);
    const uint32_t meta = (uint32_t)(g.mins_bytes + g.lens_bytes);
    // ---- the codes, minimum and width of the lane's pack ----
    const uint8_t *rows = codes + ((size_t)cb * (8 * P) + (size_t)r * P + (size_t)(c >> 2)) * hidden_dim + (size_t)hb * 64 + 16 * (c & 3);
    uint8_t *mine = s_tile[bw * 8 + r];
    uint32_t pk[P / 4];
    uint32_t lo = 255u, hi = 0u;
    // two tiles are requested ahead of the one being turned (named registers: an array here ends up in scratch memory)
    uint4 t0 = *reinterpret_cast<const uint4 *>(rows);
    uint4 t1 = *reinterpret_cast<const uint4 *>(rows + (size_t)16 * hidden_dim);          // (NSUB >= 2)
#pragma unroll
    for (int j = 0; j < NSUB; j++) {
        uint4 t2 = t1;
        if (j + 2 < NSUB) t2 = *reinterpret_cast<const uint4 *>(rows + (size_t)(16 * (j + 2)) * hidden_dim);
        *reinterpret_cast<uint4 *>(mine + (c >> 2) * kRow + 16 * (c & 3)) = t0;
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        uint32_t e[16];
#pragma unroll
        for (int k = 0; k < 16; k++) e[k] = mine[k * kRow + c];
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int k = 0; k < 16; k++) { lo = min(lo, e[k]); hi = max(hi, e[k]); }
#pragma unroll
        for (int q = 0; q < 4; q++) {
            pk[4 * j + q] = e[4 * q] | (e[4 * q + 1] << 8) | (e[4 * q + 2] << 16) | (e[4 * q + 3] << 24);
            asm volatile("" : "+v"(pk[4 * j + q]));          // (kept packed: the compiler would carry the bytes apart)
        }
        t0 = t1;
        t1 = t2;
    }
    const uint32_t mn = lo, len = (uint32_t)bit_length_u32(hi - lo);
    s_len[bw][r][c] = (uint8_t)len;
    __syncthreads();
    uint32_t len4[4], off4[4], payload;
#pragma unroll
    for (int i = 0; i < 4; i++) len4[i] = s_len[bw][seg * 4 + i][c];
    pack_offsets(len4, off4, payload);
    payload *= (uint32_t)NSUB;
    if (slot == 0 && t == 0) s_unit[bw][u] = meta + payload;
    long_put_meta(s_meta[bw][u], t, W, (mn & ((1u << W) - 1u)) << (slot * W));
    long_put_meta(s_meta[bw][u] + g.mins_bytes / 4, t, g.LB, len << (slot * g.LB));
    __syncthreads();
    // the blocks lie one behind the other in the image, as in the stream
    uint32_t blk_bytes[NB], bytes = 0, blk0 = 0;
#pragma unroll
    for (int j = 0; j < NB; j++) {
        blk_bytes[j] = 8u + s_unit[j][0] + s_unit[j][1] + s_unit[j][2] + s_unit[j][3];
        if (j < bw) blk0 += blk_bytes[j];
        bytes += blk_bytes[j];
    }
    if (tid == 0) lookback_publish(st, tk, bytes);
    // ---- the blocks in LDS: header, metadata, words ----
    if (r == 0 && c < 4) {
        uint32_t cum = 0;
        for (int q = 0; q <= c; q++) cum += s_unit[bw][q];
        *reinterpret_cast<uint16_t *>(image + long_swz(blk0 + 2u * (uint32_t)c)) = (uint16_t)(cum >> 2);
    }
    uint32_t ustart = blk0 + 8u;
    for (int q = 0; q < u; q++) ustart += s_unit[bw][q];
    if (slot == 0)
        for (uint32_t q = (uint32_t)t; q < meta / 4u; q += 32u)
            *reinterpret_cast<uint32_t *>(image + long_swz(ustart + 4u * q)) = s_meta[bw][u][q];
    const uint32_t my_off = slot == 0 ? off4[0] : slot == 1 ? off4[1] : slot == 2 ? off4[2] : off4[3];
    const uint32_t pay = ustart + meta + my_off * (uint32_t)NSUB;      // byte offset of the lane's pack inside the image
    const uint32_t mn4 = mn * 0x01010101u;
#pragma unroll
    for (int j = 0; j < NSUB; j++) {
        uint32_t e[16];
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const uint32_t w = pk[4 * j + q] - mn4;         // no byte borrows: every code is at least the minimum
            e[4 * q] = w & 0xFFu; e[4 * q + 1] = (w >> 8) & 0xFFu; e[4 * q + 2] = (w >> 16) & 0xFFu; e[4 * q + 3] = w >> 24;
        }
        long_put_sub_swz(image, pay + (uint32_t)(NSUB - 1 - j) * 2u * len, e, len);     // tokens 16 j .. are sub-word NSUB - 1 - j
    }
    if (tid < 64) {
        const uint64_t o = lookback_offset(st, tk, bytes, true);
        if (tid == 0) {
            s_off = o;
            uint32_t run = 0;
#pragma unroll
            for (int j = 0; j < NB; j++) {
                info[2 * (size_t)(tk * NB + j)] = (uint32_t)(o + run);
                info[2 * (size_t)(tk * NB + j) + 1] = blk_bytes[j];
                run += blk_bytes[j];
            }
            if (tk == ntickets - 1) st->total = o + bytes;
            if (o + bytes > capacity) atomicExch(&st->error, (uint32_t)PKV_ERR_CAPACITY);
        }
    }
    __syncthreads();
    const uint64_t o = s_off;
    if (o + bytes > capacity) return;
    long_copy_out(stream + o, image, bytes, tid, 512 * NB);
}

__global__ void __launch_bounds__(1024) unpack_long_v_plain_kernel(const uint8_t *__restrict__ stream, const uint32_t *__restrict__ info,
                                                          uint8_t *__restrict__ codes, int hidden_dim, int P, int W,
                                                          uint64_t stream_bytes) {
    __shared__ uint32_t s_meta[4][kLongMetaWords];
    const int tid = threadIdx.x, u = (tid >> 5) & 3, t = tid & 31;
    const int chunk = tid >> 7, nch = (int)blockDim.x >> 7;       // as in the encoder
    const uint32_t b = blockIdx.x;
    const int hid_blk = 64, ctx_blk = 8 * P;
    const int n_hid = hidden_dim / hid_blk;
    const uint32_t cb = b / (uint32_t)n_hid, hb = b % (uint32_t)n_hid;
    uint8_t *tile = codes + (size_t)cb * ctx_blk * hidden_dim + (size_t)hb * hid_blk;
    const UnitGeom g = unit_geom(W);
    const uint32_t meta = (uint32_t)(g.mins_bytes + g.lens_bytes);
    const uint64_t boff = info[2 * (size_t)b];
    const uint32_t bsize = info[2 * (size_t)b + 1];
    // a block_info row that points outside the stream decodes nothing (the codes of the block stay as they are)
    if (boff + bsize > stream_bytes || bsize < 8u + 4u * meta) return;
    const uint16_t *hdr = reinterpret_cast<const uint16_t *>(stream + boff);
    const uint32_t gran = P == 16 ? 1u : 4u;
    const uint32_t ustart = 8u + (u ? (uint32_t)hdr[u - 1] * gran : 0u);
    const uint32_t uend = 8u + (uint32_t)hdr[u] * gran;
    const bool sane = ustart + meta <= uend && uend <= bsize;      // uniform per half-wavefront
    uint32_t *area = s_meta[u];
    const uint8_t *src_u = stream + boff + ustart;
    if (sane && chunk == 0)
        for (uint32_t q = (uint32_t)t; q < meta / 2u; q += 32u)
            reinterpret_cast<uint16_t *>(area)[q] = reinterpret_cast<const uint16_t *>(src_u)[q];
    __syncthreads();
    if (!sane) return;
    const uint32_t minsw = lds_meta_word(reinterpret_cast<const uint8_t *>(area), t, W);
    const uint32_t lensw = lds_meta_word(reinterpret_cast<const uint8_t *>(area) + g.mins_bytes, t, g.LB);
    uint32_t mn[4], len[4], off[4], payload;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        mn[i] = (minsw >> (i * W)) & ((1u << W) - 1u);
        len[i] = min((lensw >> (i * g.LB)) & ((1u << g.LB) - 1u), (uint32_t)kMaxBits);
    }
    pack_offsets(len, off, payload);
    const uint32_t nsub = (uint32_t)P / 16u;
    if (ustart + meta + payload * nsub > uend) return;             // (uniform) widths that overrun the unit
    const uint32_t s0 = nsub * (uint32_t)chunk / (uint32_t)nch, s1 = nsub * (uint32_t)(chunk + 1) / (uint32_t)nch;
    const uint8_t *pay = src_u + meta;
    {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            int tok0, ch;
            long_pack_at<false>(u, t, i, P, tok0, ch);
            for (uint32_t s = s0; s < s1; s++) {
                uint32_t c[16];
                long_get_sub(reinterpret_cast<const uint16_t *>(pay + off[i] * nsub + s * 2u * len[i]), c, len[i]);
                uint8_t *col = tile + (size_t)(tok0 + P - 16 * (int)(s + 1)) * hidden_dim + ch;
#pragma unroll
                for (int k = 0; k < 16; k++) col[(size_t)k * hidden_dim] = (uint8_t)(c[k] + mn[i]);
            }
        }
    }
}

// ---- decoders that stage the stream through LDS ----------------------------------------------------------------
// A pack of P tokens is P / 16 sub-words of the 16-token shape, so sub-word s of all packs of a unit is a 16-token
// unit whose words sit at payload + off[i] * nsub + s * 2 len[i] instead of payload + off[i]: decoded with the
// windows of the 16-token codec (sub_codes), 16 tokens x 4 slots per lane at a time.  What differs from the kernel
// above is where the bytes come from and go to: the unit (K) or one slot of four units (V) is copied into LDS in
// aligned 16-byte pieces first -- a lane's pack is a contiguous run of up to 256 bytes in the stream, so lanes that
// fetch their own words touch a cache line each per load -- and V, whose units are 32 channels wide, goes through
// an LDS tile of 128 channels (two adjacent blocks) so that whole 128-byte lines are written.

// codes of sub-word `word_off` (LDS byte offsets, even) of the lane's four packs: c4[k] = the four slots' codes of
// token k, one per byte.  W <= 4: words of at most 8 bytes, 16-bit windows of four tokens; else field by field.
__device__ __forceinline__ void sub_codes(const uint8_t *lds, const uint32_t word_off[4], const uint32_t len[4], const uint32_t mn[4],
                                          bool wide, uint32_t c4[16]) {
    typedef unsigned short u16pair __attribute__((ext_vector_type(2)));
    if (!wide) {
        uint32_t hlf[4][2];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint64_t w = lds_load64(lds, word_off[i]);
            hlf[i][0] = (uint32_t)(w >> (8u * len[i]));   // tokens 0..7
            hlf[i][1] = (uint32_t)w;                      // tokens 8..15
        }
        const uint32_t len01 = len[0] | (len[1] << 16), len23 = len[2] | (len[3] << 16);
        const uint32_t mq = ((1u << len[0]) - 1u) | (((1u << len[1]) - 1u) << 8) | (((1u << len[2]) - 1u) << 16) |
                            (((1u << len[3]) - 1u) << 24);
        const uint32_t minq = mn[0] | (mn[1] << 8) | (mn[2] << 16) | (mn[3] << 24);
#pragma unroll
        for (int q = 0; q < 4; q++) {
            uint32_t qd[4];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const uint32_t src = hlf[i][q >> 1];
                qd[i] = (q & 1) ? src : (src >> (4u * len[i]));
            }
            const uint32_t w01 = __builtin_amdgcn_perm(qd[1], qd[0], 0x05040100u);   // tokens 4q..4q+3 of packs 0 | 1
            const uint32_t w23 = __builtin_amdgcn_perm(qd[3], qd[2], 0x05040100u);
#pragma unroll
            for (int pp = 0; pp < 4; pp++) {
                const u16pair s01 = __builtin_bit_cast(u16pair, len01 * (uint32_t)(3 - pp));
                const u16pair s23 = __builtin_bit_cast(u16pair, len23 * (uint32_t)(3 - pp));
                const uint32_t x01 = __builtin_bit_cast(uint32_t, (u16pair)(__builtin_bit_cast(u16pair, w01) >> s01));
                const uint32_t x23 = __builtin_bit_cast(uint32_t, (u16pair)(__builtin_bit_cast(u16pair, w23) >> s23));
                c4[4 * q + pp] = (__builtin_amdgcn_perm(x23, x01, 0x06040200u) & mq) + minq;
            }
        }
    } else {
#pragma unroll
        for (int k = 0; k < 16; k++) c4[k] = 0u;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint64_t lo = lds_load64(lds, word_off[i]), hi = lds_load64(lds, word_off[i] + 8u);
            uint32_t d0 = (uint32_t)lo, d1 = (uint32_t)(lo >> 32), d2 = (uint32_t)hi, d3 = (uint32_t)(hi >> 32);
            const uint32_t mask = (1u << len[i]) - 1u, sh = len[i];
#pragma unroll
            for (int k = 15; k >= 0; k--) {
                c4[k] |= (((d0 & mask) + mn[i]) & 0xFFu) << (8 * i);
                d0 = __builtin_amdgcn_alignbit(d1, d0, sh);
                d1 = __builtin_amdgcn_alignbit(d2, d1, sh);
                d2 = __builtin_amdgcn_alignbit(d3, d2, sh);
                d3 >>= sh;
            }
        }
    }
}

// codes of one 16-token sub-word of a single pack (V works slot by slot: a lane's four packs are four token groups)
__device__ __forceinline__ void sub_codes1(const uint8_t *lds, uint32_t word_off, uint32_t len, uint32_t mn, bool wide, uint32_t c[16]) {
    const uint32_t mask = (1u << len) - 1u;
    if (!wide) {
        const uint64_t w = lds_load64(lds, word_off);
#pragma unroll
        for (int k = 0; k < 16; k++) c[k] = ((uint32_t)(w >> ((15 - k) * len)) & mask) + mn;
    } else {
        const uint64_t lo = lds_load64(lds, word_off), hi = lds_load64(lds, word_off + 8u);
        uint32_t d0 = (uint32_t)lo, d1 = (uint32_t)(lo >> 32), d2 = (uint32_t)hi, d3 = (uint32_t)(hi >> 32);
#pragma unroll
        for (int k = 15; k >= 0; k--) {
            c[k] = (d0 & mask) + mn;
            d0 = __builtin_amdgcn_alignbit(d1, d0, len);
            d1 = __builtin_amdgcn_alignbit(d2, d1, len);
            d2 = __builtin_amdgcn_alignbit(d3, d2, len);
            d3 >>= len;
        }
    }
}

// Where unit u of block b lies in the stream, made safe: false when block_info or the header cannot be right
// (the codes of the unit then stay as they are).  ustart / ubytes: offset inside the block and size of the unit.
__device__ __forceinline__ bool long_unit_span(const uint8_t *stream, uint64_t stream_bytes, const uint32_t *info, uint32_t b, int u,
                                               int P, uint32_t meta, uint64_t &boff, uint32_t &ustart, uint32_t &ubytes) {
    boff = info[2 * (size_t)b];
    const uint32_t bsize = info[2 * (size_t)b + 1];
    if (boff + bsize > stream_bytes || bsize < 8u + 4u * meta) return false;
    const uint16_t *hdr = reinterpret_cast<const uint16_t *>(stream + boff);
    const uint32_t gran = P == 16 ? 1u : 4u;
    ustart = 8u + (u ? (uint32_t)hdr[u - 1] * gran : 0u);
    const uint32_t uend = 8u + (uint32_t)hdr[u] * gran;
    if (!(ustart + meta <= uend && uend <= bsize)) return false;
    ubytes = uend - ustart;
    return true;
}

// K: one workgroup per unit (P tokens x 128 channels); half-wavefront h decodes sub-words h, h + nhw, ... and
// writes their 16 rows of 128 bytes.  Dynamic LDS: the unit's bytes + 48.
__global__ void __launch_bounds__(256) unpack_long_k_kernel(const uint8_t *__restrict__ stream, const uint32_t *__restrict__ info,
                                                           uint8_t *__restrict__ codes, int hidden_dim, int P, int W,
                                                           uint64_t stream_bytes, uint32_t unit_cap) {
    extern __shared__ __align__(16) uint8_t lds[];
    const int tid = threadIdx.x, hw = tid >> 5, nhw = (int)blockDim.x >> 5, t = tid & 31;
    const uint32_t b = blockIdx.x >> 2;
    const int u = (int)(blockIdx.x & 3u);
    const int n_hid = hidden_dim / 128;
    const uint32_t cb = b / (uint32_t)n_hid, hb = b % (uint32_t)n_hid;
    const UnitGeom g = unit_geom(W);
    const uint32_t meta = (uint32_t)(g.mins_bytes + g.lens_bytes);
    uint64_t boff;
    uint32_t ustart, ubytes;
    if (!long_unit_span(stream, stream_bytes, info, b, u, P, meta, boff, ustart, ubytes)) return;      // uniform
    ubytes = min(ubytes, unit_cap);
    const uint32_t phase = stage_to_lds(stream + boff + ustart, ubytes, lds, tid, (int)blockDim.x);
    __syncthreads();
    const uint32_t minsw = lds_meta_word(lds + phase, t, W);
    const uint32_t lensw = lds_meta_word(lds + phase + g.mins_bytes, t, g.LB);
    uint32_t mn[4], len[4], off[4], payload;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        mn[i] = (minsw >> (i * W)) & ((1u << W) - 1u);
        len[i] = min((lensw >> (i * g.LB)) & ((1u << g.LB) - 1u), (uint32_t)kMaxBits);
    }
    pack_offsets(len, off, payload);
    const uint32_t nsub = (uint32_t)P / 16u;
    if (meta + payload * nsub > ubytes) return;                    // (uniform) widths that overrun the unit
    const uint32_t pay = phase + meta;
    uint8_t *tile = codes + (size_t)cb * (4 * P) * hidden_dim + (size_t)hb * 128 + (size_t)(u * P) * hidden_dim + 4 * t;
    for (uint32_t s = (uint32_t)hw; s < nsub; s += (uint32_t)nhw) {
        uint32_t wo[4], c4[16];
#pragma unroll
        for (int i = 0; i < 4; i++) wo[i] = pay + off[i] * nsub + s * 2u * len[i];
        sub_codes(lds, wo, len, mn, W > 4, c4);
        uint8_t *row = tile + (size_t)(P - 16 * (int)(s + 1)) * hidden_dim;
#pragma unroll
        for (int k = 0; k < 16; k++) *reinterpret_cast<uint32_t *>(row + (size_t)k * hidden_dim) = c4[k];
    }
}

// V: one workgroup of 256 threads per (pair of adjacent blocks, token half `seg`): half-wavefront h serves unit
// q = h % 4 of the pair (block q / 2, channel half q % 2).  The bytes of `sps` slots of the four units (the whole
// unit with its metadata when all four slots fit the staging area, one or two slots at a time for the longest packs,
// the next stage requested into registers while the current one is decoded) go to LDS.  A unit's work is cut into
// items (slot, sub-word) of 16 tokens x 32 channels; a lane decodes FOUR ADJACENT CHANNELS of one item -- it reads
// their (offset, width, minimum) from a table the unit's lanes fill after the offset scan -- so the codes come out
// as the 16-token codec's K side produces them, a dword of four channels per token, and go into the tile as dwords.
// A step is eight items per unit (the two half-wavefronts of a unit take four each): eight tiles of 16 tokens x 128
// channels that are written out as whole lines.  Dynamic LDS: 4 staging regions, 8 tiles, the table, metadata.
constexpr int kLongVTile = 16 * 128 + 32;                  // tile pitch: 32 bytes of padding keep the four items of a half-wavefront on different banks
__global__ void __launch_bounds__(256) unpack_long_v_kernel(const uint8_t *__restrict__ stream, const uint32_t *__restrict__ info,
                                                           uint8_t *__restrict__ codes, int hidden_dim, int P, int W,
                                                           uint64_t stream_bytes, uint32_t stage_cap, int sps) {
    extern __shared__ __align__(16) uint8_t lds[];
    const int tid = threadIdx.x, hw = tid >> 5, t = tid & 31;
    const int q = hw & 3, sp = hw >> 2;                    // unit of the pair, half of a step's items
    const int seg = (int)(blockIdx.x & 1u);
    const uint32_t pair = blockIdx.x >> 1;
    const int n_pair = hidden_dim / 128;
    const uint32_t cb = pair / (uint32_t)n_pair, hp = pair % (uint32_t)n_pair;
    const uint32_t b = cb * (uint32_t)(2 * n_pair) + 2u * hp + (uint32_t)(q >> 1);
    const int u = 2 * (q & 1) + seg;                       // unit of block b: channel half q % 2, token half seg
    const UnitGeom g = unit_geom(W);
    const uint32_t meta = (uint32_t)(g.mins_bytes + g.lens_bytes);
    const uint32_t meta16 = (meta + 15u) & ~15u;
    const uint32_t region = stage_cap + meta16 + 48u;      // LDS bytes of one unit's staged slots (with its metadata when the unit is staged whole)
    uint8_t *tiles = lds + 4 * region;                     // [8 items][16 tokens][128 channels], padded
    uint32_t *table = reinterpret_cast<uint32_t *>(tiles + 8 * kLongVTile);     // [4 units][4 slots][32 channels]: offset | width << 16 | minimum << 24
    uint8_t *metas = reinterpret_cast<uint8_t *>(table + 4 * 4 * 32);          // [4 units][meta rounded up to 16 + 32]
    const uint32_t meta_stride = meta16 + 32u;
    uint64_t boff = 0;
    uint32_t ustart = 0, ubytes = 0;
    bool ok = long_unit_span(stream, stream_bytes, info, b, u, P, meta, boff, ustart, ubytes);          // uniform per half-wavefront
    uint8_t *reg = lds + q * region;
    const int l64 = t + 32 * sp;
    // all four slots fit the staging area: the unit goes to LDS in one piece, metadata and words (one trip to memory
    // instead of two); else the metadata first (the two half-wavefronts of a unit share the copies)
    const bool whole = sps == 4;
    uint32_t mphase = 0;
    if (ok) mphase = whole ? stage_to_lds(stream + boff + ustart, min(ubytes, meta + stage_cap), reg, l64, 64)
                           : stage_to_lds(stream + boff + ustart, meta, metas + q * meta_stride, l64, 64);
    __syncthreads();
    const uint32_t nsub = (uint32_t)P / 16u;
    uint32_t base0, base1, base2, base3, base4;       // (scalars, not an array: indexed by the stage below it would live in scratch memory)
    {
        uint32_t mn[4], len[4], off[4], payload = 0;
        const uint8_t *m = (whole ? reg : metas + q * meta_stride) + mphase;
        const uint32_t minsw = ok ? lds_meta_word(m, t, W) : 0u;
        const uint32_t lensw = ok ? lds_meta_word(m + g.mins_bytes, t, g.LB) : 0u;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            mn[i] = (minsw >> (i * W)) & ((1u << W) - 1u);
            len[i] = min((lensw >> (i * g.LB)) & ((1u << g.LB) - 1u), (uint32_t)kMaxBits);
        }
        pack_offsets(len, off, payload);                   // (whole wavefronts: every lane takes part)
        ok = ok && meta + payload * nsub <= ubytes;        // widths that overrun the unit
        if (sp == 0)
#pragma unroll
            for (int i = 0; i < 4; i++) table[(q * 4 + i) * 32 + t] = off[i] | (len[i] << 16) | (mn[i] << 24);
        // slot i of this unit: bytes [base[i], base[i + 1]) * nsub of the payload; the slot bases are the offsets of the
        // half-wavefront's first lane (swizzle within 32 lanes: every lane reads lane 0 of its half)
        base0 = (uint32_t)__builtin_amdgcn_ds_swizzle((int)off[0], 0);
        base1 = (uint32_t)__builtin_amdgcn_ds_swizzle((int)off[1], 0);
        base2 = (uint32_t)__builtin_amdgcn_ds_swizzle((int)off[2], 0);
        base3 = (uint32_t)__builtin_amdgcn_ds_swizzle((int)off[3], 0);
        base4 = payload;
    }
    uint8_t *out = codes + (size_t)cb * (8 * P) * hidden_dim + (size_t)hp * 128;
    uint32_t sphase = mphase + meta, b_stage = 0;          // phase of the staged words, payload offset (/ nsub) they start at
    // Longer packs are staged `sps` slots at a time.  The 16-byte pieces of the next stage are requested into
    // registers before the current one is decoded (up to kPre per thread: 64 threads x 5 x 16 bytes cover 4 KiB and
    // the phase), so that the trip to memory runs under the decode; larger stages are fetched when they are needed.
    constexpr int kPre = 5;
    const bool pre = !whole && stage_cap + 16u <= 64u * kPre * 16u;
    uint4 pv[kPre];
    uint32_t ld_phase = 0, ld_n16 = 0, ld_b = 0;
    auto slot_base = [&](int i) { return i == 0 ? base0 : i == 1 ? base1 : i == 2 ? base2 : i == 3 ? base3 : base4; };
    auto pre_load = [&](int i) {
        const uint32_t b_lo = slot_base(i), b_hi = slot_base(i + sps);
        const uint32_t sbytes = min((b_hi - b_lo) * nsub, stage_cap);
        const uint8_t *src = stream + boff + ustart + meta + b_lo * nsub;
        ld_phase = (uint32_t)(reinterpret_cast<uintptr_t>(src) & 15u);
        ld_n16 = ok ? (ld_phase + sbytes + 15u) >> 4 : 0u;
        ld_b = b_lo;
        const uint4 *s16 = reinterpret_cast<const uint4 *>(src - ld_phase);
#pragma unroll
        for (int v = 0; v < kPre; v++) {
            const uint32_t idx = (uint32_t)l64 + 64u * (uint32_t)v;
            pv[v] = idx < ld_n16 ? s16[idx] : make_uint4(0u, 0u, 0u, 0u);
        }
    };
    if (pre) pre_load(0);
    const int m4 = t & 7, sel = t >> 3;                    // the lane's four channels 4 m4 .. 4 m4 + 3 and which of the half-wavefront's four items
    const uint32_t steps_per_stage = nsub * (uint32_t)sps / 8u;      // (the launcher sees to nsub * sps >= 8)
#pragma unroll 1
    for (int i0 = 0; i0 < 4; i0 += sps) {                  // a stage: slots i0 .. i0 + sps - 1
        if (!whole) {
            __syncthreads();                               // the bytes staged before are no longer read
            if (pre) {
#pragma unroll
                for (int v = 0; v < kPre; v++) {
                    const uint32_t idx = (uint32_t)l64 + 64u * (uint32_t)v;
                    if (idx < ld_n16) reinterpret_cast<uint4 *>(reg)[idx] = pv[v];
                }
                sphase = ld_phase;
                b_stage = ld_b;
            } else {
                const uint32_t b_lo = slot_base(i0), b_hi = slot_base(i0 + sps);
                const uint32_t sbytes = min((b_hi - b_lo) * nsub, stage_cap);
                if (ok) sphase = stage_to_lds(stream + boff + ustart + meta + b_lo * nsub, sbytes, reg, l64, 64);
                b_stage = b_lo;
            }
        }
        __syncthreads();                                   // the stage and the table are there
        if (pre && i0 + sps < 4) pre_load(i0 + sps);
#pragma unroll 1
        for (uint32_t j = 0; j < steps_per_stage; j++) {
            const uint32_t item0 = (uint32_t)i0 * nsub + 8u * j;            // the step's first item: slot item / nsub, sub-word item % nsub
            if (ok) {
                const uint32_t item = item0 + 4u * (uint32_t)sp + (uint32_t)sel;
                const uint32_t i = item / nsub, s = item % nsub;
                const uint4 tb = *reinterpret_cast<const uint4 *>(table + (q * 4 + (int)i) * 32 + 4 * m4);
                const uint32_t e4[4] = {tb.x, tb.y, tb.z, tb.w};
                uint32_t wo[4], len[4], mn[4], c4[16];
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    len[c] = (e4[c] >> 16) & 0xFFu;
                    mn[c] = e4[c] >> 24;
                    wo[c] = sphase + ((e4[c] & 0xFFFFu) - b_stage) * nsub + s * 2u * len[c];
                }
                sub_codes(reg, wo, len, mn, W > 4, c4);
                uint8_t *tile = tiles + (4 * sp + sel) * kLongVTile + 32 * q + 4 * m4;
#pragma unroll
                for (int k = 0; k < 16; k++) *reinterpret_cast<uint32_t *>(tile + k * 128) = c4[k];
            }
            __syncthreads();                               // the tiles are complete
            // 8 tiles of 16 rows x 128 bytes = 1024 pieces of 16 bytes: four per thread
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int idx = tid + 256 * r;
                const int tl = idx >> 7, row = (idx >> 3) & 15, c16 = idx & 7;
                const uint32_t item = item0 + (uint32_t)tl;
                const uint32_t i = item / nsub, s = item % nsub;
                const uint4 v = *reinterpret_cast<const uint4 *>(tiles + tl * kLongVTile + row * 128 + 16 * c16);
                *reinterpret_cast<uint4 *>(out + ((size_t)(seg * 4 + (int)i) * P + (size_t)(P - 16 * (int)(s + 1)) + row) * hidden_dim + 16 * c16) = v;
            }
            __syncthreads();                               // ... and read before the next step writes them
        }
    }
}

static int check_long(bool is_k, const void *codes, const void *stream, const void *info, int ctx_len, int hidden_dim,
                      int P, int bits) {
    PKV_REQUIRE(codes && stream && info, PKV_ERR_INVALID, "null pointer argument");
    PKV_REQUIRE(P == 32 || P == 64 || P == 128 || P == 256, PKV_ERR_UNSUPPORTED,
                "not supported: pack_len %d (16, 32, 64, 128 or 256 tokens)", P);
    PKV_REQUIRE(bits >= 2 && bits <= kMaxBits, PKV_ERR_UNSUPPORTED, "not supported: bits_len %d (2..8)", bits);
    PKV_REQUIRE(ctx_len > 0 && hidden_dim > 0, PKV_ERR_INVALID, "sizes must be positive");
    PKV_REQUIRE(ctx_len % ((is_k ? 4 : 8) * P) == 0, PKV_ERR_INVALID,
                "ctx_len must be divisible by the block's tokens (%d packs of pack_len)", is_k ? 4 : 8);
    PKV_REQUIRE(hidden_dim % (is_k ? 128 : 64) == 0, PKV_ERR_INVALID, "hidden_dim must be divisible by %d", is_k ? 128 : 64);
    PKV_REQUIRE((reinterpret_cast<uintptr_t>(stream) & 1u) == 0, PKV_ERR_INVALID,
                "compressed_buffer must start at an even address (blocks are written in 2-byte units)");
    PKV_REQUIRE(!is_k || (reinterpret_cast<uintptr_t>(codes) & 3u) == 0, PKV_ERR_INVALID,
                "the code matrix must start at a 4-byte boundary");
    return PKV_OK;
}

static int run_pack_long(bool is_k, const uint8_t *codes, uint8_t *stream, uint64_t capacity, uint32_t *info, int ctx_len,
                         int hidden_dim, int P, int bits, uint64_t *size_out, float *ms_out, hipStream_t s) {
    int rc = check_long(is_k, codes, stream, info, ctx_len, hidden_dim, P, bits);
    if (rc) return rc;
    PKV_REQUIRE(capacity > 0, PKV_ERR_INVALID, "compressed_buffer must be a non-empty tensor");
    if (capacity > (1ull << 32)) capacity = 1ull << 32;          // block_info offsets are 32 bits: never wrapped
    const uint32_t nblocks = (uint32_t)(ctx_len / ((is_k ? 4 : 8) * P)) * (uint32_t)(hidden_dim / (is_k ? 128 : 64));
    ScanState *st = nullptr;
    if ((rc = prepare_scan_state(nblocks, &st, s))) return rc;
    LaunchTimer tm(s, ms_out != nullptr);
    if ((rc = tm.begin())) return rc;
    const int threads = 128 * long_chunks(P);
    // the block image in LDS: the block's bound and what the copy reads past the last byte
    const uint32_t image_bytes = ((uint32_t)pkv_block_bound_p(P, bits) + 32u + 127u) & ~127u;      // (whole 128-byte rows: the swizzle stays inside a row)
    if (is_k) {
        // packs of 32 tokens: four consecutive blocks per workgroup (1024 threads) while the number of blocks allows --
        // 0.41 -> 0.28 ms per 512 MiB; at 64 tokens two blocks per workgroup lose, 0.25 -> 0.28 ms.  NT = tokens of a
        // pack per thread: 16, or 32 for packs of 256
        const int nb = P != 32 ? 1 : nblocks % 4 == 0 ? 4 : nblocks % 2 == 0 ? 2 : 1;
        const uint32_t lds_k = (uint32_t)nb * (((uint32_t)pkv_block_bound_p(P, bits) + 127u) & ~127u) + 128u;
#define PKV_LAUNCH_LONG_K(NT_, NB_)                                                                                            \
    do {                                                                                                                       \
        PKV_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(pack_long_k_kernel<NT_, NB_>),                          \
                                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_k));                             \
        pack_long_k_kernel<NT_, NB_><<<nblocks / NB_, threads * NB_, lds_k, s>>>(codes, stream, capacity, info, st, hidden_dim, \
                                                                                P, bits, nblocks / NB_);                        \
    } while (0)
        if (P == 256) PKV_LAUNCH_LONG_K(32, 1);
        else if (nb == 4) PKV_LAUNCH_LONG_K(16, 4);
        else if (nb == 2) PKV_LAUNCH_LONG_K(16, 2);
        else PKV_LAUNCH_LONG_K(16, 1);
#undef PKV_LAUNCH_LONG_K
    } else if ((reinterpret_cast<uintptr_t>(codes) & 15u) == 0) {
        // two adjacent blocks per workgroup for packs of 32 and 64 tokens when every row of blocks is even (512 MiB of
        // 4-bit codes: 0.42 -> 0.32 ms and 0.27 -> 0.23 ms; longer packs lose by it -- 0.23 -> 0.26 ms at 128 tokens,
        // 0.27 -> 0.29 ms at 256 -- because two images leave one workgroup per CU)
        const bool pair = hidden_dim % 128 == 0 && P <= 64;
        const uint32_t lds_v = pair ? 2u * image_bytes : image_bytes;
#define PKV_LAUNCH_LONG_V(PP)                                                                                                  \
    do {                                                                                                                       \
        if (pair) {                                                                                                            \
            PKV_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(pack_long_v_kernel<PP, 2>),                        \
                                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_v));                         \
            pack_long_v_kernel<PP, 2><<<nblocks / 2, 1024, lds_v, s>>>(codes, stream, capacity, info, st, hidden_dim, bits,      \
                                                                       nblocks / 2);                                           \
        } else {                                                                                                               \
            PKV_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(pack_long_v_kernel<PP, 1>),                        \
                                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_v));                         \
            pack_long_v_kernel<PP, 1><<<nblocks, 512, lds_v, s>>>(codes, stream, capacity, info, st, hidden_dim, bits, nblocks); \
        }                                                                                                                      \
    } while (0)
        if (P == 32) PKV_LAUNCH_LONG_V(32);
        else if (P == 64) PKV_LAUNCH_LONG_V(64);
        else if (P == 128) PKV_LAUNCH_LONG_V(128);
        else PKV_LAUNCH_LONG_V(256);
#undef PKV_LAUNCH_LONG_V
    } else {
        // a code matrix that does not start at a 16-byte boundary: the plain kernel (byte loads)
        pack_long_v_plain_kernel<<<nblocks, threads, 0, s>>>(codes, stream, capacity, info, st, hidden_dim, P, bits, nblocks);
    }
    PKV_HIP_CHECK(hipGetLastError());
    if ((rc = tm.end(ms_out))) return rc;
    return finish_encode(st, size_out, 0, s);
}

static int run_unpack_long(bool is_k, const uint8_t *stream, uint64_t stream_bytes, const uint32_t *info, uint8_t *codes,
                           int ctx_len, int hidden_dim, int P, int bits, float *ms_out, hipStream_t s) {
    int rc = check_long(is_k, codes, stream, info, ctx_len, hidden_dim, P, bits);
    if (rc) return rc;
    const uint32_t nblocks = (uint32_t)(ctx_len / ((is_k ? 4 : 8) * P)) * (uint32_t)(hidden_dim / (is_k ? 128 : 64));
    LaunchTimer tm(s, ms_out != nullptr);
    if ((rc = tm.begin())) return rc;
    const uint32_t meta = 16u * (uint32_t)(bits + len_field_bits(bits));
    const uint32_t slot_cap = 4u * (uint32_t)P * (uint32_t)bits;              // 32 packs of P tokens at full width
    if (is_k) {
        // a workgroup per unit, staged through LDS; a half-wavefront per sub-word, at most eight
        const uint32_t unit_cap = meta + 4u * slot_cap;
        const int threads = 32 * (P / 16 < 8 ? P / 16 : 8);
        unpack_long_k_kernel<<<4 * nblocks, threads < 64 ? 64 : threads, unit_cap + 48u, s>>>(stream, info, codes, hidden_dim, P, bits,
                                                                                          stream_bytes, unit_cap);
    } else if (hidden_dim % 128 == 0 && (reinterpret_cast<uintptr_t>(codes) & 15u) == 0) {
        // pairs of adjacent blocks (whole 128-byte lines), a workgroup per token half; all four slots of a unit are
        // staged at once while they fit 4 KiB per unit, else two or one at a time -- but never less than the eight
        // (slot, sub-word) items of a step
        const uint32_t stage_max = 4096u;        // (8 KiB: 5 % slower at 128 and 256 tokens, two trips to memory per stage; 2 KiB: 15 % slower at 64)
        int sps = 4u * slot_cap <= stage_max ? 4 : 2u * slot_cap <= stage_max ? 2 : 1;
        while (sps * (P / 16) < 8) sps *= 2;
        const uint32_t stage_cap = (uint32_t)sps * slot_cap;
        const uint32_t meta16 = (meta + 15u) & ~15u;
        const uint32_t lds_bytes = 4u * (stage_cap + meta16 + 48u) + 8u * (uint32_t)kLongVTile + 4u * 4u * 32u * 4u + 4u * (meta16 + 32u);
        PKV_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(unpack_long_v_kernel),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
        unpack_long_v_kernel<<<nblocks, 256, lds_bytes, s>>>(stream, info, codes, hidden_dim, P, bits, stream_bytes, stage_cap, sps);
    } else {
        const int threads = 128 * long_chunks(P);
        unpack_long_v_plain_kernel<<<nblocks, threads, 0, s>>>(stream, info, codes, hidden_dim, P, bits, stream_bytes);
    }
    PKV_HIP_CHECK(hipGetLastError());
    return tm.end(ms_out);
}

}  // namespace pkv

extern "C" {

int pkv_k_encode_p(const uint8_t *codes, uint8_t *stream, uint64_t capacity, uint32_t *block_info, int ctx_len,
                   int hidden_dim, int pack_len, int bits, uint64_t *size_out, float *ms_out, pkv_stream_t s) {
    if (pack_len == 16)
        return pkv_k_encode(codes, stream, capacity, block_info, ctx_len, hidden_dim, 64, 128, bits, size_out, ms_out, s);
    return pkv::run_pack_long(true, codes, stream, capacity, block_info, ctx_len, hidden_dim, pack_len, bits, size_out,
                              ms_out, (hipStream_t)s);
}

int pkv_v_encode_p(const uint8_t *codes, uint8_t *stream, uint64_t capacity, uint32_t *block_info, int ctx_len,
                   int hidden_dim, int pack_len, int bits, uint64_t *size_out, float *ms_out, pkv_stream_t s) {
    if (pack_len == 16)
        return pkv_v_encode(codes, stream, capacity, block_info, ctx_len, hidden_dim, 128, 64, bits, size_out, ms_out, s);
    return pkv::run_pack_long(false, codes, stream, capacity, block_info, ctx_len, hidden_dim, pack_len, bits, size_out,
                              ms_out, (hipStream_t)s);
}

int pkv_k_decode_p(const uint8_t *stream, uint64_t stream_bytes, const uint32_t *block_info, uint8_t *codes, int ctx_len,
                   int hidden_dim, int pack_len, int bits, float *ms_out, pkv_stream_t s) {
    if (pack_len == 16)
        return pkv_k_decode(stream, stream_bytes, block_info, codes, ctx_len, hidden_dim, 64, 128, bits, ms_out, s);
    return pkv::run_unpack_long(true, stream, stream_bytes, block_info, codes, ctx_len, hidden_dim, pack_len, bits, ms_out,
                                (hipStream_t)s);
}

int pkv_v_decode_p(const uint8_t *stream, uint64_t stream_bytes, const uint32_t *block_info, uint8_t *codes, int ctx_len,
                   int hidden_dim, int pack_len, int bits, float *ms_out, pkv_stream_t s) {
    if (pack_len == 16)
        return pkv_v_decode(stream, stream_bytes, block_info, codes, ctx_len, hidden_dim, 128, 64, bits, ms_out, s);
    return pkv::run_unpack_long(false, stream, stream_bytes, block_info, codes, ctx_len, hidden_dim, pack_len, bits, ms_out,
                                (hipStream_t)s);
}

uint64_t pkv_block_bound_p(int pack_len, int bits) {
    if (pack_len < 16 || bits < 2 || bits > pkv::kMaxBits) return 0;
    return 8ull + 4ull * (uint64_t)(bits + pkv::len_field_bits(bits)) * 16ull + 512ull * (uint64_t)pack_len * (uint64_t)bits / 8ull;
}

}  // extern "C"
