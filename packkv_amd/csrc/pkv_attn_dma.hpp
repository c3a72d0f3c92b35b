// Fused decompress-attention decode, asynchronous-copy kernel.  The compressed blocks of a tile
// travel global memory -> LDS with LDS-direct buffer loads (no registers, 16 bytes per lane,
// fully coalesced) into one of two tile slots, one tile ahead of their use; lanes then parse their
// packs out of LDS.  Included by pkv_attn.hip after pkv_attn_direct.hpp (shares UnitRegs,
// meta_fields, unit_windows, pack_offsets8 and the fused DPP reductions).
//
// Tile = 128 tokens of one (sequence, KV head) = 2 K blocks (64 x 128) + 2 V blocks (128 x 64);
// wave w copies block w (0, 1: K; 2, 3: V) and quantizer-parameter array w of the tile.
// Per tile and half-wavefront hw (0..7): K unit = round hw%4 of K block hw/4, V unit = segment
// hw%4 of V block hw/4 -- both blocks are wave-uniform (hw/4 == wave/2).
//
// Step s of the pipeline (slot = s & 1 holds tile s, already parsed into registers):
//   K stage      packs -> int8 K tile, written OVER the block bytes of slot s (dead once parsed),
//                scores on the matrix cores; then wait for this wave's share of the copy of
//                tile s+1                                                           | barrier 1
//   softmax      reads scores and the slot's parameters, together with the parse of tile s+1
//                out of the other slot                                              | barrier 2
//   issue the copy of tile s+2 into slot s (its scores and parameters are consumed); V stage.
// LDS per workgroup is 2 slots + 2 KiB: four workgroups fit a CU.
//
// Ordering.  The copies are issued from inline assembly, so the compiler neither sees them nor
// waits for them; every wait on a copy is written out here (s_waitcnt vmcnt(0): the loop has no
// other vector memory instruction, block_info comes through scalar loads).  The barriers are bare
// s_barrier with an LDS-only wait: a workgroup fence would also drain the copies in flight.
// The slots sit at the bottom of LDS, below 64 KiB.
#pragma once

namespace pkv {

// Wave priorities of the pipeline stages (s_setprio).  With four workgroups per CU (groups of up to 4 query heads,
// the reference's widths) the further a wavefront is in its tile the sooner it issues, so the resident workgroups
// drift apart instead of competing stage for stage -- wavefronts reach their barriers earlier and the vector ALUs
// idle less: 142.5 us with equal priorities, 129.5 us with (K 1, softmax 2, copy issue 0, V 3) on the 16 x 8 x
// 32768-token workload (a sweep over the 2-bit range; copy issue lowest was best).  The setting does not carry over
// to fewer resident workgroups: with three (groups of 8) equal priorities are best (197 us against 218), with two
// (widths 5 and 6) the K stage first (211 us against 218).
template <int G, bool WIDE> struct StagePrio {                       // 4 workgroups per CU
    static constexpr int K = 1, S = 2, D = 0, V = 3;                 // K stage, parse + softmax, copy issue and waits, V stage
};
template <int G> struct StagePrio<G, true> { static constexpr int K = 2, S = 1, D = 0, V = 0; };
template <> struct StagePrio<8, false> { static constexpr int K = 0, S = 0, D = 0, V = 0; };
#define PKV_LDS_BARRIER() asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory")
// A wave-uniform value the compiler may not look through: keeps scalar min / max chains on the scalar unit (it forms
// three-operand vector instructions plus a v_readfirstlane out of them otherwise) and keeps cheap address arithmetic
// inside the loop instead of in scalar registers that live across it.
#define PKV_SCALAR(x) asm volatile("" : "+s"(x))

// PKV_ATTN_PROBE (measurement builds only, results are then meaningless): bit mask of pipeline stages to leave out
// of the tile loop -- 1 the copies (the first two tiles are re-used), 2 the K stage, 4 the softmax, 8 the V stage,
// 16 the parse, 32 the wait for the copies.  30 = "loads only", 1 = "arithmetic only".
#ifndef PKV_ATTN_PROBE
#define PKV_ATTN_PROBE 0
#endif

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// Raw buffer descriptor (base, stride 0, num_records = bytes, 32-bit raw format): reads past
// `bytes` return zero instead of touching memory.
__device__ __forceinline__ u32x4 dma_rsrc(const void *base, uint32_t bytes) {
    const uintptr_t a = reinterpret_cast<uintptr_t>(base);
    return (u32x4){(uint32_t)a, (uint32_t)(a >> 32) & 0xFFFFu, bytes, 0x00020000u};
}

// One LDS-direct load: lane l's 16 (4) bytes at buffer offset voff (+ soff) land at LDS byte
// lds_addr + 16 l (4 l).  lds_addr, rsrc and soff are wave-uniform.  M0 (the LDS base of the copy)
// is written and consumed inside the one asm statement; nothing else in these kernels depends on M0.
// The compiler does not see inside the statement, so it pads no hazards for it: the s_mov and the s_nop 3 are the
// five wait states a memory instruction needs after a VALU instruction wrote one of its scalar operands (which is
// what the compiler's restore of a spilled scalar register is).
// M0 is on the clobber list: the compiler reserves the register for its own short-lived uses (lane-indexed writes, LDS
// parameters) and may merge or hoist the initialisations it emits for them; told about the write, it keeps none of them
// alive across these statements.  (It warns that a reserved register is named; that is the point.)
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
__device__ __forceinline__ void dma_b128(u32x4 rsrc, uint32_t lds_addr, uint32_t voff) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 3\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
                 :: "s"(lds_addr), "v"(voff), "s"(rsrc) : "memory", "m0");
}
// The same with an immediate offset, which the hardware adds on both sides: to the buffer offset (and its range
// check) and to the LDS address (measured: data of `offset:1024` lands 1 KiB behind M0's address).
template <int IMM>
__device__ __forceinline__ void dma_b128_imm(u32x4 rsrc, uint32_t lds_addr, uint32_t voff) {
    static_assert(IMM >= 0 && IMM < 4096, "12-bit immediate");
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 3\n\tbuffer_load_dwordx4 %1, %2, 0 offen offset:%3 lds"
                 :: "s"(lds_addr), "v"(voff), "s"(rsrc), "n"(IMM) : "memory", "m0");
}
__device__ __forceinline__ void dma_b32(u32x4 rsrc, uint32_t lds_addr, uint32_t voff, uint32_t soff) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 3\n\tbuffer_load_dword %1, %2, %3 offen lds"
                 :: "s"(lds_addr), "v"(voff), "s"(rsrc), "s"(soff) : "memory", "m0");
}
#pragma clang diagnostic pop

// The same descriptor moved `add` bytes forward and cut to `bytes`: scalar arithmetic only.  A copy whose lanes address
// `16 lane` through such a descriptor needs no per-lane address arithmetic and no per-lane clamp: lanes past the end
// get zeroes (and touch no memory).
__device__ __forceinline__ u32x4 dma_rsrc_at(u32x4 r, uint32_t add, uint32_t bytes) {
    const uint64_t a = (((uint64_t)r[1] << 32) | r[0]) + add;
    return (u32x4){(uint32_t)a, (uint32_t)(a >> 32), bytes, r[3]};
}

template <int N> struct IntC { static constexpr int value = N; };

template <int KW, int VW>
struct DmaGeom {
    static constexpr int kMaxBlock = k_block_bound(64, KW) > v_block_bound(64, VW) ? k_block_bound(64, KW) : v_block_bound(64, VW);
    // a block is copied from the 16-byte boundary below its start: up to 14 bytes of phase in front
    static constexpr int kRegion = (kMaxBlock + 14 + 511) / 512 * 512;      // LDS bytes per block
    static constexpr int kMaxInstr = (kRegion + 1023) / 1024;              // 64-lane copy instructions per block
    static constexpr int kKTile = 8 * 16 * 136;                            // the int8 K tile shares the block regions
    static constexpr int kParOff = 4 * kRegion > kKTile ? 4 * kRegion : kKTile;   // then 4 arrays x 128 tokens x 2 bytes
    static constexpr int kSlot = kParOff + 4 * kTile * 2;
    static_assert(2 * kSlot <= 65536, "the slots must stay below 64 KiB of LDS");
    static_assert(kKTile == 8 * 16 * kKtStride, "K tile geometry");
};

// One unit's packs in registers: pack words, the four widths as two 16-bit pairs, minima as bytes.
struct UnitPairs {
    uint64_t word[4];
    uint32_t len01, len23;   // widths of packs (0, 1) and (2, 3), one per 16-bit half
    uint32_t mins;           // the four minima, one per byte
};

__device__ __forceinline__ uint32_t pk_mask16(uint32_t len_pair) {   // (1 << len) - 1 in both halves
    const ushort2v one = {1, 1};
    return __builtin_bit_cast(uint32_t, (ushort2v)((ushort2v)(one << __builtin_bit_cast(ushort2v, len_pair)) - one));
}

__device__ __forceinline__ int4v pair128(long a, long b) {
    return (int4v){(int)a, (int)(a >> 32), (int)b, (int)(b >> 32)};
}

// 64 bits at byte offset `off` (even) of an LDS array whose base is 4-byte aligned: the three
// aligned dwords that cover it, funnel-shifted by bytes (a misaligned DS read stalls the LDS pipe).
__device__ __forceinline__ uint64_t lds_word64(const uint8_t *base, uint32_t off) {   // base: a 4-byte aligned array; pass every
    const uint32_t *q = reinterpret_cast<const uint32_t *>(base + (off & ~3u));      // variable part of the address in `off`
    const uint32_t d0 = q[0], d1 = q[1], d2 = q[2];
    const uint32_t lo = __builtin_amdgcn_alignbyte(d1, d0, off), hi = __builtin_amdgcn_alignbyte(d2, d1, off);
    return ((uint64_t)hi << 32) | lo;
}

// Lane t's 4*NB-bit metadata word of an LSB-first bit array in LDS.  `base` is 4-byte aligned and holds everything the
// compiler knows of the address (it becomes the instruction's offset field); `a` = byte offset of the array (even)
// + meta_lane_byte<NB>(t), everything that varies; the word starts meta_lane_bit<NB>(t) bits into that byte.
template <int NB> __device__ __forceinline__ uint32_t meta_lane_byte(int t) { return (uint32_t)(t * 4 * NB) >> 3; }
template <int NB> __device__ __forceinline__ uint32_t meta_lane_bit(int t) { return (uint32_t)(t * 4 * NB) & 7u; }
template <int NB>
__device__ __forceinline__ uint32_t lds_meta(const uint8_t *base, uint32_t a, uint32_t lane_bit) {
    if (NB == 4) return *reinterpret_cast<const uint16_t *>(base + a);
    if (NB == 2) return base[a];
    // 4 NB bits, then 0 or 4 bits further (4 NB + 4 <= 32 for NB <= 7)
    const uint32_t *q = reinterpret_cast<const uint32_t *>(base + (a & ~3u));
    const uint32_t v = __builtin_amdgcn_alignbyte(q[1], q[0], a);
    return (v >> lane_bit) & ((1u << (4 * NB)) - 1u);
}

template <int W, typename U>
__device__ __forceinline__ void meta_pairs(uint32_t minsw, uint32_t lensw, U &u) {
    constexpr int LB = len_field_bits(W);
    u.len01 = __builtin_amdgcn_ubfe(lensw, 0, LB) | (__builtin_amdgcn_ubfe(lensw, LB, LB) << 16);
    u.len23 = __builtin_amdgcn_ubfe(lensw, 2 * LB, LB) | (__builtin_amdgcn_ubfe(lensw, 3 * LB, LB) << 16);
    if (W == 4) {   // four nibbles -> four bytes
        const uint32_t y = (minsw | (minsw << 8)) & 0x00FF00FFu;
        u.mins = (y | (y << 4)) & 0x0F0F0F0Fu;
    } else {
        u.mins = __builtin_amdgcn_ubfe(minsw, 0, W) | (__builtin_amdgcn_ubfe(minsw, W, W) << 8) |
                 (__builtin_amdgcn_ubfe(minsw, 2 * W, W) << 16) | (__builtin_amdgcn_ubfe(minsw, 3 * W, W) << 24);
    }
}

// win01[q] = tokens 4q..4q+3 of packs 0 and 1 in the low / high 16 bits (token 4q on top), win23
// likewise; bits above 4*len in a half are other tokens' fields, every consumer masks.
__device__ __forceinline__ void pair_windows(const UnitPairs &u, uint32_t win01[4], uint32_t win23[4]) {
    // shift amounts, two to a register like the widths: 8 len (the upper eight tokens) and 4 len (the upper four of
    // eight).  A shift takes the low six (five) bits of its amount, and 8 len <= 32 leaves the bits above untouched,
    // so the low half of a pair serves as it stands and the high half is one byte-select away.
    const uint32_t s8[2] = {u.len01 << 3, u.len23 << 3}, s4[2] = {u.len01 << 2, u.len23 << 2};
    uint32_t hlf[4][2];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const uint32_t a8 = (i & 1) ? s8[i >> 1] >> 16 : s8[i >> 1];
        hlf[i][0] = (uint32_t)(u.word[i] >> (a8 & 63u));    // tokens 0..7
        hlf[i][1] = (uint32_t)u.word[i];                      // tokens 8..15
    }
#pragma unroll
    for (int q = 0; q < 4; q++) {
        uint32_t qd[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t src = hlf[i][q >> 1];
            const uint32_t a4 = (i & 1) ? s4[i >> 1] >> 16 : s4[i >> 1];
            qd[i] = (q & 1) ? src : (src >> (a4 & 31u));
        }
        win01[q] = __builtin_amdgcn_perm(qd[1], qd[0], 0x05040100u);
        win23[q] = __builtin_amdgcn_perm(qd[3], qd[2], 0x05040100u);
    }
}

// Widths 5 and 6 (this build's extension of the format): a quarter of a pack no longer fits a 16-bit lane, so the
// windows hold TWO tokens each.  e01[e] = tokens 2e, 2e+1 of packs 0 and 1 in the low / high 16 bits (token 2e on
// top), e23 likewise; bits above 2*len in a half are other tokens' fields, every consumer masks.
struct UnitWide {
    uint32_t e01[8], e23[8];
    uint32_t len01, len23;
    uint32_t mins;
};

// The eight two-token windows of the four packs whose words start at byte pay0 + 2 * off2[i] of `base`.  A word is
// up to 12 bytes long, so it is not assembled: each quarter (four tokens, 4 * len bits starting (3 - q) * 4 * len
// bits into the word, i.e. at a byte or a nibble boundary) is fetched on its own as the 32 bits at its byte
// address -- two aligned dwords and a byte funnel shift -- and moved down by the odd nibble.
__device__ __forceinline__ void wide_windows(const uint8_t *base, uint32_t pay0, const uint32_t off2[4], UnitWide &u) {
    const uint32_t len[4] = {u.len01 & 0xFFFFu, u.len01 >> 16, u.len23 & 0xFFFFu, u.len23 >> 16};
    uint32_t hi[4][4], lo[4][4];       // [pack][quarter]: tokens 4q, 4q+1 and 4q+2, 4q+3
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const uint32_t a = pay0 + 2u * off2[i], L = len[i], nib = (L & 1u) * 4u;
        const uint32_t at[4] = {a + ((3u * L) >> 1), a + L, a + (L >> 1), a};      // byte address of quarter q
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const uint32_t *dq = reinterpret_cast<const uint32_t *>(base + (at[q] & ~3u));
            uint32_t v = __builtin_amdgcn_alignbyte(dq[1], dq[0], at[q]);
            if (q == 0 || q == 2) v >>= nib;
            lo[i][q] = v;
            hi[i][q] = v >> (2u * L);
        }
    }
#pragma unroll
    for (int q = 0; q < 4; q++) {
        u.e01[2 * q] = __builtin_amdgcn_perm(hi[1][q], hi[0][q], 0x05040100u);
        u.e01[2 * q + 1] = __builtin_amdgcn_perm(lo[1][q], lo[0][q], 0x05040100u);
        u.e23[2 * q] = __builtin_amdgcn_perm(hi[3][q], hi[2][q], 0x05040100u);
        u.e23[2 * q + 1] = __builtin_amdgcn_perm(lo[3][q], lo[2][q], 0x05040100u);
    }
}

// Wavefronts per SIMD the register allocation aims for: four workgroups per CU for the reference's widths (three for
// groups of 8 query heads); the two-token windows of widths 5 and 6 need about 210 VGPRs, two workgroups per CU
// (at three, 168 VGPRs, the compiler spills 47 of them and the kernel is 2.4 times slower).
#define PKV_DMA_WAVES(KW, G) ((KW) > 4 ? ((G) <= 4 ? 2 : 1) : ((G) <= 4 ? 4 : 3))
template <bool WIDE> struct UnitOf { typedef UnitPairs type; };
template <> struct UnitOf<true> { typedef UnitWide type; };

template <int G, int KW, int VW>
constexpr int dma_lds_bytes() {          // static LDS of attn_dma_kernel: two slots, weights, round sums, state
    constexpr int GP = (G + 3) / 4 * 4;
    return 2 * DmaGeom<KW, VW>::kSlot + GP * (kTile + 4) * 2 + 2 * GP * 8 * 2 + 8 * 8 * 4;
}

template <int G, int KW, int VW, bool BF>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(PKV_DMA_WAVES((KW > VW ? KW : VW), G), 4))) attn_dma_kernel(const AttnParams p) {
    using Geo = DmaGeom<KW, VW>;
    constexpr bool KWIDE = KW > 4, VWIDE = VW > 4;            // widths 5, 6: two-token windows (K and V independently)
    constexpr bool WIDE = KWIDE || VWIDE;
    static_assert(KW <= 6 && VW <= 6, "widths 2..6");
    constexpr int KTPW = KWIDE ? 2 : 4, VTPW = VWIDE ? 2 : 4;  // tokens per window
    constexpr int KNWIN = 16 / KTPW, VNWIN = 16 / VTPW;
    typedef typename UnitOf<KWIDE>::type KUnit;
    typedef typename UnitOf<VWIDE>::type VUnit;
    typedef StagePrio<G, WIDE> Prio;
    constexpr int ROWS = 4 * G;                   // MFMA row 4 g + digit (row 4 g + 3 stays zero): the three digits of a
    constexpr int NSETS = (ROWS + 15) / 16;       // head come out in one lane
    constexpr bool SCORE_INT = KW <= 4;           // 128 x 64 x 15 x 2^14 < 2^31: the digits combine in int32
    constexpr int NG4 = (G + 3) / 4;
    constexpr int GP = NG4 * 4;
    constexpr int GW = (G + 3) / 4;
    constexpr int KLB = len_field_bits(KW), VLB = len_field_bits(VW);
    constexpr uint32_t K_META = KW * 16 + KLB * 16, V_META = VW * 16 + VLB * 16;
    constexpr int kRoundBytes = 16 * kKtStride;
    static_assert(NSETS * 256 <= kRoundBytes, "score rows must fit the K-tile rows they reuse");

    constexpr int kPStride = kTile + 4;          // halves per head row of the weights: rows 8 bytes apart in bank space
    constexpr int kLdsBytes = dma_lds_bytes<G, KW, VW>();
    static_assert(kLdsBytes == 2 * Geo::kSlot + GP * kPStride * 2 + 2 * GP * 8 * 2 + 8 * 8 * 4, "LDS layout");
    __shared__ __attribute__((aligned(16))) uint8_t smem[kLdsBytes];
    uint8_t *ring = smem;                                                    // [2 slots][4 block regions | parameters]
    _Float16 *pbuf = reinterpret_cast<_Float16 *>(smem + 2 * Geo::kSlot);    // [GP][128 + 4]
    _Float16 *p16hi = pbuf + GP * kPStride;                                     // [GP][8]
    _Float16 *p16lo = p16hi + GP * 8;
    float *st_m = reinterpret_cast<float *>(p16lo + GP * 8);                 // 8 floats each
    float *st_l = st_m + 8, *st_z = st_l + 8, *qsum = st_z + 8, *qs = qsum + 8;
    float *st_a = qs + 8;                                                    // [2 slot parities][8]: accumulator factors of a step
    uint32_t *resc = reinterpret_cast<uint32_t *>(st_a + 16);                // [2]: some head's factor of that step is not 1
    const uint32_t ring_lds = (uint32_t)reinterpret_cast<uintptr_t>(ring);   // LDS byte address of the slots

    // Workgroup L of the launch is member L / (B Hkv) of (sequence, KV head) L % (B Hkv): the members of one head are
    // spread over the launch, so that each head has members among the workgroups a CU starts first and among those
    // it starts last (the former run faster), and they even it out by taking tiles from a common counter.
    // Which head: workgroups go round-robin over the 8 XCDs (each with an L2 of its own), and neighbouring heads
    // should share one -- a block copy reads whole 1 KiB pieces, so it runs into the next block of the stream, which
    // is the next head's; on the same XCD that piece is the neighbour's own copy a moment later (an L2 hit), on
    // another it crosses HBM twice (measured: 1.13 x the algorithmic bytes, 1.01 x with this assignment).
    const int n_heads = p.B * p.Hkv;
    const int split = (int)blockIdx.x / n_heads, slot_ = (int)blockIdx.x % n_heads;
    const int bh_ = (n_heads & 7) == 0 ? (slot_ & 7) * (n_heads >> 3) + (slot_ >> 3) : slot_;
    const int h = bh_ % p.Hkv, b = bh_ / p.Hkv;
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    __builtin_assume(wave >= 0 && wave < 4);
    const int t = tid & 31, hw = tid >> 5;
    const int bh = b * p.Hkv + h;
    const int n_hid_k = p.B * p.Hkv;

    // the stream this wave copies from, range-checked: block_info is never trusted with an address
    // (the size is rounded up to whole dwords: a copy is range-checked dword by dword, and the aligned dword that
    // holds the buffer's last byte lies in the same page as that byte -- a buffer that ends with its stream loses
    // nothing and nothing unmapped is touched)
    const uint32_t blk_bytes4 = ((wave < 2 ? p.k_bytes : p.v_bytes) + 3u) & ~3u;
    const u32x4 blk_rsrc = dma_rsrc(wave < 2 ? p.k_stream : p.v_stream, blk_bytes4);
    const uint16_t *par_arr = wave == 0 ? p.k_scale : wave == 1 ? p.k_zero : wave == 2 ? p.v_scale : p.v_zero;
    const u32x4 par_rsrc = dma_rsrc(par_arr, (uint32_t)(p.B * p.par_stride * 2));
    const uint32_t par_row = (uint32_t)(b * p.par_stride * 2);        // byte offset of this sequence's parameter rows

    // Tiles this member works on, by position in its own sequence.  Static split (p.dynamic == 0): the contiguous
    // range [tile0, tile_end).  Dynamic: positions 0..4 are tiles split + k * nsplit (known at once, they fill the
    // pipeline); every further position comes out of the head's counter, which counts the tiles handed out so far:
    // a member adds the size of the batch it wants (up to four tiles while many are left, single tiles towards the
    // end, so that the members finish together) and owns tiles 5 nsplit + [old value, old value + size); a faster
    // member simply comes back sooner.  The request for the next batch goes out when the current one is first drawn
    // on, so its round trip lies at least a whole step before the value is needed.  Sequences are increasing, a
    // tile number >= tile_end ends them, and attention does not depend on the order of the tokens.
    const int n_tiles = p.T_c / kTile;
    const int tile0 = split * p.tiles_per_split;
    const int tile_end = p.dynamic ? n_tiles : min(n_tiles, tile0 + p.tiles_per_split);
    auto first_tiles = [&](int k) -> int { return p.dynamic ? split + k * p.nsplit : tile0 + k; };
    __shared__ int tau_lds[2];

    // ---- block_info: wave-uniform scalar loads, fetched well before use ----
    // this wave copies block `wave` of a tile and parses K block wave/2 and V block 2 + wave/2
    // (read through the constant address space: block_info is read-only for the whole launch, and
    // only loads known to be unclobbered are issued as scalar loads; a vector load here would make
    // every later vmcnt wait drain the copies in flight)
    typedef const __attribute__((address_space(4))) uint32_t *const_u32_ptr;
    const int kj = wave >> 1;
    const const_u32_ptr k_info_c = reinterpret_cast<const_u32_ptr>(reinterpret_cast<uintptr_t>(p.k_info));
    const const_u32_ptr v_info_c = reinterpret_cast<const_u32_ptr>(reinterpret_cast<uintptr_t>(p.v_info));
    // entry of this wave's blocks for tile 0; a tile further on is 2 K rows = 1 V row = 4 B Hkv words further
    const const_u32_ptr dma_info0 = wave < 2 ? k_info_c + 2 * (size_t)(bh + wave * n_hid_k) : v_info_c + 2 * (size_t)(2 * bh + wave - 2);
    const const_u32_ptr k_info0 = k_info_c + 2 * (size_t)(bh + kj * n_hid_k), v_info0 = v_info_c + 2 * (size_t)(2 * bh + kj);
    const uint32_t info_stride = 4u * (uint32_t)n_hid_k;
    const uint32_t last_tile = (uint32_t)(n_tiles - 1);
    struct RawInfo { uint32_t dma_off, dma_size, k_off, v_off; };          // as loaded
    struct TileInfo { uint32_t dma_off, dma_size, ph; };                    // ph: k_off % 16 | v_off % 16 << 4
    auto load_info = [&](int tile) -> RawInfo {
        const size_t o = (size_t)min((uint32_t)tile, last_tile) * info_stride;   // past the end (or a damaged counter): the last tile again, never used
        RawInfo ri;
        ri.dma_off = dma_info0[o];
        ri.dma_size = dma_info0[o + 1];
        ri.k_off = k_info0[o];
        ri.v_off = v_info0[o];
        return ri;
    };
    auto pack_info = [&](const RawInfo &ri) -> TileInfo {
        return TileInfo{ri.dma_off, ri.dma_size, (ri.k_off & 15u) | ((ri.v_off & 15u) << 4)};
    };

    // ---- copy of one tile into slot `slot` ----
    // The block gets a descriptor of its own (scalar arithmetic): base = the 16-byte boundary below the block, length
    // = what the block and the stream hold from there.  Every copy instruction then uses the same per-lane offset,
    // 16 lane, plus 1 KiB per instruction as an immediate; lanes past the end fetch nothing and store zeroes.
    const uint32_t lane16 = 16u * (uint32_t)lane;
    const uint32_t dst_wave = ring_lds + (uint32_t)wave * (uint32_t)Geo::kRegion;
    auto dma_issue = [&](auto slot_c, int tile, const TileInfo &ti) {
        constexpr int slot = decltype(slot_c)::value;
        const uint32_t phase = ti.dma_off & 15u;                  // the streams themselves are 16-byte aligned
        const uint32_t src = ti.dma_off - phase;
        uint32_t nb = (phase + ti.dma_size + 15u) & ~15u;         // bytes to copy: whole 16-byte quads
        nb = max(nb, 16u);
        PKV_SCALAR(nb);
        nb = min(nb, (uint32_t)Geo::kRegion);                     // corrupt block_info must not overrun the region
        PKV_SCALAR(nb);
        uint32_t have = src < blk_bytes4 ? min(nb, blk_bytes4 - src) : 0u;   // ... nor the stream
        PKV_SCALAR(have);
        uint32_t dst = dst_wave;                                  // (kept out of the loop-invariant code: ten LDS
        PKV_SCALAR(dst);                                          // addresses held in scalar registers were spilled)
        dst += (uint32_t)(slot * Geo::kSlot);
        const u32x4 rs = dma_rsrc_at(blk_rsrc, src, have);
        dma_b128_imm<0>(rs, dst, lane16);
        if (nb > 1024u) dma_b128_imm<1024>(rs, dst, lane16);      // wave-uniform
        if (Geo::kRegion > 2048 && nb > 2048u) dma_b128_imm<2048>(rs, dst, lane16);
        if (Geo::kRegion > 3072 && nb > 3072u) dma_b128_imm<3072>(rs, dst, lane16);
#pragma unroll
        for (int i = 4; i < Geo::kMaxInstr; i++) {                // beyond the immediate's reach: rare, large blocks
            if ((uint32_t)(i * 1024) < nb) {
                uint32_t len = max(have, (uint32_t)(i * 1024));        // (a conditional difference becomes a saturating
                PKV_SCALAR(len);                                       // subtraction, which only the vector unit has)
                len -= (uint32_t)(i * 1024);
                // (the lane test of a partial last instruction is made here, from a value the compiler cannot trace
                // back to the lane number: as loop-invariant code it would hold a register pair for its mask)
                uint32_t l16 = lane16;
                if (i * 1024 + 1024 > Geo::kRegion) asm volatile("" : "+v"(l16));
                const u32x4 rs_i = dma_rsrc_at(blk_rsrc, src + (uint32_t)(i * 1024), len);     // scalar: before the lane test
                const uint32_t dst_i = dst + (uint32_t)(i * 1024);
                if (i * 1024 + 1024 <= Geo::kRegion || l16 < (uint32_t)(Geo::kRegion - i * 1024))
                    dma_b128(rs_i, dst_i, lane16);
            }
        }
        // parameter array `wave` of the tile: 128 tokens x 2 bytes = 16 lanes x 16 bytes
        const uint32_t tile_off = par_row + min((uint32_t)tile, last_tile) * (uint32_t)(kTile * 2);
        const u32x4 rs_p = dma_rsrc_at(par_rsrc, tile_off, 256u);
        const uint32_t dst_p = dst + (uint32_t)Geo::kParOff - (uint32_t)wave * (uint32_t)(Geo::kRegion - 256);
        uint32_t l16p = lane16;
        asm volatile("" : "+v"(l16p));
        if (l16p < 256u) dma_b128(rs_p, dst_p, lane16);
    };

    // tile 0 starts its way into slot 0 now, under the prologue's arithmetic
    int t_cur = first_tiles(0), t1 = first_tiles(1), t2 = first_tiles(2), t3 = first_tiles(3);
    TileInfo i0 = pack_info(load_info(t_cur)), i1 = pack_info(load_info(t1)), i2 = pack_info(load_info(t2));
    dma_issue(IntC<0>{}, t_cur, i0);

    auto cvt2 = [&](uint32_t w, float &lo, float &hi) {
        if (!BF) {
            lo = __half2float(__ushort_as_half((unsigned short)(w & 0xFFFFu)));
            hi = __half2float(__ushort_as_half((unsigned short)(w >> 16)));
        } else {
            lo = __uint_as_float(w << 16);
            hi = __uint_as_float(w & 0xFFFF0000u);
        }
    };

    // ---- prologue: LDS state; q split into signed 7-bit digits, staged through slot 1 (tile 0 is on its way into
    // slot 0 meanwhile) ----
    uint8_t *aq = ring + Geo::kSlot;
    for (int i = tid; i < NSETS * 4 * 16 * 32 / 4; i += 256) reinterpret_cast<uint32_t *>(aq)[i] = 0u;
    for (int i = tid; i < GP * kPStride / 2; i += 256) reinterpret_cast<uint32_t *>(pbuf)[i] = 0u;
    for (int i = tid; i < GP * 8; i += 256) reinterpret_cast<uint32_t *>(p16hi)[i] = 0u;   // hi and lo
    if (tid < 8) { st_m[tid] = -INFINITY; st_l[tid] = 0.f; st_z[tid] = 0.f; st_a[tid] = 1.f; st_a[8 + tid] = 1.f; resc[tid] = 0u; }
    __builtin_amdgcn_s_waitcnt(0xC07F);       // lgkmcnt(0): the zeroes are written; the copy in flight is not waited for
    __builtin_amdgcn_s_barrier();
    for (int g = wave; g < G; g += 4) {
        if (g >= p.Gq) {                       // an idle head slot (group of 3 in the kernel of 4, ...): a query of zeros
            if (lane == 0) { qsum[g] = 0.f; qs[g] = 0.f; }
            continue;
        }
        const size_t qoff = ((size_t)b * p.Hq + (size_t)h * p.Gq + g) * kHeadDim;
        const float q0 = a_ld16(p.q, qoff + lane, p.dtype), q1 = a_ld16(p.q, qoff + 64 + lane, p.dtype);
        const float mx = wave_max(fmaxf(fabsf(q0), fabsf(q1)));
        const float sm = wave_sum(q0 + q1);
        const float inv = mx > 0.f ? 1048576.f / mx : 0.f;
        if (lane == 0) { qsum[g] = sm; qs[g] = mx * (1.f / 1048576.f); }
#pragma unroll
        for (int e = 0; e < 2; e++) {
            const int d = lane + 64 * e;
            int Q = (int)rintf((e ? q1 : q0) * inv);
            const int d2 = ((Q + 64) & 127) - 64;
            Q = (Q - d2) >> 7;
            const int d1 = ((Q + 64) & 127) - 64;
            const int d0 = (Q - d1) >> 7;
            const int dig[3] = {d0, d1, d2};
#pragma unroll
            for (int pp = 0; pp < 3; pp++) {
                const int m = 4 * g + pp;
                aq[(((m >> 4) * 4 + (d >> 5)) * 16 + (m & 15)) * 32 + (d & 31)] = (uint8_t)(int8_t)dig[pp];
            }
        }
    }
    PKV_LDS_BARRIER();
    long aop[NSETS][4];
#pragma unroll
    for (int s = 0; s < NSETS; s++)
#pragma unroll
        for (int sl = 0; sl < 4; sl++)
            aop[s][sl] = *reinterpret_cast<const long *>(aq + ((s * 4 + sl) * 16 + (lane & 15)) * 32 + 8 * (lane >> 4));
    // score of a token in the log2 domain: (k_scale * c1) * (D + k_zero * c2), D = the integer dot product of the digits
    float c1_r[GW], c2_r[GW];
#pragma unroll
    for (int gi = 0; gi < GW; gi++) {
        const int g = min(wave + 4 * gi, G - 1);
        c1_r[gi] = p.sm_scale * qs[g] * 1.44269504088896341f;
        c2_r[gi] = qs[g] > 0.f ? qsum[g] / qs[g] : 0.f;
    }
    // The softmax weights reach the matrix cores as fp16(p * v_scale * wscale), wscale = 2^(kWExp - emax), emax = the
    // largest biased exponent of v_scale met so far: p * v_scale * wscale < 2^11 whatever the magnitude of V, at full
    // fp16 precision, and the sum of a round's 16 weights (the pack-minimum term takes it as fp16) stays below 2^15.
    // When a tile brings a larger exponent the accumulators are rescaled like for a new maximum.
    constexpr int kWExp = BF ? 137 : 25;
    uint32_t emax_pair = 0u;                      // emax in both 16-bit halves
    float wscale = 0.f, wscale_inv = 0.f;

    // ---- parse of this half-wave's K unit and V unit out of a landed slot ----
    const int ku = hw & 3;
    // what a lane adds to a unit's offset inside its block region to reach its own metadata (the region of K block
    // kj included; V block 2 + kj lies two regions further, a constant)
    const uint32_t kj_region = (uint32_t)(kj * Geo::kRegion);
    const uint32_t hdr_c = kj_region + 2u * (uint32_t)max(ku - 1, 0);
    const uint32_t kmin_c = kj_region + meta_lane_byte<KW>(t), klen_c = kj_region + meta_lane_byte<KLB>(t);
    const uint32_t vmin_c = VW == KW ? kmin_c : kj_region + meta_lane_byte<VW>(t);
    const uint32_t vlen_c = VLB == KLB ? klen_c : kj_region + meta_lane_byte<VLB>(t);
    const uint32_t kmin_b = meta_lane_bit<KW>(t), klen_b = meta_lane_bit<KLB>(t), vmin_b = meta_lane_bit<VW>(t), vlen_b = meta_lane_bit<VLB>(t);
    auto parse = [&](auto slot_c, const TileInfo &ti, KUnit &kr, VUnit &vr) {
        constexpr int slot = decltype(slot_c)::value;
        const uint8_t *kb0 = ring + slot * Geo::kSlot, *vb0 = kb0 + 2 * Geo::kRegion;   // region of K block 0 / V block 0
        const uint8_t *kb = kb0 + kj * Geo::kRegion;
        const uint8_t *vb = vb0 + kj * Geo::kRegion;
        const uint32_t kph = ti.ph & 15u, vph = ti.ph >> 4;
        // header: four cumulative u16 unit sizes; unit u starts at 8 + cum[u - 1] (read unconditionally, then selected)
        uint32_t kc = *reinterpret_cast<const uint16_t *>(kb0 + (kph + hdr_c));
        uint32_t vc = *reinterpret_cast<const uint16_t *>(vb0 + (vph + hdr_c));
        kc = ku ? kc : 0u;
        vc = ku ? vc : 0u;
        // A corrupt header must not send the metadata reads out of the block's region.  The pack
        // reads below start less than 1.1 KiB behind the unit, which keeps them inside this
        // workgroup's LDS (2.3 KiB follow the last region); garbage in, garbage out, no fault.
        const uint32_t k_unit = min(kph + 8u + kc, (uint32_t)(Geo::kRegion - K_META - 16));
        const uint32_t v_unit = min(vph + 8u + vc, (uint32_t)(Geo::kRegion - V_META - 16));
        const uint32_t k_mins = lds_meta<KW>(kb0, k_unit + kmin_c, kmin_b), k_lens = lds_meta<KLB>(kb0 + KW * 16, k_unit + klen_c, klen_b);
        const uint32_t v_mins = lds_meta<VW>(vb0, v_unit + vmin_c, vmin_b), v_lens = lds_meta<VLB>(vb0 + VW * 16, v_unit + vlen_c, vlen_b);
        uint32_t koff[4], voff[4];
        meta_pairs<KW>(k_mins, k_lens, kr);
        meta_pairs<VW>(v_mins, v_lens, vr);
        pack_offsets8(__builtin_amdgcn_perm(kr.len23, kr.len01, 0x06040200u), koff);
        pack_offsets8(__builtin_amdgcn_perm(vr.len23, vr.len01, 0x06040200u), voff);
        // pack words are addressed from the start of LDS (the slots sit at its bottom), region base included, so that
        // one shift-add and one mask make the aligned address
        const uint32_t kpay0 = k_unit + K_META, vpay0 = v_unit + V_META;
        const uint32_t kabs = (uint32_t)(slot * Geo::kSlot + kj * Geo::kRegion) + kpay0;
        const uint32_t vabs = (uint32_t)(slot * Geo::kSlot + (2 + kj) * Geo::kRegion) + vpay0;
        if constexpr (KWIDE) {
            wide_windows(kb, kpay0, koff, kr);
        } else {
#pragma unroll
            for (int i = 0; i < 4; i++) kr.word[i] = lds_word64(ring, kabs + 2u * koff[i]);
        }
        if constexpr (VWIDE) {
            wide_windows(vb, vpay0, voff, vr);
        } else {
#pragma unroll
            for (int i = 0; i < 4; i++) vr.word[i] = lds_word64(ring, vabs + 2u * voff[i]);
        }
    };


    float4v acc[NG4];
#pragma unroll
    for (int i = 0; i < NG4; i++) acc[i] = (float4v){0.f, 0.f, 0.f, 0.f};
    float m_run[GW], l_part[GW], z_part[GW];
#pragma unroll
    for (int i = 0; i < GW; i++) { m_run[i] = -INFINITY; l_part[i] = 0.f; z_part[i] = 0.f; }

    // ---- stage 1: K round hw -> int8 tile rows [hw*16, hw*16+16), then scores on the matrix cores ----
    auto k_stage = [&](const KUnit &kr, uint8_t *kt) {
        {
            constexpr int TPW = KTPW, NWIN = KNWIN;
            uint32_t w01[NWIN], w23[NWIN];
            if constexpr (KWIDE) {
#pragma unroll
                for (int e = 0; e < NWIN; e++) { w01[e] = kr.e01[e]; w23[e] = kr.e23[e]; }
            } else {
                pair_windows(kr, w01, w23);
            }
            const uint32_t len01 = kr.len01, len23 = kr.len23;
            const uint32_t mq = __builtin_amdgcn_perm(pk_mask16(len23), pk_mask16(len01), 0x06040200u);   // byte masks
            uint32_t *dst = reinterpret_cast<uint32_t *>(kt) + (hw * 16) * kKtDw + t;
#pragma unroll
            for (int q = 0; q < NWIN; q++) {
                uint32_t x01 = w01[q], x23 = w23[q];      // the window's last token first, one width further per token
#pragma unroll
                for (int pp = TPW - 1; pp >= 0; pp--) {
                    dst[(q * TPW + pp) * kKtDw] = (__builtin_amdgcn_perm(x23, x01, 0x06040200u) & mq) + kr.mins;
                    if (pp) { x01 = pk_shr16(x01, len01); x23 = pk_shr16(x23, len23); }
                }
            }
        }
        // the rounds a wavefront multiplies are the two its own halves just wrote: LDS executes a
        // wavefront's accesses in order, so only the compiler must be kept from reordering
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        // both rounds' operands first, then the products of the two rounds in turn: a round's second product waits
        // for its first, the other round's fills the gap
        long bop[2][4];
#pragma unroll
        for (int rr = 0; rr < 2; rr++) {
            const uint8_t *row = kt + ((2 * wave + rr) * 16 + (lane & 15)) * kKtStride + 8 * (lane >> 4);
#pragma unroll
            for (int sl = 0; sl < 4; sl++) bop[rr][sl] = *reinterpret_cast<const long *>(row + 32 * sl);
        }
#pragma unroll
        for (int s = 0; s < NSETS; s++) {
            int4v d[2] = {{0, 0, 0, 0}, {0, 0, 0, 0}};
            // two K = 64 products per round: which 64 channels an instruction contracts does not matter as long
            // as A and B pair up the same ones, and both operands were loaded in the same pattern
            // (the 8 channels at 32 sl + 8 (lane / 16)), so slices (0, 1) and (2, 3) simply concatenate
#pragma unroll
            for (int sl = 0; sl < 4; sl += 2)
#pragma unroll
                for (int rr = 0; rr < 2; rr++)
                    d[rr] = __builtin_amdgcn_mfma_i32_16x16x64_i8(pair128(aop[s][sl], aop[s][sl + 1]), pair128(bop[rr][sl], bop[rr][sl + 1]), d[rr], 0, 0, 0);
#pragma unroll
            for (int rr = 0; rr < 2; rr++) {
                const int R = 2 * wave + rr;
                // lane group lg = lane / 16 holds rows 4 lg .. 4 lg + 3 = the three digits of head 4 s + lg for token
                // lane % 16: one score per lane.  Row of 16 tokens per (round, head); the head rows of a round rotate
                // with the round number so that the softmax reads (one head, all rounds) spread over the banks.
                const int lg = lane >> 4;
                int lo = (d[rr][1] << 7) + d[rr][2];
                asm volatile("" : "+v"(lo));         // two shift-adds; the compiler makes two shifts and a three-operand add of them
                uint32_t *o = reinterpret_cast<uint32_t *>(kt + R * kRoundBytes + 256 * s + 64 * ((lg + R) & 3)) + (lane & 15);
                if constexpr (SCORE_INT)
                    *o = (uint32_t)((d[rr][0] << 14) + lo);
                else
                    *o = __float_as_uint(fmaf((float)d[rr][0], 16384.f, (float)lo));
            }
        }
    };

    // ---- stage 2: online softmax; wave <-> query head, lane <-> tokens 2*lane, 2*lane+1 ----
    // The usual tile changes neither the running maximum of its head nor the largest exponent of v_scale: then no
    // cross-lane maximum is formed, nothing is rescaled and the V stage is told nothing.  A tile in which some lane
    // sees a larger score or a larger exponent takes the full update instead (about 1 / n of the tiles at position n
    // of a member's sequence).  Both tests are per lane and meet in one branch.
    // ethr_pair: in both halves the largest raw 16-bit pattern whose exponent does not exceed emax (a negative
    // v_scale, which no quantiser produces, compares above it and merely takes the full update every time).
    constexpr int kMant = BF ? 7 : 10;
    uint32_t ethr_pair = 0u;
    int stale_factors = 0;           // this wave published factors != 1 in the previous step: put them back to 1
    auto softmax_stage = [&](auto slot_c, const uint8_t *kt) {
        constexpr int slot = decltype(slot_c)::value;
        const uint32_t *par = reinterpret_cast<const uint32_t *>(ring + slot * Geo::kSlot + Geo::kParOff) + lane;
        const uint32_t vs_raw = par[128];
        float ks0, ks1, kz0, kz1, vs0, vs1, vz0, vz1;
        cvt2(par[0], ks0, ks1); cvt2(par[64], kz0, kz1); cvt2(vs_raw, vs0, vs1); cvt2(par[192], vz0, vz1);
        if (stale_factors) {         // rare; the V stage that read them lies before this step's first barrier
            if (lane == 0) {
#pragma unroll
                for (int gi = 0; gi < GW; gi++)
                    if (wave + 4 * gi < G) st_a[(slot ^ 1) * 8 + wave + 4 * gi] = 1.f;
                resc[slot ^ 1] = 0u;
            }
            stale_factors = 0;
        }
        float sv0[GW], sv1[GW];
        const ushort2v cap = __builtin_elementwise_max(__builtin_bit_cast(ushort2v, vs_raw), __builtin_bit_cast(ushort2v, ethr_pair));
        bool up = __builtin_bit_cast(uint32_t, cap) != ethr_pair;
#pragma unroll
        for (int gi = 0; gi < GW; gi++) {
            const int g = min(wave + 4 * gi, G - 1);
            const int R = lane >> 3;
            const uint2v raw = *reinterpret_cast<const uint2v *>(
                kt + R * kRoundBytes + 256 * (g >> 2) + 64 * (((g & 3) + R) & 3) + 8 * (lane & 7));
            const float D0 = SCORE_INT ? (float)(int)raw[0] : __uint_as_float(raw[0]);
            const float D1 = SCORE_INT ? (float)(int)raw[1] : __uint_as_float(raw[1]);
            // log2-domain scores
            sv0[gi] = fmaf(ks0, c1_r[gi], 0.f) * fmaf(kz0, c2_r[gi], D0);     // (a fused multiply-add takes the 16-bit
            sv1[gi] = fmaf(ks1, c1_r[gi], 0.f) * fmaf(kz1, c2_r[gi], D1);     // operand as it is: no conversion first)
            if (wave + 4 * gi < G) up = up || fmaxf(sv0[gi], sv1[gi]) > m_run[gi];
        }
        const bool full = __builtin_amdgcn_ballot_w64(up) != 0;
        float grow = 1.f;
        if (full) {
            // biased exponents of the v_scale of this lane's two tokens against the largest met so far (every wave
            // sees the same tokens, so all four take the same decision)
            const uint32_t ex = (vs_raw >> kMant) & (BF ? 0x00FF00FFu : 0x001F001Fu);
            const ushort2v mxp = __builtin_elementwise_max(__builtin_bit_cast(ushort2v, ex), __builtin_bit_cast(ushort2v, emax_pair));
            if (__builtin_amdgcn_ballot_w64(__builtin_bit_cast(uint32_t, mxp) != emax_pair) != 0) {
                const uint32_t mine = max(__builtin_bit_cast(uint32_t, mxp) & 0xFFFFu, __builtin_bit_cast(uint32_t, mxp) >> 16);
                uint32_t e = (uint32_t)__builtin_bit_cast(int, wave_max(__builtin_bit_cast(float, mine)));   // small positive ints order like floats
                e = max(e, BF ? 14u : 1u);
                const uint32_t old = emax_pair & 0xFFFFu;
                grow = __builtin_amdgcn_exp2f(-(float)(int)(e - old));       // 0 on the first tile (nothing accumulated yet)
                emax_pair = e | (e << 16);
                wscale = __uint_as_float((uint32_t)(kWExp - (int)e + 127) << 23);
                wscale_inv = __uint_as_float((uint32_t)((int)e - kWExp + 127) << 23);
                const uint32_t thr = ((e + 1u) << kMant) - 1u;
                ethr_pair = thr | (thr << 16);
            }
        }
#pragma unroll
        for (int gi = 0; gi < GW; gi++) {
            const int g = wave + 4 * gi;
            if (g < G) {
                float alpha = 1.f, beta = 1.f;
                if (full) {
                    const float mx = wave_max_fused(fmaxf(sv0[gi], sv1[gi]));
                    const float m_new = fmaxf(m_run[gi], mx);
                    alpha = __builtin_amdgcn_exp2f(m_run[gi] - m_new);    // exp2(-inf) = 0 on the first tile
                    m_run[gi] = m_new;
                    beta = alpha * grow;     // what the weighted sums so far are multiplied by
                }
                const float p0 = __builtin_amdgcn_exp2f(sv0[gi] - m_run[gi]), p1 = __builtin_amdgcn_exp2f(sv1[gi] - m_run[gi]);
                const _Float16 h0 = (_Float16)(p0 * fmaf(vs0, wscale, 0.f)), h1 = (_Float16)(p1 * fmaf(vs1, wscale, 0.f));
                const float f0 = (float)h0, f1 = (float)h1;
                // V-side order: MFMA k of a segment contracts token k of its four rounds
                const int tok0 = 2 * lane;
                _Float16 *pb = pbuf + g * kPStride + (tok0 & 64) + ((tok0 & 15) << 2) + ((tok0 >> 4) & 3);
                pb[0] = h0;
                pb[4] = h1;      // token 2*lane+1: same round, next k
                if (full) {
                    l_part[gi] = l_part[gi] * alpha + (p0 + p1);
                    z_part[gi] = z_part[gi] * beta + (f0 * vz0 + f1 * vz1);
                    if (lane == 0) { st_a[slot * 8 + g] = beta; resc[slot] = 1u; }
                } else {
                    l_part[gi] += p0 + p1;
                    z_part[gi] += f0 * vz0 + f1 * vz1;
                }
                // per-round sums (16 tokens = 8 lanes) of the rounded weights, for the pack-minimum term
                const float r16 = oct_sum_fused(f0 + f1);
                if ((lane & 7) == 0) {
                    const _Float16 hi = (_Float16)r16;
                    p16hi[g * 8 + (lane >> 3)] = hi;
                    p16lo[g * 8 + (lane >> 3)] = (_Float16)(r16 - (float)hi);
                }
            }
        }
        if (full) stale_factors = 1;
    };

    // ---- stage 3: V segment hw; lane = channel, MFMA k contracts token k of the lane's four packs ----
    // A operands of the V-side MFMAs (4 heads x 4 tokens of weights): every block of 4 lanes wants
    // the same values, so only lanes 0..3 of each half-wavefront read them from LDS and the MFMA
    // broadcasts block 0 of each group of 8 blocks (cbsz = 3, abid = 0).  The other lanes' copies
    // are never read; they stay at their initial zero.
    half4v a_w[4][NG4], a_hi[NG4], a_lo[NG4];
#pragma unroll
    for (int i4 = 0; i4 < NG4; i4++) {
        a_hi[i4] = a_lo[i4] = (half4v){0, 0, 0, 0};
#pragma unroll
        for (int pp = 0; pp < 4; pp++) a_w[pp][i4] = (half4v){0, 0, 0, 0};
    }
    const bool a_loader = (lane & 31) < 4;
    // LDS address of this lane's weights (head lane % 4, segment half hw % 2), handed to the compiler as a value it
    // cannot split: it would otherwise keep the per-lane part and add the array's base again at every read
    typedef const __attribute__((address_space(3))) half4v *lds_half4_ptr;
    uint32_t aw_addr = (uint32_t)reinterpret_cast<uintptr_t>(pbuf + (lane & 3) * kPStride + 64 * (hw & 1));
    asm volatile("" : "+v"(aw_addr));
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Wint-to-pointer-cast"      // the host pass sees a 64-bit pointer here; LDS pointers are 32 bits wide
    const lds_half4_ptr aw_ptr = (lds_half4_ptr)aw_addr;
#pragma clang diagnostic pop
    auto v_stage = [&](auto slot_c, const VUnit &vr) {
        constexpr int slot = decltype(slot_c)::value;
        constexpr int TPW = VTPW, NWIN = VNWIN;
        const int seg = hw & 1;
        uint32_t w01[NWIN], w23[NWIN];
        if constexpr (VWIDE) {
#pragma unroll
            for (int e = 0; e < NWIN; e++) { w01[e] = vr.e01[e]; w23[e] = vr.e23[e]; }
        } else {
            pair_windows(vr, w01, w23);
        }
        const uint32_t len01 = vr.len01, len23 = vr.len23;
        const uint32_t m01 = pk_mask16(len01), m23 = pk_mask16(len23);
        // rescale the accumulators only when the softmax of this step said that some head's factor is not 1
        if (__builtin_amdgcn_readfirstlane(resc[slot]) != 0u) {
#pragma unroll
            for (int i4 = 0; i4 < NG4; i4++) {
                const float4v al = *reinterpret_cast<const float4v *>(st_a + slot * 8 + 4 * i4);
                acc[i4] *= al;
            }
        }
        const int gl = lane & 3;
        // pack minima: raw bits are the same fp16-subnormal encoding as the fields
        const half4v mins = __builtin_bit_cast(half4v, make_uint2(__builtin_amdgcn_perm(0u, vr.mins, 0x0C010C00u),
                                                                  __builtin_amdgcn_perm(0u, vr.mins, 0x0C030C02u)));
        if (a_loader) {
#pragma unroll
            for (int i4 = 0; i4 < NG4; i4++) {
                a_hi[i4] = *reinterpret_cast<const half4v *>(p16hi + (4 * i4 + gl) * 8 + 4 * seg);
                a_lo[i4] = *reinterpret_cast<const half4v *>(p16lo + (4 * i4 + gl) * 8 + 4 * seg);
            }
        }
#pragma unroll
        for (int i4 = 0; i4 < NG4; i4++) {
            acc[i4] = __builtin_amdgcn_mfma_f32_4x4x4f16(a_hi[i4], mins, acc[i4], 3, 0, 0);
            acc[i4] = __builtin_amdgcn_mfma_f32_4x4x4f16(a_lo[i4], mins, acc[i4], 3, 0, 0);
        }
#pragma unroll
        for (int q = 0; q < 4; q++) {
            if (a_loader) {
#pragma unroll
                for (int pp = 0; pp < 4; pp++)
#pragma unroll
                    for (int i4 = 0; i4 < NG4; i4++)
                        a_w[pp][i4] = aw_ptr[i4 * kPStride + 4 * q + pp];     // head 4 i4 + lane % 4, tokens 4 (4 q + pp) ..+3 of the segment half
            }
            uint32_t x01 = 0, x23 = 0;
#pragma unroll
            for (int pp = 3; pp >= 0; pp--) {
                constexpr int SH_MAX = TPW - 1;
                const int wi = (4 * q + pp) / TPW, ps = (4 * q + pp) % TPW;      // window and position of token 4q + pp
                if (ps == SH_MAX) { x01 = w01[wi]; x23 = w23[wi]; }             // a window's last token first,
                else { x01 = pk_shr16(x01, len01); x23 = pk_shr16(x23, len23); }  // then one width further per token
                const half4v bop = __builtin_bit_cast(half4v, make_uint2(x01 & m01, x23 & m23));
#pragma unroll
                for (int i4 = 0; i4 < NG4; i4++)
                    acc[i4] = __builtin_amdgcn_mfma_f32_4x4x4f16(a_w[pp][i4], bop, acc[i4], 3, 0, 0);
            }
        }
    };

    // ---- pipeline ----
    KUnit k_a, k_b;               // the units of the tile a step works on and of the one it parses alternate between
    VUnit v_a, v_b;               // the two sets; the loop below is written out twice so that nothing is copied
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");     // tile 0 (issued before the prologue's arithmetic)
    PKV_LDS_BARRIER();                                    // ... and every wave has its q operands out of slot 1
    dma_issue(IntC<1>{}, t1, i1);
    parse(IntC<0>{}, i0, k_a, v_a);
    // the head's counter: tiles 5 nsplit + [old value, old value + size) belong to whoever added `size`
    const int n_dyn = n_tiles - 5 * p.nsplit;                   // tiles that are handed out by counter
    uint32_t fetched = 0u;        // wave 0, lane 0: old counter value of the request in flight
    int pend_n = 0, cur_base = 0, cur_left = 0;                 // size of that request; the batch being drawn on
    auto batch_of = [&](int handed) -> int {
        int n = (n_dyn - handed) >> p.batch_shift;
        n = max(n, 1);
        PKV_SCALAR(n);
        return min(n, 4);
    };
    // (the counter's index goes through a vector register the compiler cannot see into: with an address it knows to be
    // the same in every lane it rewrites the atomic as a reduction over the active lanes whose epilogue waits for the
    // answer on the spot -- and with it for the copies just issued.  And it does so where it is used: an address
    // formed once before the loop is a register pair that lives through it, and the 3-bit kernels spilled it, which
    // put a scratch reload and its wait for every outstanding copy in here)
    auto request = [&](int n) {
        if (wave == 0 && lane == 0) {
            uint32_t ctr_idx = (uint32_t)bh;
            asm volatile("" : "+v"(ctr_idx));
            fetched = __hip_atomic_fetch_add(p.counters + ctr_idx, (uint32_t)n, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        pend_n = n;
    };
    if (p.dynamic) request(batch_of(0));
    PKV_LDS_BARRIER();

    // Step s works on position s of the sequence (tile t_cur); t1, t2, t3 = the tiles of positions s+1 .. s+3, i1, i2 =
    // block_info of t1, t2.  Position s+4 becomes known in the middle of the step: from the batch being drawn on, or,
    // when that is used up, from the request wave 0 sent at least a step ago -- its answer has arrived with the
    // copies the wave waits for before barrier 1 and is handed to the other waves through LDS.
    int s = 0;
    auto step = [&](auto slot_c, KUnit &kcur, VUnit &vcur, KUnit &knext, VUnit &vnext) {
        constexpr int slot = decltype(slot_c)::value;
        uint8_t *kt = ring + slot * Geo::kSlot;
        const RawInfo i3 = load_info(t3);
        const bool take = p.dynamic && s > 0 && cur_left == 0;       // this step starts on the next batch
        __builtin_amdgcn_s_setprio(Prio::K);
        if (!(PKV_ATTN_PROBE & 2)) k_stage(kcur, kt);
        __builtin_amdgcn_s_setprio(0);
        if (!(PKV_ATTN_PROBE & 32)) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");     // this wave's part of tile t1 has landed
        if (take && wave == 0 && lane == 0) tau_lds[slot] = (int)fetched;
        PKV_LDS_BARRIER();                                    // publishes the scores, tile t1 and the new batch
        int t4;
        if (!p.dynamic) {
            t4 = t3 + 1;
        } else if (s == 0) {
            t4 = first_tiles(4);
        } else {
            if (take) { cur_base = __builtin_amdgcn_readfirstlane(tau_lds[slot]); cur_left = pend_n; }
            t4 = 5 * p.nsplit + cur_base;
            cur_base++;
            cur_left--;
        }
        __builtin_amdgcn_s_setprio(Prio::S);
        if (!(PKV_ATTN_PROBE & 16)) parse(IntC<slot ^ 1>{}, i1, knext, vnext); else { knext = kcur; vnext = vcur; }
        if (!(PKV_ATTN_PROBE & 4)) softmax_stage(slot_c, kt);
        // the pack words of tile t1 are put together here, not wherever the compiler finds room before their first
        // use: it kept the three raw dwords of every word alive through the V stage (24 registers instead of 16)
        if constexpr (!KWIDE) {
#pragma unroll
            for (int i = 0; i < 4; i++) asm volatile("" : "+v"(knext.word[i]));
        }
        if constexpr (!VWIDE) {
#pragma unroll
            for (int i = 0; i < 4; i++) asm volatile("" : "+v"(vnext.word[i]));
        }
        __builtin_amdgcn_s_setprio(0);
        PKV_LDS_BARRIER();                                    // publishes the weights; slot s is free, tile t1 is parsed
        __builtin_amdgcn_s_setprio(Prio::D);
        if (!(PKV_ATTN_PROBE & 1)) dma_issue(slot_c, t2, i2);
        if (take) request(batch_of(cur_base));                // collected at the wait above, a step or more from now
        __builtin_amdgcn_s_setprio(Prio::V);
        if (!(PKV_ATTN_PROBE & 8)) v_stage(slot_c, vcur);
        __builtin_amdgcn_s_setprio(0);
        t_cur = t1; t1 = t2; t2 = t3; t3 = t4;
        i1 = i2; i2 = pack_info(i3);
        s++;
    };
    while ((uint32_t)t_cur < (uint32_t)tile_end) {
        step(IntC<0>{}, k_a, v_a, k_b, v_b);
        if (!((uint32_t)t_cur < (uint32_t)tile_end)) break;
        step(IntC<1>{}, k_b, v_b, k_a, v_a);
    }
    // drain: the copy issued in the last step must land before the workgroup's LDS is released
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    // the last member of the head to get here (every request of the others has been answered) zeroes the head's two
    // counters for the next launch
    if (p.dynamic && tid == 0) {
        uint32_t *done = p.counters + n_heads + bh;
        if (atomicAdd(done, 1u) + 1u == (uint32_t)p.nsplit) {
            atomicExch(p.counters + bh, 0u);
            atomicExch(done, 0u);
        }
    }

    // ---- epilogue ----
#pragma unroll
    for (int gi = 0; gi < GW; gi++) {
        const int g = wave + 4 * gi;
        if (g < G) {
            const float l = wave_sum(l_part[gi]), z = wave_sum(z_part[gi]);
            if (lane == 0) { st_m[g] = m_run[gi] * 0.693147180559945309f; st_l[g] = l; st_z[g] = z; }   // natural-log domain for the merge
        }
    }
    PKV_LDS_BARRIER();
#pragma unroll
    for (int i4 = 0; i4 < NG4; i4++)
#pragma unroll
        for (int m = 0; m < 4; m++) acc[i4][m] += __shfl_xor(acc[i4][m], 32, 64);
    if ((lane >> 5) == 0) {
        const int j = hw >> 2, w = (hw & 3) >> 1;
        const int ch = 64 * j + 32 * w + t;
#pragma unroll
        for (int g = 0; g < G; g++) {
            if (g >= p.Gq) break;
            const size_t hq = (size_t)b * p.Hq + (size_t)h * p.Gq + g;
            // fields were consumed as fp16 subnormals (delta * 2^-24)
            const float val = (acc[g >> 2][g & 3] * 16777216.f + st_z[g]) * wscale_inv;
            if (p.direct_out) {                // one split and no window: this is the result, no merge launch follows
                p.out[hq * kHeadDim + ch] = a_st16(val / st_l[g], p.dtype);
                continue;
            }
            float *dst = p.part + (hq * p.nparts + split) * kPartStride;
            dst[2 + ch] = val;
            if (ch == 0) { dst[0] = st_m[g]; dst[1] = st_l[g]; }
        }
    }
    // this split's share of the 16-bit tail window, as a partial of its own (the slots are free: every
    // wave drained its copies before the barrier above)
    if (p.win_piece > 0) {
        const int t0 = split * p.win_piece, t1 = min(t0 + p.win_piece, p.T_w);
        window_body<G>(p, smem, h, b, t0, t1, p.nsplit + split);
    }
}

}  // namespace pkv
