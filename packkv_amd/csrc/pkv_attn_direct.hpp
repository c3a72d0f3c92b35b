// Fused decompress-attention decode, "direct" kernel: the compressed stream is never staged in
// LDS.  Every lane fetches its own metadata words and pack words straight into registers with
// range-checked buffer loads, two tiles (metadata) and one tile (pack words) ahead of their use,
// so the parse of a tile costs no LDS round trip and no wait.  Included by pkv_attn.hip after the
// shared helpers (AttnParams, wave_max, row16_sum, pack_windows, pk_shr16 ...).
//
// Tile = 128 tokens of one (sequence, KV head) = 2 K blocks (64 x 128) + 2 V blocks (128 x 64).
// Per tile and half-wavefront hw (0..7):  K unit = round hw%4 of K block hw/4 (16 tokens x 128
// channels, lane t = channels 4t..4t+3);  V unit = segment hw%4 of V block hw/4 (64 tokens x 32
// channels, lane t = channel).  Where a unit starts inside the stream comes from a small LDS
// table built per chunk of 16 tiles from block_info and the blocks' 8-byte headers.
#pragma once

namespace pkv {

constexpr int kChunk = 16;     // tiles per table chunk
constexpr int kRing = 32;      // table ring: two chunks

// One unit's state in registers.
struct UnitRegs {
    uint64_t word[4];
    uint32_t lens;     // the four bit widths, one per byte
    uint32_t mins;     // the four minima, one per byte
};

template <int W>
__device__ __forceinline__ void meta_fields(uint32_t minsw, uint32_t lensw, uint32_t len[4], uint32_t &lens_b,
                                            uint32_t &mins_b) {
    constexpr int LB = len_field_bits(W);
#pragma unroll
    for (int i = 0; i < 4; i++) len[i] = __builtin_amdgcn_ubfe(lensw, i * LB, LB);
    lens_b = len[0] | (len[1] << 8) | (len[2] << 16) | (len[3] << 24);
    if (W == 4) {   // four nibbles -> four bytes
        uint32_t y = (minsw | (minsw << 8)) & 0x00FF00FFu;
        mins_b = (y | (y << 4)) & 0x0F0F0F0Fu;
    } else {
        mins_b = __builtin_amdgcn_ubfe(minsw, 0, W) | (__builtin_amdgcn_ubfe(minsw, W, W) << 8) |
                 (__builtin_amdgcn_ubfe(minsw, 2 * W, W) << 16) | (__builtin_amdgcn_ubfe(minsw, 3 * W, W) << 24);
    }
}

// Windows of a unit held as UnitRegs (see pack_windows): win01[q] = tokens 4q..4q+3 of packs 0, 1.
__device__ __forceinline__ void unit_windows(const UnitRegs &u, uint32_t win01[4], uint32_t win23[4]) {
    uint32_t hlf[4][2], len4[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const uint32_t len = (u.lens >> (8 * i)) & 0xFFu;
        len4[i] = 4u * len;
        hlf[i][0] = (uint32_t)(u.word[i] >> (8u * len));   // tokens 0..7
        hlf[i][1] = (uint32_t)u.word[i];                   // tokens 8..15
    }
#pragma unroll
    for (int q = 0; q < 4; q++) {
        uint32_t qd[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t src = hlf[i][q >> 1];
            qd[i] = (q & 1) ? src : (src >> len4[i]);
        }
        win01[q] = __builtin_amdgcn_perm(qd[1], qd[0], 0x05040100u);
        win23[q] = __builtin_amdgcn_perm(qd[3], qd[2], 0x05040100u);
    }
}

typedef uint32_t uint2v __attribute__((ext_vector_type(2)));

// Cross-lane float reductions with the lane permutation fused into the arithmetic instruction
// (one VALU instruction per step).  Lanes whose row is masked off keep their value.  The leading
// s_nop covers the two wait states a DPP read needs after the VALU write of its source.
#define PKV_DPP_STEP(op, x, ctrl) asm("s_nop 1\n\t" op " %0, %0, %0 " ctrl : "+v"(x))

__device__ __forceinline__ float wave_max_fused(float x) {
    PKV_DPP_STEP("v_max_f32_dpp", x, "quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf");
    PKV_DPP_STEP("v_max_f32_dpp", x, "quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf");
    PKV_DPP_STEP("v_max_f32_dpp", x, "row_half_mirror row_mask:0xf bank_mask:0xf");
    PKV_DPP_STEP("v_max_f32_dpp", x, "row_mirror row_mask:0xf bank_mask:0xf");
    PKV_DPP_STEP("v_max_f32_dpp", x, "row_bcast:15 row_mask:0xa bank_mask:0xf");
    PKV_DPP_STEP("v_max_f32_dpp", x, "row_bcast:31 row_mask:0xc bank_mask:0xf");
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), 63));
}

__device__ __forceinline__ float oct_sum_fused(float x) {   // every lane gets the sum over its 8-lane group
    PKV_DPP_STEP("v_add_f32_dpp", x, "quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf");
    PKV_DPP_STEP("v_add_f32_dpp", x, "quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf");
    PKV_DPP_STEP("v_add_f32_dpp", x, "row_half_mirror row_mask:0xf bank_mask:0xf");
    return x;
}

// Payload offsets (in 2-byte units) of a lane's four packs from their widths `lens_b` (one per
// byte): a single packed scan over the 32 lanes of the half-wavefront.  A slot's widths sum to at
// most 32 * 4 = 128, so the four running sums never carry into each other.
__device__ __forceinline__ void pack_offsets8(uint32_t lens_b, uint32_t off2[4]) {
    const uint32_t incl = half_incl_scan(lens_b);
    const uint32_t excl = incl - lens_b;
    // the four slot totals of this lane's half = the running sums of its lane 31: one cross-lane read on the LDS
    // crossbar (bit-mask swizzle within 32 lanes: lane | 31), no memory access, no scalar round trip, and the slot
    // bases are byte-select additions
    const uint32_t tot = (uint32_t)__builtin_amdgcn_ds_swizzle((int)incl, 0x03E0);
    const uint32_t a0 = tot & 0xFFu, a01 = a0 + ((tot >> 8) & 0xFFu), a012 = a01 + ((tot >> 16) & 0xFFu);
    off2[0] = excl & 0xFFu;
    off2[1] = ((excl >> 8) & 0xFFu) + a0;
    off2[2] = ((excl >> 16) & 0xFFu) + a01;
    off2[3] = (excl >> 24) + a012;
}

template <int G, int KW, int VW, bool BF>
__global__ void __launch_bounds__(256) attn_direct_kernel(const AttnParams p) {
    constexpr int ROWS = 3 * G;
    constexpr int NSETS = (ROWS + 15) / 16;
    constexpr int NG4 = (G + 3) / 4;
    constexpr int GP = NG4 * 4;
    constexpr int GW = (G + 3) / 4;
    constexpr int KLB = len_field_bits(KW), VLB = len_field_bits(VW);
    constexpr uint32_t K_META = KW * 16 + KLB * 16, V_META = VW * 16 + VLB * 16;   // mins + lens bytes of a unit
    constexpr int kRoundBytes = 16 * kKtStride;
    static_assert(16 * NSETS * 16 * 4 + 64 <= kRoundBytes, "score rows must fit the K-tile rows they reuse");

    extern __shared__ __align__(16) uint8_t lds[];
    uint8_t *kt = lds;                                            // [8 rounds][16 tok][136] int8 (+ scores)
    uint8_t *aq = lds;                                            // q digits, prologue only
    uint32_t *tab = reinterpret_cast<uint32_t *>(kt + 8 * kRoundBytes);       // [kRing][4 blocks][4 units]
    _Float16 *pbuf = reinterpret_cast<_Float16 *>(tab + kRing * 16);          // [GP][128]
    _Float16 *p16hi = pbuf + GP * kTile;                                      // [GP][8]
    _Float16 *p16lo = p16hi + GP * 8;
    float *st_m = reinterpret_cast<float *>(p16lo + GP * 8);                  // 8 floats each
    float *st_l = st_m + 8, *st_a = st_l + 8, *st_z = st_a + 8, *qsum = st_z + 8, *qs = qsum + 8;

    const int split = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int t = tid & 31, hw = tid >> 5;
    const int bh = b * p.Hkv + h;
    const int n_hid_k = p.B * p.Hkv, n_hid_v = 2 * p.B * p.Hkv;

    const __amdgpu_buffer_rsrc_t k_rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(p.k_stream), 0, (int)p.k_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t v_rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(p.v_stream), 0, (int)p.v_bytes, 0x00020000);

    const int par_bytes = p.B * p.par_stride * 2, info_bytes = (p.T_c / 64) * p.B * p.Hkv * 8;
    const __amdgpu_buffer_rsrc_t ks_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t *>(p.k_scale), 0, par_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t kz_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t *>(p.k_zero), 0, par_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t vs_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t *>(p.v_scale), 0, par_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t vz_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t *>(p.v_zero), 0, par_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t ki_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint32_t *>(p.k_info), 0, info_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t vi_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint32_t *>(p.v_info), 0, info_bytes, 0x00020000);

    // ---- prologue: split q into digits (through LDS, aliased onto the K tile) ----
    for (int i = tid; i < NSETS * 4 * 16 * 32 / 4; i += 256) reinterpret_cast<uint32_t *>(aq)[i] = 0u;
    for (int i = tid; i < GP * kTile / 2; i += 256) reinterpret_cast<uint32_t *>(pbuf)[i] = 0u;
    for (int i = tid; i < GP * 8; i += 256) reinterpret_cast<uint32_t *>(p16hi)[i] = 0u;   // hi and lo
    if (tid < 8) { st_m[tid] = -INFINITY; st_l[tid] = 0.f; st_z[tid] = 0.f; st_a[tid] = 0.f; }
    __syncthreads();
    for (int g = wave; g < G; g += 4) {
        if (g >= p.Gq) {                       // an idle head slot: a query of zeros
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
                const int m = pp * G + g;
                aq[(((m >> 4) * 4 + (d >> 5)) * 16 + (m & 15)) * 32 + (d & 31)] = (uint8_t)(int8_t)dig[pp];
            }
        }
    }
    __syncthreads();
    long aop[NSETS][4];
#pragma unroll
    for (int s = 0; s < NSETS; s++)
#pragma unroll
        for (int sl = 0; sl < 4; sl++)
            aop[s][sl] = *reinterpret_cast<const long *>(aq + ((s * 4 + sl) * 16 + (lane & 15)) * 32 + 8 * (lane >> 4));
    float qs_r[GW], qsum_r[GW];
#pragma unroll
    for (int gi = 0; gi < GW; gi++) {
        const int g = min(wave + 4 * gi, G - 1);
        qs_r[gi] = qs[g];
        qsum_r[gi] = qsum[g];
    }

    const int n_tiles = p.T_c / kTile;
    const int tile0 = split * p.tiles_per_split;
    const int tile1 = min(n_tiles, tile0 + p.tiles_per_split);
    const int ntl = tile1 - tile0;                 // tiles of this split (>= 1)

    // ---- unit-start table: ring of kRing tiles x 4 blocks x 4 units (byte offsets into the streams) ----
    // Thread (tile i = tid >> 2, block j = tid & 3) looks a block up in block_info, reads the block's
    // 8-byte header (cumulative unit sizes) and stores where the four units start.  The first
    // kChunk tiles are filled here, blocking; the main loop then adds one tile per iteration,
    // kChunk tiles ahead, with the two dependent loads spread over three iterations.
    auto block_index = [&](int tau, int j) -> uint32_t {
        return j < 2 ? (uint32_t)((2 * tau + j) * n_hid_k + bh) : (uint32_t)(tau * n_hid_v + 2 * bh + (j - 2));
    };
    const int f_j = tid & 3;
    auto fill_info = [&](int rel) -> uint32_t {              // byte offset of block f_j of tile rel (clamped)
        const uint32_t bi = block_index(tile0 + min(rel, ntl - 1), f_j);
        // the two tables have the same number of entries, so either index is in range for both
        const uint32_t ko = __builtin_amdgcn_raw_buffer_load_b32(ki_rsrc, 8u * bi, 0, 0);
        const uint32_t vo = __builtin_amdgcn_raw_buffer_load_b32(vi_rsrc, 8u * bi, 0, 0);
        return f_j < 2 ? ko : vo;
    };
    auto fill_header = [&](uint32_t off) -> uint2v {         // the block's four cumulative u16 sizes
        const uint2v hk = __builtin_amdgcn_raw_buffer_load_b64(k_rsrc, off, 0, 0);
        const uint2v hv = __builtin_amdgcn_raw_buffer_load_b64(v_rsrc, off, 0, 0);
        return f_j < 2 ? hk : hv;
    };
    auto fill_store = [&](int rel, uint32_t off, uint2v hdr, bool mine) {
        if (mine) {
            uint4 st;
            st.x = off + 8u;
            st.y = off + 8u + (hdr[0] & 0xFFFFu);
            st.z = off + 8u + (hdr[0] >> 16);
            st.w = off + 8u + (hdr[1] & 0xFFFFu);
            *reinterpret_cast<uint4 *>(tab + ((rel & (kRing - 1)) * 4 + f_j) * 4) = st;
        }
    };
    uint32_t f0_off, f1_off;      // refill pipeline: info of tile r+kChunk-1, (info, header) of tile r+kChunk-2
    uint2v f1_hdr;
    {
        const int i = (tid >> 2) & (kChunk - 1);
        const uint32_t o = fill_info(i);
        const uint2v hd = fill_header(o);
        fill_store(i, o, hd, tid < 4 * kChunk);
        f1_off = fill_info(kChunk - 2);
        f0_off = fill_info(kChunk - 1);
        f1_hdr = fill_header(f1_off);
    }
    __syncthreads();

    // ---- per-lane constants of the metadata fetch ----
    const int kj = hw >> 2, ku = hw & 3;                        // block and unit of this half-wave
    const uint32_t k_mins_off = (uint32_t)(t * 4 * KW) >> 3, k_mins_sh = (uint32_t)(t * 4 * KW) & 7u;
    const uint32_t k_lens_off = KW * 16 + ((uint32_t)(t * 4 * KLB) >> 3), k_lens_sh = (uint32_t)(t * 4 * KLB) & 7u;
    const uint32_t v_mins_off = (uint32_t)(t * 4 * VW) >> 3, v_mins_sh = (uint32_t)(t * 4 * VW) & 7u;
    const uint32_t v_lens_off = VW * 16 + ((uint32_t)(t * 4 * VLB) >> 3), v_lens_sh = (uint32_t)(t * 4 * VLB) & 7u;

    struct Meta { uint32_t k_start, v_start, k_mins, k_lens, v_mins, v_lens; };
    auto tab_read = [&](int rel, uint32_t &k_start, uint32_t &v_start) {     // rel may run past the split: clamped
        const int r = min(rel, ntl - 1) & (kRing - 1);
        k_start = tab[(r * 4 + kj) * 4 + ku];
        v_start = tab[(r * 4 + 2 + kj) * 4 + ku];
    };
    auto meta_issue = [&](uint32_t k_start, uint32_t v_start, Meta &m) {
        m.k_start = k_start;
        m.v_start = v_start;
        m.k_mins = __builtin_amdgcn_raw_buffer_load_b32(k_rsrc, m.k_start + k_mins_off, 0, 0);
        m.k_lens = __builtin_amdgcn_raw_buffer_load_b32(k_rsrc, m.k_start + k_lens_off, 0, 0);
        m.v_mins = __builtin_amdgcn_raw_buffer_load_b32(v_rsrc, m.v_start + v_mins_off, 0, 0);
        m.v_lens = __builtin_amdgcn_raw_buffer_load_b32(v_rsrc, m.v_start + v_lens_off, 0, 0);
    };
    auto words_issue = [&](const Meta &m, UnitRegs &ku_r, UnitRegs &vu_r) {
        uint32_t klen[4], vlen[4], koff[4], voff[4];
        meta_fields<KW>((m.k_mins >> k_mins_sh) & ((1u << (4 * KW)) - 1u), (m.k_lens >> k_lens_sh) & ((1u << (4 * KLB)) - 1u),
                        klen, ku_r.lens, ku_r.mins);
        meta_fields<VW>((m.v_mins >> v_mins_sh) & ((1u << (4 * VW)) - 1u), (m.v_lens >> v_lens_sh) & ((1u << (4 * VLB)) - 1u),
                        vlen, vu_r.lens, vu_r.mins);
        pack_offsets8(ku_r.lens, koff);
        pack_offsets8(vu_r.lens, voff);
        const uint32_t kpay0 = m.k_start + K_META, vpay0 = m.v_start + V_META;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint2v kwd = __builtin_amdgcn_raw_buffer_load_b64(k_rsrc, kpay0 + 2u * koff[i], 0, 0);
            const uint2v vwd = __builtin_amdgcn_raw_buffer_load_b64(v_rsrc, vpay0 + 2u * voff[i], 0, 0);
            ku_r.word[i] = ((uint64_t)kwd[1] << 32) | kwd[0];
            vu_r.word[i] = ((uint64_t)vwd[1] << 32) | vwd[0];
        }
    };
    // quantizer parameters of the two tokens (2*lane, 2*lane+1) this lane handles in the softmax stage
    struct QPar { uint32_t ks, kz, vs, vz; };
    auto qpar_issue = [&](int rel, QPar &q) {
        const int tile_off = (b * p.par_stride + (tile0 + min(rel, ntl - 1)) * kTile) * 2;     // bytes, wave-uniform
        q.ks = __builtin_amdgcn_raw_buffer_load_b32(ks_rsrc, 4 * lane, tile_off, 0);
        q.kz = __builtin_amdgcn_raw_buffer_load_b32(kz_rsrc, 4 * lane, tile_off, 0);
        q.vs = __builtin_amdgcn_raw_buffer_load_b32(vs_rsrc, 4 * lane, tile_off, 0);
        q.vz = __builtin_amdgcn_raw_buffer_load_b32(vz_rsrc, 4 * lane, tile_off, 0);
    };
    auto cvt2 = [&](uint32_t w, float &lo, float &hi) {
        if (!BF) {
            lo = __half2float(__ushort_as_half((unsigned short)(w & 0xFFFFu)));
            hi = __half2float(__ushort_as_half((unsigned short)(w >> 16)));
        } else {
            lo = __uint_as_float(w << 16);
            hi = __uint_as_float(w & 0xFFFF0000u);
        }
    };

    float4v acc[NG4];
#pragma unroll
    for (int i = 0; i < NG4; i++) acc[i] = (float4v){0.f, 0.f, 0.f, 0.f};
    float m_run[GW], l_part[GW], z_part[GW];
#pragma unroll
    for (int i = 0; i < GW; i++) { m_run[i] = -INFINITY; l_part[i] = 0.f; z_part[i] = 0.f; }
    // The softmax weights reach the matrix cores as fp16(p * v_scale * wscale), wscale = 2^(kWExp - emax), emax = the
    // largest biased exponent of v_scale among the tokens met so far: weights stay below 2^11 and a round's 16-weight
    // sum below 2^15 whatever the magnitude of V; when emax grows the running sums are rescaled (factor `grow`).
    constexpr int kWExp = BF ? 137 : 25;
    uint32_t emax = 0u;
    float wscale = 0.f, wscale_inv = 0.f;

    // ---- one tile: consume (K unit, V unit, parameters) that are already in registers ----
    auto process = [&](const UnitRegs &ku_r, const UnitRegs &vu_r, const QPar &qp) {
        // K round hw -> int8 tile rows [hw*16, hw*16+16)
        {
            uint32_t w01[4], w23[4];
            unit_windows(ku_r, w01, w23);
            const uint32_t len01 = (ku_r.lens & 0xFFu) | ((ku_r.lens & 0xFF00u) << 8);
            const uint32_t len23 = ((ku_r.lens >> 16) & 0xFFu) | ((ku_r.lens >> 8) & 0xFF0000u);
            const uint32_t l0 = ku_r.lens & 0xFFu, l1 = (ku_r.lens >> 8) & 0xFFu, l2 = (ku_r.lens >> 16) & 0xFFu,
                           l3 = ku_r.lens >> 24;
            const uint32_t mq = ((1u << l0) - 1u) | (((1u << l1) - 1u) << 8) | (((1u << l2) - 1u) << 16) |
                                (((1u << l3) - 1u) << 24);
            uint32_t *dst = reinterpret_cast<uint32_t *>(kt) + (hw * 16) * kKtDw + t;
#pragma unroll
            for (int q = 0; q < 4; q++) {
#pragma unroll
                for (int pp = 0; pp < 4; pp++) {
                    const uint32_t x01 = pp == 3 ? w01[q] : pk_shr16(w01[q], len01 * (uint32_t)(3 - pp));
                    const uint32_t x23 = pp == 3 ? w23[q] : pk_shr16(w23[q], len23 * (uint32_t)(3 - pp));
                    dst[(q * 4 + pp) * kKtDw] = (__builtin_amdgcn_perm(x23, x01, 0x06040200u) & mq) + ku_r.mins;
                }
            }
        }
        // the rounds a wavefront multiplies are the two its own halves just wrote: LDS executes a
        // wavefront's accesses in order, so only the compiler must be kept from reordering
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int rr = 0; rr < 2; rr++) {
            const int R = 2 * wave + rr;
            const uint8_t *row = kt + (R * 16 + (lane & 15)) * kKtStride + 8 * (lane >> 4);
            long bop[4];
#pragma unroll
            for (int sl = 0; sl < 4; sl++) bop[sl] = *reinterpret_cast<const long *>(row + 32 * sl);
#pragma unroll
            for (int s = 0; s < NSETS; s++) {
                int4v d = {0, 0, 0, 0};
#pragma unroll
                for (int sl = 0; sl < 4; sl++) d = __builtin_amdgcn_mfma_i32_16x16x32_i8(aop[s][sl], bop[sl], d, 0, 0, 0);
                // row-major [m][token]; odd rounds sit 16 banks further so the softmax reads spread over all banks
                int32_t *o = reinterpret_cast<int32_t *>(kt + R * kRoundBytes + (R & 1) * 64) +
                             (s * 16 + 4 * (lane >> 4)) * 16 + (lane & 15);
#pragma unroll
                for (int jj = 0; jj < 4; jj++) o[jj * 16] = d[jj];
            }
        }
        __syncthreads();

        // online softmax: wave <-> query head, lane <-> tokens 2*lane, 2*lane+1 (round lane / 8)
        float ks0, ks1, kz0, kz1, vs0, vs1, vz0, vz1;
        cvt2(qp.ks, ks0, ks1); cvt2(qp.kz, kz0, kz1); cvt2(qp.vs, vs0, vs1); cvt2(qp.vz, vz0, vz1);
        float grow = 1.f;
        {   // every wavefront sees the same 128 tokens, so all four take the same decision
            const uint32_t ex = (qp.vs >> (BF ? 7 : 10)) & (BF ? 0x00FF00FFu : 0x001F001Fu);
            const uint32_t mine = max(ex & 0xFFFFu, ex >> 16);
            uint32_t e = (uint32_t)__builtin_bit_cast(int, wave_max_fused(__builtin_bit_cast(float, mine)));   // small positive ints order like floats
            e = max(e, BF ? 14u : 1u);
            if (e > emax) {
                grow = emax ? __builtin_amdgcn_exp2f(-(float)(int)(e - emax)) : 1.f;    // nothing accumulated before the first tile
                emax = e;
                wscale = __uint_as_float((uint32_t)(kWExp - (int)e + 127) << 23);
                wscale_inv = __uint_as_float((uint32_t)((int)e - kWExp + 127) << 23);
            }
        }
#pragma unroll
        for (int gi = 0; gi < GW; gi++) {
            const int g = wave + 4 * gi;
            if (g < G) {
                const int32_t *r =
                    reinterpret_cast<const int32_t *>(kt + (lane >> 3) * kRoundBytes + ((lane >> 3) & 1) * 64) + 2 * (lane & 7);
                float sv[2];
#pragma unroll
                for (int e = 0; e < 2; e++) {
                    const float d0 = (float)r[g * 16 + e], d1 = (float)r[(G + g) * 16 + e], d2 = (float)r[(2 * G + g) * 16 + e];
                    const float dot = qs_r[gi] * (d0 * 16384.f + d1 * 128.f + d2);
                    sv[e] = p.sm_scale * (e ? ks1 : ks0) * (dot + (e ? kz1 : kz0) * qsum_r[gi]);
                }
                const float mx = wave_max_fused(fmaxf(sv[0], sv[1]));
                const float m_new = fmaxf(m_run[gi], mx);
                const float alpha = __expf(m_run[gi] - m_new);    // exp(-inf) = 0 on the first tile
                m_run[gi] = m_new;
                const float p0 = __expf(sv[0] - m_new), p1 = __expf(sv[1] - m_new);
                const _Float16 h0 = (_Float16)(p0 * vs0 * wscale), h1 = (_Float16)(p1 * vs1 * wscale);
                const float f0 = (float)h0, f1 = (float)h1;
                // V-side order: MFMA k of a segment contracts token k of its four rounds
                const int tok0 = 2 * lane;
                _Float16 *pb = pbuf + g * kTile + (tok0 & 64) + ((tok0 & 15) << 2) + ((tok0 >> 4) & 3);
                pb[0] = h0;
                pb[4] = h1;      // token 2*lane+1: same round, next k
                l_part[gi] = l_part[gi] * alpha + (p0 + p1);
                z_part[gi] = z_part[gi] * (alpha * grow) + (f0 * vz0 + f1 * vz1);
                // per-round sums (16 tokens = 8 lanes) of the rounded weights, for the pack-minimum term
                const float r16 = oct_sum_fused(f0 + f1);
                if ((lane & 7) == 0) {
                    const _Float16 hi = (_Float16)r16;
                    p16hi[g * 8 + (lane >> 3)] = hi;
                    p16lo[g * 8 + (lane >> 3)] = (_Float16)(r16 - (float)hi);
                }
                if (lane == 0) st_a[g] = alpha * grow;
            }
        }
        __syncthreads();

        // V segment hw: lane = channel; MFMA k contracts token k of the lane's four packs
        {
            const int seg = hw & 1;
            uint32_t w01[4], w23[4];
            unit_windows(vu_r, w01, w23);
            const uint32_t len01 = (vu_r.lens & 0xFFu) | ((vu_r.lens & 0xFF00u) << 8);
            const uint32_t len23 = ((vu_r.lens >> 16) & 0xFFu) | ((vu_r.lens >> 8) & 0xFF0000u);
            const uint32_t m01 = ((1u << (vu_r.lens & 7u)) - 1u) | (((1u << ((vu_r.lens >> 8) & 7u)) - 1u) << 16);
            const uint32_t m23 = ((1u << ((vu_r.lens >> 16) & 7u)) - 1u) | (((1u << ((vu_r.lens >> 24) & 7u)) - 1u) << 16);
#pragma unroll
            for (int i4 = 0; i4 < NG4; i4++) {
                const float4v al = *reinterpret_cast<const float4v *>(st_a + 4 * i4);
                acc[i4] *= al;
            }
            const int gl = lane & 3;
            // pack minima: raw bits are the same fp16-subnormal encoding as the fields
            const half4v mins = __builtin_bit_cast(
                half4v, make_uint2((vu_r.mins & 0xFFu) | ((vu_r.mins & 0xFF00u) << 8),
                                   ((vu_r.mins >> 16) & 0xFFu) | ((vu_r.mins >> 8) & 0xFF0000u)));
#pragma unroll
            for (int i4 = 0; i4 < NG4; i4++) {
                const half4v ahi = *reinterpret_cast<const half4v *>(p16hi + (4 * i4 + gl) * 8 + 4 * seg);
                const half4v alo = *reinterpret_cast<const half4v *>(p16lo + (4 * i4 + gl) * 8 + 4 * seg);
                acc[i4] = __builtin_amdgcn_mfma_f32_4x4x4f16(ahi, mins, acc[i4], 0, 0, 0);
                acc[i4] = __builtin_amdgcn_mfma_f32_4x4x4f16(alo, mins, acc[i4], 0, 0, 0);
            }
#pragma unroll
            for (int q = 0; q < 4; q++) {
#pragma unroll
                for (int pp = 0; pp < 4; pp++) {
                    const uint32_t x01 = pp == 3 ? w01[q] : pk_shr16(w01[q], len01 * (uint32_t)(3 - pp));
                    const uint32_t x23 = pp == 3 ? w23[q] : pk_shr16(w23[q], len23 * (uint32_t)(3 - pp));
                    const half4v bop = __builtin_bit_cast(half4v, make_uint2(x01 & m01, x23 & m23));
#pragma unroll
                    for (int i4 = 0; i4 < NG4; i4++) {
                        const half4v aopv = *reinterpret_cast<const half4v *>(
                            pbuf + (4 * i4 + gl) * kTile + 64 * seg + 4 * (4 * q + pp));
                        acc[i4] = __builtin_amdgcn_mfma_f32_4x4x4f16(aopv, bop, acc[i4], 0, 0, 0);
                    }
                }
            }
        }
    };

    // ---- software pipeline: pack words one tile ahead, metadata two tiles ahead ----
    UnitRegs kA, vA, kB, vB;
    QPar qA, qB;
    Meta mA, mB;
    {
        uint32_t ks0, vs0, ks1, vs1;
        tab_read(0, ks0, vs0);
        tab_read(1, ks1, vs1);
        meta_issue(ks0, vs0, mA);
        meta_issue(ks1, vs1, mB);
    }
    words_issue(mA, kA, vA);      // tile 0 (waits for its metadata here, once)
    qpar_issue(0, qA);
    // step(rel): tile rel is in (kc, vc, qc), metadata of rel+1 in mnext.  Issue the pack words of
    // rel+1 into (kn, vn, qn) and the metadata of rel+2 into mfree, advance the table refill by one
    // tile, then process tile rel.
    auto step = [&](int rel, UnitRegs &kc, UnitRegs &vc, QPar &qc, UnitRegs &kn, UnitRegs &vn, QPar &qn,
                    Meta &mnext, Meta &mfree) {
        uint32_t ks2, vs2;
        tab_read(rel + 2, ks2, vs2);
        words_issue(mnext, kn, vn);
        qpar_issue(rel + 1, qn);
        meta_issue(ks2, vs2, mfree);
        fill_store(min(rel + kChunk - 2, ntl - 1), f1_off, f1_hdr, tid < 4);
        f1_hdr = fill_header(f0_off);
        f1_off = f0_off;
        f0_off = fill_info(rel + kChunk);
        process(kc, vc, qc);
    };
    for (int rel = 0; rel < ntl; rel += 2) {
        step(rel, kA, vA, qA, kB, vB, qB, mB, mA);
        if (rel + 1 < ntl) step(rel + 1, kB, vB, qB, kA, vA, qA, mA, mB);
    }

    // ---- epilogue ----
#pragma unroll
    for (int gi = 0; gi < GW; gi++) {
        const int g = wave + 4 * gi;
        if (g < G) {
            const float l = wave_sum(l_part[gi]), z = wave_sum(z_part[gi]);
            if (lane == 0) { st_m[g] = m_run[gi]; st_l[g] = l; st_z[g] = z; }
        }
    }
    __syncthreads();
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
            float *dst = p.part + (hq * p.nparts + split) * kPartStride;
            // fields were consumed as fp16 subnormals (delta * 2^-24)
            dst[2 + ch] = (acc[g >> 2][g & 3] * 16777216.f + st_z[g]) * wscale_inv;
            if (ch == 0) { dst[0] = st_m[g]; dst[1] = st_l[g]; }
        }
    }
}

}  // namespace pkv
