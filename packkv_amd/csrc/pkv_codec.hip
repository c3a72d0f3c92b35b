// Bit-unpack (stream -> uint8 codes) and bit-pack (uint8 codes -> stream) kernels: one 32-lane
// half-wavefront per round (K) or segment (V); one workgroup per block, except the encoder of
// the standard block shapes, which takes eight consecutive blocks per workgroup.
//
// Replaces the reference's scalar CPU codec on the device:
//   packkv_cuda_ext/src/k_encode_cpu.cpp:203-231, v_encode_cpu.cpp:230-259  (encode drivers)
//   packkv_cuda_ext/src/k_decode_cpu.cpp:201-225, v_decode_cpu.cpp:184-216  (decode drivers)
#include "pkv_block.hpp"
#include "pkv_runtime.hpp"

namespace pkv {

// LDS layout of both kernels: [code tile: ctx_blk*hid_blk][block buffer: bound + 32][unit_bytes]
__host__ __device__ inline uint32_t round_up16(uint32_t v) { return (v + 15u) & ~15u; }

template <bool IS_K>
__global__ void unpack_kernel(const uint8_t *__restrict__ stream, uint64_t stream_bytes, const uint32_t *__restrict__ info,
                              uint8_t *__restrict__ codes, int hidden_dim, int ctx_blk, int hid_blk,
                              int nunits, int W, uint32_t blk_cap) {
    extern __shared__ __align__(16) uint8_t lds[];
    uint8_t *tile = lds;
    uint8_t *blk = lds + round_up16((uint32_t)(ctx_blk * hid_blk));
    const int n_hid = hidden_dim / hid_blk;
    const uint32_t b = blockIdx.x;
    const uint32_t cb = b / n_hid, hb = b % n_hid;
    uint32_t off, size;
    block_span(info, b, blk_cap, stream_bytes, off, size);
    const uint32_t phase = stage_to_lds(stream + off, size, blk, threadIdx.x, blockDim.x);
    __syncthreads();
    block_decode<IS_K>(blk, phase, nunits, W, tile, hid_blk);
    __syncthreads();
    uint8_t *base = codes + (size_t)cb * ctx_blk * hidden_dim + (size_t)hb * hid_blk;
    // coalesced write-back: rows of hid_blk bytes, 16 bytes per lane where rows start on 16-byte boundaries
    if (((hid_blk | hidden_dim) & 15) == 0 && (reinterpret_cast<uintptr_t>(codes) & 15u) == 0) {
        const int row16 = hid_blk >> 4;
        const uint4 *t16 = reinterpret_cast<const uint4 *>(tile);
        for (int i = threadIdx.x; i < ctx_blk * row16; i += blockDim.x)
            *reinterpret_cast<uint4 *>(base + (size_t)(i / row16) * hidden_dim + 16 * (i % row16)) = t16[i];
        return;
    }
    const int row_dw = hid_blk >> 2;
    const uint32_t *t4 = reinterpret_cast<const uint32_t *>(tile);
    // (row, column) advance by the workgroup size without a division per element
    const int step_row = (int)blockDim.x / row_dw, step_c = (int)blockDim.x % row_dw;
    int row = (int)threadIdx.x / row_dw, c = (int)threadIdx.x % row_dw;
    for (int i = threadIdx.x; i < ctx_blk * row_dw; i += blockDim.x) {
        reinterpret_cast<uint32_t *>(base + (size_t)row * hidden_dim)[c] = t4[i];
        row += step_row;
        c += step_c;
        if (c >= row_dw) { c -= row_dw; row++; }
    }
}

// V blocks of 64 channels, two adjacent ones (the two halves of a head) per workgroup of 256 threads: the pair
// decodes into one tile of 128 tokens x 128 channels, so the write-back stores whole 128-byte lines.  In tile
// addressing the pair is a V block of 128 channels whose units 4 j + u are the units u of block j.
__global__ void __launch_bounds__(256) unpack_v_pair_kernel(const uint8_t *__restrict__ stream, uint64_t stream_bytes,
                                                            const uint32_t *__restrict__ info,
                                                            uint8_t *__restrict__ codes, int hidden_dim, int W,
                                                            uint32_t blk_cap) {
    constexpr int kCtx = 128, kPairHid = 128;
    extern __shared__ __align__(16) uint8_t lds[];
    uint8_t *tile = lds;
    const uint32_t blk_stride = round_up16(blk_cap) + 32u;
    const int n_pair = hidden_dim / kPairHid;
    const uint32_t cb = blockIdx.x / n_pair, hp = blockIdx.x % n_pair;
    const uint32_t b0 = cb * (uint32_t)(2 * n_pair) + 2u * hp;
    const int tid = threadIdx.x;
    const int j = tid >> 7;                                   // which block of the pair this half of the workgroup serves
    uint8_t *blk = lds + kCtx * kPairHid + j * blk_stride;
    uint32_t off, size;
    block_span(info, b0 + j, blk_cap, stream_bytes, off, size);
    const uint32_t phase = stage_to_lds(stream + off, size, blk, tid & 127, 128);
    __syncthreads();
    {
        const UnitGeom g = unit_geom(W);
        const int t = tid & 31, u = (tid >> 5) & 3;
        const uint16_t *cum = reinterpret_cast<const uint16_t *>(blk + phase);
        const uint32_t start = phase + 8u + (u ? (uint32_t)cum[u - 1] : 0u);
        unit_decode<false>(blk, min(start, blk_cap), 4 * j + u, t, g, tile, kPairHid);
    }
    __syncthreads();
    const uint4 *t16 = reinterpret_cast<const uint4 *>(tile);
    uint8_t *base = codes + (size_t)cb * kCtx * hidden_dim + (size_t)hp * kPairHid;
#pragma unroll
    for (int i = 0; i < kCtx * kPairHid / 16 / 256; i++) {     // 8 rows of 128 bytes per step, 16 bytes per thread
        const int idx = tid + 256 * i;
        *reinterpret_cast<uint4 *>(base + (size_t)(idx >> 3) * hidden_dim + 16 * (idx & 7)) = t16[idx];
    }
}

template <bool IS_K>
__global__ void pack_kernel(const uint8_t *__restrict__ codes, uint8_t *__restrict__ stream,
                            uint64_t capacity, uint32_t *__restrict__ info, ScanState *st,
                            int hidden_dim, int ctx_blk, int hid_blk, int nunits, int W,
                            uint32_t nblocks) {
    extern __shared__ __align__(16) uint8_t lds[];
    __shared__ uint32_t s_idx;
    __shared__ uint64_t s_off;
    __shared__ uint32_t unit_bytes[16];
    uint8_t *tile = lds;
    uint8_t *blk = lds + round_up16((uint32_t)(ctx_blk * hid_blk));
    if (threadIdx.x == 0) s_idx = atomicAdd(&st->ticket, 1u);
    __syncthreads();
    const uint32_t b = s_idx;
    if (b >= nblocks) return;
    const int n_hid = hidden_dim / hid_blk;
    const uint32_t cb = b / n_hid, hb = b % n_hid;
    const int row_dw = hid_blk >> 2;
    uint32_t *t4 = reinterpret_cast<uint32_t *>(tile);
    {   // (row, column) advance by the workgroup size without a division per element; four loads in flight
        const int step_row = (int)blockDim.x / row_dw, step_c = (int)blockDim.x % row_dw;
        int row = (int)threadIdx.x / row_dw, c = (int)threadIdx.x % row_dw;
        const uint8_t *base = codes + (size_t)cb * ctx_blk * hidden_dim + (size_t)hb * hid_blk;
        const int n = ctx_blk * row_dw;
        for (int i = threadIdx.x; i < n; i += 4 * (int)blockDim.x) {
            uint32_t v[4];
#pragma unroll
            for (int u = 0; u < 4; u++) {
                v[u] = i + u * (int)blockDim.x < n ? reinterpret_cast<const uint32_t *>(base + (size_t)row * hidden_dim)[c] : 0u;
                row += step_row;
                c += step_c;
                if (c >= row_dw) { c -= row_dw; row++; }
            }
#pragma unroll
            for (int u = 0; u < 4; u++)
                if (i + u * (int)blockDim.x < n) t4[i + u * (int)blockDim.x] = v[u];
        }
    }
    __syncthreads();
    block_finish<IS_K>(tile, blk, unit_bytes, &s_off, st, b, nblocks, stream, capacity, info, hid_blk,
                       nunits, W);
}

// ---- the same encode, eight blocks per workgroup (blocks of four units) ----------------------------------------
// With one ticket per block a launch has tens of thousands of status words in flight and a block's look-back walks
// far before it meets an inclusive prefix: the per-block kernel spends most of its time there (vector ALUs 24 %
// busy).  Here a workgroup of 256 threads takes eight consecutive blocks of the stream -- two at a time: load the
// two code tiles with 16-byte loads, analyse, emit behind the blocks already in LDS -- and then asks ONE offset for
// all of them and writes their bytes, contiguous in the stream, in one sweep of aligned 16-byte stores.
constexpr int kPackGroup = 8;

template <bool IS_K, bool WIDE>
__global__ void __launch_bounds__(256) pack_group_kernel(const uint8_t *__restrict__ codes, uint8_t *__restrict__ stream,
                                                         uint64_t capacity, uint32_t *__restrict__ info, ScanState *st,
                                                         int hidden_dim, int /* ctx_blk */, int /* hid_blk */, int W, uint32_t nblocks,
                                                         uint32_t ngroups, const Stagger stagger) {
    // blocks of four units are 64 tokens x 128 channels (K) or 128 tokens x 64 channels (V): as constants, the tile
    // offsets of a lane's codes are immediates of its loads instead of an address register each
    constexpr int ctx_blk = IS_K ? 64 : 128, hid_blk = IS_K ? 128 : 64;
    extern __shared__ __align__(16) uint8_t lds[];         // two code tiles | the group's bytes
    __shared__ uint32_t s_idx;
    __shared__ uint64_t s_off;
    __shared__ uint32_t unit_bytes[2][4];
    __shared__ uint32_t blk_off[kPackGroup + 1];
    const int tid = threadIdx.x;
    stagger_first_generation(stagger);
    if (tid == 0) { s_idx = atomicAdd(&st->ticket, 1u); blk_off[0] = 0u; }
    __syncthreads();
    const uint32_t gidx = s_idx;
    if (gidx >= ngroups) return;
    const uint32_t b0 = gidx * (uint32_t)kPackGroup;
    const int nb = (int)min((uint32_t)kPackGroup, nblocks - b0);
    const int tile_bytes = ctx_blk * hid_blk;              // a multiple of 16
    uint8_t *gbuf = lds + 2 * tile_bytes;
    const UnitGeom g = unit_geom(W);
    const uint32_t meta = (uint32_t)(g.mins_bytes + g.lens_bytes);
    const int n_hid = hidden_dim / hid_blk;
    const int jl = tid >> 7, lt = tid & 127, unit = lt >> 5, t = tid & 31;
    const uint8_t *tile = lds + jl * tile_bytes;
    const int row16 = hid_blk >> 4, n16 = ctx_blk * row16;
    // the tile of a thread's block of the pair that starts at block j0: four 16-byte pieces (tiles are 8 KiB: 512
    // pieces over the 128 threads of a block), loaded a pair ahead so that the loads fly while the current pair is
    // analysed and emitted
#define PKV_FETCH_PAIR(j0_)                                                                                              \
    {                                                                                                                    \
        const uint32_t b = b0 + (uint32_t)min((j0_) + jl, nb - 1); /* clamped: the loads are unconditional */           \
        const uint32_t cb = b / (uint32_t)n_hid, hb = b % (uint32_t)n_hid;                                               \
        const uint8_t *src = codes + (size_t)cb * ctx_blk * hidden_dim + (size_t)hb * hid_blk;                           \
        const int i0 = min(lt, n16 - 1), i1 = min(lt + 128, n16 - 1), i2 = min(lt + 256, n16 - 1), i3 = min(lt + 384, n16 - 1); \
        a0 = *reinterpret_cast<const uint4 *>(src + (size_t)(i0 / row16) * hidden_dim + 16 * (i0 % row16));              \
        a1 = *reinterpret_cast<const uint4 *>(src + (size_t)(i1 / row16) * hidden_dim + 16 * (i1 % row16));              \
        a2 = *reinterpret_cast<const uint4 *>(src + (size_t)(i2 / row16) * hidden_dim + 16 * (i2 % row16));              \
        a3 = *reinterpret_cast<const uint4 *>(src + (size_t)(i3 / row16) * hidden_dim + 16 * (i3 % row16));              \
    }
    uint4 a0, a1, a2, a3;
    PKV_FETCH_PAIR(0)
    for (int j0 = 0; j0 < nb; j0 += 2) {
        const int jj = j0 + jl;
        const bool active = jj < nb;
        uint4 *t16 = reinterpret_cast<uint4 *>(lds + jl * tile_bytes);
        if (lt < n16) t16[lt] = a0;
        if (lt + 128 < n16) t16[lt + 128] = a1;
        if (lt + 256 < n16) t16[lt + 256] = a2;
        if (lt + 384 < n16) t16[lt + 384] = a3;
        __syncthreads();
        if (j0 + 2 < nb) PKV_FETCH_PAIR(j0 + 2)
        UnitPacks u;
        constexpr bool wide = WIDE;                       // the field-by-field code of the extension widths (W > 4)
        if (active) {
            if constexpr (wide) {
                const uint32_t usz = unit_encode_wide<IS_K>(tile, hid_blk, unit, t, g, nullptr, 0u);
                if (t == 0) unit_bytes[jl][unit] = usz;
            } else {
                unit_analyse<IS_K>(tile, hid_blk, unit, t, u);
                if (t == 0) unit_bytes[jl][unit] = meta + u.payload;
            }
        }
        __syncthreads();
        if (tid == 0) {                                   // block sizes of this pair -> offsets inside the group
            uint32_t off = blk_off[j0] + 8u + unit_bytes[0][0] + unit_bytes[0][1] + unit_bytes[0][2] + unit_bytes[0][3];
            blk_off[j0 + 1] = off;
            if (j0 + 1 < nb) blk_off[j0 + 2] = off + 8u + unit_bytes[1][0] + unit_bytes[1][1] + unit_bytes[1][2] + unit_bytes[1][3];
            // the group's size is known here, before its last pair is written: the successors' look-backs wait less
            if (j0 + 2 >= nb) lookback_publish(st, gidx, blk_off[nb]);
        }
        __syncthreads();
        if (active) {
            uint8_t *blk = gbuf + blk_off[jj];
            uint32_t base = 8u;
#pragma unroll
            for (int q = 0; q < 4; q++) base += q < unit ? unit_bytes[jl][q] : 0u;
            if (t == 0) reinterpret_cast<uint16_t *>(blk)[unit] = (uint16_t)(base - 8u + unit_bytes[jl][unit]);
            if constexpr (wide) unit_encode_wide<IS_K>(tile, hid_blk, unit, t, g, blk, base);
            else unit_emit(blk, base, t, g, u);
        }
        __syncthreads();
    }
#undef PKV_FETCH_PAIR
    const uint32_t bytes = blk_off[nb];
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
    if (tid < nb) {
        info[2 * (size_t)(b0 + tid)] = (uint32_t)(off + blk_off[tid]);
        info[2 * (size_t)(b0 + tid) + 1] = blk_off[tid + 1] - blk_off[tid];
    }
    // head (to the first 16-byte boundary of the stream) and tail in 2-byte pieces, the body as aligned 16-byte
    // stores fed by aligned LDS reads and byte funnel shifts
    uint8_t *dst = stream + off;
    const uint32_t head = min(bytes, (uint32_t)((16u - (uint32_t)(reinterpret_cast<uintptr_t>(dst) & 15u)) & 15u));
    const uint32_t nq = (bytes - head) >> 4;
    for (uint32_t i = tid; i < (head >> 1); i += 256)
        reinterpret_cast<uint16_t *>(dst)[i] = reinterpret_cast<const uint16_t *>(gbuf)[i];
    const uint32_t *src32 = reinterpret_cast<const uint32_t *>(gbuf + (head & ~3u));
    for (uint32_t i = tid; i < nq; i += 256) {
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
    for (uint32_t i = tid; i < ((bytes - done) >> 1); i += 256)
        reinterpret_cast<uint16_t *>(dst + done)[i] = reinterpret_cast<const uint16_t *>(gbuf + done)[i];
}

__global__ void zero_state_kernel(uint64_t *p, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0;
}

struct CodecShape {
    int nunits, threads, nblocks;
    uint32_t blk_cap, lds_bytes;
};

static int codec_shape(bool is_k, int ctx_len, int hidden_dim, int ctx_blk, int hid_blk, int bits,
                       CodecShape *o) {
    PKV_REQUIRE(bits >= 2 && bits <= kMaxBits, PKV_ERR_UNSUPPORTED, "not supported: bits_len %d (need 2..8)", bits);
    PKV_REQUIRE(ctx_len > 0 && hidden_dim > 0 && ctx_blk > 0 && hid_blk > 0, PKV_ERR_INVALID,
                "sizes must be positive");
    PKV_REQUIRE(ctx_len % ctx_blk == 0, PKV_ERR_INVALID, "ctx_len must be divisible by ctx_len_block_size");
    PKV_REQUIRE(hidden_dim % hid_blk == 0, PKV_ERR_INVALID,
                "hidden_dim must be divisible by hidden_dim_block_size");
    PKV_REQUIRE(ctx_blk % kPackTok == 0, PKV_ERR_INVALID, "ctx_len_block_size must be divisible by 16");
    if (is_k) {
        PKV_REQUIRE(hid_blk == kHeadDim, PKV_ERR_UNSUPPORTED,
                    "not supported: K hidden_dim_block_size must be 128");
        PKV_REQUIRE(ctx_blk <= 256, PKV_ERR_UNSUPPORTED, "not supported: K ctx_len_block_size > 256");
        o->nunits = ctx_blk / kPackTok;
        o->blk_cap = (uint32_t)k_block_bound(ctx_blk, bits);
    } else {
        PKV_REQUIRE(ctx_blk == 128, PKV_ERR_UNSUPPORTED, "not supported: V ctx_len_block_size must be 128");
        PKV_REQUIRE(hid_blk % kLanes == 0 && hid_blk <= 256, PKV_ERR_UNSUPPORTED,
                    "not supported: V hidden_dim_block_size must be a multiple of 32, at most 256");
        o->nunits = 2 * (hid_blk / kLanes);
        o->blk_cap = (uint32_t)v_block_bound(hid_blk, bits);
    }
    o->threads = ((32 * o->nunits + 63) / 64) * 64;
    o->nblocks = (ctx_len / ctx_blk) * (hidden_dim / hid_blk);
    o->lds_bytes = round_up16((uint32_t)(ctx_blk * hid_blk)) + round_up16(o->blk_cap) + 32u;
    return PKV_OK;
}

static int run_unpack(bool is_k, const uint8_t *stream, uint64_t stream_bytes, const uint32_t *info, uint8_t *codes,
                      int ctx_len, int hidden_dim, int ctx_blk, int hid_blk, int bits, float *ms_out,
                      hipStream_t s) {
    PKV_REQUIRE(stream && info && codes, PKV_ERR_INVALID, "null pointer argument");
    PKV_REQUIRE(stream_bytes > 0 && stream_bytes < (1ull << 32), PKV_ERR_INVALID, "stream size must be in 1 .. 4 GiB - 1");
    CodecShape cs;
    int rc = codec_shape(is_k, ctx_len, hidden_dim, ctx_blk, hid_blk, bits, &cs);
    if (rc) return rc;
    LaunchTimer tm(s, ms_out != nullptr);
    if ((rc = tm.begin())) return rc;
    if (is_k)
        unpack_kernel<true><<<cs.nblocks, cs.threads, cs.lds_bytes, s>>>(
            stream, stream_bytes, info, codes, hidden_dim, ctx_blk, hid_blk, cs.nunits, bits, cs.blk_cap);
    else if (hid_blk == 64 && hidden_dim % 128 == 0 && (reinterpret_cast<uintptr_t>(codes) & 15u) == 0)
        unpack_v_pair_kernel<<<cs.nblocks / 2, 256, 128 * 128 + 2 * (round_up16(cs.blk_cap) + 32u), s>>>(
            stream, stream_bytes, info, codes, hidden_dim, bits, cs.blk_cap);
    else
        unpack_kernel<false><<<cs.nblocks, cs.threads, cs.lds_bytes, s>>>(
            stream, stream_bytes, info, codes, hidden_dim, ctx_blk, hid_blk, cs.nunits, bits, cs.blk_cap);
    PKV_HIP_CHECK(hipGetLastError());
    return tm.end(ms_out);
}

// Shared tail of every encoder: read back {error, total} when the caller wants the size.
int finish_encode(ScanState *st, uint64_t *size_out, int bits, hipStream_t s) {
    if (!size_out) return PKV_OK;
    struct { uint32_t ticket, error; uint64_t total; uint32_t max_code, pad; } h;
    PKV_HIP_CHECK(hipMemcpyAsync(&h, st, sizeof(h), hipMemcpyDeviceToHost, s));
    PKV_HIP_CHECK(hipStreamSynchronize(s));
    if (h.error == (uint32_t)PKV_ERR_CAPACITY) {
        set_error("compressed stream does not fit the output buffer");
        return PKV_ERR_CAPACITY;
    }
    if (h.error) {
        set_error("device-side encode failure (code %u)", h.error);
        return (int)h.error;
    }
    if (bits > 0 && h.max_code >= (1u << bits)) {
        set_error("not supported: code %u does not fit bits_len %d", h.max_code, bits);
        return PKV_ERR_UNSUPPORTED;
    }
    *size_out = h.total;
    return PKV_OK;
}

int prepare_scan_state(uint32_t nblocks, ScanState **out, hipStream_t s) {
    void *p = nullptr;
    const size_t bytes = sizeof(ScanState) + (size_t)nblocks * sizeof(uint64_t);
    int rc = scratch_get(bytes, s, &p, kScratchEncoder);
    if (rc) return rc;
    const size_t n64 = (bytes + 7) / 8;
    zero_state_kernel<<<(unsigned)((n64 + 255) / 256), 256, 0, s>>>((uint64_t *)p, n64);
    PKV_HIP_CHECK(hipGetLastError());
    *out = (ScanState *)p;
    return PKV_OK;
}

static int run_pack(bool is_k, const uint8_t *codes, uint8_t *stream, uint64_t capacity, uint32_t *info,
                    int ctx_len, int hidden_dim, int ctx_blk, int hid_blk, int bits, uint64_t *size_out,
                    float *ms_out, hipStream_t s) {
    PKV_REQUIRE(stream && info && codes, PKV_ERR_INVALID, "null pointer argument");
    PKV_REQUIRE((reinterpret_cast<uintptr_t>(stream) & 1u) == 0, PKV_ERR_INVALID,
                "compressed_buffer must start at an even address (blocks are written in 2-byte units)");
    PKV_REQUIRE(capacity > 0, PKV_ERR_INVALID, "compressed_buffer must be a non-empty tensor");
    // block_info holds 32-bit byte offsets: a stream past 4 GiB is reported as a full buffer, never wrapped
    if (capacity > (1ull << 32)) capacity = 1ull << 32;
    CodecShape cs;
    int rc = codec_shape(is_k, ctx_len, hidden_dim, ctx_blk, hid_blk, bits, &cs);
    if (rc) return rc;
    ScanState *st = nullptr;
    // blocks of four units, 16-byte aligned rows: eight blocks per workgroup (not at 8 bits, where the group's 88 KB
    // of LDS leave one workgroup per CU and the per-block kernel is 10 % faster)
    const bool grouped = cs.nunits == 4 && bits <= 7 && hid_blk % 16 == 0 && hidden_dim % 16 == 0 &&
                         (reinterpret_cast<uintptr_t>(codes) & 15u) == 0;
    // the reference's block shapes over rows that are whole groups of 1024 channels: the cells kernels (no code tile
    // in LDS, the next round in flight while packs are formed)
    const bool cells = bits <= 6 && hidden_dim % 1024 == 0 && (reinterpret_cast<uintptr_t>(codes) & 3u) == 0 &&
                       (is_k ? (ctx_blk == 64 && hid_blk == 128) : (ctx_blk == 128 && hid_blk == 64));
    if (cells) {
        const uint32_t ngroups = (uint32_t)cs.nblocks / (is_k ? 8u : 16u);
        if ((rc = prepare_scan_state(ngroups, &st, s))) return rc;
        LaunchTimer tm(s, ms_out != nullptr);
        if ((rc = tm.begin())) return rc;
        if ((rc = launch_code_cells(is_k, codes, ctx_len, hidden_dim, bits, cs.blk_cap, stream, capacity, info, st, ngroups, s))) return rc;
        if ((rc = tm.end(ms_out))) return rc;
        return finish_encode(st, size_out, 0, s);
    }
    if (grouped) {
        const uint32_t ngroups = ((uint32_t)cs.nblocks + kPackGroup - 1) / kPackGroup;
        const uint32_t lds = 2u * (uint32_t)(ctx_blk * hid_blk) + (uint32_t)kPackGroup * cs.blk_cap + 32u;
        if ((rc = prepare_scan_state(ngroups, &st, s))) return rc;
        auto kern = bits > 4 ? (is_k ? pack_group_kernel<true, true> : pack_group_kernel<false, true>)
                             : (is_k ? pack_group_kernel<true, false> : pack_group_kernel<false, false>);
        if (lds > 48u * 1024u)
            PKV_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        Stagger sg;
        if ((rc = stagger_for(reinterpret_cast<const void *>(kern), 256, lds, ngroups, &sg))) return rc;
        LaunchTimer tm(s, ms_out != nullptr);
        if ((rc = tm.begin())) return rc;
        kern<<<ngroups, 256, lds, s>>>(codes, stream, capacity, info, st, hidden_dim, ctx_blk, hid_blk, bits,
                                       (uint32_t)cs.nblocks, ngroups, sg);
        PKV_HIP_CHECK(hipGetLastError());
        if ((rc = tm.end(ms_out))) return rc;
        return finish_encode(st, size_out, 0, s);
    }
    if ((rc = prepare_scan_state((uint32_t)cs.nblocks, &st, s))) return rc;
    LaunchTimer tm(s, ms_out != nullptr);
    if ((rc = tm.begin())) return rc;
    if (is_k)
        pack_kernel<true><<<cs.nblocks, cs.threads, cs.lds_bytes, s>>>(
            codes, stream, capacity, info, st, hidden_dim, ctx_blk, hid_blk, cs.nunits, bits,
            (uint32_t)cs.nblocks);
    else
        pack_kernel<false><<<cs.nblocks, cs.threads, cs.lds_bytes, s>>>(
            codes, stream, capacity, info, st, hidden_dim, ctx_blk, hid_blk, cs.nunits, bits,
            (uint32_t)cs.nblocks);
    PKV_HIP_CHECK(hipGetLastError());
    if ((rc = tm.end(ms_out))) return rc;
    return finish_encode(st, size_out, 0, s);
}

}  // namespace pkv

extern "C" {

int pkv_k_encode(const uint8_t *codes, uint8_t *stream, uint64_t capacity, uint32_t *block_info,
                 int ctx_len, int hidden_dim, int ctx_blk, int hid_blk, int bits, uint64_t *size_out,
                 float *ms_out, pkv_stream_t s) {
    return pkv::run_pack(true, codes, stream, capacity, block_info, ctx_len, hidden_dim, ctx_blk, hid_blk,
                         bits, size_out, ms_out, (hipStream_t)s);
}

int pkv_v_encode(const uint8_t *codes, uint8_t *stream, uint64_t capacity, uint32_t *block_info,
                 int ctx_len, int hidden_dim, int ctx_blk, int hid_blk, int bits, uint64_t *size_out,
                 float *ms_out, pkv_stream_t s) {
    return pkv::run_pack(false, codes, stream, capacity, block_info, ctx_len, hidden_dim, ctx_blk, hid_blk,
                         bits, size_out, ms_out, (hipStream_t)s);
}

int pkv_k_decode(const uint8_t *stream, uint64_t stream_bytes, const uint32_t *block_info, uint8_t *codes, int ctx_len,
                 int hidden_dim, int ctx_blk, int hid_blk, int bits, float *ms_out, pkv_stream_t s) {
    return pkv::run_unpack(true, stream, stream_bytes, block_info, codes, ctx_len, hidden_dim, ctx_blk, hid_blk, bits,
                           ms_out, (hipStream_t)s);
}

int pkv_v_decode(const uint8_t *stream, uint64_t stream_bytes, const uint32_t *block_info, uint8_t *codes, int ctx_len,
                 int hidden_dim, int ctx_blk, int hid_blk, int bits, float *ms_out, pkv_stream_t s) {
    return pkv::run_unpack(false, stream, stream_bytes, block_info, codes, ctx_len, hidden_dim, ctx_blk, hid_blk, bits,
                           ms_out, (hipStream_t)s);
}

int pkv_encode_status(pkv_stream_t s_, int bits, uint64_t *size_out) {
    using namespace pkv;
    hipStream_t s = (hipStream_t)s_;
    PKV_REQUIRE(size_out != nullptr, PKV_ERR_INVALID, "null pointer argument");
    void *st = nullptr;
    int rc = encoder_state_peek(s, &st);
    if (rc) return rc;
    return finish_encode(static_cast<ScanState *>(st), size_out, bits, s);
}

uint64_t pkv_block_bound(int is_k, int ctx_blk, int hid_blk, int bits) {
    return is_k ? (uint64_t)pkv::k_block_bound(ctx_blk, bits) : (uint64_t)pkv::v_block_bound(hid_blk, bits);
}

}  // extern "C"
