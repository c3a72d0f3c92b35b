/*
 * TEST INFRASTRUCTURE ONLY -- CPU restatement of the PackKV block codec.
 *
 * This file is the parity oracle for the HIP codec kernels.  Only tests, the
 * smoke check and the benchmark's CPU-baseline leg may link or call it; the
 * product library never does.
 *
 * It restates, from the stream layout, what the reference scalar codec does:
 *   K encode  packkv_cuda_ext/src/k_encode_cpu.cpp:12-31 (pack min / bit width),
 *             :34-52 (pack word), :55-95 (metadata bit arrays), :98-119 (payload
 *             order), :122-161 (round layout + cumulative header), :203-231
 *             (block loop, block_info)
 *   K decode  packkv_cuda_ext/src/k_decode_cpu.cpp:102-142, :145-165, :201-225
 *   V encode  packkv_cuda_ext/src/v_encode_cpu.cpp:69-91, :94-132, :135-187,
 *             :230-259
 *   V decode  packkv_cuda_ext/src/v_decode_cpu.cpp:12-32, :111-147, :184-216
 *   constants packkv_cuda_ext/include/static_def.h:4-6, include/utils.h:24-36
 *
 * Pinned by: the compiled reference templates (oracle/_ref, byte-for-byte on
 * stream + block_info for W in {2,3,4}), the committed golden vectors made
 * from that build, and closed-form block sizes / byte patterns in the tests.
 *
 * W in 5..8 is a FORMAT EXTENSION of this build (the reference stops at 16 * W <= 64 bits
 * per pack word, k_encode_cpu.cpp:211): the same layout rules with pack words of up to 128
 * bits.  No reference exists for it -- parity unpinned; it is pinned by encode -> decode round
 * trips, by the closed-form block sizes and by the reference's analytic size model
 * (utils/compute.py:272-297), which has no width limit.
 *
 * Layout facts restated here:
 *   - a pack is 16 consecutive tokens of one channel; min, len = bit_length(max-min);
 *     word = sum_k (code_k - min) << ((15-k)*len); stored as the low 2*len bytes, LE.
 *   - metadata arrays (mins: W bits per pack, lens: LB(W) bits per pack) are plain
 *     LSB-first bit arrays.
 *   - K block: u16 cumulative round sizes, then per round: mins | lens | payload,
 *     payload order j = 0..HDB-1 -> channel (j % 32) * (HDB/32) + j / 32.
 *   - V block (128 tokens): u16 cumulative segment sizes in (warp, seg) order, then per
 *     (warp, seg): mins | lens | payload; metadata field (lane t, slot i) at bit
 *     index t*4+i; payload order slot-major, lane-minor.
 */
#include <stdint.h>
#include <stddef.h>
#include <string.h>

#define PACK_TOK 16
typedef unsigned __int128 pkv_word;   /* 16 fields of up to 8 bits */
#define LANES 32

static int len_field_bits(int W) { /* include/utils.h:24-36 with n = W */
    int bits = 0;
    unsigned v = (unsigned)W;
    while (v) { v >>= 1; bits++; }
    return bits ? bits : 1;
}

static int bit_length(unsigned v) {
    int n = 0;
    while (v) { v >>= 1; n++; }
    return n;
}

static void put_bits(uint8_t *base, size_t bitpos, int nbits, unsigned value) {
    for (int b = 0; b < nbits; b++) {
        if ((value >> b) & 1u) base[(bitpos + b) >> 3] |= (uint8_t)(1u << ((bitpos + b) & 7));
    }
}

static unsigned get_bits(const uint8_t *base, size_t bitpos, int nbits) {
    unsigned v = 0;
    for (int b = 0; b < nbits; b++) {
        v |= (unsigned)((base[(bitpos + b) >> 3] >> ((bitpos + b) & 7)) & 1u) << b;
    }
    return v;
}

/* min, len and word of the pack holding tokens tok0..tok0+15 of channel ch. */
static void pack_stats(const uint8_t *codes, size_t row_stride, size_t tok0, size_t ch,
                       unsigned *mn_out, int *len_out, pkv_word *word_out) {
    unsigned mn = 255, mx = 0;
    for (int k = 0; k < PACK_TOK; k++) {
        unsigned c = codes[(tok0 + k) * row_stride + ch];
        if (c < mn) mn = c;
        if (c > mx) mx = c;
    }
    int len = bit_length(mx - mn);
    pkv_word word = 0;
    for (int k = 0; k < PACK_TOK; k++) {
        unsigned c = codes[(tok0 + k) * row_stride + ch];
        word = (len ? (word << len) : 0) | (pkv_word)(c - mn);
    }
    *mn_out = mn; *len_out = len; *word_out = word;
}

static size_t put_word(uint8_t *dst, pkv_word word, int len) {
    size_t n = (size_t)len * PACK_TOK / 8;
    for (size_t i = 0; i < n; i++) { dst[i] = (uint8_t)(word & 0xFF); word >>= 8; }
    return n;
}

static pkv_word get_word(const uint8_t *src, int len) {
    size_t n = (size_t)len * PACK_TOK / 8;
    pkv_word w = 0;
    for (size_t i = 0; i < n; i++) w |= (pkv_word)src[i] << (8 * i);
    return w;
}

static void unpack_word(uint8_t *codes, size_t row_stride, size_t tok0, size_t ch,
                        pkv_word word, int len, unsigned mn) {
    unsigned mask = len ? ((1u << len) - 1) : 0;
    for (int k = PACK_TOK - 1; k >= 0; k--) {
        codes[(tok0 + k) * row_stride + ch] = (uint8_t)(((unsigned)word & mask) + mn);
        word = len ? (word >> len) : 0;
    }
}

/* ------------------------------------------------------------------ K ---- */

size_t pkv_oracle_k_block_encode(const uint8_t *codes, size_t row_stride, int ctx_blk,
                                 int hid_blk, int W, uint8_t *out) {
    const int rounds = ctx_blk / PACK_TOK;
    const int LB = len_field_bits(W);
    const size_t mins_bytes = (size_t)W * hid_blk / 8;
    const size_t lens_bytes = (size_t)LB * hid_blk / 8;
    const int per_lane = hid_blk / LANES;
    size_t off = 2 * (size_t)rounds;
    unsigned cum = 0;
    for (int r = 0; r < rounds; r++) {
        uint8_t *mins = out + off;
        uint8_t *lens = mins + mins_bytes;
        uint8_t *payload = lens + lens_bytes;
        memset(mins, 0, mins_bytes + lens_bytes);
        size_t pay = 0;
        for (int j = 0; j < hid_blk; j++) {
            int ch = (j % LANES) * per_lane + j / LANES;
            unsigned mn; int len; pkv_word word;
            pack_stats(codes, row_stride, (size_t)r * PACK_TOK, (size_t)ch, &mn, &len, &word);
            put_bits(mins, (size_t)ch * W, W, mn);
            put_bits(lens, (size_t)ch * LB, LB, (unsigned)len);
            pay += put_word(payload + pay, word, len);
        }
        size_t round_bytes = mins_bytes + lens_bytes + pay;
        cum += (unsigned)round_bytes;
        out[2 * r] = (uint8_t)(cum & 0xFF);
        out[2 * r + 1] = (uint8_t)((cum >> 8) & 0xFF);
        off += round_bytes;
    }
    return off;
}

void pkv_oracle_k_block_decode(const uint8_t *in, int ctx_blk, int hid_blk, int W,
                               uint8_t *codes, size_t row_stride) {
    const int rounds = ctx_blk / PACK_TOK;
    const int LB = len_field_bits(W);
    const size_t mins_bytes = (size_t)W * hid_blk / 8;
    const size_t lens_bytes = (size_t)LB * hid_blk / 8;
    const int per_lane = hid_blk / LANES;
    size_t off = 2 * (size_t)rounds;
    unsigned prev = 0;
    for (int r = 0; r < rounds; r++) {
        unsigned cum = (unsigned)in[2 * r] | ((unsigned)in[2 * r + 1] << 8);
        const uint8_t *mins = in + off;
        const uint8_t *lens = mins + mins_bytes;
        const uint8_t *payload = lens + lens_bytes;
        size_t pay = 0;
        for (int j = 0; j < hid_blk; j++) {
            int ch = (j % LANES) * per_lane + j / LANES;
            unsigned mn = get_bits(mins, (size_t)ch * W, W);
            int len = (int)get_bits(lens, (size_t)ch * LB, LB);
            pkv_word word = get_word(payload + pay, len);
            pay += (size_t)len * PACK_TOK / 8;
            unpack_word(codes, row_stride, (size_t)r * PACK_TOK, (size_t)ch, word, len, mn);
        }
        off += (size_t)(uint16_t)(cum - prev);
        prev = cum;
    }
}

/* ------------------------------------------------------------------ V ---- */

#define V_SLOTS 4   /* packs per lane per segment  */
#define V_SEGS 2    /* segments per warp: 2 * 4 * 16 = 128 tokens */

size_t pkv_oracle_v_block_encode(const uint8_t *codes, size_t row_stride, int ctx_blk,
                                 int hid_blk, int W, uint8_t *out) {
    (void)ctx_blk; /* fixed at 128 by the layout */
    const int warps = hid_blk / LANES;
    const int LB = len_field_bits(W);
    const size_t mins_bytes = (size_t)W * V_SLOTS * LANES / 8;
    const size_t lens_bytes = (size_t)LB * V_SLOTS * LANES / 8;
    size_t off = 2 * (size_t)warps * V_SEGS;
    unsigned cum = 0;
    for (int w = 0; w < warps; w++) {
        for (int s = 0; s < V_SEGS; s++) {
            uint8_t *mins = out + off;
            uint8_t *lens = mins + mins_bytes;
            uint8_t *payload = lens + lens_bytes;
            memset(mins, 0, mins_bytes + lens_bytes);
            size_t pay = 0;
            for (int i = 0; i < V_SLOTS; i++) {
                for (int t = 0; t < LANES; t++) {
                    unsigned mn; int len; pkv_word word;
                    pack_stats(codes, row_stride, (size_t)(s * V_SLOTS + i) * PACK_TOK,
                               (size_t)(w * LANES + t), &mn, &len, &word);
                    put_bits(mins, (size_t)(t * V_SLOTS + i) * W, W, mn);
                    put_bits(lens, (size_t)(t * V_SLOTS + i) * LB, LB, (unsigned)len);
                    pay += put_word(payload + pay, word, len);
                }
            }
            size_t seg_bytes = mins_bytes + lens_bytes + pay;
            cum += (unsigned)seg_bytes;
            int idx = w * V_SEGS + s;
            out[2 * idx] = (uint8_t)(cum & 0xFF);
            out[2 * idx + 1] = (uint8_t)((cum >> 8) & 0xFF);
            off += seg_bytes;
        }
    }
    return off;
}

void pkv_oracle_v_block_decode(const uint8_t *in, int ctx_blk, int hid_blk, int W,
                               uint8_t *codes, size_t row_stride) {
    (void)ctx_blk;
    const int warps = hid_blk / LANES;
    const int LB = len_field_bits(W);
    const size_t mins_bytes = (size_t)W * V_SLOTS * LANES / 8;
    const size_t lens_bytes = (size_t)LB * V_SLOTS * LANES / 8;
    size_t off = 2 * (size_t)warps * V_SEGS;
    for (int w = 0; w < warps; w++) {
        for (int s = 0; s < V_SEGS; s++) {
            const uint8_t *mins = in + off;
            const uint8_t *lens = mins + mins_bytes;
            const uint8_t *payload = lens + lens_bytes;
            size_t pay = 0;
            for (int i = 0; i < V_SLOTS; i++) {
                for (int t = 0; t < LANES; t++) {
                    unsigned mn = get_bits(mins, (size_t)(t * V_SLOTS + i) * W, W);
                    int len = (int)get_bits(lens, (size_t)(t * V_SLOTS + i) * LB, LB);
                    pkv_word word = get_word(payload + pay, len);
                    pay += (size_t)len * PACK_TOK / 8;
                    unpack_word(codes, row_stride, (size_t)(s * V_SLOTS + i) * PACK_TOK,
                                (size_t)(w * LANES + t), word, len, mn);
                }
            }
            off += mins_bytes + lens_bytes + pay;
        }
    }
}

/* ------------------------------------------------- whole-tensor drivers -- */

static int check_shape(int is_k, int ctx_len, int hidden_dim, int ctx_blk, int hid_blk, int W) {
    if (W < 2 || W > 8) return -1;
    if (ctx_len <= 0 || hidden_dim <= 0 || ctx_blk <= 0 || hid_blk <= 0) return -1;
    if (ctx_len % ctx_blk || hidden_dim % hid_blk || ctx_blk % PACK_TOK) return -1;
    if (is_k) { if (hid_blk != 128) return -1; }
    else { if (ctx_blk != 128 || hid_blk % LANES) return -1; }
    return 0;
}

/* Returns the stream size in bytes, or (uint64_t)-1 for an unsupported shape. */
uint64_t pkv_oracle_encode(int is_k, const uint8_t *codes, uint8_t *stream, uint32_t *block_info,
                           int ctx_len, int hidden_dim, int ctx_blk, int hid_blk, int W) {
    if (check_shape(is_k, ctx_len, hidden_dim, ctx_blk, hid_blk, W)) return (uint64_t)-1;
    const int n_ctx = ctx_len / ctx_blk, n_hid = hidden_dim / hid_blk;
    uint64_t total = 0;
    for (int cb = 0; cb < n_ctx; cb++) {
        for (int hb = 0; hb < n_hid; hb++) {
            const uint8_t *tile = codes + (size_t)cb * ctx_blk * hidden_dim + (size_t)hb * hid_blk;
            size_t sz = is_k
                ? pkv_oracle_k_block_encode(tile, (size_t)hidden_dim, ctx_blk, hid_blk, W, stream + total)
                : pkv_oracle_v_block_encode(tile, (size_t)hidden_dim, ctx_blk, hid_blk, W, stream + total);
            size_t idx = (size_t)cb * n_hid + hb;
            block_info[2 * idx] = (uint32_t)total;
            block_info[2 * idx + 1] = (uint32_t)sz;
            total += sz;
        }
    }
    return total;
}

int pkv_oracle_decode(int is_k, const uint8_t *stream, const uint32_t *block_info, uint8_t *codes,
                      int ctx_len, int hidden_dim, int ctx_blk, int hid_blk, int W) {
    if (check_shape(is_k, ctx_len, hidden_dim, ctx_blk, hid_blk, W)) return -1;
    const int n_ctx = ctx_len / ctx_blk, n_hid = hidden_dim / hid_blk;
    for (int cb = 0; cb < n_ctx; cb++) {
        for (int hb = 0; hb < n_hid; hb++) {
            size_t idx = (size_t)cb * n_hid + hb;
            uint8_t *tile = codes + (size_t)cb * ctx_blk * hidden_dim + (size_t)hb * hid_blk;
            const uint8_t *src = stream + block_info[2 * idx];
            if (is_k) pkv_oracle_k_block_decode(src, ctx_blk, hid_blk, W, tile, (size_t)hidden_dim);
            else pkv_oracle_v_block_decode(src, ctx_blk, hid_blk, W, tile, (size_t)hidden_dim);
        }
    }
    return 0;
}

/* ------------------------------------------------- packs longer than 16 tokens --
 *
 * FORMAT EXTENSION of this build (the reference fixes PACK_ELE_NUM = 16, include/static_def.h:6, and only its
 * analytic size model, utils/compute.py:272-297, knows other pack lengths).  No reference exists for it -- parity
 * unpinned; it is pinned by the definition below restated with big integers in the tests, by the closed-form size
 * (stream bytes - 8 per block == the size model's bytes), by round trips, and by P = 16 reproducing the format above.
 *
 * A pack is P consecutive tokens of one channel, P in {16, 32, 64, 128, 256}; min and len as before over the P
 * tokens; word = sum_k (code_k - min) << ((P-1-k) * len), P * len bits, stored as its low P * len / 8 bytes,
 * little-endian (so the last 16 tokens of the pack come first in the stream).  Everything else scales with it: a
 * K block is 4 rounds of P tokens x 128 channels, a V block 2 warps x 2 segments of 4 slots of P tokens (8 P
 * tokens x 64 channels); metadata arrays and payload order as above.  The header keeps four u16 cumulative unit
 * sizes; for P >= 32 they count 4-byte words (every unit size is then a multiple of 4), since a unit can exceed
 * 65535 / 4 bytes.
 */
static void long_stats(const uint8_t *codes, size_t row_stride, size_t tok0, size_t ch, int P,
                       unsigned *mn_out, int *len_out) {
    unsigned mn = 255, mx = 0;
    for (int k = 0; k < P; k++) {
        unsigned c = codes[(tok0 + k) * row_stride + ch];
        if (c < mn) mn = c;
        if (c > mx) mx = c;
    }
    *mn_out = mn;
    *len_out = bit_length(mx - mn);
}

/* payload bytes of one pack at dst (zeroed by the caller); returns their count */
static size_t long_put(uint8_t *dst, const uint8_t *codes, size_t row_stride, size_t tok0, size_t ch, int P,
                       unsigned mn, int len) {
    for (int k = 0; k < P; k++)
        put_bits(dst, (size_t)(P - 1 - k) * len, len, codes[(tok0 + k) * row_stride + ch] - mn);
    return (size_t)P * len / 8;
}

static size_t long_get(const uint8_t *src, uint8_t *codes, size_t row_stride, size_t tok0, size_t ch, int P,
                       unsigned mn, int len) {
    for (int k = 0; k < P; k++)
        codes[(tok0 + k) * row_stride + ch] = (uint8_t)(get_bits(src, (size_t)(P - 1 - k) * len, len) + mn);
    return (size_t)P * len / 8;
}

static void put_cum(uint8_t *hdr, int idx, size_t cum, int P) {
    unsigned v = (unsigned)(P == 16 ? cum : cum / 4);
    hdr[2 * idx] = (uint8_t)(v & 0xFF);
    hdr[2 * idx + 1] = (uint8_t)((v >> 8) & 0xFF);
}

/* Unit u of a block (K: round u; V: warp u / 2, segment u % 2): pack (lane t, slot i) -> first token, channel. */
static void long_pack_at(int is_k, int u, int t, int i, int P, size_t *tok0, size_t *ch) {
    if (is_k) { *tok0 = (size_t)u * P; *ch = (size_t)(t * 4 + i); }
    else { *tok0 = (size_t)((u % V_SEGS) * V_SLOTS + i) * P; *ch = (size_t)((u / V_SEGS) * LANES + t); }
}

size_t pkv_oracle_long_block_encode(int is_k, const uint8_t *codes, size_t row_stride, int P, int W, uint8_t *out,
                                    size_t out_cap) {
    const int LB = len_field_bits(W);
    const size_t mins_bytes = (size_t)W * 128 / 8, lens_bytes = (size_t)LB * 128 / 8;
    size_t off = 8, cum = 0;
    for (int u = 0; u < 4; u++) {
        uint8_t *mins = out + off, *lens = mins + mins_bytes, *payload = lens + lens_bytes;
        memset(mins, 0, mins_bytes + lens_bytes);
        size_t pay = 0;
        for (int i = 0; i < 4; i++) {           /* payload order: slot-major, lane-minor */
            for (int t = 0; t < LANES; t++) {
                size_t tok0, ch; unsigned mn; int len;
                long_pack_at(is_k, u, t, i, P, &tok0, &ch);
                long_stats(codes, row_stride, tok0, ch, P, &mn, &len);
                put_bits(mins, (size_t)(t * 4 + i) * W, W, mn);
                put_bits(lens, (size_t)(t * 4 + i) * LB, LB, (unsigned)len);
                if ((size_t)(payload - out) + pay + (size_t)P * len / 8 > out_cap) return 0;
                memset(payload + pay, 0, (size_t)P * len / 8);
                pay += long_put(payload + pay, codes, row_stride, tok0, ch, P, mn, len);
            }
        }
        cum += mins_bytes + lens_bytes + pay;
        put_cum(out, u, cum, P);
        off += mins_bytes + lens_bytes + pay;
    }
    return off;
}

void pkv_oracle_long_block_decode(int is_k, const uint8_t *in, int P, int W, uint8_t *codes, size_t row_stride) {
    const int LB = len_field_bits(W);
    const size_t mins_bytes = (size_t)W * 128 / 8, lens_bytes = (size_t)LB * 128 / 8;
    size_t off = 8;
    for (int u = 0; u < 4; u++) {
        const uint8_t *mins = in + off, *lens = mins + mins_bytes, *payload = lens + lens_bytes;
        size_t pay = 0;
        for (int i = 0; i < 4; i++) {
            for (int t = 0; t < LANES; t++) {
                size_t tok0, ch;
                long_pack_at(is_k, u, t, i, P, &tok0, &ch);
                unsigned mn = get_bits(mins, (size_t)(t * 4 + i) * W, W);
                int len = (int)get_bits(lens, (size_t)(t * 4 + i) * LB, LB);
                pay += long_get(payload + pay, codes, row_stride, tok0, ch, P, mn, len);
            }
        }
        off += mins_bytes + lens_bytes + pay;
    }
}

static int check_long(int is_k, int ctx_len, int hidden_dim, int P, int W) {
    if (W < 2 || W > 8) return -1;
    if (P != 16 && P != 32 && P != 64 && P != 128 && P != 256) return -1;
    if (ctx_len <= 0 || hidden_dim <= 0) return -1;
    if (ctx_len % ((is_k ? 4 : 8) * P) || hidden_dim % (is_k ? 128 : 64)) return -1;
    return 0;
}

/* Whole tensor with packs of P tokens: K blocks of 4 P x 128, V blocks of 8 P x 64, in (context block, hidden block)
 * order.  Returns the stream size in bytes, or (uint64_t)-1 for an unsupported shape or a stream buffer too small. */
uint64_t pkv_oracle_long_encode(int is_k, const uint8_t *codes, uint8_t *stream, uint64_t capacity, uint32_t *block_info,
                                int ctx_len, int hidden_dim, int P, int W) {
    if (check_long(is_k, ctx_len, hidden_dim, P, W)) return (uint64_t)-1;
    const int ctx_blk = (is_k ? 4 : 8) * P, hid_blk = is_k ? 128 : 64;
    const int n_ctx = ctx_len / ctx_blk, n_hid = hidden_dim / hid_blk;
    uint64_t total = 0;
    for (int cb = 0; cb < n_ctx; cb++) {
        for (int hb = 0; hb < n_hid; hb++) {
            const uint8_t *tile = codes + (size_t)cb * ctx_blk * hidden_dim + (size_t)hb * hid_blk;
            size_t sz = pkv_oracle_long_block_encode(is_k, tile, (size_t)hidden_dim, P, W, stream + total,
                                                     (size_t)(capacity - total));
            if (!sz) return (uint64_t)-1;
            size_t idx = (size_t)cb * n_hid + hb;
            block_info[2 * idx] = (uint32_t)total;
            block_info[2 * idx + 1] = (uint32_t)sz;
            total += sz;
        }
    }
    return total;
}

int pkv_oracle_long_decode(int is_k, const uint8_t *stream, const uint32_t *block_info, uint8_t *codes,
                           int ctx_len, int hidden_dim, int P, int W) {
    if (check_long(is_k, ctx_len, hidden_dim, P, W)) return -1;
    const int ctx_blk = (is_k ? 4 : 8) * P, hid_blk = is_k ? 128 : 64;
    const int n_ctx = ctx_len / ctx_blk, n_hid = hidden_dim / hid_blk;
    for (int cb = 0; cb < n_ctx; cb++)
        for (int hb = 0; hb < n_hid; hb++) {
            size_t idx = (size_t)cb * n_hid + hb;
            pkv_oracle_long_block_decode(is_k, stream + block_info[2 * idx], P, W,
                                         codes + (size_t)cb * ctx_blk * hidden_dim + (size_t)hb * hid_blk,
                                         (size_t)hidden_dim);
        }
    return 0;
}

/* Worst case of one block with packs of P tokens: header, metadata of 512 packs, every pack at full width. */
uint64_t pkv_oracle_long_block_bound(int P, int W) {
    return 8ull + 4ull * (uint64_t)(W + len_field_bits(W)) * 128 / 8 + 512ull * (uint64_t)P * W / 8;
}

/* Worst-case bytes one block can take (every pack at full width W). */
uint64_t pkv_oracle_block_bound(int is_k, int ctx_blk, int hid_blk, int W) {
    const int LB = len_field_bits(W);
    const uint64_t packs = (uint64_t)(ctx_blk / PACK_TOK) * hid_blk;
    uint64_t header = is_k ? 2ull * (ctx_blk / PACK_TOK) : 2ull * V_SEGS * (hid_blk / LANES);
    return header + packs * (W + LB) / 8 + packs * 2ull * W;
}
