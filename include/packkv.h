/*
 * packkv.h -- C ABI of libpackkv_hip.so: the PackKV compressed-KV-cache hot path on one
 * AMD gfx950 GPU (quantize -> bit-pack encode, bit-unpack decode, fused
 * decompress-attention decode).
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless the parameter is documented as host;
 *     buffers are caller-allocated and written in place, nothing is returned but a status;
 *   - `s` is a hipStream_t (NULL = the default stream); work is enqueued on it;
 *   - `ms_out` (host, may be NULL): when non-NULL the call brackets its kernels with HIP
 *     events, waits for them and stores the elapsed milliseconds -- the reference's
 *     launchers are synchronous and return milliseconds the same way
 *     (packkv_cuda_ext/src/kernels.cu:560-608, src/fused_kernels.cu:118-168);
 *   - return value 0 = success, otherwise a PKV_ERR_* code with text in pkv_last_error();
 *     the library never aborts the process (the reference's CPU codec aborts on a failed
 *     precondition, include/utils.h:8-16, and throws "not supported" for shapes outside
 *     its dispatch table, src/k_encode_cpu.cpp:328-330 -- both map to error codes here);
 *   - `dtype`: PKV_F16 or PKV_BF16, the 16-bit storage type of q / scale / zero / outputs
 *     (the reference dispatches on at::Half / at::BFloat16, src/kernels.cu:622-629);
 *   - code matrices are uint8 [ctx_len, hidden_dim] row-major with channel index
 *     (b * H + h) * 128 + d (evaluation/evaluation.py:406); streams and block_info are laid
 *     out exactly as the reference encoders write them (block_info[i] = (byte offset, byte
 *     size) as uint32, i = ctx_blk * n_hid_blk + hid_blk).
 */
#ifndef PACKKV_H
#define PACKKV_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PKV_ABI_VERSION 3

#define PKV_F16 0
#define PKV_BF16 1

#define PKV_OK 0
#define PKV_ERR_UNSUPPORTED 1 /* shape / width outside what the kernels implement */
#define PKV_ERR_INVALID 2     /* bad argument */
#define PKV_ERR_HIP 3         /* a HIP runtime call failed */
#define PKV_ERR_CAPACITY 4    /* output buffer too small for the produced stream */
#define PKV_ERR_INTERNAL 5    /* device-side protocol failure */

typedef void *pkv_stream_t;

int pkv_abi_version(void);
/* Text of the last error raised on the calling thread. */
const char *pkv_last_error(void);
/* Worst-case bytes of one block (every pack at full width). */
uint64_t pkv_block_bound(int is_k, int ctx_blk, int hid_blk, int bits);

/* ---- bit-pack / bit-unpack of uint8 code matrices ---------------------------------
 * Device counterparts of k_encode_cpu / v_encode_cpu / k_decode_cpu / v_decode_cpu
 * (packkv_cuda_ext/packkv_cuda.pyi:4-24, :38-58; src/k_encode_cpu.cpp:286-331,
 * src/v_encode_cpu.cpp:301-346, src/k_decode_cpu.cpp:281-326, src/v_decode_cpu.cpp:258-303).
 * Generalised from the reference's dispatch table to any hidden_dim that is a multiple of
 * the block width, bits in 2..8; K blocks are ctx_blk x 128 (ctx_blk a multiple of 16,
 * at most 256), V blocks are 128 x hid_blk (hid_blk a multiple of 32, at most 256).
 * bits 5..8 are an extension of the format: the reference stops at 16 * bits <= 64 bits per
 * pack word (src/k_encode_cpu.cpp:211); here the same layout rules run on with pack words of
 * up to 128 bits and a 4-bit length field at bits = 8.  A stream of such codes can be larger
 * than the code matrix: size the buffer with pkv_block_bound.
 * `capacity` = bytes available at `stream` (which must start at an even address); `size_out` (host, may be NULL)
 * receives the stream size and makes the call synchronous.  With size_out = NULL nothing is reported by the call
 * itself, not even a stream that did not fit: ask pkv_encode_status afterwards.
 * The decoders (and the kq / wv products further down) take `stream_bytes`, the size of the buffer at `stream` --
 * what the reference's binding knows as compressed_buffer.numel(): a block whose block_info entry points outside
 * the buffer decodes to arbitrary codes, it is never read from there. */
int pkv_k_encode(const uint8_t *codes, uint8_t *stream, uint64_t capacity, uint32_t *block_info,
                 int ctx_len, int hidden_dim, int ctx_blk, int hid_blk, int bits, uint64_t *size_out,
                 float *ms_out, pkv_stream_t s);
int pkv_v_encode(const uint8_t *codes, uint8_t *stream, uint64_t capacity, uint32_t *block_info,
                 int ctx_len, int hidden_dim, int ctx_blk, int hid_blk, int bits, uint64_t *size_out,
                 float *ms_out, pkv_stream_t s);
/* Outcome of the last encode launched on stream `s` (any of pkv_{k,v}_encode, pkv_{k,v}_quant_encode and their
 * _append forms) -- for callers that passed size_out = NULL to keep the launch asynchronous: waits for the stream,
 * then returns what the encoder itself would have returned with size_out (PKV_ERR_CAPACITY when the stream did not
 * fit, PKV_ERR_INTERNAL, and with bits > 0 PKV_ERR_UNSUPPORTED when a code of a fused encode does not fit `bits`)
 * and stores the stream size.  No counterpart in the reference, whose encoders are synchronous host code. */
int pkv_encode_status(pkv_stream_t s, int bits, uint64_t *size_out);
int pkv_k_decode(const uint8_t *stream, uint64_t stream_bytes, const uint32_t *block_info, uint8_t *codes, int ctx_len,
                 int hidden_dim, int ctx_blk, int hid_blk, int bits, float *ms_out, pkv_stream_t s);
int pkv_v_decode(const uint8_t *stream, uint64_t stream_bytes, const uint32_t *block_info, uint8_t *codes, int ctx_len,
                 int hidden_dim, int ctx_blk, int hid_blk, int bits, float *ms_out, pkv_stream_t s);

/* ---- packs longer than 16 tokens ------------------------------------------------------
 * The block codec for pack_len in {32, 64, 128, 256} tokens: an extension of the stream format.  No counterpart in the
 * reference's codec, which fixes PACK_ELE_NUM = 16 (packkv_cuda_ext/include/static_def.h:6); they realise what the
 * reference only prices, bit_pack(tensor, pack_len) (utils/compute.py:272-297): the stream holds 8 bytes per block
 * plus exactly that model's bytes.  A pack is pack_len consecutive tokens of one channel, its word
 * sum_k (code_k - min) << ((pack_len - 1 - k) * len) stored as pack_len * len / 8 little-endian bytes; K blocks are
 * 4 pack_len tokens x 128 channels, V blocks 8 pack_len tokens x 64 channels (ctx_len / hidden_dim must be
 * multiples), units, metadata arrays and payload order as in the 16-token format; the four u16 cumulative unit sizes
 * of a block header count 4-byte words.  codes: uint8 [ctx_len, hidden_dim] (4-byte aligned for K); block_info:
 * uint32 [n_blocks, 2]; bits 2..8; the stream starts at an even address.  pack_len 16 forwards to the functions
 * above with the reference's block shapes (64 x 128, 128 x 64).  The decoders take the stream's size and skip blocks
 * whose block_info row or header points outside it. */
int pkv_k_encode_p(const uint8_t *codes, uint8_t *stream, uint64_t capacity, uint32_t *block_info, int ctx_len,
                   int hidden_dim, int pack_len, int bits, uint64_t *size_out, float *ms_out, pkv_stream_t s);
int pkv_v_encode_p(const uint8_t *codes, uint8_t *stream, uint64_t capacity, uint32_t *block_info, int ctx_len,
                   int hidden_dim, int pack_len, int bits, uint64_t *size_out, float *ms_out, pkv_stream_t s);
int pkv_k_decode_p(const uint8_t *stream, uint64_t stream_bytes, const uint32_t *block_info, uint8_t *codes, int ctx_len,
                   int hidden_dim, int pack_len, int bits, float *ms_out, pkv_stream_t s);
int pkv_v_decode_p(const uint8_t *stream, uint64_t stream_bytes, const uint32_t *block_info, uint8_t *codes, int ctx_len,
                   int hidden_dim, int pack_len, int bits, float *ms_out, pkv_stream_t s);
/* Worst-case bytes of one block with packs of pack_len tokens (K and V blocks both hold 512 packs). */
uint64_t pkv_block_bound_p(int pack_len, int bits);

/* ---- per-token affine quantizer ------------------------------------------------------
 * Device counterpart of quant_ints(..., QuantMode.TokenQuant) and of the dequantisation
 * (code + zero) * scale (utils/compute.py:84-112, :173-179): x is [B, H, T, 128] in
 * `dtype`; scale and zero are [B, T] in `dtype` (one pair per batch and token, shared by
 * all heads and channels); every intermediate is rounded to `dtype` exactly where the
 * PyTorch op chain rounds it.  `codes` is the uint8 code matrix [T, B*H*128].
 * `max_code_out` (device uint32, may be NULL) receives the largest code produced. */
int pkv_quant_params(const void *x, int dtype, int B, int H, int T, float rel, void *scale, void *zero,
                     float *ms_out, pkv_stream_t s);
int pkv_quantize(const void *x, int dtype, int B, int H, int T, const void *scale, const void *zero,
                 uint8_t *codes, uint32_t *max_code_out, float *ms_out, pkv_stream_t s);
int pkv_dequantize(const uint8_t *codes, int dtype, int B, int H, int T, const void *scale,
                   const void *zero, void *x_out, float *ms_out, pkv_stream_t s);

/* ---- fused quantize + encode (the encode hot path) -----------------------------------
 * x [B, H, T, 128] `dtype` -> stream + block_info + scale/zero [B, T], never materialising
 * the code matrix.  Same stream as pkv_quant_params + pkv_quantize + pkv_{k,v}_encode.
 * K uses blocks of 64 x 128, V blocks of 128 x 64 (the shapes the reference's kernels
 * consume, src/kernels.cu:564-589, :795-818).  `bits` is the raw code width W: 2..4, and the
 * extension widths 5 and 6 (7 and 8 go through pkv_quant_params + pkv_quantize +
 * pkv_{k,v}_encode); a code that does not fit W bits raises PKV_ERR_UNSUPPORTED when size_out
 * is requested. */
int pkv_k_quant_encode(const void *x, int dtype, int B, int H, int T, float rel, int bits, uint8_t *stream,
                       uint64_t capacity, uint32_t *block_info, void *scale, void *zero,
                       uint64_t *size_out, float *ms_out, pkv_stream_t s);
int pkv_v_quant_encode(const void *x, int dtype, int B, int H, int T, float rel, int bits, uint8_t *stream,
                       uint64_t capacity, uint32_t *block_info, void *scale, void *zero,
                       uint64_t *size_out, float *ms_out, pkv_stream_t s);

/* ---- incremental encode: append T_new more tokens to an existing stream ----------------
 * For a cache that grows (models/cache/packkv_quant.py:45-85 re-quantizes each cut of the
 * buffer, utils/compute.py:54-67; per-token parameters make a chunked encode produce the
 * codes of a one-shot encode).  x [B, H, T_new, 128] are the new tokens (T_new a multiple
 * of 64 for K, 128 for V).  Their blocks are written back-to-back from byte `stream_used`
 * of `stream`; `block_info_tail` points at the entry after the last existing block (entries
 * hold offsets from the start of `stream`), `scale_tail` / `zero_tail` at the first new
 * token of row 0 of arrays [B, par_stride].  Appending chunk after chunk gives the stream,
 * block_info and parameters of one pkv_{k,v}_quant_encode call over all tokens.  size_out
 * receives the bytes in use after the append. */
int pkv_k_quant_encode_append(const void *x, int dtype, int B, int H, int T_new, float rel, int bits,
                               uint8_t *stream, uint64_t capacity, uint64_t stream_used, uint32_t *block_info_tail,
                               void *scale_tail, void *zero_tail, int par_stride, uint64_t *size_out,
                               float *ms_out, pkv_stream_t s);
int pkv_v_quant_encode_append(const void *x, int dtype, int B, int H, int T_new, float rel, int bits,
                               uint8_t *stream, uint64_t capacity, uint64_t stream_used, uint32_t *block_info_tail,
                               void *scale_tail, void *zero_tail, int par_stride, uint64_t *size_out,
                               float *ms_out, pkv_stream_t s);

/* ---- the decode step's write into a cache's 16-bit window ------------------------------
 * pkv_window_append: rows win_pos .. win_pos + n - 1 of the windows k_win / v_win [B, H, win_stride, 128] receive the
 * new tokens k_new / v_new [B, H, n, 128] (element strides stride_b / stride_h / stride_t, channels contiguous; the
 * same for both).  With cos / sin [B, n, 128] (batch stride rot_stride_b elements, 0 for one shared table) the K rows
 * get the rotary embedding first, rounded like the reference's chain of 16-bit elementwise kernels
 * (`apply_rotary_pos_emb_single`, utils/compute.py:35-43, applied by the cache itself,
 * models/cache/packkv_quant.py:59-60); cos = sin = NULL copies K as it is.  Stands in for that embedding plus the
 * torch.cat growth of the reference's buffer (packkv_quant.py:62-83) on a decode step that cuts nothing. */
int pkv_window_append(const void *k_new, const void *v_new, const void *cos, const void *sin, int dtype, int B, int H,
                      int n, int64_t stride_b, int64_t stride_h, int64_t stride_t, int64_t rot_stride_b, void *k_win,
                      void *v_win, int win_pos, int win_stride, pkv_stream_t s);

/* ---- token repacking and the analytic pack-size model ---------------------------------
 * On the uint8 code matrix [ctx_len, hidden_dim] (channel = (b * H + h) * 128 + d).
 * pkv_bit_pack_size (utils/compute.py:272-297, `bit_pack`, one of its two halves): packs are
 *   `pack_len` consecutive tokens of one channel; returns  len_sum = sum over packs of
 *   bit_length(max - min)  and the number of distinct code values, from which the caller forms
 *   bytes = (len_sum * pack_len + n_packs * (W + ceil(log2(W + 1)))) / 8,  W = ceil(log2(n_unique)).
 * pkv_median_repack (utils/compute.py:262-270, `median_repacking`): inside every block of
 *   `block_size` tokens the tokens of K and V are reordered together by descending lower median
 *   of the token's V codes over all hidden_dim channels.  Equal medians keep their original order
 *   (the reference leaves that order to torch.sort's backend).  perm[blk * block_size + r] is
 *   the index inside the block of the token that moves to position r. */
/* Median repacking inside the fused encode (north-star "quantize, token repack, bit-pack" as one encode; reference
 * order utils/compute.py:329-357: quantise, repack, bit-pack): no code matrix is formed.
 * pkv_median_order: the permutation pkv_median_repack would produce for V [B, H, T, 128] quantised at `rel` -- the
 *   medians are counted straight from V (every value quantised in registers).  H <= 8, bits 2..6.  scale_out /
 *   zero_out (both or neither; [B, T] of V's type) receive V's per-token parameters as pkv_quant_params writes them.
 * pkv_{k,v}_quant_encode_perm: pkv_{k,v}_quant_encode on the tokens in that order: position p of the stream, of
 *   block_info's blocks and of scale / zero holds token (p / perm_block) * perm_block + perm[p] of x (perm_block a
 *   multiple of 64 that divides T).  The stream equals pkv_quant_params + pkv_quantize + pkv_median_repack +
 *   pkv_{k,v}_encode.  H <= 8.  The V form takes the parameters pkv_median_order wrote (scale_in / zero_in, [B, T]
 *   in the order of x; both NULL: computed again) and then reads V once instead of going over every row twice.
 *   No counterpart in the reference, which repacks only to price the packs. */
int pkv_median_order(const void *v, int dtype, int B, int H, int T, float rel, int bits, int block_size, uint32_t *perm,
                     void *scale_out, void *zero_out, float *ms_out, pkv_stream_t s);
int pkv_k_quant_encode_perm(const void *x, int dtype, int B, int H, int T, float rel, int bits, const uint32_t *perm,
                            int perm_block, uint8_t *stream, uint64_t capacity, uint32_t *block_info, void *scale,
                            void *zero, uint64_t *size_out, float *ms_out, pkv_stream_t s);
int pkv_v_quant_encode_perm(const void *x, int dtype, int B, int H, int T, float rel, int bits, const uint32_t *perm,
                            int perm_block, const void *scale_in, const void *zero_in, uint8_t *stream, uint64_t capacity,
                            uint32_t *block_info, void *scale, void *zero, uint64_t *size_out, float *ms_out, pkv_stream_t s);
int pkv_bit_pack_size(const uint8_t *codes, int ctx_len, int hidden_dim, int pack_len, uint64_t *len_sum_out,
                      uint32_t *n_unique_out, float *ms_out, pkv_stream_t s);
int pkv_median_repack(const uint8_t *k_codes, const uint8_t *v_codes, uint8_t *k_out, uint8_t *v_out, uint32_t *perm,
                      int ctx_len, int hidden_dim, int block_size, float *ms_out, pkv_stream_t s);
/* pkv_greedy_repack (utils/compute.py:210-260, `greedy_repacking`, with `_batched_pick` :186-208): every block of
 *   `block_size` tokens (at most 256, a multiple of pack_len) is rebuilt pack by pack -- a pack starts from the
 *   remaining token with the largest cosine to the rounded mean of the remaining tokens (rows = K codes then V
 *   codes of all channels) and then takes, pack_len - 1 times, the remaining token that adds the fewest payload
 *   bits, sum over channels of bit_length(max - min).  Integer arithmetic throughout, cosines compared exactly,
 *   every tie to the earlier token (the reference computes both criteria in fp32 and leaves ties to the backend).
 *   Same outputs as pkv_median_repack.  Blocks of up to 64 tokens keep their rows in registers (any hidden_dim whose
 *   channel slices fit the device at once as one group of workgroups); longer blocks need hidden_dim <= 32768.
 *   With ms_out the call waits for the kernels and also reports a device-side failure of the group exchange.
 *   k_out = v_out = NULL: the order only (perm), for the fused encoders' pkv_*_quant_encode_perm. */
int pkv_greedy_repack(const uint8_t *k_codes, const uint8_t *v_codes, uint8_t *k_out, uint8_t *v_out, uint32_t *perm,
                      int ctx_len, int hidden_dim, int block_size, int pack_len, float *ms_out, pkv_stream_t s);

/* ---- the reference's GEMV surface -----------------------------------------------------
 * kq_mat_vec_mul (packkv_cuda.pyi:26-36, src/kernels.cu:611-630):
 *     kq_out[h, tok] = sum_d q[h, d] * code[tok, h*128 + d]        (dtype, [H, ctx_len])
 *   q_interleaved != 0: q is in the lane order the reference kernel expects
 *   (evaluation/evaluation.py:465-468); 0: plain [H, 128].
 * wv_mat_vec_mul (packkv_cuda.pyi:60-70, src/kernels.cu:840-859):
 *     wv_out[c] += sum_tok w[c / 128, tok] * code[tok, c]          (fp32 [hidden_dim], caller
 *   zeroes it; accumulated with atomics like the reference, src/kernels.cu:756-763)
 * fused_kq (packkv_cuda.pyi:72-78, src/fused_kernels.cu:13-76):
 *     our_kq[m, n] = (sum_d q[m, d] * zero[n] + t[m, n]) * scale[n]
 * fused_wv (packkv_cuda.pyi:80-86, src/fused_kernels.cu:187-261):
 *     our_wv[m, d] = sum_n w[m, n] * zero[n] * scale[n] + term1[m, d]
 * Any head count M and any hidden_dim multiple of 128 are accepted (the reference
 * instantiates hidden_dim in {5120, 1024}, M in {40, 8} only). */
int pkv_kq_mat_vec_mul(const uint8_t *stream, uint64_t stream_bytes, const uint32_t *block_info, const void *q, void *kq_out,
                       int ctx_len, int hidden_dim, int ctx_blk, int hid_blk, int bits, int dtype,
                       int q_interleaved, float *ms_out, pkv_stream_t s);
int pkv_wv_mat_vec_mul(const uint8_t *stream, uint64_t stream_bytes, const uint32_t *block_info, const void *w, float *wv_out,
                       int ctx_len, int hidden_dim, int ctx_blk, int hid_blk, int bits, int dtype,
                       float *ms_out, pkv_stream_t s);
int pkv_fused_kq(void *our_kq, const void *q, const void *k_zero, const void *k_scale, const void *t, int M,
                 int K, int N, int dtype, float *ms_out, pkv_stream_t s);
int pkv_fused_wv(void *our_wv, const void *w, const void *v_zero, const void *v_scale, const void *term1,
                 int M, int N, int D, int dtype, float *ms_out, pkv_stream_t s);

/* ---- fused decompress-attention decode ------------------------------------------------
 * One decode step over a compressed cache, without materialising K or V:
 *   out[b, hq, :] = softmax_t( sm_scale * q[b, hq, :] . K[b, hq / G, t, :] ) @ V[b, hq / G, t, :]
 * with K = (k_code + k_zero) * k_scale, V likewise, G = Hq / Hkv, fp32 accumulation.
 * It fuses what the reference runs as kq_mat_vec_mul -> fused_kq -> softmax
 * (models/llama.py:202-209) -> w * v_scale (evaluation/evaluation.py:661) ->
 * wv_mat_vec_mul -> fused_wv, and adds the batch and GQA-group dimensions.
 *
 *   k_stream/k_info   K stream of the code matrix [T_c, B*Hkv*128], blocks 64 x 128
 *   v_stream/v_info   V stream of the same shape, blocks 128 x 64
 *   k_bytes, v_bytes  readable bytes of each stream BUFFER (below 4 GiB).  The kernels never read past
 *                     this (rounded up to a whole dword), whatever block_info says.  The default
 *                     kernel and variant 1 take a buffer that ends with its stream; variant 2 (and
 *                     variant 0 on streams that are not 16-byte aligned, which runs it) fetches pack
 *                     words as whole 8-byte words, so for it the buffer must extend at least 7 bytes
 *                     past the encoded size (size_out of the encoder) or the last block decodes wrongly
 *   k_scale..v_zero   [B, T_c] `dtype`
 *   q, out            [B, Hq, 128] `dtype`
 *   k_win, v_win      optional uncompressed tail [B, Hkv, T_w, 128] `dtype`, k_win 16-byte aligned (the residual
 *                     window the cache keeps in 16-bit, utils/compute.py:54-67); T_w may be 0
 *   T_c               compressed tokens, a multiple of 128 (may be 0 when T_w > 0)
 *   par_stride        tokens per row of the scale / zero arrays when they are allocated longer than
 *                     T_c (a cache that grows); 0 = T_c
 *   win_stride        tokens per (sequence, KV head) row of k_win / v_win; 0 = T_w
 *   variant           0 = default (asynchronous-copy matrix-core kernel; streams must be 16-byte
 *                     aligned, otherwise variant 2 runs); 1 = plain VALU kernel; 2 = matrix-core
 *                     kernel that gathers straight from global memory.  All three implement the
 *                     same contract; tests cross-check them.  The matrix-core kernels take the reference's
 *                     widths (k_bits, v_bits in 2..4, any mix); variant 0 also takes the extension widths 5
 *                     and 6 on either side with 4, 5 or 6 on the other.  Any other combination with an
 *                     extension width runs the plain kernel whatever `variant` says.
 *   flags             PKV_ATTN_OUT_F32: `out` is [B, Hq, 128] fp32 instead of `dtype` (the result before its
 *                     rounding to 16 bits).  PKV_ATTN_REF_ROUNDING (variant 1 only, otherwise PKV_ERR_INVALID):
 *                     decompress-then-attend to the letter -- every K and V element is formed as the reference
 *                     stores it, dtype(dtype(code + zero) * scale) (utils/compute.py:173-179), before the fp32
 *                     dot products, instead of folding scale and zero into the scores and weights.  This is the
 *                     checking mode: slow, and equal to the reference path up to fp32 summation order.
 */
#define PKV_ATTN_REF_ROUNDING 1
#define PKV_ATTN_OUT_F32 2

typedef struct pkv_attn_args {
    const uint8_t *k_stream;
    const uint32_t *k_info;
    const uint8_t *v_stream;
    const uint32_t *v_info;
    uint64_t k_bytes, v_bytes;
    const void *k_scale, *k_zero, *v_scale, *v_zero;
    const void *q;
    void *out;
    const void *k_win, *v_win;
    int B, Hq, Hkv, T_c, T_w;
    int k_bits, v_bits;
    int dtype;
    float sm_scale;
    int variant;
    int par_stride, win_stride;
    int flags;
} pkv_attn_args;

int pkv_attn_decode(const pkv_attn_args *args, float *ms_out, pkv_stream_t s);

/* pkv_attn_decode_noalloc: pkv_attn_decode for callers that cannot allocate device memory -- code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference.  Same
 * arguments, kernels and results, but the per-split partial results ([B, Hq, partials, 130] fp32) and the tile
 * counters, which pkv_attn_decode keeps in memory the library allocates per stream and grows on demand, live in a
 * fixed 8 MiB device array inside the library (7.75 MiB of it for the partials); the call allocates and frees
 * nothing and creates no events (hence no ms_out).  A step whose partials do not fit is rejected with
 * PKV_ERR_UNSUPPORTED and a message (B * Hq * partials * 520 bytes; partials = splits, twice that with a tail
 * window; splits ~ 1024 / (B * Hkv), at most T_c / 128).  All calls on one GPU share the one array: calls that
 * overlap on a GPU (two streams, two threads) race; calls on one stream are ordered.  Every partial a launch reads
 * was written by that launch and the counters are left at zero, so nothing needs clearing between calls.
 * pkv_attn_decode itself uses the same array when its stream is capturing a graph and has no scratch of its own. */
int pkv_attn_decode_noalloc(const pkv_attn_args *args, pkv_stream_t s);

/* pkv_stream_release: gives back the device memory the library keeps for stream `s` of the current device -- its
 * scratch buffers (attention partials, the encoders' look-back state), its tile counters and every buffer it has
 * outgrown (kept until now because a captured HIP graph might still hold its address).  It has no counterpart in the
 * reference (whose extension allocates per call through torch).  Call it before destroying a stream the library has
 * been used on -- a server that creates and destroys streams would otherwise accumulate one workspace per stream
 * handle -- and only when no graph captured on `s` will be replayed again.  Waits for the stream's work; a stream the
 * library has never seen is not an error.  The stream can be used with the library again afterwards (its scratch is
 * allocated afresh). */
int pkv_stream_release(pkv_stream_t s);

#ifdef __cplusplus
}
#endif
#endif /* PACKKV_H */
