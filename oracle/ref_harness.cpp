// TEST INFRASTRUCTURE ONLY.
// Builds the reference's own scalar CPU codec (the namespace templates in
// packkv_cuda_ext/src/{k,v}_{encode,decode}_cpu.cpp) from the sources where
// they lie under the reference checkout, behind a small C ABI, so that the
// restated oracle and the HIP kernels can be compared with the reference
// byte-for-byte at shapes its Python dispatch does not reach.  Nothing from
// the reference is copied: the sources are #included by path at build time
// (see oracle/Makefile, REF=...), and the result goes to oracle/_ref/.
#include <cstdint>
#include <cstddef>

#include "src/utils.cpp"
#include "src/k_encode_cpu.cpp"
#include "src/k_decode_cpu.cpp"
#include "src/v_encode_cpu.cpp"
#include "src/v_decode_cpu.cpp"

// (W, HIDDEN) grid instantiated for both tensors.
#define PKV_FOR_HIDDEN(X, W) \
    X(W, 128) X(W, 256) X(W, 512) X(W, 1024) X(W, 2048) X(W, 4096) X(W, 5120) X(W, 16384)
#define PKV_FOR_ALL(X) PKV_FOR_HIDDEN(X, 2) PKV_FOR_HIDDEN(X, 3) PKV_FOR_HIDDEN(X, 4)

extern "C" {

// Returns stream bytes, or (uint64_t)-1 when the shape is not instantiated here.
uint64_t pkv_ref_encode(int is_k, const uint8_t *codes, uint8_t *stream, uint32_t *info,
                        int ctx_len, int hidden_dim, int ctx_blk, int hid_blk, int W) {
#define K_CASE(W_, H_) \
    if (is_k && W == W_ && hidden_dim == H_ && hid_blk == 128 && ctx_blk == 64) \
        return k_cpu::k_encode_cpu<W_, H_, 128, 64>(codes, stream, info, (size_t)ctx_len); \
    if (is_k && W == W_ && hidden_dim == H_ && hid_blk == 128 && ctx_blk == 32) \
        return k_cpu::k_encode_cpu<W_, H_, 128, 32>(codes, stream, info, (size_t)ctx_len); \
    if (is_k && W == W_ && hidden_dim == H_ && hid_blk == 128 && ctx_blk == 128) \
        return k_cpu::k_encode_cpu<W_, H_, 128, 128>(codes, stream, info, (size_t)ctx_len);
#define V_CASE(W_, H_) \
    if (!is_k && W == W_ && hidden_dim == H_ && hid_blk == 64 && ctx_blk == 128) \
        return v_cpu::v_encode_cpu<W_, H_, 64, 128>(codes, stream, info, (size_t)ctx_len); \
    if (!is_k && W == W_ && hidden_dim == H_ && hid_blk == 32 && ctx_blk == 128) \
        return v_cpu::v_encode_cpu<W_, H_, 32, 128>(codes, stream, info, (size_t)ctx_len); \
    if (!is_k && W == W_ && hidden_dim == H_ && hid_blk == 128 && ctx_blk == 128) \
        return v_cpu::v_encode_cpu<W_, H_, 128, 128>(codes, stream, info, (size_t)ctx_len);
    PKV_FOR_ALL(K_CASE)
    PKV_FOR_ALL(V_CASE)
#undef K_CASE
#undef V_CASE
    return (uint64_t)-1;
}

int pkv_ref_decode(int is_k, const uint8_t *stream, const uint32_t *info, uint8_t *codes,
                   int ctx_len, int hidden_dim, int ctx_blk, int hid_blk, int W) {
#define K_CASE(W_, H_) \
    if (is_k && W == W_ && hidden_dim == H_ && hid_blk == 128 && ctx_blk == 64) { \
        k_cpu::k_decode_cpu<W_, H_, 128, 64>(stream, info, codes, (size_t)ctx_len); return 0; } \
    if (is_k && W == W_ && hidden_dim == H_ && hid_blk == 128 && ctx_blk == 32) { \
        k_cpu::k_decode_cpu<W_, H_, 128, 32>(stream, info, codes, (size_t)ctx_len); return 0; } \
    if (is_k && W == W_ && hidden_dim == H_ && hid_blk == 128 && ctx_blk == 128) { \
        k_cpu::k_decode_cpu<W_, H_, 128, 128>(stream, info, codes, (size_t)ctx_len); return 0; }
#define V_CASE(W_, H_) \
    if (!is_k && W == W_ && hidden_dim == H_ && hid_blk == 64 && ctx_blk == 128) { \
        v_cpu::v_decode_cpu<W_, H_, 64, 128>(stream, info, codes, (size_t)ctx_len); return 0; } \
    if (!is_k && W == W_ && hidden_dim == H_ && hid_blk == 32 && ctx_blk == 128) { \
        v_cpu::v_decode_cpu<W_, H_, 32, 128>(stream, info, codes, (size_t)ctx_len); return 0; } \
    if (!is_k && W == W_ && hidden_dim == H_ && hid_blk == 128 && ctx_blk == 128) { \
        v_cpu::v_decode_cpu<W_, H_, 128, 128>(stream, info, codes, (size_t)ctx_len); return 0; }
    PKV_FOR_ALL(K_CASE)
    PKV_FOR_ALL(V_CASE)
#undef K_CASE
#undef V_CASE
    return -1;
}

}  // extern "C"
