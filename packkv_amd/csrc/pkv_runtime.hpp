// Host-side runtime shared by the C-ABI entry points: last-error text, per-device scratch
// for the single-pass encoders, and event-based timing of a launch.
#pragma once
#include "pkv_common.hpp"

namespace pkv {

// A device buffer of at least `bytes` that belongs to (current device, stream `s`): calls on different streams get
// different buffers and may overlap; calls on one stream share it and are ordered by the stream.  Buffers grow on
// demand; one that has been handed out is never freed or moved while the process lives (a larger one is allocated
// beside it), so an address captured in a HIP graph stays valid and growing never synchronises.
// While `s` is capturing a HIP graph nothing can be allocated: a request the stream's buffer cannot serve then
// returns PKV_ERR_CAPTURING (library-internal; callers fall back or report it as PKV_ERR_HIP).
constexpr int PKV_ERR_CAPTURING = 100;
// Two buffers per stream: the encoders' look-back state has one of its own, so that it (and the status it ends with)
// survives whatever else runs on the stream until the next encode.
constexpr int kScratchGeneral = 0, kScratchEncoder = 1;
int scratch_get(size_t bytes, hipStream_t s, void **out, int kind = kScratchGeneral);
// Start of the encoder-state buffer of stream `s` (the ScanState of the last encode launched on it).
int encoder_state_peek(hipStream_t s, void **out);
// Capacity after growing a buffer of `have` bytes to hold `want` (geometric, at least 1 MiB): host arithmetic only.
size_t scratch_grown_size(size_t have, size_t want);

// Tile counters of the attention kernel for (current device, stream `s`): kAttnCounters zeroed 32-bit words,
// allocated on first use; the attention kernel leaves every counter it used at zero again.
constexpr int kAttnCounters = 65536;
int attn_counters_get(hipStream_t s, uint32_t **out);
int stream_release(hipStream_t s);

// Per-call timing: records start/stop events on `stream` around fn() and returns elapsed ms
// after synchronising on the stop event (mirrors the reference launchers, which time every
// launch with events and return milliseconds: packkv_cuda_ext/src/kernels.cu:560-608).
struct LaunchTimer {
    hipEvent_t start = nullptr, stop = nullptr;
    hipStream_t stream;
    bool enabled;
    LaunchTimer(hipStream_t s, bool on) : stream(s), enabled(on) {}
    int begin();
    int end(float *ms_out);   // synchronises when enabled
    ~LaunchTimer();
};

// perm[blk * block_size + r] = index inside block blk of the token that moves to position r: descending median, equal
// medians in their original order (pkv_repack.hip).
int launch_block_order(const uint8_t *median, int ctx_len, int block_size, uint32_t *perm, hipStream_t s);

struct ScanState;
struct Stagger;
// Zeroed look-back state for `nblocks` blocks, from the per-device scratch.
// The stagger of the first resident generation (stagger_first_generation, pkv_block.hpp) for `kernel` launched with
// `threads` threads and `lds` bytes of dynamic LDS over `nwg` workgroups: CU count and workgroups per CU from the
// occupancy query (looked up once per device, kernel and LDS size); zeros -- no stagger -- for launches of fewer
// than four generations.
int stagger_for(const void *kernel, int threads, uint32_t lds, uint32_t nwg, Stagger *out);
int prepare_scan_state(uint32_t nblocks, ScanState **out, hipStream_t s);
// Reads back {error, total, max_code}; when `size_out` is NULL returns at once (no sync).
// `bits` > 0 additionally rejects a launch whose largest code does not fit `bits` bits.
int finish_encode(ScanState *st, uint64_t *size_out, int bits, hipStream_t s);
// The block codec from a code matrix through the cells kernels (pkv_quant.hip): eight K / sixteen V blocks per group,
// for hidden a multiple of 1024, the reference's block shapes, widths up to 6.  `st` holds one status word per group.
int launch_code_cells(bool is_k, const uint8_t *codes, int ctx_len, int hidden, int bits, uint32_t bound, uint8_t *stream,
                      uint64_t capacity, uint32_t *info, ScanState *st, uint32_t ngroups, hipStream_t s);

}  // namespace pkv
