// Host-side runtime shared by the C-ABI entry points: last-error text, per-device scratch
// for the single-pass encoders, and event-based timing of a launch.
#pragma once
#include "pkv_common.hpp"

namespace pkv {

// Returns a device buffer of at least `bytes` on the current device, grown on demand and
// kept until the process ends.  Not safe for concurrent encodes on one device.
int scratch_get(size_t bytes, void **out);

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

struct ScanState;
// Zeroed look-back state for `nblocks` blocks, from the per-device scratch.
int prepare_scan_state(uint32_t nblocks, ScanState **out, hipStream_t s);
// Reads back {error, total, max_code}; when `size_out` is NULL returns at once (no sync).
// `bits` > 0 additionally rejects a launch whose largest code does not fit `bits` bits.
int finish_encode(ScanState *st, uint64_t *size_out, int bits, hipStream_t s);

}  // namespace pkv
