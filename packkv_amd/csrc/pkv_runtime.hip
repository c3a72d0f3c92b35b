// Host-side runtime for the C-ABI library: last-error text, scratch, launch timing.
#include "pkv_runtime.hpp"

#include <cstdarg>
#include <cstdio>
#include <mutex>

namespace pkv {

static thread_local char g_error[512] = "";

void set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

namespace {
constexpr int kMaxDevices = 16;
struct Scratch { void *ptr = nullptr; size_t bytes = 0; };
Scratch g_scratch[kMaxDevices];
std::mutex g_scratch_mu;
}  // namespace

int scratch_get(size_t bytes, void **out) {
    int dev = 0;
    PKV_HIP_CHECK(hipGetDevice(&dev));
    PKV_REQUIRE(dev >= 0 && dev < kMaxDevices, PKV_ERR_INVALID, "device index %d out of range", dev);
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    Scratch &sc = g_scratch[dev];
    if (sc.bytes < bytes) {
        if (sc.ptr) {
            PKV_HIP_CHECK(hipDeviceSynchronize());
            PKV_HIP_CHECK(hipFree(sc.ptr));
            sc.ptr = nullptr;
            sc.bytes = 0;
        }
        size_t want = bytes < (size_t)(1 << 20) ? (size_t)(1 << 20) : bytes + bytes / 4;
        PKV_HIP_CHECK(hipMalloc(&sc.ptr, want));
        sc.bytes = want;
    }
    *out = sc.ptr;
    return PKV_OK;
}

int LaunchTimer::begin() {
    if (!enabled) return PKV_OK;
    PKV_HIP_CHECK(hipEventCreate(&start));
    PKV_HIP_CHECK(hipEventCreate(&stop));
    PKV_HIP_CHECK(hipEventRecord(start, stream));
    return PKV_OK;
}

int LaunchTimer::end(float *ms_out) {
    if (!enabled) return PKV_OK;
    PKV_HIP_CHECK(hipEventRecord(stop, stream));
    PKV_HIP_CHECK(hipEventSynchronize(stop));
    float ms = 0.f;
    PKV_HIP_CHECK(hipEventElapsedTime(&ms, start, stop));
    if (ms_out) *ms_out = ms;
    return PKV_OK;
}

LaunchTimer::~LaunchTimer() {
    if (start) (void)hipEventDestroy(start);
    if (stop) (void)hipEventDestroy(stop);
}

}  // namespace pkv

extern "C" {

int pkv_abi_version(void) { return PKV_ABI_VERSION; }

const char *pkv_last_error(void) { return pkv::g_error; }

}  // extern "C"
