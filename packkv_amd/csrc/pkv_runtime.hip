// Host-side runtime for the C-ABI library: last-error text, scratch, launch timing.
#include "pkv_block.hpp"
#include "pkv_runtime.hpp"
#include <utility>
#include <tuple>
#include <map>

#include <cstdarg>
#include <cstdio>
#include <mutex>
#include <vector>

namespace pkv {

static thread_local char g_error[512] = "";

void set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

namespace {
// One workspace per (device, stream): calls on different streams of one device never share scratch, so they may
// overlap.  A buffer that has been handed out is never freed or moved while the process lives: a request for more
// allocates a larger buffer beside it and retires the old one (a captured HIP graph may still hold its address), so
// growth costs memory (at most twice the largest request, growth is geometric) but never a synchronisation.
struct Workspace {
    int dev;
    hipStream_t stream;
    void *ptr[2];           // kScratchGeneral, kScratchEncoder
    size_t bytes[2];
    uint32_t *counters;     // kAttnCounters tile counters of the attention kernel, zero between launches
    bool encoded;           // an encoder has run on this stream: ptr[kScratchEncoder] starts with its ScanState
};
std::vector<Workspace> g_ws;
struct Retired { int dev; hipStream_t stream; void *ptr; };
std::vector<Retired> g_retired;     // superseded buffers, kept until their stream is released (a captured graph may hold them)
std::mutex g_ws_mu;

int workspace_for(hipStream_t s, Workspace **out) {     // caller holds g_ws_mu
    int dev = 0;
    PKV_HIP_CHECK(hipGetDevice(&dev));
    for (Workspace &w : g_ws)
        if (w.dev == dev && w.stream == s) { *out = &w; return PKV_OK; }
    g_ws.push_back(Workspace{dev, s, {nullptr, nullptr}, {0, 0}, nullptr, false});
    *out = &g_ws.back();
    return PKV_OK;
}
}  // namespace

size_t scratch_grown_size(size_t have, size_t want) {
    if (want <= have) return have;
    size_t n = have ? have : (size_t)(1 << 20);
    while (n < want) n += n / 2 + (size_t)(1 << 20);
    return n;
}

// True when `s` is recording a HIP graph: nothing may be allocated then.
static bool capturing(hipStream_t s) {
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    return hipStreamIsCapturing(s, &st) == hipSuccess && st != hipStreamCaptureStatusNone;
}

int scratch_get(size_t bytes, hipStream_t s, void **out, int kind) {
    std::lock_guard<std::mutex> lock(g_ws_mu);
    Workspace *w = nullptr;
    int rc = workspace_for(s, &w);
    if (rc) return rc;
    if (kind == kScratchEncoder) w->encoded = true;
    if (w->bytes[kind] < bytes) {
        if (capturing(s)) {
            set_error("stream is capturing a graph and has no scratch buffer of %zu bytes yet: make one eager call "
                      "of the same shape on this stream first", bytes);
            return PKV_ERR_CAPTURING;
        }
        const size_t want = scratch_grown_size(w->bytes[kind], bytes);
        void *fresh = nullptr;
        PKV_HIP_CHECK(hipMalloc(&fresh, want));
        if (w->ptr[kind]) g_retired.push_back(Retired{w->dev, s, w->ptr[kind]});
        w->ptr[kind] = fresh;
        w->bytes[kind] = want;
    }
    *out = w->ptr[kind];
    return PKV_OK;
}

int encoder_state_peek(hipStream_t s, void **out) {
    std::lock_guard<std::mutex> lock(g_ws_mu);
    Workspace *w = nullptr;
    int rc = workspace_for(s, &w);
    if (rc) return rc;
    PKV_REQUIRE(w->encoded && w->ptr[kScratchEncoder], PKV_ERR_INVALID, "no encode has been launched on this stream");
    *out = w->ptr[kScratchEncoder];
    return PKV_OK;
}

int attn_counters_get(hipStream_t s, uint32_t **out) {
    std::lock_guard<std::mutex> lock(g_ws_mu);
    Workspace *w = nullptr;
    int rc = workspace_for(s, &w);
    if (rc) return rc;
    if (!w->counters) {
        if (capturing(s)) {
            set_error("stream is capturing a graph and has no attention counters yet: make one eager call on this "
                      "stream first");
            return PKV_ERR_CAPTURING;
        }
        void *c = nullptr;
        PKV_HIP_CHECK(hipMalloc(&c, (size_t)kAttnCounters * sizeof(uint32_t)));
        PKV_HIP_CHECK(hipMemset(c, 0, (size_t)kAttnCounters * sizeof(uint32_t)));
        w->counters = (uint32_t *)c;
    }
    *out = w->counters;
    return PKV_OK;
}

// Gives back everything the library holds for (current device, stream `s`): waits for the stream, frees its scratch
// buffers, its tile counters and the buffers it has outgrown, and forgets the stream.
int stream_release(hipStream_t s) {
    std::lock_guard<std::mutex> lock(g_ws_mu);
    int dev = 0;
    PKV_HIP_CHECK(hipGetDevice(&dev));
    PKV_REQUIRE(!capturing(s), PKV_ERR_INVALID, "the stream is capturing a graph");
    size_t at = g_ws.size();
    for (size_t i = 0; i < g_ws.size(); i++)
        if (g_ws[i].dev == dev && g_ws[i].stream == s) at = i;
    bool any = at < g_ws.size();
    for (const Retired &r : g_retired) any = any || (r.dev == dev && r.stream == s);
    if (!any) return PKV_OK;
    PKV_HIP_CHECK(hipStreamSynchronize(s));
    if (at < g_ws.size()) {
        Workspace &w = g_ws[at];
        for (int k = 0; k < 2; k++)
            if (w.ptr[k]) PKV_HIP_CHECK(hipFree(w.ptr[k]));
        if (w.counters) PKV_HIP_CHECK(hipFree(w.counters));
        g_ws.erase(g_ws.begin() + (long)at);
    }
    for (size_t i = 0; i < g_retired.size();) {
        if (g_retired[i].dev == dev && g_retired[i].stream == s) {
            PKV_HIP_CHECK(hipFree(g_retired[i].ptr));
            g_retired.erase(g_retired.begin() + (long)i);
        } else {
            i++;
        }
    }
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

int stagger_for(const void *kernel, int threads, uint32_t lds, uint32_t nwg, Stagger *out) {
    out->cus = out->slots = 0u;
    if (nwg < 1024u) return PKV_OK;                         // the appends of a growing cache: a handful of workgroups
    int dev = 0, cus = 0, per_cu = 0;
    PKV_HIP_CHECK(hipGetDevice(&dev));
    {   // the two figures are looked up once per (device, kernel, LDS size)
        static std::mutex mu;
        static std::map<std::tuple<int, const void *, uint32_t>, std::pair<int, int>> known;
        std::lock_guard<std::mutex> lock(mu);
        const auto key = std::make_tuple(dev, kernel, lds);
        auto it = known.find(key);
        if (it == known.end()) {
            PKV_HIP_CHECK(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
            PKV_HIP_CHECK(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, threads, (size_t)lds));
            it = known.emplace(key, std::make_pair(cus, per_cu)).first;
        }
        cus = it->second.first;
        per_cu = it->second.second;
    }
    if (cus > 0 && per_cu > 1 && (uint64_t)nwg >= 4ull * (uint64_t)cus * (uint64_t)per_cu) {
        out->cus = (uint32_t)cus;
        out->slots = (uint32_t)per_cu;
    }
    return PKV_OK;
}

}  // namespace pkv

extern "C" {

int pkv_abi_version(void) { return PKV_ABI_VERSION; }

const char *pkv_last_error(void) { return pkv::g_error; }

}  // extern "C"

extern "C" int pkv_stream_release(pkv_stream_t s) { return pkv::stream_release((hipStream_t)s); }
