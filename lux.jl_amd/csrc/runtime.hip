// libluxhip runtime: context, error reporting, streams, events, pooled device memory and
// the per-stream workspace used by the reduction kernels.
#include <stdarg.h>
#include <stdlib.h>
#include <stdio.h>
#include <string.h>

#include <atomic>
#include <map>
#include <string>
#include <mutex>
#include <unordered_map>
#include <vector>

#include "common.h"

namespace luxhip {

namespace {
thread_local char g_err[512] = "";
std::mutex g_mu;
bool g_init = false;
int g_device = -1;
int g_cus = 0;

struct Pool {
    std::multimap<size_t, void*> free_blocks;       // rounded size -> block
    std::unordered_map<void*, size_t> live;         // block -> rounded size
} g_pool;

// A workspace block that has been replaced by a larger one: kernels queued before the switch may
// still use it until `done` has passed.
struct RetiredBlock {
    void* p;
    size_t bytes;
    hipEvent_t done;
};
struct WsEntry {
    void* base = nullptr;
    size_t data_bytes = 0;
    uint32_t* counters = nullptr;   // kWorkspaceCounters words, zero between kernels, then kWorkspaceFlags words
    uint32_t epoch = 0;
    std::vector<RetiredBlock> retired;
    bool recorded = false;          // a graph recorded on this stream holds the address of `base`
    std::vector<void*> pinned;      // outgrown blocks that recorded graphs still write to: kept until luxhip_shutdown
};
std::map<hipStream_t, WsEntry> g_ws;
std::vector<void*> g_pinned;        // pinned blocks of destroyed streams (a graph outlives the stream it was recorded on)

// One event is recorded after every profiled launch; a launch that directly follows another
// profiled launch on the same stream takes that event as its start, so a launch costs one event
// record and its time runs from the end of its predecessor to its own end (the kernel plus the gap
// between dependent launches).  Exact scopes hand two events to the dispatch itself instead
// (hipExtLaunchKernelGGL): the time between them is the kernel's alone, what a kernel trace reports.
struct ProfEntry {
    const char* name;
    hipStream_t stream;
    int a, b;   // indices into g_prof_events, b < 0 while the scope is open
};
bool g_prof = false;
std::vector<ProfEntry> g_prof_entries;
std::vector<hipEvent_t> g_prof_events;

size_t round_size(size_t b) {
    if (b == 0) b = 1;
    if (b <= (1u << 20)) return (b + 511) & ~size_t(511);               // 512 B granules
    return (b + (size_t(2) << 20) - 1) & ~((size_t(2) << 20) - 1);      // 2 MiB granules
}
}  // namespace

static int prof_record(hipStream_t s) {   // g_mu held
    hipEvent_t e;
    if (hipEventCreate(&e) != hipSuccess) return -1;
    if (hipEventRecord(e, s) != hipSuccess) { (void)hipEventDestroy(e); return -1; }
    g_prof_events.push_back(e);
    return (int)g_prof_events.size() - 1;
}
ProfScope::ProfScope(const char* n, hipStream_t s, bool exact) : name(n), stream(s), active(g_prof) {
    if (!active) return;
    std::lock_guard<std::mutex> lk(g_mu);
    if (exact) {
        hipEvent_t a = nullptr, b = nullptr;
        if (hipEventCreate(&a) != hipSuccess) { active = false; return; }
        if (hipEventCreate(&b) != hipSuccess) { (void)hipEventDestroy(a); active = false; return; }
        g_prof_events.push_back(a);
        g_prof_events.push_back(b);
        g_prof_entries.push_back(ProfEntry{n, s, (int)g_prof_events.size() - 2, (int)g_prof_events.size() - 1});
        start = a;
        stop = b;
        return;
    }
    int a = -1;
    if (!g_prof_entries.empty() && g_prof_entries.back().stream == s && g_prof_entries.back().b >= 0)
        a = g_prof_entries.back().b;
    else
        a = prof_record(s);
    if (a < 0) { active = false; return; }
    g_prof_entries.push_back(ProfEntry{n, s, a, -1});
}
ProfScope::~ProfScope() {
    if (!active || start != nullptr) return;
    std::lock_guard<std::mutex> lk(g_mu);
    // the matching entry is the last one with this name still open
    for (auto it = g_prof_entries.rbegin(); it != g_prof_entries.rend(); ++it)
        if (it->name == name && it->b < 0) { it->b = prof_record(stream); break; }
}

int set_error(int status, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return status;
}

bool initialized() { return g_init; }
int num_cus() { return g_cus; }

namespace {
std::atomic<int64_t> g_opt_bn_resident{1}, g_opt_bn_spin_limit{int64_t(1) << 22}, g_opt_gemm_tile{-1}, g_opt_conv_tile{0},
    g_opt_gemm_pretranspose{1};
}
int64_t option_bn_resident() { return g_opt_bn_resident.load(); }
int64_t option_bn_spin_limit() { return g_opt_bn_spin_limit.load(); }
int64_t option_conv_tile() { return g_opt_conv_tile.load(); }
int64_t option_gemm_pretranspose() { return g_opt_gemm_pretranspose.load(); }
int64_t option_gemm_tile() {
    int64_t v = g_opt_gemm_tile.load();
    if (v < 0) {   // not set through the API: the environment variable LUXHIP_GEMM_TILE, read once
        const char* e = getenv("LUXHIP_GEMM_TILE");
        v = e ? atoll(e) : 0;
        g_opt_gemm_tile.store(v);
    }
    return v;
}

__global__ void fill_zero_kernel(uint32_t* p, size_t nwords);
int noalloc_setup(int device);   // elementwise.hip: device address of the fixed scratch block

bool stream_capturing(hipStream_t s) {
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(s, &st) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    return st != hipStreamCaptureStatusNone;
}

// Retired blocks whose last kernels have finished go to the allocator's pool: no wait and no hipFree
// (which would synchronise the device) on an operator's path.  g_mu held.
static void collect_retired(WsEntry& e, bool wait) {
    for (size_t i = 0; i < e.retired.size();) {
        RetiredBlock& r = e.retired[i];
        if (wait) (void)hipEventSynchronize(r.done);
        if (wait || hipEventQuery(r.done) == hipSuccess) {
            (void)hipEventDestroy(r.done);
            g_pool.free_blocks.emplace(r.bytes, r.p);
            e.retired[i] = e.retired.back();
            e.retired.pop_back();
        } else {
            (void)hipGetLastError();   // hipErrorNotReady is not an error here
            ++i;
        }
    }
}

// The workspace never makes the host wait for the device: a block that has become too small is
// retired behind an event on the stream and a new one is taken from the pool or the driver.  While
// the stream records a graph nothing may be allocated (and an allocation inside a recording would
// be replayed as a stale pointer): the caller sizes the workspace before, with one eager call of
// the operator or luxhip_reserve.
int get_workspace(hipStream_t s, size_t bytes, Workspace* out) {
    std::lock_guard<std::mutex> lk(g_mu);
    WsEntry& e = g_ws[s];
    if (!e.retired.empty()) collect_retired(e, false);
    const bool grow = e.base == nullptr || e.data_bytes < bytes;
    const bool capturing = stream_capturing(s);
    if (capturing) e.recorded = true;
    if ((grow || e.counters == nullptr) && capturing)
        return set_error(LUXHIP_INVALID,
                         "the stream is recording a graph and its workspace (%zu bytes) is smaller than the %zu bytes this call "
                         "needs: call luxhip_reserve(stream, bytes) or run the operator once eagerly before recording",
                         e.data_bytes, bytes);
    if (grow) {
        const size_t want = bytes < (size_t(8) << 20) ? (size_t(8) << 20) : round_size(bytes);
        void* p = nullptr;
        auto it = g_pool.free_blocks.find(want);
        if (it != g_pool.free_blocks.end()) {
            p = it->second;
            g_pool.free_blocks.erase(it);
        } else {
            hipError_t rc = hipMalloc(&p, want);
            if (rc != hipSuccess) {
                // out of memory: give the pooled blocks back to the driver and try once more, as luxhip_malloc does
                (void)hipGetLastError();
                for (auto& kv : g_pool.free_blocks) (void)hipFree(kv.second);
                g_pool.free_blocks.clear();
                rc = hipMalloc(&p, want);
            }
            LUX_CHECK_HIP(rc);
        }
        if (e.base != nullptr && e.recorded) {
            // a graph recorded on this stream has the old block's address in its kernels: the block is
            // never handed out again, so a replay still writes to memory that nobody else owns
            e.pinned.push_back(e.base);
            e.recorded = false;
        } else if (e.base != nullptr) {
            // the old block may still be in use by kernels queued on this stream
            hipEvent_t done;
            hipError_t rc = hipEventCreateWithFlags(&done, hipEventDisableTiming);
            if (rc == hipSuccess) rc = hipEventRecord(done, s);
            if (rc != hipSuccess) { g_pool.free_blocks.emplace(want, p); LUX_CHECK_HIP(rc); }
            e.retired.push_back(RetiredBlock{e.base, e.data_bytes, done});
        }
        e.base = p;
        e.data_bytes = want;
    }
    if (e.counters == nullptr) {
        void* c = nullptr;
        constexpr size_t words = kWorkspaceCounters + kWorkspaceFlags + kWorkspaceZeroBytes / 4;
        LUX_CHECK_HIP(hipMalloc(&c, words * sizeof(uint32_t)));
        fill_zero_kernel<<<dim3(64), dim3(256), 0, s>>>(reinterpret_cast<uint32_t*>(c), words);
        hipError_t rc = hipGetLastError();
        if (rc != hipSuccess) { (void)hipFree(c); LUX_CHECK_HIP(rc); }
        e.counters = reinterpret_cast<uint32_t*>(c);
    }
    out->data = reinterpret_cast<char*>(e.base);
    out->counters = e.counters;
    out->flags = e.counters + kWorkspaceCounters;
    out->zeros = e.counters + kWorkspaceCounters + kWorkspaceFlags;
    if (++e.epoch == 0) {
        // the 32-bit epoch has wrapped: words tagged during the previous cycle must not be taken for
        // new ones, so the exchange words are cleared (on the stream, behind every kernel that used
        // them) and the count starts again at 1; 0 is what cleared words hold
        fill_zero_kernel<<<dim3(16), dim3(256), 0, s>>>(e.counters + kWorkspaceCounters, kWorkspaceFlags);
        LUX_CHECK_LAUNCH();
        e.epoch = 1;
    }
    out->epoch = e.epoch;
    return LUXHIP_OK;
}

__global__ void fill_zero_kernel(uint32_t* p, size_t nwords) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < nwords; i += stride) p[i] = 0u;
}
__global__ void fill_zero_bytes_kernel(uint8_t* p, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0;
}

}  // namespace luxhip

using namespace luxhip;

extern "C" {

int luxhip_init(int device) {
    std::lock_guard<std::mutex> lk(g_mu);
    int n = 0;
    LUX_CHECK_HIP(hipGetDeviceCount(&n));
    if (n <= 0) return set_error(LUXHIP_HIP_ERROR, "no HIP device visible");
    if (device < 0 || device >= n) return set_error(LUXHIP_INVALID, "device %d out of range (0..%d)", device, n - 1);
    if (g_init && device == g_device) return LUXHIP_OK;
    if (g_init) return set_error(LUXHIP_INVALID, "already initialised on device %d", g_device);
    LUX_CHECK_HIP(hipSetDevice(device));
    hipDeviceProp_t prop;
    LUX_CHECK_HIP(hipGetDeviceProperties(&prop, device));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return set_error(LUXHIP_UNSUPPORTED, "device %d is %s; this library is built for gfx950 only", device,
                         prop.gcnArchName);
    {
        const int rc = noalloc_setup(device);
        if (rc != LUXHIP_OK) return rc;
    }
    g_cus = prop.multiProcessorCount;
    g_device = device;
    g_init = true;
    return LUXHIP_OK;
}

int luxhip_shutdown(void) {
    std::lock_guard<std::mutex> lk(g_mu);
    if (!g_init) return LUXHIP_OK;
    (void)hipDeviceSynchronize();
    for (auto& kv : g_ws) {
        collect_retired(kv.second, true);       // into the pool, which is released below
        if (kv.second.base) (void)hipFree(kv.second.base);
        if (kv.second.counters) (void)hipFree(kv.second.counters);
        for (void* p : kv.second.pinned) (void)hipFree(p);
    }
    g_ws.clear();
    for (void* p : g_pinned) (void)hipFree(p);
    g_pinned.clear();
    for (auto& kv : g_pool.free_blocks) (void)hipFree(kv.second);
    g_pool.free_blocks.clear();
    for (auto& kv : g_pool.live) (void)hipFree(kv.first);
    g_pool.live.clear();
    g_init = false;
    g_device = -1;
    return LUXHIP_OK;
}

const char* luxhip_last_error(void) { return g_err; }

int luxhip_set_option(const char* name, int64_t value) {
    LUX_INVALID_IF(name == nullptr, "set_option: name must not be NULL");
    if (strcmp(name, "bn_resident") == 0) {
        g_opt_bn_resident.store(value != 0);
    } else if (strcmp(name, "bn_spin_limit") == 0) {
        LUX_INVALID_IF(value < 0 || value > (int64_t(1) << 30), "set_option: bn_spin_limit out of range");
        g_opt_bn_spin_limit.store(value);
    } else if (strcmp(name, "gemm_tile") == 0) {
        LUX_INVALID_IF(value != 0 && value != 82 && value != 42 && value != 22 && value != 11,
                       "set_option: gemm_tile must be 0, 82, 42, 22 or 11");
        g_opt_gemm_tile.store(value);
    } else if (strcmp(name, "conv_tile") == 0) {
        LUX_INVALID_IF(value != 0 && value != 1 && value != 2 && value != 82 && value != 83 && value != 84 && value != 42,
                       "set_option: conv_tile must be 0, 1, 2, 82, 83, 84 or 42");
        g_opt_conv_tile.store(value);
    } else if (strcmp(name, "gemm_pretranspose") == 0) {
        LUX_INVALID_IF(value != 0 && value != 1, "set_option: gemm_pretranspose must be 0 or 1");
        g_opt_gemm_pretranspose.store(value);
    } else if (strcmp(name, "workspace_epoch") == 0) {
        // for tests: the next call on every stream continues from this epoch (e.g. just below 2^32)
        LUX_INVALID_IF(value < 0 || value > (int64_t)0xffffffffll, "set_option: workspace_epoch out of range");
        std::lock_guard<std::mutex> lk(g_mu);
        for (auto& kv : g_ws) kv.second.epoch = (uint32_t)value;
    } else {
        return set_error(LUXHIP_INVALID, "set_option: unknown option '%s'", name);
    }
    return LUXHIP_OK;
}

int luxhip_device_info(char* name, size_t name_len, int* compute_units, int64_t* total_mem) {
    LUX_REQUIRE_INIT();
    hipDeviceProp_t prop;
    LUX_CHECK_HIP(hipGetDeviceProperties(&prop, g_device));
    if (name && name_len) snprintf(name, name_len, "%s (%s)", prop.name, prop.gcnArchName);
    if (compute_units) *compute_units = prop.multiProcessorCount;
    if (total_mem) *total_mem = (int64_t)prop.totalGlobalMem;
    return LUXHIP_OK;
}

int luxhip_stream_create(luxhip_stream_t* out) {
    LUX_REQUIRE_INIT();
    LUX_INVALID_IF(out == nullptr, "null output pointer");
    hipStream_t s;
    LUX_CHECK_HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));  // default priority
    *out = s;
    return LUXHIP_OK;
}
int luxhip_stream_synchronize(luxhip_stream_t s) {
    LUX_REQUIRE_INIT();
    LUX_CHECK_HIP(hipStreamSynchronize((hipStream_t)s));
    return LUXHIP_OK;
}
int luxhip_stream_destroy(luxhip_stream_t s) {
    LUX_REQUIRE_INIT();
    if (s == nullptr) return LUXHIP_OK;
    LUX_CHECK_HIP(hipStreamSynchronize((hipStream_t)s));
    {
        std::lock_guard<std::mutex> lk(g_mu);
        auto it = g_ws.find((hipStream_t)s);
        if (it != g_ws.end()) {
            collect_retired(it->second, true);  // the stream has been synchronised: into the pool
            WsEntry& e = it->second;
            g_pinned.insert(g_pinned.end(), e.pinned.begin(), e.pinned.end());
            if (e.recorded) {
                // graphs recorded on this stream can still be launched (on any stream): their scratch memory stays
                if (e.base) g_pinned.push_back(e.base);
                if (e.counters) g_pinned.push_back(e.counters);
            } else {
                if (e.base) (void)hipFree(e.base);
                if (e.counters) (void)hipFree(e.counters);
            }
            g_ws.erase(it);
        }
    }
    LUX_CHECK_HIP(hipStreamDestroy((hipStream_t)s));
    return LUXHIP_OK;
}

int luxhip_reserve(luxhip_stream_t s, size_t bytes) {
    LUX_REQUIRE_INIT();
    Workspace ws;
    return get_workspace((hipStream_t)s, bytes, &ws);
}

int luxhip_event_create(luxhip_event_t* out) {
    LUX_REQUIRE_INIT();
    LUX_INVALID_IF(out == nullptr, "null output pointer");
    hipEvent_t e;
    LUX_CHECK_HIP(hipEventCreate(&e));
    *out = e;
    return LUXHIP_OK;
}
int luxhip_event_record(luxhip_event_t e, luxhip_stream_t s) {
    LUX_REQUIRE_INIT();
    LUX_CHECK_HIP(hipEventRecord((hipEvent_t)e, (hipStream_t)s));
    return LUXHIP_OK;
}
int luxhip_event_elapsed_ms(float* ms, luxhip_event_t start, luxhip_event_t stop) {
    LUX_REQUIRE_INIT();
    LUX_INVALID_IF(ms == nullptr, "null output pointer");
    LUX_CHECK_HIP(hipEventSynchronize((hipEvent_t)stop));
    LUX_CHECK_HIP(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
    return LUXHIP_OK;
}
int luxhip_event_destroy(luxhip_event_t e) {
    LUX_REQUIRE_INIT();
    LUX_CHECK_HIP(hipEventDestroy((hipEvent_t)e));
    return LUXHIP_OK;
}

int luxhip_profile_enable(int on) {
    LUX_REQUIRE_INIT();
    std::lock_guard<std::mutex> lk(g_mu);
    g_prof = on != 0;
    return LUXHIP_OK;
}

int luxhip_profile_report(char* buf, size_t len) {
    LUX_REQUIRE_INIT();
    LUX_INVALID_IF(buf == nullptr || len < 3, "profile_report: buffer too small");
    LUX_CHECK_HIP(hipDeviceSynchronize());
    std::lock_guard<std::mutex> lk(g_mu);
    struct Agg { int count = 0; double total = 0, mn = 1e30, mx = 0; };
    std::map<std::string, Agg> agg;
    for (auto& e : g_prof_entries) {
        float ms = 0.0f;
        if (e.a >= 0 && e.b >= 0 && hipEventElapsedTime(&ms, g_prof_events[e.a], g_prof_events[e.b]) == hipSuccess) {
            Agg& a = agg[e.name];
            a.count++; a.total += ms;
            if (ms < a.mn) a.mn = ms;
            if (ms > a.mx) a.mx = ms;
        }
    }
    for (hipEvent_t ev : g_prof_events) (void)hipEventDestroy(ev);
    g_prof_events.clear();
    g_prof_entries.clear();
    size_t off = 0;
    off += snprintf(buf + off, len - off, "[");
    bool first = true;
    for (auto& kv : agg) {
        if (off + 200 >= len) break;
        off += snprintf(buf + off, len - off, "%s{\"kernel\": \"%s\", \"count\": %d, \"total_ms\": %.6f, \"min_ms\": %.6f, \"max_ms\": %.6f}",
                        first ? "" : ", ", kv.first.c_str(), kv.second.count, kv.second.total, kv.second.mn, kv.second.mx);
        first = false;
    }
    snprintf(buf + off, len - off, "]");
    return LUXHIP_OK;
}

int luxhip_malloc(void** out, size_t bytes) {
    LUX_REQUIRE_INIT();
    LUX_INVALID_IF(out == nullptr, "null output pointer");
    const size_t r = round_size(bytes);
    std::lock_guard<std::mutex> lk(g_mu);
    auto it = g_pool.free_blocks.find(r);
    if (it != g_pool.free_blocks.end()) {
        *out = it->second;
        g_pool.free_blocks.erase(it);
        g_pool.live[*out] = r;
        return LUXHIP_OK;
    }
    void* p = nullptr;
    hipError_t e = hipMalloc(&p, r);
    if (e != hipSuccess) {
        // give the pool back to the driver and retry once
        for (auto& kv : g_pool.free_blocks) (void)hipFree(kv.second);
        g_pool.free_blocks.clear();
        e = hipMalloc(&p, r);
        if (e != hipSuccess)
            return set_error(LUXHIP_HIP_ERROR, "hipMalloc(%zu) failed: %s", r, hipGetErrorString(e));
    }
    g_pool.live[p] = r;
    *out = p;
    return LUXHIP_OK;
}

int luxhip_free(void* p) {
    LUX_REQUIRE_INIT();
    if (p == nullptr) return LUXHIP_OK;
    std::lock_guard<std::mutex> lk(g_mu);
    auto it = g_pool.live.find(p);
    LUX_INVALID_IF(it == g_pool.live.end(), "luxhip_free: %p was not allocated by luxhip_malloc", p);
    g_pool.free_blocks.emplace(it->second, p);
    g_pool.live.erase(it);
    return LUXHIP_OK;
}

int luxhip_trim(void) {
    LUX_REQUIRE_INIT();
    std::lock_guard<std::mutex> lk(g_mu);
    LUX_CHECK_HIP(hipDeviceSynchronize());
    for (auto& kv : g_pool.free_blocks) (void)hipFree(kv.second);
    g_pool.free_blocks.clear();
    return LUXHIP_OK;
}

int luxhip_memcpy_h2d(void* dst, const void* src, size_t bytes, luxhip_stream_t s) {
    LUX_REQUIRE_INIT();
    if (bytes == 0) return LUXHIP_OK;
    LUX_CHECK_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, (hipStream_t)s));
    LUX_CHECK_HIP(hipStreamSynchronize((hipStream_t)s));
    return LUXHIP_OK;
}
int luxhip_memcpy_d2h(void* dst, const void* src, size_t bytes, luxhip_stream_t s) {
    LUX_REQUIRE_INIT();
    if (bytes == 0) return LUXHIP_OK;
    LUX_CHECK_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, (hipStream_t)s));
    LUX_CHECK_HIP(hipStreamSynchronize((hipStream_t)s));
    return LUXHIP_OK;
}
int luxhip_memcpy_d2d(void* dst, const void* src, size_t bytes, luxhip_stream_t s) {
    LUX_REQUIRE_INIT();
    if (bytes == 0) return LUXHIP_OK;
    LUX_CHECK_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, (hipStream_t)s));
    return LUXHIP_OK;
}
int luxhip_fill_zero(void* dst, size_t bytes, luxhip_stream_t s) {
    LUX_REQUIRE_INIT();
    if (bytes == 0) return LUXHIP_OK;
    LUX_INVALID_IF((reinterpret_cast<uintptr_t>(dst) & 3u) != 0, "luxhip_fill_zero: destination must be 4-byte aligned");
    const size_t nwords = bytes / 4, tail = bytes % 4;
    if (nwords) {
        size_t blocks = (nwords + 255) / 256;
        if (blocks > 4096) blocks = 4096;
        fill_zero_kernel<<<dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)s>>>(reinterpret_cast<uint32_t*>(dst), nwords);
        LUX_CHECK_LAUNCH();
    }
    if (tail) {
        fill_zero_bytes_kernel<<<dim3(1), dim3(64), 0, (hipStream_t)s>>>(reinterpret_cast<uint8_t*>(dst) + nwords * 4, tail);
        LUX_CHECK_LAUNCH();
    }
    return LUXHIP_OK;
}

}  // extern "C"
