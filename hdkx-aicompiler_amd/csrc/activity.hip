// activity.hip -- record of what the library asks of the HIP runtime and what the GPU then does, for the
// profiling bundle's "backend.hip" events.  GPU counterpart of the reference's CUPTI activity adapter
// (src/base/profiling.cc:250-695: runtime API, memcpy, memset and kernel records with start / end times), built
// from the library's own call sites instead of a tool library: every HIP runtime call of the device API and the
// module loader is timed on the host, and every copy, fill and kernel launch they enqueue is bracketed by two HIP
// events on its stream.  Off by default and free while off (one relaxed atomic load per call).
#include <atomic>
#include <chrono>
#include <mutex>
#include <thread>
#include <vector>

#include "common.h"

namespace kxc_hip {

namespace {

std::atomic<bool> g_on{false};
std::atomic<uint64_t> g_correlation{1};

struct Pending {
    kxc_hip_activity_record rec;
    hipEvent_t start = nullptr, stop = nullptr;     // device activities measured on the GPU
};

struct State {
    std::mutex mu;
    std::vector<kxc_hip_activity_record> done;
    std::vector<Pending> pending;
    hipEvent_t base = nullptr;      // recorded and waited for at enable: GPU time zero
    int64_t base_host_ns = 0;
};
State& S() {
    static State* s = new State();  // never destroyed: records may arrive during process exit
    return *s;
}

int64_t NowNs() {
    return std::chrono::duration_cast<std::chrono::nanoseconds>(std::chrono::steady_clock::now().time_since_epoch()).count();
}

uint64_t ThreadId() { return static_cast<uint64_t>(std::hash<std::thread::id>()(std::this_thread::get_id())); }

void Fill(kxc_hip_activity_record* r, int32_t kind, const char* name) {
    std::memset(r, 0, sizeof(*r));
    r->kind = kind;
    std::snprintf(r->name, sizeof(r->name), "%s", name ? name : "");
    r->thread_id = ThreadId();
    int dev = 0;
    if (hipGetDevice(&dev) == hipSuccess) r->device_id = dev;
}

thread_local int t_suppress = 0;

}  // namespace

bool ActivityOn() { return g_on.load(std::memory_order_relaxed) && t_suppress == 0; }
ActivitySuppress::ActivitySuppress() { ++t_suppress; }
ActivitySuppress::~ActivitySuppress() { --t_suppress; }

ApiScope::ApiScope(const char* name) : on_(ActivityOn()), name_(name) {
    if (!on_) return;
    correlation_ = g_correlation.fetch_add(1);
    start_ns_ = NowNs();
}
ApiScope::~ApiScope() {
    if (!on_) return;
    kxc_hip_activity_record r;
    Fill(&r, KXC_HIP_ACTIVITY_RUNTIME_API, name_);
    r.start_ns = start_ns_;
    r.end_ns = NowNs();
    r.correlation_id = correlation_;
    r.return_value = result_;
    std::lock_guard<std::mutex> lock(S().mu);
    S().done.push_back(r);
}

DeviceScope::DeviceScope(int32_t kind, const char* name, hipStream_t stream, uint64_t correlation)
    : on_(ActivityOn()), kind_(kind), name_(name), stream_(stream), correlation_(correlation) {
    if (!on_) return;
    host_start_ns_ = NowNs();
    // (no events under stream capture: a captured record would become a graph node)
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    if (stream_ && hipStreamIsCapturing(stream_, &st) == hipSuccess && st != hipStreamCaptureStatusNone) { on_ = false; return; }
    if (hipEventCreate(&start_) != hipSuccess || hipEventCreate(&stop_) != hipSuccess || hipEventRecord(start_, stream_) != hipSuccess) {
        (void)hipGetLastError();
        if (start_) (void)hipEventDestroy(start_);
        if (stop_) (void)hipEventDestroy(stop_);
        start_ = stop_ = nullptr;
    }
}
DeviceScope::~DeviceScope() {
    if (!on_) return;
    Pending p;
    Fill(&p.rec, kind_, name_);
    p.rec.bytes = bytes; p.rec.value = value; p.rec.copy_kind = copy_kind;
    for (int i = 0; i < 3; ++i) { p.rec.grid[i] = grid[i]; p.rec.block[i] = block[i]; }
    p.rec.dynamic_shared_memory = dynamic_shared_memory;
    p.rec.correlation_id = correlation_;
    p.rec.stream = reinterpret_cast<uint64_t>(stream_);
    p.rec.start_ns = host_start_ns_;
    p.rec.end_ns = NowNs();              // replaced by GPU times when the events resolve
    if (start_ && stop_ && hipEventRecord(stop_, stream_) == hipSuccess) {
        p.start = start_; p.stop = stop_;
    } else {
        if (start_) (void)hipEventDestroy(start_);
        if (stop_) (void)hipEventDestroy(stop_);
        (void)hipGetLastError();
    }
    std::lock_guard<std::mutex> lock(S().mu);
    S().pending.push_back(p);
}

}  // namespace kxc_hip

using namespace kxc_hip;

extern "C" {

int32_t kxc_hip_activity_enable(int32_t enable) {
    State& s = S();
    std::lock_guard<std::mutex> lock(s.mu);
    if (enable) {
        if (!s.base) {
            // GPU time zero: an event that has completed, and the host time at which it was seen complete
            KXC_HIP_CALL(hipEventCreate(&s.base), "hipEventCreate");
            KXC_HIP_CALL(hipEventRecord(s.base, nullptr), "hipEventRecord");
            KXC_HIP_CALL(hipEventSynchronize(s.base), "hipEventSynchronize");
            s.base_host_ns = NowNs();
        }
        g_on.store(true);
    } else {
        g_on.store(false);
    }
    return KXC_HIP_OK;
}

int32_t kxc_hip_activity_drain(kxc_hip_activity_record* records, int32_t capacity, int32_t* count) {
    KXC_HIP_REQUIRE(count != nullptr && (capacity == 0 || records != nullptr), "kxc_hip_activity_drain: NULL output");
    State& s = S();
    std::lock_guard<std::mutex> lock(s.mu);
    // resolve the device activities whose events have completed (waiting for each: a drain follows a stream sync)
    for (Pending& p : s.pending) {
        if (p.start && p.stop && s.base) {
            float to_start = 0.0f, dur = 0.0f;
            if (hipEventSynchronize(p.stop) == hipSuccess && hipEventElapsedTime(&to_start, s.base, p.start) == hipSuccess &&
                hipEventElapsedTime(&dur, p.start, p.stop) == hipSuccess) {
                p.rec.start_ns = s.base_host_ns + static_cast<int64_t>(static_cast<double>(to_start) * 1e6);
                p.rec.end_ns = p.rec.start_ns + static_cast<int64_t>(static_cast<double>(dur) * 1e6);
                p.rec.timed_on_gpu = 1;
            } else {
                (void)hipGetLastError();
            }
        }
        if (p.start) (void)hipEventDestroy(p.start);
        if (p.stop) (void)hipEventDestroy(p.stop);
        s.done.push_back(p.rec);
    }
    s.pending.clear();
    const int32_t n = static_cast<int32_t>(s.done.size());
    *count = n;
    if (capacity == 0) return KXC_HIP_OK;           // size query
    KXC_HIP_REQUIRE(capacity >= n, "kxc_hip_activity_drain: %d records, room for %d", n, capacity);
    for (int32_t i = 0; i < n; ++i) records[i] = s.done[static_cast<size_t>(i)];
    s.done.clear();
    return KXC_HIP_OK;
}

int64_t kxc_hip_activity_now_ns(void) { return NowNs(); }

}  // extern "C"
