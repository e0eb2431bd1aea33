// activity.hip -- record of what the library asks of the HIP runtime and what the GPU then does, for the
// profiling bundle's "backend.hip" events.  GPU counterpart of the reference's CUPTI activity adapter
// (src/base/profiling.cc:250-695: runtime API, memcpy, memset and kernel records with start / end times), built
// from the library's own call sites instead of a tool library: every HIP runtime call of the device API and the
// module loader is timed on the host, and every copy, fill and kernel launch they enqueue is bracketed by two HIP
// events on its stream.  Off by default and free while off (one relaxed atomic load per call).
//
// Mode 2 takes the records from rocprofiler-sdk instead (libkxc_hip_rocprof.so, rocprof_tool.cpp): buffered tracing
// of kernel dispatches, memory copies and HIP runtime calls of the WHOLE process, which is what the reference's
// adapter does with CUPTI.  The tool library is loaded on request only, and it has to be registered before the
// process makes its first HIP call.
#include <dlfcn.h>

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
    uint64_t dropped = 0;           // device records not kept because kMaxPending were already waiting for a drain
};
constexpr size_t kMaxPending = 1u << 16;
// hipEventElapsedTime returns float milliseconds: 24 bits of mantissa are a microsecond at 16 s from the base event
// and worse beyond, so the base is renewed when it is older than this and no record still refers to it
constexpr int64_t kBaseMaxAgeNs = 4000000000LL;
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

// ---- mode 2: the rocprofiler-sdk tool library, loaded from this library's own directory
struct SdkTool {
    void* handle = nullptr;
    int32_t (*prepare)() = nullptr;
    int32_t (*start)() = nullptr;
    int32_t (*stop)() = nullptr;
    int32_t (*drain)(kxc_hip_activity_record*, int32_t, int32_t*) = nullptr;
    const char* (*status)() = nullptr;
    std::string error;
    bool running = false;
};
SdkTool& Sdk() {
    static SdkTool* t = new SdkTool();
    return *t;
}

// (caller holds S().mu or runs before main)
bool LoadSdkTool() {
    SdkTool& t = Sdk();
    if (t.handle) return true;
    Dl_info info;
    std::string path = "libkxc_hip_rocprof.so";
    if (dladdr(reinterpret_cast<const void*>(&LoadSdkTool), &info) && info.dli_fname) {
        const std::string self = info.dli_fname;
        const size_t slash = self.rfind('/');
        if (slash != std::string::npos) path = self.substr(0, slash + 1) + path;
    }
    void* h = dlopen(path.c_str(), RTLD_NOW | RTLD_GLOBAL);
    if (!h) { t.error = std::string("cannot load ") + path + ": " + dlerror(); return false; }
    t.prepare = reinterpret_cast<int32_t (*)()>(dlsym(h, "kxc_rocprof_prepare"));
    t.start = reinterpret_cast<int32_t (*)()>(dlsym(h, "kxc_rocprof_start"));
    t.stop = reinterpret_cast<int32_t (*)()>(dlsym(h, "kxc_rocprof_stop"));
    t.drain = reinterpret_cast<int32_t (*)(kxc_hip_activity_record*, int32_t, int32_t*)>(dlsym(h, "kxc_rocprof_drain"));
    t.status = reinterpret_cast<const char* (*)()>(dlsym(h, "kxc_rocprof_status"));
    if (!t.prepare || !t.start || !t.stop || !t.drain || !t.status) { t.error = path + " lacks the kxc_rocprof_* entry points"; dlclose(h); return false; }
    t.handle = h;
    return true;
}

// KXC_PROFILE_GPU_ACTIVITY=2 in the environment: register the tool while this library is being loaded, which is
// before any HIP call this library makes (a failure shows when mode 2 is asked for).
__attribute__((constructor)) void RegisterSdkToolEarly() {
    const char* e = std::getenv("KXC_PROFILE_GPU_ACTIVITY");
    if (e && e[0] == '2' && e[1] == 0 && LoadSdkTool()) (void)Sdk().prepare();
}

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
    if (S().pending.size() >= kMaxPending) {
        // nobody drains: keep the newest kMaxPending device records' worth of events at most
        if (p.start) (void)hipEventDestroy(p.start);
        if (p.stop) (void)hipEventDestroy(p.stop);
        ++S().dropped;
        return;
    }
    S().pending.push_back(p);
}

}  // namespace kxc_hip

using namespace kxc_hip;

extern "C" {

int32_t kxc_hip_activity_enable(int32_t enable) {
    State& s = S();
    std::lock_guard<std::mutex> lock(s.mu);
    KXC_HIP_REQUIRE(enable >= 0 && enable <= 2, "kxc_hip_activity_enable: mode %d (0 off, 1 call sites of this library, 2 rocprofiler-sdk)", enable);
    SdkTool& tool = Sdk();
    if (enable != 2 && tool.running) {
        (void)tool.stop();
        tool.running = false;
    }
    if (enable == 2) {
        // no HIP call before the tool is registered
        g_on.store(false);
        KXC_HIP_REQUIRE(LoadSdkTool(), "kxc_hip_activity_enable(2): %s", tool.error.c_str());
        KXC_HIP_REQUIRE(tool.prepare() == 0, "kxc_hip_activity_enable(2): %s", tool.status());
        KXC_HIP_REQUIRE(tool.start() == 0, "kxc_hip_activity_enable(2): %s", tool.status());
        // A tool registered after the HIP runtime initialised is accepted by rocprofiler-sdk and then never hears of
        // anything.  One harmless runtime call shows which case this is: its record has to come back.
        int version = 0;
        (void)hipDriverGetVersion(&version);
        bool heard = false;
        for (int tries = 0; tries < 40 && !heard; ++tries) {
            int32_t m = 0;
            heard = tool.drain(nullptr, 0, &m) == 0 && m > 0;
            if (!heard) std::this_thread::sleep_for(std::chrono::milliseconds(5));
        }
        if (!heard) {
            (void)tool.stop();
            KXC_HIP_REQUIRE(false, "kxc_hip_activity_enable(2): rocprofiler-sdk does not see this process's HIP calls -- the tool was "
                                   "registered after the HIP runtime had initialised; ask for mode 2 before the first HIP call "
                                   "(or set KXC_PROFILE_GPU_ACTIVITY=2 in the environment)");
        }
        tool.running = true;
        return KXC_HIP_OK;
    }
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
    if (s.base && g_on.load() && NowNs() - s.base_host_ns > kBaseMaxAgeNs) {
        if (hipEventRecord(s.base, nullptr) == hipSuccess && hipEventSynchronize(s.base) == hipSuccess) s.base_host_ns = NowNs();
        else (void)hipGetLastError();
    }
    // mode 2: what rocprofiler-sdk has delivered so far (timed_on_gpu = 2 marks the source)
    SdkTool& tool = Sdk();
    if (tool.handle) {
        int32_t m = 0;
        if (tool.drain(nullptr, 0, &m) == 0 && m > 0) {
            std::vector<kxc_hip_activity_record> more(static_cast<size_t>(m) + 256);
            if (tool.drain(more.data(), static_cast<int32_t>(more.size()), &m) == 0)
                for (int32_t i = 0; i < m; ++i) {
                    if (more[static_cast<size_t>(i)].timed_on_gpu) more[static_cast<size_t>(i)].timed_on_gpu = 2;
                    s.done.push_back(more[static_cast<size_t>(i)]);
                }
        }
    }
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
