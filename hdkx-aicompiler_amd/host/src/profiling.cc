// profiling.cc -- bundle writer and thread-local span stack (see kxc/profiling.h).
#include "kxc/profiling.h"

#include "kxc_hip.h"

#include <dlfcn.h>
#include <unistd.h>

#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <filesystem>
#include <fstream>
#include <map>
#include <sstream>
#include <thread>

namespace kxc {
namespace profiling {

namespace {

struct ThreadState {
    std::shared_ptr<ProfileContext> ctx;
    std::string run_id;
    std::vector<std::string> span_stack;
};
ThreadState& TLS() {
    static thread_local ThreadState s;
    return s;
}
const std::string kEmpty;

std::int64_t SteadyNs() {
    return std::chrono::duration_cast<std::chrono::nanoseconds>(std::chrono::steady_clock::now().time_since_epoch()).count();
}
std::int64_t WallNs() {
    return std::chrono::duration_cast<std::chrono::nanoseconds>(std::chrono::system_clock::now().time_since_epoch()).count();
}

std::string Escape(const std::string& in) {
    std::string out;
    out.reserve(in.size() + 8);
    for (unsigned char ch : in) {
        switch (ch) {
            case '"': out += "\\\""; break;
            case '\\': out += "\\\\"; break;
            case '\n': out += "\\n"; break;
            case '\r': out += "\\r"; break;
            case '\t': out += "\\t"; break;
            default:
                if (ch < 0x20) { char b[8]; std::snprintf(b, sizeof(b), "\\u%04x", ch); out += b; }
                else out += static_cast<char>(ch);
        }
    }
    return out;
}

std::string Number(double v) {
    if (v != v || v > 1.7e308 || v < -1.7e308) return "null";
    char b[40];
    if (v == static_cast<double>(static_cast<long long>(v)) && v > -9e15 && v < 9e15)
        std::snprintf(b, sizeof(b), "%lld", static_cast<long long>(v));
    else
        std::snprintf(b, sizeof(b), "%.9g", v);
    return b;
}

// Objects are written with sorted keys so that a bundle is reproducible.
std::string ObjectOf(const StringMap& m) {
    std::map<std::string, std::string> sorted(m.begin(), m.end());
    std::string out = "{";
    bool first = true;
    for (const auto& kv : sorted) {
        out += (first ? "\"" : ",\"") + Escape(kv.first) + "\":\"" + Escape(kv.second) + "\"";
        first = false;
    }
    return out + "}";
}
std::string ObjectOf(const MetricMap& m) {
    std::map<std::string, double> sorted(m.begin(), m.end());
    std::string out = "{";
    bool first = true;
    for (const auto& kv : sorted) {
        out += (first ? "\"" : ",\"") + Escape(kv.first) + "\":" + Number(kv.second);
        first = false;
    }
    return out + "}";
}

std::string EventLine(const std::string& trace_id, const std::string& session_id, const std::string& run_id,
                      const std::string& span_id, const std::string& parent, const EventSpec& e, std::int64_t ts_ns,
                      std::int64_t dur_ns) {
    StringMap fields = e.fields;
    fields["schema_version"] = "1";
    std::ostringstream os;
    os << "{\"trace_id\":\"" << Escape(trace_id) << "\",\"session_id\":\"" << Escape(session_id) << "\",\"run_id\":\""
       << Escape(run_id) << "\",\"span_id\":\"" << Escape(span_id) << "\",\"parent_span_id\":\"" << Escape(parent)
       << "\",\"component\":\"" << Escape(e.component) << "\",\"event_type\":\"" << Escape(e.event_type)
       << "\",\"phase\":\"" << Escape(e.phase) << "\",\"ts_ns\":" << ts_ns << ",\"duration_ns\":" << dur_ns
       << ",\"status\":\"" << Escape(e.status) << "\",\"severity\":\"" << LogSeverityToString(e.severity)
       << "\",\"device\":\"" << Escape(e.device) << "\",\"worker_id\":" << e.worker_id << ",\"op_name\":\""
       << Escape(e.op_name) << "\",\"pass_name\":\"" << Escape(e.pass_name) << "\",\"kernel_symbol\":\""
       << Escape(e.kernel_symbol) << "\",\"shape_signature\":\"" << Escape(e.shape_signature) << "\",\"message\":\""
       << Escape(e.message) << "\",\"fields\":" << ObjectOf(fields) << ",\"metrics\":" << ObjectOf(e.metrics) << "}";
    return os.str();
}

std::string TraceEvent(const EventSpec& e, std::int64_t ts_ns, std::int64_t dur_ns, bool device_track) {
    const bool span = e.phase != "instant" && dur_ns > 0;
    std::ostringstream os;
    const std::string name = !e.kernel_symbol.empty() ? e.kernel_symbol : (e.event_type.empty() ? e.component : e.event_type);
    os << "{\"name\":\"" << Escape(name) << "\",\"cat\":\"" << Escape(e.component) << "\",\"ph\":\"" << (span ? "X" : "i")
       << "\",\"ts\":" << (ts_ns / 1000) << ",\"dur\":" << (dur_ns / 1000) << ",\"pid\":" << static_cast<long>(getpid())
       << ",\"tid\":" << (device_track ? 1000000L : static_cast<long>(std::hash<std::thread::id>()(std::this_thread::get_id()) % 100000))
       << ",\"s\":\"t\",\"args\":{\"status\":\"" << Escape(e.status) << "\",\"severity\":\""
       << LogSeverityToString(e.severity) << "\",\"message\":\"" << Escape(e.message) << "\"}}";
    return os.str();
}

// roctx ranges, if the library is on the machine (no link-time dependency).
struct Roctx {
    int (*push)(const char*) = nullptr;
    int (*pop)() = nullptr;
    Roctx() {
        for (const char* name : {"libroctx64.so", "libroctx64.so.4", "librocprofiler-sdk-roctx.so"}) {
            if (void* h = dlopen(name, RTLD_LAZY | RTLD_LOCAL)) {
                push = reinterpret_cast<int (*)(const char*)>(dlsym(h, "roctxRangePushA"));
                pop = reinterpret_cast<int (*)()>(dlsym(h, "roctxRangePop"));
                if (push && pop) return;
                push = nullptr; pop = nullptr;
            }
        }
    }
};
Roctx& RoctxLib() {
    static Roctx r;
    return r;
}

bool EnvBool(const char* key, bool fallback) {
    const char* v = std::getenv(key);
    if (!v || !*v) return fallback;
    const std::string s(v);
    if (s == "1" || s == "true" || s == "TRUE" || s == "on" || s == "ON" || s == "yes") return true;
    if (s == "0" || s == "false" || s == "FALSE" || s == "off" || s == "OFF" || s == "no") return false;
    return fallback;
}

}  // namespace

std::string LogSeverityToString(LogSeverity s) {
    switch (s) {
        case LogSeverity::kDebug: return "debug";
        case LogSeverity::kInfo: return "info";
        case LogSeverity::kWarn: return "warn";
        case LogSeverity::kError: return "error";
    }
    return "info";
}

std::string IRCaptureModeToString(IRCaptureMode m) {
    switch (m) {
        case IRCaptureMode::kDisabled: return "disabled";
        case IRCaptureMode::kChangedOrFailed: return "changed_or_failed";
        case IRCaptureMode::kVerbose: return "verbose";
    }
    return "disabled";
}

std::string HashText(const std::string& text) {      // FNV-1a, 64 bit
    std::uint64_t h = 1469598103934665603ULL;
    for (unsigned char c : text) { h ^= c; h *= 1099511628211ULL; }
    char b[20];
    std::snprintf(b, sizeof(b), "%016llx", static_cast<unsigned long long>(h));
    return b;
}

std::string ShapeSignatureToString(const std::vector<std::vector<int64_t>>& shapes) {
    std::string out;
    for (size_t i = 0; i < shapes.size(); ++i) {
        out += i ? ";[" : "[";
        for (size_t k = 0; k < shapes[i].size(); ++k) out += (k ? "," : "") + std::to_string(shapes[i][k]);
        out += "]";
    }
    return out;
}

StringMap MakeFields(std::initializer_list<std::pair<std::string, std::string>> init) {
    StringMap m;
    for (const auto& kv : init) m[kv.first] = kv.second;
    return m;
}

bool ShouldCaptureIR(const std::shared_ptr<ProfileContext>& ctx, bool changed, bool failed) {
    if (!ctx || !ctx->options().record_pass_ir) return false;
    switch (ctx->options().ir_capture_mode) {
        case IRCaptureMode::kDisabled: return false;
        case IRCaptureMode::kChangedOrFailed: return changed || failed;
        case IRCaptureMode::kVerbose: return true;
    }
    return false;
}

ProfileOptions ApplyEnvironmentOverrides(ProfileOptions o) {
    o.enabled = EnvBool("KXC_PROFILE_ENABLE", o.enabled);
    if (const char* d = std::getenv("KXC_PROFILE_BUNDLE_DIR")) if (*d) o.bundle_dir = d;
    if (const char* l = std::getenv("KXC_PROFILE_LOG_LEVEL")) {
        const std::string s(l);
        if (s == "debug") o.log_level = LogSeverity::kDebug;
        else if (s == "info") o.log_level = LogSeverity::kInfo;
        else if (s == "warn") o.log_level = LogSeverity::kWarn;
        else if (s == "error") o.log_level = LogSeverity::kError;
    }
    if (const char* m = std::getenv("KXC_PROFILE_IR_MODE")) {
        const std::string s(m);
        if (s == "disabled") o.ir_capture_mode = IRCaptureMode::kDisabled;
        else if (s == "changed_or_failed") o.ir_capture_mode = IRCaptureMode::kChangedOrFailed;
        else if (s == "verbose") o.ir_capture_mode = IRCaptureMode::kVerbose;
    }
    o.enable_roctx = EnvBool("KXC_PROFILE_ROCTX", o.enable_roctx);
    if (const char* v = std::getenv("KXC_PROFILE_GPU_ACTIVITY"); v && v[0] == '2' && v[1] == 0) o.enable_gpu_activity = 2;
    else o.enable_gpu_activity = EnvBool("KXC_PROFILE_GPU_ACTIVITY", o.enable_gpu_activity != 0) ? std::max(o.enable_gpu_activity, 1) : 0;
    o.record_pass_ir = EnvBool("KXC_PROFILE_RECORD_PASS_IR", o.record_pass_ir);
    o.record_execution_plan_details = EnvBool("KXC_PROFILE_EXEC_PLAN_DETAILS", o.record_execution_plan_details);
    return o;
}

std::shared_ptr<ProfileContext> CurrentContext() { return TLS().ctx; }
const std::string& CurrentRunId() { return TLS().run_id; }
const std::string& CurrentSpanId() { return TLS().span_stack.empty() ? kEmpty : TLS().span_stack.back(); }

ScopedSpan CurrentSpan(EventSpec spec) {
    auto ctx = CurrentContext();
    if (!ctx) return ScopedSpan();
    return ScopedSpan(std::move(ctx), std::move(spec));
}

// ---------------------------------------------------------------- ActivationScope
ActivationScope::ActivationScope(std::shared_ptr<ProfileContext> ctx, std::string run_id) {
    ThreadState& t = TLS();
    previous_ctx_ = t.ctx;
    previous_run_id_ = t.run_id;
    previous_span_stack_ = t.span_stack;
    t.ctx = std::move(ctx);
    t.run_id = std::move(run_id);
    t.span_stack.clear();
}
ActivationScope::~ActivationScope() {
    ThreadState& t = TLS();
    t.ctx = previous_ctx_;
    t.run_id = previous_run_id_;
    t.span_stack = previous_span_stack_;
}

// ---------------------------------------------------------------- ScopedSpan
ScopedSpan::ScopedSpan(std::shared_ptr<ProfileContext> ctx, EventSpec spec, std::string run_id, std::string parent)
    : ctx_(std::move(ctx)), spec_(std::move(spec)) {
    if (!ctx_ || !ctx_->options().enabled) { ctx_.reset(); return; }
    run_id_ = run_id.empty() ? CurrentRunId() : std::move(run_id);
    parent_span_id_ = parent.empty() ? CurrentSpanId() : std::move(parent);
    span_id_ = ctx_->NextSpanId();
    start_ns_ = ctx_->NowNs();
    active_ = true;
    if (TLS().ctx == ctx_) { TLS().span_stack.push_back(span_id_); pushed_ = true; }
    if (ctx_->options().enable_roctx && RoctxLib().push) {
        const std::string label = spec_.component + ":" + (spec_.kernel_symbol.empty() ? spec_.event_type : spec_.kernel_symbol);
        RoctxLib().push(label.c_str());
        roctx_pushed_ = true;
    }
}
ScopedSpan::~ScopedSpan() { Close(); }
void ScopedSpan::MoveFrom(ScopedSpan& o) {
    ctx_ = std::move(o.ctx_); spec_ = std::move(o.spec_); run_id_ = std::move(o.run_id_); span_id_ = std::move(o.span_id_);
    parent_span_id_ = std::move(o.parent_span_id_); start_ns_ = o.start_ns_; active_ = o.active_; pushed_ = o.pushed_;
    roctx_pushed_ = o.roctx_pushed_;
    o.active_ = false; o.pushed_ = false; o.roctx_pushed_ = false;
}
ScopedSpan::ScopedSpan(ScopedSpan&& o) noexcept { MoveFrom(o); }
ScopedSpan& ScopedSpan::operator=(ScopedSpan&& o) noexcept {
    if (this != &o) { Close(); MoveFrom(o); }
    return *this;
}
void ScopedSpan::Close() {
    if (!active_) return;
    active_ = false;
    if (roctx_pushed_ && RoctxLib().pop) RoctxLib().pop();
    if (pushed_) {
        auto& st = TLS().span_stack;
        if (!st.empty() && st.back() == span_id_) st.pop_back();
    }
    ctx_->RecordCompletedSpan(spec_, run_id_, span_id_, parent_span_id_, start_ns_, ctx_->NowNs());
}

// ---------------------------------------------------------------- ProfileContext
ProfileContext::ProfileContext(ProfileOptions options) : options_(std::move(options)) {
    start_wall_ns_ = WallNs();
    start_mono_ns_ = SteadyNs();
    const std::string seed = std::to_string(start_wall_ns_) + ":" + std::to_string(static_cast<long>(getpid())) + ":" +
                             std::to_string(reinterpret_cast<std::uintptr_t>(this));
    trace_id_ = "trace-" + HashText(seed);
    session_id_ = "session-" + HashText(seed + ":s");
    bundle_dir_ = options_.bundle_dir.empty()
                      ? (std::filesystem::temp_directory_path() / ("kxc_profile_" + HashText(seed))).string()
                      : options_.bundle_dir;
}
namespace {
std::mutex g_activity_mu;
int g_activity_users = 0;      // contexts that asked the HIP library to record activity
}  // namespace

ProfileContext::~ProfileContext() {
    try {
        if (options_.enabled && !event_lines_.empty()) Flush();
    } catch (...) {
    }
    if (gpu_activity_on_) {
        std::lock_guard<std::mutex> lock(g_activity_mu);
        if (--g_activity_users == 0) kxc_hip_activity_enable(0);
    }
}
std::shared_ptr<ProfileContext> ProfileContext::Create(const ProfileOptions& options) {
    std::shared_ptr<ProfileContext> ctx(new ProfileContext(options));
    if (options.enabled && options.enable_gpu_activity) {
        std::lock_guard<std::mutex> lock(g_activity_mu);
        int mode = options.enable_gpu_activity >= 2 ? 2 : 1;
        std::string why;
        // (the rocprofiler-sdk tool has to be registered before the first HIP call: nothing may ask the runtime
        // anything before this)
        if (mode == 2 && kxc_hip_activity_enable(2) != 0) {
            why = kxc_hip_last_error();
            mode = 1;
        }
        int32_t devices = 0;
        if (kxc_hip_device_count(&devices) == 0 && devices > 0 && (mode == 2 || kxc_hip_activity_enable(1) == 0)) {
            ++g_activity_users;
            ctx->gpu_activity_on_ = true;
            ctx->gpu_activity_mode_ = mode;
        } else if (mode == 2) {
            kxc_hip_activity_enable(0);
        }
        if (!why.empty()) {
            EventSpec e;
            e.component = "backend.hip";
            e.event_type = "activity_source_fallback";
            e.status = "degraded";
            e.severity = LogSeverity::kWarn;
            e.message = "rocprofiler-sdk tracing not available, recording at the HIP library's call sites: " + why;
            const std::int64_t now = ctx->NowNs();
            ctx->RecordCompletedSpan(e, "", ctx->NextSpanId(), "", now, now);
        }
    }
    return ctx;
}

void ProfileContext::CollectGpuActivity() {
    if (!gpu_activity_on_) return;
    int32_t count = 0;
    if (kxc_hip_activity_drain(nullptr, 0, &count) != 0 || count == 0) return;
    std::vector<kxc_hip_activity_record> records(static_cast<size_t>(count) + 64);
    if (kxc_hip_activity_drain(records.data(), static_cast<int32_t>(records.size()), &count) != 0) return;
    // the library's clock -> this context's time base
    const std::int64_t offset = NowNs() - kxc_hip_activity_now_ns();
    static const char* const kTypes[4] = {"hip_runtime_api", "hip_memcpy", "hip_memset", "hip_kernel"};
    for (int32_t i = 0; i < count; ++i) {
        const kxc_hip_activity_record& r = records[static_cast<size_t>(i)];
        if (r.kind < 0 || r.kind > 3) continue;
        EventSpec e;
        e.component = "backend.hip";
        e.event_type = kTypes[r.kind];
        e.device = r.kind == KXC_HIP_ACTIVITY_RUNTIME_API ? "hip" : "hip:" + std::to_string(r.device_id);
        e.fields["backend.hip.correlation_id"] = std::to_string(r.correlation_id);
        e.fields["backend.hip.thread_id"] = std::to_string(r.thread_id);
        if (r.kind == KXC_HIP_ACTIVITY_RUNTIME_API) {
            e.fields["backend.hip.api"] = r.name;
            e.fields["backend.hip.return_value"] = std::to_string(r.return_value);
            if (r.return_value != 0) { e.status = "error"; e.severity = LogSeverity::kWarn; }
        } else {
            e.fields["backend.hip.stream_id"] = std::to_string(r.stream);
            e.fields["backend.hip.timing_source"] = r.timed_on_gpu == 2 ? "rocprofiler_sdk" : r.timed_on_gpu ? "hip_events" : "host_clock";
        }
        if (r.kind == KXC_HIP_ACTIVITY_MEMCPY) {
            e.fields["backend.hip.copy_kind"] = std::to_string(r.copy_kind);
            e.metrics["bytes"] = static_cast<double>(r.bytes);
            e.metrics["copy_count"] = 1.0;
        } else if (r.kind == KXC_HIP_ACTIVITY_MEMSET) {
            e.metrics["bytes"] = static_cast<double>(r.bytes);
            e.metrics["value"] = static_cast<double>(r.value);
        } else if (r.kind == KXC_HIP_ACTIVITY_KERNEL) {
            e.kernel_symbol = r.name;
            e.metrics["grid_x"] = r.grid[0]; e.metrics["grid_y"] = r.grid[1]; e.metrics["grid_z"] = r.grid[2];
            e.metrics["block_x"] = r.block[0]; e.metrics["block_y"] = r.block[1]; e.metrics["block_z"] = r.block[2];
            e.metrics["dynamic_shared_memory"] = r.dynamic_shared_memory;
        }
        RecordCompletedSpan(e, CurrentRunId(), NextSpanId(), "", r.start_ns + offset, r.end_ns + offset);
    }
}

std::vector<DiagnosticEntry> ProfileContext::DiagnoseDeviceOverheads() const {
    constexpr double kCopyDominanceRatio = 0.40, kSyncDominanceRatio = 0.25;
    constexpr std::int64_t kSmallKernelRunNs = 200000;
    std::int64_t copy = 0, device = 0, sync = 0, total = 0;
    int tiny_runs = 0;
    {
        std::lock_guard<std::mutex> lock(mu_);
        for (const EventDigest& d : digests_) {
            total += d.duration_ns;
            if (d.component == "device_api") {
                device += d.duration_ns;
                if (d.event_type == "copy") copy += d.duration_ns;
            }
            if (d.event_type == "stream_sync" || d.event_type == "execute_barrier_node") sync += d.duration_ns;
            if ((d.event_type == "compiled_module_run" || d.event_type == "adaptive_module_run") && d.duration_ns < kSmallKernelRunNs) ++tiny_runs;
        }
    }
    std::vector<DiagnosticEntry> out;
    if (device > 0 && static_cast<double>(copy) / static_cast<double>(device) >= kCopyDominanceRatio)
        out.push_back({"copy_dominance", "warn", "device_api", "Device copy time dominates device API activity."});
    if (total > 0 && static_cast<double>(sync) / static_cast<double>(total) >= kSyncDominanceRatio)
        out.push_back({"sync_overhead", "warn", "runtime", "Synchronization overhead is a large portion of the run."});
    if (tiny_runs >= 5)
        out.push_back({"kernel_launch_overhead", "info", "runtime", "Many very short module runs suggest launch overhead may dominate."});
    return out;
}
std::int64_t ProfileContext::NowNs() const { return SteadyNs() - start_mono_ns_; }
std::string ProfileContext::NextRunId(const std::string& prefix) {
    std::lock_guard<std::mutex> lock(mu_);
    return prefix + "-" + std::to_string(++run_counter_);
}
std::string ProfileContext::NextSpanId() {
    std::lock_guard<std::mutex> lock(mu_);
    return "span-" + std::to_string(++span_counter_);
}
std::size_t ProfileContext::event_count() const {
    std::lock_guard<std::mutex> lock(mu_);
    return event_lines_.size();
}
void ProfileContext::RecordCompletedSpan(const EventSpec& spec, const std::string& run_id, const std::string& span_id,
                                         const std::string& parent, std::int64_t start_ns, std::int64_t end_ns) {
    if (!options_.enabled || static_cast<int>(spec.severity) < static_cast<int>(options_.log_level)) return;
    const std::int64_t dur = end_ns > start_ns ? end_ns - start_ns : 0;
    std::lock_guard<std::mutex> lock(mu_);
    event_lines_.push_back(EventLine(trace_id_, session_id_, run_id, span_id, parent, spec, start_ns, dur));
    trace_events_.push_back(TraceEvent(spec, start_ns, dur, spec.component == "backend.hip"));
    digests_.push_back({spec.component, spec.event_type, dur});
}
void ProfileContext::RecordInstant(EventSpec spec, const std::string& run_id, const std::string& parent) {
    if (!options_.enabled || static_cast<int>(spec.severity) < static_cast<int>(options_.log_level)) return;
    const std::string run = run_id.empty() ? CurrentRunId() : run_id;
    const std::string par = parent.empty() ? CurrentSpanId() : parent;
    const std::int64_t ts = NowNs();
    const std::string span = NextSpanId();
    std::lock_guard<std::mutex> lock(mu_);
    event_lines_.push_back(EventLine(trace_id_, session_id_, run, span, par, spec, ts, 0));
    trace_events_.push_back(TraceEvent(spec, ts, 0, false));
}
void ProfileContext::RecordLog(LogSeverity severity, const std::string& component, const std::string& message,
                               StringMap fields, MetricMap metrics, const std::string& run_id) {
    EventSpec spec;
    spec.component = component;
    spec.event_type = "log";
    spec.phase = "instant";
    spec.severity = severity;
    spec.message = message;
    spec.fields = std::move(fields);
    spec.metrics = std::move(metrics);
    RecordInstant(std::move(spec), run_id);
}
void ProfileContext::EnsureLayoutLocked() {
    if (layout_done_) return;
    std::filesystem::create_directories(std::filesystem::path(bundle_dir_) / "artifacts");
    layout_done_ = true;
}
std::string ProfileContext::WriteArtifact(const std::string& relative_path, const std::string& content) {
    std::lock_guard<std::mutex> lock(mu_);
    EnsureLayoutLocked();
    const std::filesystem::path path = std::filesystem::path(bundle_dir_) / "artifacts" / relative_path;
    std::filesystem::create_directories(path.parent_path());
    std::ofstream out(path, std::ios::out | std::ios::trunc);
    out << content;
    return path.string();
}
void ProfileContext::PublishDiagnostics(const std::vector<DiagnosticEntry>& diagnostics) {
    std::lock_guard<std::mutex> lock(mu_);
    diagnostics_ = diagnostics;
    auto_diagnosed_ = false;
    EnsureLayoutLocked();
    WriteAllLocked();
}
void ProfileContext::Flush() {
    CollectGpuActivity();
    // unless a caller published a diagnosis of its own, the device-side rules are evaluated on what was recorded
    bool published = false;
    {
        std::lock_guard<std::mutex> lock(mu_);
        published = !diagnostics_.empty() && !auto_diagnosed_;
    }
    std::vector<DiagnosticEntry> found;
    if (!published) found = DiagnoseDeviceOverheads();
    std::lock_guard<std::mutex> lock(mu_);
    if (!published) {
        diagnostics_ = found;
        auto_diagnosed_ = true;
    }
    EnsureLayoutLocked();
    WriteAllLocked();
}
void ProfileContext::WriteAllLocked() {
    const std::filesystem::path dir(bundle_dir_);
    {
        std::ofstream f(dir / "manifest.json", std::ios::out | std::ios::trunc);
        f << "{\"schema_version\":" << options_.schema_version << ",\"trace_id\":\"" << Escape(trace_id_)
          << "\",\"session_id\":\"" << Escape(session_id_) << "\",\"bundle_dir\":\"" << Escape(bundle_dir_)
          << "\",\"log_level\":\"" << LogSeverityToString(options_.log_level) << "\",\"ir_capture_mode\":\""
          << IRCaptureModeToString(options_.ir_capture_mode) << "\",\"enable_roctx\":" << (options_.enable_roctx ? "true" : "false")
          << ",\"roctx_available\":" << (RoctxLib().push ? "true" : "false")
          << ",\"enable_gpu_activity\":" << (options_.enable_gpu_activity ? "true" : "false")
          << ",\"gpu_activity_source\":\"" << (gpu_activity_mode_ == 2 ? "rocprofiler_sdk" : "hip_events")
          << "\",\"record_execution_plan_details\":"
          << (options_.record_execution_plan_details ? "true" : "false") << ",\"event_count\":" << event_lines_.size() << "}";
    }
    {
        std::ofstream f(dir / "events.jsonl", std::ios::out | std::ios::trunc);
        for (const auto& line : event_lines_) f << line << "\n";
    }
    {
        std::ofstream f(dir / "trace.json", std::ios::out | std::ios::trunc);
        f << "{\"traceEvents\":[";
        for (size_t i = 0; i < trace_events_.size(); ++i) f << (i ? "," : "") << trace_events_[i];
        f << "],\"metadata\":{\"trace_id\":\"" << Escape(trace_id_) << "\",\"session_id\":\"" << Escape(session_id_)
          << "\",\"start_time_ns\":" << start_wall_ns_ << "}}";
    }
    {
        std::map<std::string, std::uint64_t> counts;
        const std::string key = "\"component\":\"";
        for (const auto& line : event_lines_) {
            const size_t pos = line.find(key);
            if (pos == std::string::npos) continue;
            const size_t b = pos + key.size(), e = line.find('"', b);
            ++counts[line.substr(b, e - b)];
        }
        std::ofstream f(dir / "summary.json", std::ios::out | std::ios::trunc);
        f << "{\"trace_id\":\"" << Escape(trace_id_) << "\",\"session_id\":\"" << Escape(session_id_)
          << "\",\"event_count\":" << event_lines_.size() << ",\"component_counts\":{";
        bool first = true;
        for (const auto& kv : counts) { f << (first ? "\"" : ",\"") << Escape(kv.first) << "\":" << kv.second; first = false; }
        f << "}}";
    }
    {
        std::vector<DiagnosticEntry> items = diagnostics_;
        if (items.empty())
            items.push_back({"no_findings", "info", "analysis",
                             "The device-side rules (kernel_launch_overhead, copy_dominance, sync_overhead) found nothing."});
        std::ofstream f(dir / "diagnosis.json", std::ios::out | std::ios::trunc);
        f << "{\"trace_id\":\"" << Escape(trace_id_) << "\",\"diagnostics\":[";
        for (size_t i = 0; i < items.size(); ++i) {
            const auto& d = items[i];
            f << (i ? "," : "") << "{\"category\":\"" << Escape(d.category) << "\",\"severity\":\"" << Escape(d.severity)
              << "\",\"component\":\"" << Escape(d.component) << "\",\"summary\":\"" << Escape(d.summary) << "\"}";
        }
        f << "]}";
        std::ofstream md(dir / "diagnosis.md", std::ios::out | std::ios::trunc);
        md << "# Diagnostics\n\n";
        for (const auto& d : items)
            md << "- [" << d.severity << "] " << d.category << " (" << d.component << "): " << d.summary << "\n";
    }
}

}  // namespace profiling
}  // namespace kxc
