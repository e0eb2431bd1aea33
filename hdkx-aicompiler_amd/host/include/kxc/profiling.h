// profiling.h -- profiling bundle of the host layer: event model, RAII spans, bundle writer.
// Mirrors the reference's public profiling API (include/base/profiling.h:24-236) for the part the
// lowered-operator path touches, and writes the same bundle (manifest.json, events.jsonl, trace.json,
// summary.json, diagnosis.json, diagnosis.md, artifacts/) with the same event fields (src/base/profiling.cc:740-771),
// so the reference's bundle consumers read a HIP run unchanged.  Differences, all on the GPU side:
//   * device activity is component "backend.hip" with event types hip_kernel / hip_memcpy (the reference's
//     CUPTI adapter emits "backend.cuda" / cuda_kernel, profiling.cc:623-651); the records come from HIP
//     events placed between the launches of a plan (kxc_hip_plan_run_profiled), not from an activity API,
//     so they need no tool library and cost nothing when profiling is off;
//   * ProfileOptions::enable_gpu_activity replaces enable_cupti, enable_roctx replaces enable_nvtx
//     (ranges through the roctx library, looked up at run time; absent library = no ranges).
//     enable_gpu_activity = 2 takes the activity records from rocprofiler-sdk's buffered tracing instead of the
//     HIP library's own call sites (every HIP call of the process is then seen, as with CUPTI); the context must
//     be created before the process's first HIP call for that, or KXC_PROFILE_GPU_ACTIVITY=2 set in the
//     environment.  If the tool cannot be registered any more the context falls back to 1 and records a warning.
#pragma once

#include <cstdint>
#include <initializer_list>
#include <memory>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

namespace kxc {
namespace profiling {

enum class LogSeverity : int { kDebug = 0, kInfo = 1, kWarn = 2, kError = 3 };
enum class IRCaptureMode : int { kDisabled = 0, kChangedOrFailed = 1, kVerbose = 2 };

using StringMap = std::unordered_map<std::string, std::string>;
using MetricMap = std::unordered_map<std::string, double>;

struct EventSpec {
    std::string component;
    std::string event_type;
    std::string phase{"complete"};
    std::string status{"ok"};
    LogSeverity severity{LogSeverity::kInfo};
    std::string device;
    int worker_id{-1};
    std::string op_name;
    std::string pass_name;
    std::string kernel_symbol;
    std::string shape_signature;
    std::string message;
    StringMap fields;
    MetricMap metrics;
};

struct ProfileOptions {
    bool enabled{false};
    std::string bundle_dir;
    LogSeverity log_level{LogSeverity::kInfo};
    IRCaptureMode ir_capture_mode{IRCaptureMode::kChangedOrFailed};
    bool enable_roctx{false};
    int enable_gpu_activity{1};       // 0 off, 1 (true) records at the HIP library's call sites, 2 rocprofiler-sdk
    bool record_pass_ir{true};
    bool record_execution_plan_details{true};
    int schema_version{1};
};

struct DiagnosticEntry {
    std::string category;
    std::string severity;
    std::string component;
    std::string summary;
};

class ProfileContext;

// Installs a context and run id as the calling thread's current ones for the scope.
class ActivationScope {
public:
    ActivationScope(std::shared_ptr<ProfileContext> ctx, std::string run_id);
    ~ActivationScope();
    ActivationScope(const ActivationScope&) = delete;
    ActivationScope& operator=(const ActivationScope&) = delete;

private:
    std::shared_ptr<ProfileContext> previous_ctx_;
    std::string previous_run_id_;
    std::vector<std::string> previous_span_stack_;
};

// A timed event: starts at construction, is written to the context at destruction.
class ScopedSpan {
public:
    ScopedSpan() = default;
    ScopedSpan(std::shared_ptr<ProfileContext> ctx, EventSpec spec, std::string run_id = "",
               std::string parent_span_id = "");
    ~ScopedSpan();
    ScopedSpan(const ScopedSpan&) = delete;
    ScopedSpan& operator=(const ScopedSpan&) = delete;
    ScopedSpan(ScopedSpan&& other) noexcept;
    ScopedSpan& operator=(ScopedSpan&& other) noexcept;

    void SetStatus(const std::string& status) { spec_.status = status; }
    void SetMessage(const std::string& message) { spec_.message = message; }
    void AddField(const std::string& key, const std::string& value) { spec_.fields[key] = value; }
    void AddMetric(const std::string& key, double value) { spec_.metrics[key] = value; }
    bool active() const { return active_; }
    const std::string& span_id() const { return span_id_; }

private:
    void Close();
    void MoveFrom(ScopedSpan& other);

    std::shared_ptr<ProfileContext> ctx_;
    EventSpec spec_;
    std::string run_id_, span_id_, parent_span_id_;
    std::int64_t start_ns_{0};
    bool active_{false};
    bool pushed_{false};
    bool roctx_pushed_{false};
};

class ProfileContext : public std::enable_shared_from_this<ProfileContext> {
public:
    static std::shared_ptr<ProfileContext> Create(const ProfileOptions& options);
    ~ProfileContext();

    const ProfileOptions& options() const { return options_; }
    const std::string& trace_id() const { return trace_id_; }
    const std::string& session_id() const { return session_id_; }
    const std::string& bundle_dir() const { return bundle_dir_; }

    std::string NextRunId(const std::string& prefix);
    std::string NextSpanId();
    // Nanoseconds since the context was created (monotonic clock): the time base of every event.
    std::int64_t NowNs() const;

    void RecordCompletedSpan(const EventSpec& spec, const std::string& run_id, const std::string& span_id,
                             const std::string& parent_span_id, std::int64_t start_ns, std::int64_t end_ns);
    void RecordInstant(EventSpec spec, const std::string& run_id = "", const std::string& parent_span_id = "");
    void RecordLog(LogSeverity severity, const std::string& component, const std::string& message,
                   StringMap fields = {}, MetricMap metrics = {}, const std::string& run_id = "");
    std::string WriteArtifact(const std::string& relative_path, const std::string& content);
    void PublishDiagnostics(const std::vector<DiagnosticEntry>& diagnostics);
    // Fetches the GPU-side activity the HIP library has recorded since the last call (runtime API calls, copies,
    // fills, kernel launches) and adds it as "backend.hip" events: hip_runtime_api / hip_memcpy / hip_memset /
    // hip_kernel, with the metric keys the reference's CUPTI adapter uses for their CUDA counterparts
    // (src/base/profiling.cc:537-651).  Flush calls it; a caller synchronises its streams first.
    void CollectGpuActivity();
    // 0: no device activity records; 1: taken at the HIP library's call sites; 2: from rocprofiler-sdk
    int gpu_activity_mode() const { return gpu_activity_mode_; }
    // The device-side diagnosis rules the reference's offline analyser applies to a bundle (kernel_launch_overhead,
    // copy_dominance, sync_overhead: python/kxc_agent/services/diagnosis_engine.py:233-297, thresholds
    // rule_library.py:22-24), evaluated on the recorded events.
    std::vector<DiagnosticEntry> DiagnoseDeviceOverheads() const;
    void Flush();
    std::size_t event_count() const;

private:
    explicit ProfileContext(ProfileOptions options);
    void EnsureLayoutLocked();
    void WriteAllLocked();

    ProfileOptions options_;
    std::string trace_id_, session_id_, bundle_dir_;
    std::int64_t start_wall_ns_{0}, start_mono_ns_{0};
    std::vector<std::string> event_lines_, trace_events_;
    struct EventDigest {            // what the diagnosis rules read
        std::string component, event_type;
        std::int64_t duration_ns;
    };
    std::vector<EventDigest> digests_;
    bool gpu_activity_on_{false};
    int gpu_activity_mode_{0};        // what Create could switch on: 0, 1 or 2
    bool auto_diagnosed_{false};     // diagnostics_ came from DiagnoseDeviceOverheads, not from PublishDiagnostics
    std::vector<DiagnosticEntry> diagnostics_;
    std::uint64_t run_counter_{0}, span_counter_{0};
    bool layout_done_{false};
    mutable std::mutex mu_;
};

// KXC_PROFILE_ENABLE, KXC_PROFILE_BUNDLE_DIR, KXC_PROFILE_LOG_LEVEL, KXC_PROFILE_IR_MODE,
// KXC_PROFILE_ROCTX, KXC_PROFILE_GPU_ACTIVITY, KXC_PROFILE_RECORD_PASS_IR, KXC_PROFILE_EXEC_PLAN_DETAILS
// (the reference reads the same names with NVTX / CUPTI for the two GPU switches, profiling.cc:1159-1194).
ProfileOptions ApplyEnvironmentOverrides(ProfileOptions options);

std::shared_ptr<ProfileContext> CurrentContext();
const std::string& CurrentRunId();
const std::string& CurrentSpanId();

std::string LogSeverityToString(LogSeverity severity);
std::string IRCaptureModeToString(IRCaptureMode mode);
std::string HashText(const std::string& text);
std::string ShapeSignatureToString(const std::vector<std::vector<int64_t>>& shapes);
StringMap MakeFields(std::initializer_list<std::pair<std::string, std::string>> init);
bool ShouldCaptureIR(const std::shared_ptr<ProfileContext>& ctx, bool changed, bool failed);

// Span on the calling thread's current context (inactive when there is none).
ScopedSpan CurrentSpan(EventSpec spec);

}  // namespace profiling
}  // namespace kxc
