// runtime_session.cc -- see kxc/runtime_session.h.
#include "kxc/runtime_session.h"

#include <algorithm>
#include <limits>
#include <sstream>
#include <stdexcept>

namespace kxc {
namespace runtime {

// ------------------------------------------------------------------ ShapeSignature
namespace {
inline void Mix(size_t* seed, size_t v) { *seed ^= v + 0x9e3779b9 + (*seed << 6) + (*seed >> 2); }
}  // namespace

size_t ShapeSignature::Hash() const {
    size_t seed = input_shapes.size();
    for (const auto& shape : input_shapes) {
        Mix(&seed, shape.size());
        for (int64_t d : shape) Mix(&seed, std::hash<int64_t>{}(d));
    }
    return seed;
}

ShapeSignature MakeShapeSignature(const std::vector<std::vector<int64_t>>& shapes) { return ShapeSignature{shapes}; }

// ------------------------------------------------------------------ ShapePredictor
void ShapePredictor::Record(const ShapeSignature& sig) {
    std::lock_guard<std::mutex> lock(mu_);
    ++seen_[sig];
    ++total_;
    recent_.push_back(sig);
    while (recent_.size() > kMaxRecent) recent_.pop_front();
}

std::vector<ShapeSignature> ShapePredictor::PredictTopK(int k) const {
    std::vector<std::pair<int, const ShapeSignature*>> order;
    std::lock_guard<std::mutex> lock(mu_);
    for (const auto& kv : seen_) order.emplace_back(kv.second, &kv.first);
    std::stable_sort(order.begin(), order.end(), [](const auto& a, const auto& b) { return a.first > b.first; });
    std::vector<ShapeSignature> top;
    for (size_t i = 0; i < order.size() && static_cast<int>(i) < k; ++i) top.push_back(*order[i].second);
    return top;
}

bool ShapePredictor::ShouldCompile(const ShapeSignature& sig, int count_threshold, double ratio_threshold) const {
    // shape_predictor.cc:44-59: below the count threshold never; at or above it the ratio test is tried first and
    // the count test decides anyway -- so the answer is "seen at least count_threshold times".
    (void)ratio_threshold;
    std::lock_guard<std::mutex> lock(mu_);
    auto it = seen_.find(sig);
    return it != seen_.end() && it->second >= count_threshold;
}

int ShapePredictor::GetCount(const ShapeSignature& sig) const {
    std::lock_guard<std::mutex> lock(mu_);
    auto it = seen_.find(sig);
    return it == seen_.end() ? 0 : it->second;
}

int ShapePredictor::TotalCount() const {
    std::lock_guard<std::mutex> lock(mu_);
    return total_;
}

// ------------------------------------------------------------------ KernelCache
int64_t KernelCache::ShapeDistance(const ShapeSignature& query, const ShapeSignature& cached) {
    if (query.input_shapes.size() != cached.input_shapes.size()) return -1;
    int64_t distance = 0;
    for (size_t i = 0; i < query.input_shapes.size(); ++i) {
        const auto& want = query.input_shapes[i];
        const auto& have = cached.input_shapes[i];
        if (want.size() != have.size()) return -1;
        for (size_t d = 0; d < want.size(); ++d) {
            if (have[d] < want[d]) return -1;          // only a module built for larger extents can serve
            distance += have[d] - want[d];
        }
    }
    return distance;
}

api::CompiledModule* KernelCache::GetExact(const ShapeSignature& sig) {
    std::lock_guard<std::mutex> lock(mu_);
    auto it = modules_.find(sig);
    return it == modules_.end() ? nullptr : &it->second;
}

api::CompiledModule* KernelCache::GetFuzzy(const ShapeSignature& sig) {
    std::lock_guard<std::mutex> lock(mu_);
    api::CompiledModule* nearest = nullptr;
    int64_t nearest_distance = std::numeric_limits<int64_t>::max();
    for (auto& kv : modules_) {
        const int64_t d = ShapeDistance(sig, kv.first);
        if (d >= 0 && d < nearest_distance) { nearest_distance = d; nearest = &kv.second; }
    }
    return nearest;
}

void KernelCache::Put(const ShapeSignature& sig, api::CompiledModule module) {
    std::lock_guard<std::mutex> lock(mu_);
    modules_[sig] = std::move(module);
}

bool KernelCache::Has(const ShapeSignature& sig) const {
    std::lock_guard<std::mutex> lock(mu_);
    return modules_.find(sig) != modules_.end();
}

size_t KernelCache::Size() const {
    std::lock_guard<std::mutex> lock(mu_);
    return modules_.size();
}

void KernelCache::Clear() {
    std::lock_guard<std::mutex> lock(mu_);
    modules_.clear();
}

// ------------------------------------------------------------------ KernelRunner
void KernelRunner::SwapKernel(std::shared_ptr<api::CompiledModule> module) {
    std::lock_guard<std::mutex> lock(mu_);
    module_.swap(module);
}

void KernelRunner::Run(const std::vector<void*>& args) {
    std::shared_ptr<api::CompiledModule> current;
    {
        std::lock_guard<std::mutex> lock(mu_);
        current = module_;       // a concurrent SwapKernel cannot free what this call runs
    }
    if (!current) throw std::runtime_error("KernelRunner: no kernel available");
    current->Run(args);
}

bool KernelRunner::HasKernel() const {
    std::lock_guard<std::mutex> lock(mu_);
    return static_cast<bool>(module_);
}

// ------------------------------------------------------------------ BackgroundCompiler
BackgroundCompiler::BackgroundCompiler(int num_threads) {
    if (num_threads <= 0) num_threads = static_cast<int>(std::max(1u, std::thread::hardware_concurrency() / 2));
    workers_.reserve(static_cast<size_t>(num_threads));
    for (int i = 0; i < num_threads; ++i) workers_.emplace_back(&BackgroundCompiler::Work, this);
}

BackgroundCompiler::~BackgroundCompiler() {
    {
        std::lock_guard<std::mutex> lock(mu_);
        stopping_ = true;
    }
    work_cv_.notify_all();
    for (std::thread& t : workers_)
        if (t.joinable()) t.join();
}

void BackgroundCompiler::Submit(CompileTask task) {
    {
        std::lock_guard<std::mutex> lock(mu_);
        queue_.push(std::move(task));
        ++unfinished_;
    }
    work_cv_.notify_one();
}

void BackgroundCompiler::WaitAll() {
    std::unique_lock<std::mutex> lock(mu_);
    idle_cv_.wait(lock, [this] { return unfinished_ == 0; });
}

int BackgroundCompiler::PendingCount() const {
    std::lock_guard<std::mutex> lock(mu_);
    return static_cast<int>(queue_.size());
}

void BackgroundCompiler::Work() {
    for (;;) {
        CompileTask task;
        {
            std::unique_lock<std::mutex> lock(mu_);
            work_cv_.wait(lock, [this] { return stopping_ || !queue_.empty(); });
            if (queue_.empty()) return;               // stopping and drained
            task = queue_.top();
            queue_.pop();
        }
        {
            profiling::ActivationScope activation(task.profile_context, task.run_id);
            profiling::EventSpec spec;
            spec.component = "background_compiler";
            spec.event_type = "background_compile_task";
            spec.shape_signature = profiling::ShapeSignatureToString(task.target_shape.input_shapes);
            profiling::ScopedSpan span(task.profile_context, std::move(spec), task.run_id, task.parent_span_id);
            try {
                api::CompiledModule module = api::Compiler::Compile(task.relay_func, task.config);
                if (task.on_complete) task.on_complete(std::move(module));
                ++completed_;
            } catch (const std::exception& e) {
                ++failed_;
                span.SetStatus("error");
                span.SetMessage(e.what());
                if (task.profile_context)
                    task.profile_context->RecordLog(profiling::LogSeverity::kError, "background_compiler", e.what(), {}, {},
                                                    task.run_id);
            }
        }
        {
            std::lock_guard<std::mutex> lock(mu_);
            --unfinished_;
        }
        idle_cv_.notify_all();
    }
}

// ------------------------------------------------------------------ RuntimeSession
namespace {
profiling::EventSpec SessionEvent(const char* event_type) {
    profiling::EventSpec spec;
    spec.component = "runtime_session";
    spec.event_type = event_type;
    return spec;
}
}  // namespace

RuntimeSession::RuntimeSession(Function relay_func, api::CompileConfig config,
                               std::shared_ptr<profiling::ProfileContext> profile_context)
    : relay_func_(std::move(relay_func)), config_(config), profile_context_(std::move(profile_context)) {
    bg_compiler_ = std::make_unique<BackgroundCompiler>(config->background_threads);
    // the session compiles ahead of time at the caller's optimisation level, whatever mode the caller's
    // configuration names (runtime_session.cc:32-33); back-end switches carry over
    internal_config_ = api::CompileConfig::AOT(config->target, config->opt_level);
    internal_config_->backend = config->backend;
    internal_config_->hip_use_handwritten = config->hip_use_handwritten;
    internal_config_->hip_fuse = config->hip_fuse;
    internal_config_->hip_concurrent_branches = config->hip_concurrent_branches;
    internal_config_->hip_winograd = config->hip_winograd;
    internal_config_->hip_batch_lanes = config->hip_batch_lanes;
    internal_config_->hip_pair_convolutions = config->hip_pair_convolutions;
    internal_config_->hip_constants_frozen = config->hip_constants_frozen;
    internal_config_->sync_after_run = config->sync_after_run;
}

RuntimeSession::~RuntimeSession() {
    if (bg_compiler_) bg_compiler_->WaitAll();      // completion callbacks touch this object
}

void RuntimeSession::Run(const std::vector<void*>& args, const std::vector<std::vector<int64_t>>& input_shapes) {
    profiling::EventSpec run_spec = SessionEvent("runtime_session_run");
    run_spec.shape_signature = profiling::ShapeSignatureToString(input_shapes);
    profiling::ScopedSpan span(profile_context_, std::move(run_spec));
    const ShapeSignature sig = MakeShapeSignature(input_shapes);
    const std::string hash = std::to_string(sig.Hash());
    predictor_.Record(sig);
    span.AddField("shape_hash", hash);
    span.AddMetric("shape_seen_count", static_cast<double>(predictor_.GetCount(sig)));

    if (api::CompiledModule* exact = cache_.GetExact(sig)) {
        profiling::ScopedSpan hit(profile_context_, SessionEvent("cache_exact_hit"));
        hit.AddField("shape_hash", hash);
        exact->Run(args);
        return;
    }
    // A fuzzy candidate was compiled for other (larger) extents.  On the host back end the reference runs it on
    // the caller's buffers (src/runtime/runtime_session.cc:63-75); on the hip target that would make device kernels
    // read and write past allocations sized for the smaller shape, so there a fuzzy candidate counts as a miss and
    // the exact shape is compiled on the calling thread.
    const bool device_buffers = config_->target.defined() && config_->target->kind == "hip";
    api::CompiledModule* fuzzy = cache_.GetFuzzy(sig);
    if (fuzzy && device_buffers) {
        if (profile_context_) {
            profiling::EventSpec skipped = SessionEvent("cache_fuzzy_skipped_device_buffers");
            skipped.fields["shape_hash"] = hash;
            profile_context_->RecordInstant(std::move(skipped), profiling::CurrentRunId(), profiling::CurrentSpanId());
        }
        fuzzy = nullptr;
    }
    if (fuzzy) {
        {
            profiling::ScopedSpan hit(profile_context_, SessionEvent("cache_fuzzy_hit"));
            hit.AddField("shape_hash", hash);
            fuzzy->Run(args);
        }
        MaybeScheduleOptimization(sig);
        return;
    }
    {
        profiling::ScopedSpan miss(profile_context_, SessionEvent("cache_miss_sync_compile"));
        miss.AddField("shape_hash", hash);
        cache_.Put(sig, api::Compiler::Compile(relay_func_, internal_config_));
        cache_.GetExact(sig)->Run(args);
    }
    MaybeScheduleOptimization(sig);
}

void RuntimeSession::WarmUp(const std::vector<std::vector<int64_t>>& input_shapes) {
    profiling::EventSpec spec = SessionEvent("runtime_session_warmup");
    spec.shape_signature = profiling::ShapeSignatureToString(input_shapes);
    profiling::ScopedSpan span(profile_context_, std::move(spec));
    const ShapeSignature sig = MakeShapeSignature(input_shapes);
    span.AddField("shape_hash", std::to_string(sig.Hash()));
    if (cache_.Has(sig)) {
        span.AddField("warmup_cache_status", "already_cached");
        return;
    }
    cache_.Put(sig, api::Compiler::Compile(relay_func_, internal_config_));
}

void RuntimeSession::WaitAll() {
    profiling::ScopedSpan span(profile_context_, SessionEvent("runtime_session_wait_all"));
    if (bg_compiler_) bg_compiler_->WaitAll();
}

std::string RuntimeSession::GetStatus() const {
    std::ostringstream os;
    os << "RuntimeSession{cached=" << cache_.Size() << ", pending=" << (bg_compiler_ ? bg_compiler_->PendingCount() : 0)
       << ", completed=" << (bg_compiler_ ? bg_compiler_->CompletedCount() : 0) << ", total_runs=" << predictor_.TotalCount()
       << "}";
    return os.str();
}

void RuntimeSession::MaybeScheduleOptimization(const ShapeSignature& sig) {
    const int seen = predictor_.GetCount(sig);
    if (!predictor_.ShouldCompile(sig, 2, 0.05)) return;
    const size_t hash = sig.Hash();
    {
        std::lock_guard<std::mutex> lock(schedule_mu_);
        if (!submitted_shapes_.insert(hash).second) return;     // one background compile per shape
    }
    BackgroundCompiler::CompileTask task;
    task.relay_func = relay_func_;
    task.config = internal_config_;
    task.target_shape = sig;
    task.priority = seen;
    task.profile_context = profile_context_;
    task.run_id = profiling::CurrentRunId();
    task.parent_span_id = profiling::CurrentSpanId();
    const std::string run_id = task.run_id, parent = task.parent_span_id;
    task.on_complete = [this, sig, run_id, parent](api::CompiledModule module) {
        cache_.Put(sig, std::move(module));
        if (!profile_context_) return;
        profiling::EventSpec done = SessionEvent("background_compile_completed");
        done.shape_signature = profiling::ShapeSignatureToString(sig.input_shapes);
        done.fields["shape_hash"] = std::to_string(sig.Hash());
        profile_context_->RecordInstant(std::move(done), run_id, parent);
    };
    if (profile_context_) {
        profiling::EventSpec submitted = SessionEvent("background_compile_submitted");
        submitted.shape_signature = profiling::ShapeSignatureToString(sig.input_shapes);
        submitted.fields["shape_hash"] = std::to_string(hash);
        submitted.metrics["priority"] = static_cast<double>(task.priority);
        submitted.metrics["seen_count"] = static_cast<double>(seen);
        profile_context_->RecordInstant(std::move(submitted), task.run_id, task.parent_span_id);
    }
    bg_compiler_->Submit(std::move(task));
}

}  // namespace runtime
}  // namespace kxc
