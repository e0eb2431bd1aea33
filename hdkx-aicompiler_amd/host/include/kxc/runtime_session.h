// runtime_session.h -- the adaptive runtime of the reference (include/runtime/runtime_session.h:24-61,
// kernel_cache.h:19-43, shape_predictor.h:19-70, background_compiler.h:24-69, kernel_runner.h:17-33) on top of
// this host layer's Compiler, so that it drives the "hip" target as it drives the CPU one:
//
//   RuntimeSession::Run(args, input_shapes)
//     1. records the shape signature in the ShapePredictor;
//     2. an exact KernelCache hit runs at once;
//     3. else a "fuzzy" hit -- the cached module whose every input dimension is >= the request, nearest by
//        summed difference -- runs, and a background compile for the exact shape may be scheduled;
//     4. else the function is compiled on the calling thread, cached, run, and the same scheduling applies.
//   A shape is scheduled once, when it has been seen at least twice; the task's priority is how often it was
//   seen.  Worker threads call Compiler::Compile concurrently with the caller's Run: for the hip target that is
//   hipRTC compilation, module loading and plan building from several threads, which the C ABI library supports
//   (independent hipRTC programs, a mutex around module loading, per-thread error and stream state).
//
// Same class names, methods, thresholds and status text as the reference, so code written against it compiles
// unchanged; profiling spans use the reference's component / event names (runtime_session.cc:17-22,44-161).
#pragma once

#include <atomic>
#include <condition_variable>
#include <deque>
#include <functional>
#include <memory>
#include <mutex>
#include <queue>
#include <string>
#include <thread>
#include <unordered_map>
#include <unordered_set>
#include <vector>

#include "kxc/compiler.h"
#include "kxc/profiling.h"

namespace kxc {
namespace runtime {

// The shapes of all inputs of one call; hashing as shape_predictor.h:24-34 (callers log the hash).
struct ShapeSignature {
    std::vector<std::vector<int64_t>> input_shapes;
    bool operator==(const ShapeSignature& other) const { return input_shapes == other.input_shapes; }
    size_t Hash() const;
};
struct ShapeSignatureHash {
    size_t operator()(const ShapeSignature& sig) const { return sig.Hash(); }
};
ShapeSignature MakeShapeSignature(const std::vector<std::vector<int64_t>>& shapes);

// Frequency statistics over the shapes a session has seen.
class ShapePredictor {
public:
    void Record(const ShapeSignature& sig);
    // The k most frequent signatures, most frequent first.
    std::vector<ShapeSignature> PredictTopK(int k = 3) const;
    // Seen at least count_threshold times (the ratio test of the reference can only confirm that: see the .cc).
    bool ShouldCompile(const ShapeSignature& sig, int count_threshold = 2, double ratio_threshold = 0.05) const;
    int GetCount(const ShapeSignature& sig) const;
    int TotalCount() const;

private:
    mutable std::mutex mu_;
    std::unordered_map<ShapeSignature, int, ShapeSignatureHash> seen_;
    std::deque<ShapeSignature> recent_;     // the last kMaxRecent calls
    int total_ = 0;
    static constexpr size_t kMaxRecent = 200;
};

// Compiled modules by shape signature.  Pointers stay valid until Clear() or a Put() of the same signature.
class KernelCache {
public:
    api::CompiledModule* GetExact(const ShapeSignature& sig);
    api::CompiledModule* GetFuzzy(const ShapeSignature& sig);
    void Put(const ShapeSignature& sig, api::CompiledModule module);
    bool Has(const ShapeSignature& sig) const;
    size_t Size() const;
    void Clear();
    // -1: `cached` cannot serve `query` (different arity or rank, or some cached dimension smaller); otherwise
    // the sum over all dimensions of cached - query.
    static int64_t ShapeDistance(const ShapeSignature& query, const ShapeSignature& cached);

private:
    mutable std::mutex mu_;
    std::unordered_map<ShapeSignature, api::CompiledModule, ShapeSignatureHash> modules_;
};

// Holder of "the module to run now", replaceable while other threads run it.
class KernelRunner {
public:
    void SwapKernel(std::shared_ptr<api::CompiledModule> module);
    void Run(const std::vector<void*>& args);       // throws "KernelRunner: no kernel available"
    bool HasKernel() const;

private:
    std::shared_ptr<api::CompiledModule> module_;
    mutable std::mutex mu_;
};

// Thread pool that compiles tasks in priority order (highest first).
class BackgroundCompiler {
public:
    struct CompileTask {
        Function relay_func;
        api::CompileConfig config;
        ShapeSignature target_shape;
        int priority{0};
        std::shared_ptr<profiling::ProfileContext> profile_context;
        std::string run_id;
        std::string parent_span_id;
        std::function<void(api::CompiledModule)> on_complete;
        bool operator<(const CompileTask& other) const { return priority < other.priority; }
    };
    explicit BackgroundCompiler(int num_threads = 0);   // 0: half the hardware threads, at least one
    ~BackgroundCompiler();                               // finishes the queue, then joins
    BackgroundCompiler(const BackgroundCompiler&) = delete;
    BackgroundCompiler& operator=(const BackgroundCompiler&) = delete;

    void Submit(CompileTask task);
    void WaitAll();
    int PendingCount() const;                 // tasks still queued (not the ones being compiled)
    int CompletedCount() const { return completed_.load(); }
    int FailedCount() const { return failed_.load(); }

private:
    void Work();
    std::vector<std::thread> workers_;
    std::priority_queue<CompileTask> queue_;
    mutable std::mutex mu_;
    std::condition_variable work_cv_, idle_cv_;
    bool stopping_ = false;
    int unfinished_ = 0;                      // queued + running
    std::atomic<int> completed_{0}, failed_{0};
};

class RuntimeSession {
public:
    explicit RuntimeSession(Function relay_func, api::CompileConfig config,
                            std::shared_ptr<profiling::ProfileContext> profile_context = nullptr);
    ~RuntimeSession();

    void Run(const std::vector<void*>& args, const std::vector<std::vector<int64_t>>& input_shapes);
    void WarmUp(const std::vector<std::vector<int64_t>>& input_shapes);
    void WaitAll();

    std::string GetStatus() const;            // "RuntimeSession{cached=.., pending=.., completed=.., total_runs=..}"
    int CachedKernelCount() const { return static_cast<int>(cache_.Size()); }
    int PendingCompileCount() const { return bg_compiler_ ? bg_compiler_->PendingCount() : 0; }

private:
    void MaybeScheduleOptimization(const ShapeSignature& sig);

    Function relay_func_;
    api::CompileConfig config_, internal_config_;
    std::shared_ptr<profiling::ProfileContext> profile_context_;
    KernelCache cache_;
    ShapePredictor predictor_;
    std::unique_ptr<BackgroundCompiler> bg_compiler_;
    std::unordered_set<size_t> submitted_shapes_;
    mutable std::mutex schedule_mu_;
};

}  // namespace runtime
}  // namespace kxc
