// compiler.h -- CompileConfig, Compiler::Compile, CompiledModule::Run.
// The user-visible entry of the reference (include/api/compiler.h:32-92, include/api/compile_config.h:34-68):
// a test that compiles for the CPU with CompileConfig::JIT(BuildTarget(kCPU)) runs on the GPU by
// changing only the target to BuildTarget(kGPU).  Compile selects the back end from
// config->target->kind: "hip" builds a launch plan of hand-written kernels (operators that register
// FHIPDispatch, with bias / residual add / ReLU fused into convolutions) and run-time compiled
// kernels from the TIR -> HIP generator (everything else); any other kind compiles the whole
// function to C with the host compiler.
//
// Run ABI (src/codegen/compiled_kernel.cc:41-55): packed_args = inputs, constants in lowering order,
// outputs.  For the "hip" target every pointer is a DEVICE pointer; Run enqueues the plan on the
// current stream and synchronises it before returning, because callers read outputs right after.
#pragma once

#include <memory>

#include "kxc/codegen.h"
#include "kxc/device_api.h"
#include "kxc/lower.h"
#include "kxc/profiling.h"

namespace kxc {
namespace runtime {
class RuntimeSession;       // kxc/runtime_session.h
}
namespace api {

enum class CompileMode { kAOT, kJIT, kAdaptive };

struct CompileConfigNode {
    CompileMode mode{CompileMode::kAOT};
    int opt_level{2};
    Target target;
    codegen::CodeGenBackend backend{codegen::CodeGenBackend::kLLVM};
    // HIP back end switches
    bool hip_use_handwritten{true};    // false: every operator goes through the TIR -> HIP generator
    bool hip_fuse{true};               // fold bias / residual add / ReLU into convolution launches
    bool hip_concurrent_branches{true};   // run a block's downsample convolution beside its first 3x3 convolution
    bool hip_pair_convolutions{true};     // a block's 1x1 downsample as a second output of its first convolution's launch
    bool hip_winograd{true};              // 3x3 stride-1 convolutions with constant weights as Winograd F(2x2,3x3) where faster
    // Shares of the batch that run side by side on streams of their own inside one launch plan (each share is the
    // whole graph on batch / lanes samples; the kernels of one share fill the compute units the other's leave idle
    // at the end of every launch).  0: two for batches of 64 samples and more when the graph is separable along the
    // batch (relay::SplitBatch), else one; 1: never; 2..8: that many (Compile throws when the graph does not allow it).
    int hip_batch_lanes{0};
    // Winograd layers transform their (constant) filters on the GPU.  false (default): at the start of every Run, from
    // the pointers passed to that Run, so a Run always sees the constants' current contents, like the CPU back end.
    // true: once, when a pointer is first seen -- the caller promises not to change the weights behind the module's
    // back (serving); CompiledModule::InvalidateConstants() announces an in-place update.
    bool hip_constants_frozen{false};
    bool sync_after_run{true};
    // Adaptive mode (include/api/compile_config.h:40-45)
    std::vector<std::vector<int64_t>> suggested_input_shapes;   // each is warmed up at Compile
    int background_threads{0};         // compile workers (0 = half the hardware threads)
    bool enable_hot_swap{true};
    std::string cache_dir;             // empty = cache in memory (the only kind either implementation has)
    // When enabled and no context is active on the calling thread, Compile creates a ProfileContext from these
    // options; the module keeps it, activates it around every Run and names its bundle in GetProfileBundlePath()
    // (include/api/compile_config.h:47, src/api/compiler.cc:32-40).
    profiling::ProfileOptions profile_options;
};
class CompileConfig : public Ref<CompileConfigNode> {
public:
    CompileConfig() = default;
    explicit CompileConfig(std::shared_ptr<CompileConfigNode> n) : Ref<CompileConfigNode>(std::move(n)) {}
    static CompileConfig AOT(Target target, int opt_level = 3);
    static CompileConfig JIT(Target target);
    // Compile returns a module backed by a runtime::RuntimeSession: Run(args, input_shapes) goes through its shape
    // cache and background compiler (src/api/compile_config.cc:38-49, src/api/compiler.cc:64-80).
    static CompileConfig Adaptive(Target target, std::vector<std::vector<int64_t>> suggested_shapes = {});
};

// One launch of a compiled module, as an execution-plan node would describe it
// (include/base/execution_plan.h:42-50): operator, kernel symbol, value ids.
struct KernelExecInfo {
    std::string op_name;
    std::string kernel_symbol;
    std::vector<int> input_values;
    std::vector<int> output_values;
};

class CompiledModuleImpl;

class CompiledModule {
public:
    CompiledModule() = default;
    explicit CompiledModule(std::shared_ptr<CompiledModuleImpl> impl) : impl_(std::move(impl)) {}
    void Run(const std::vector<void*>& packed_args);
    // Adaptive modules run only through this overload (the plain one throws "Adaptive mode requires
    // Run(args, input_shapes)..."); for other modules the shapes are ignored (src/api/compiler.cc:146-191).
    void Run(const std::vector<void*>& packed_args, const std::vector<std::vector<int64_t>>& input_shapes);
    void WarmUp(const std::vector<std::vector<int64_t>>& input_shapes);     // adaptive: compile for a shape now
    void WaitAll();                                                          // adaptive: drain background compiles
    bool IsReady() const;
    std::string GetStatus() const;
    // Directory of the profiling bundle; empty when profiling was not enabled (include/api/compiler.h:88).
    std::string GetProfileBundlePath() const;
    // The compiled function behind Run (include/api/compiler.h:96-105 holds a codegen::CompiledKernel likewise).
    const codegen::CompiledKernel& GetKernel() const;
    const tir::PrimFunc& GetPrimFunc() const;
    // Generated source: C for the host back end, HIP for the GPU back end.
    const std::string& GetSource() const;
    void SaveCSource(const std::string& path) const;
    // Constants of the graph in parameter order (host data), to be passed again at every Run.
    const Array<runtime::NDArray>& GetConstants() const;
    int64_t input_count() const;
    int64_t constant_count() const;
    // The launches Run performs, in order.
    const std::vector<KernelExecInfo>& GetKernelExecs() const;
    // Execution-plan description: the schema of src/base/execution_plan.cc:674-877 (value ids, op_name,
    // kernel_symbol per node) plus a "kxc_hip" object with everything LoadExecutionPlan needs.
    std::string ExecutionPlanJSON() const;
    size_t workspace_bytes() const;
    // hip target: later runs on a non-null stream with unchanged argument pointers replay a captured HIP graph
    // (one launch call per Run instead of one per kernel; for launch-bound, small-batch functions).
    void EnableGraphReplay(bool enable);
    // hip target: see CompileConfigNode::hip_constants_frozen.
    void FreezeConstants(bool frozen);
    void InvalidateConstants();
    // hip target: one Run with a HIP event between consecutive launches; returns each launch's duration in
    // nanoseconds, in the order of GetKernelExecs() (waits for the last launch).
    std::vector<int64_t> RunTimed(const std::vector<void*>& packed_args);

private:
    friend class Compiler;
    std::shared_ptr<CompiledModuleImpl> impl_;
    std::shared_ptr<runtime::RuntimeSession> session_;     // adaptive mode only
    std::shared_ptr<profiling::ProfileContext> session_profile_;
};

class Compiler {
public:
    static CompiledModule Compile(Function func, CompileConfig config);
    // Rebuilds a runnable module for the hip target from CompiledModule::ExecutionPlanJSON() without the
    // graph: saved kernel sources are compiled again, the launches come from the saved launch plan.  The
    // caller passes the same packed arguments (inputs, constants, outputs) to Run as for the original.
    static CompiledModule LoadExecutionPlan(const std::string& plan_json, CompileConfig config);
};

}  // namespace api
}  // namespace kxc
