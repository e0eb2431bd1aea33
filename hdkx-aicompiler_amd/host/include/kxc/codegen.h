// codegen.h -- TIR -> C text for the host, TIR -> HIP source for gfx950.
//
// CodeGenC mirrors the reference's C back end (src/codegen/codegen_c.cc:54-276): one function
// `int32_t <name>(void** packed_args)` of scalar serial loops.  Differences on purpose: buffer
// names are made unique (the reference declares same-named arrays twice for a graph that calls an
// operator twice) and intermediates are heap-allocated like its LLVM back end does
// (src/codegen/codegen_llvm.cc:578-623) instead of living on the stack.
//
// CodeGenHIP is the GPU emitter the reference reserves an enum value for
// (include/codegen/codegen.h:19-23, kCUDA "future extension").  Every top-level compute stage of
// the PrimFunc becomes one `extern "C" __global__` kernel:
//   * the stage's data-parallel loop nest is flattened to one index; a workgroup is 256 threads =
//     four 64-lane wavefronts, the innermost data axis is the lane-fastest one (coalesced stores),
//     and a grid-stride loop covers the rest;
//   * reduce loops stay inside the thread, in the CPU order, accumulating through the output
//     element exactly as the lowered TIR does -- so a generated kernel is bit-identical to the CPU
//     loop nest (the source is compiled without multiply-add contraction);
//   * LDS staging: a reduction whose source rows are contiguous in memory (global average pool,
//     reduce_mean over trailing axes, row sums) is scheduled as a cooperative, coalesced load of the
//     workgroup's rows into LDS followed by per-thread sequential sums from LDS (odd row stride, no
//     bank conflicts), which keeps the order and removes the strided global reads; a reduction whose innermost
//     axis walks an operand contiguously per thread (dense / matmul against a transposed operand, long rows) stages
//     that operand a chunk of the axis at a time the same way ("lds_k_stage"), again adding in the CPU order.
#pragma once

#include "kxc/tir.h"

namespace kxc {
namespace codegen {

enum class CodeGenBackend { kLLVM, kC, kCUDA, kHIP };

class CodeGenC {
public:
    std::string Generate(const tir::PrimFunc& func, const std::string& name = "main");
};

struct HIPKernelSpec {
    std::string symbol;
    uint32_t grid[3] = {1, 1, 1};
    uint32_t block[3] = {256, 1, 1};
    uint32_t shared_bytes = 0;
    // kernel parameters: the buffer variables of the PrimFunc (parameters or Allocate'd intermediates)
    std::vector<const tir::ExprNode*> buffers;
    std::string schedule;     // "flat", "lds_row_reduce" or "lds_k_stage"
};

struct HIPModuleSource {
    std::string source;
    std::vector<HIPKernelSpec> kernels;      // in execution order
};

// One compiled function behind the Run ABI `int32_t f(void** packed_args)`: what the reference's CompiledKernelNode
// is for its LLVM JIT and C back ends (include/codegen/compiled_kernel.h:19-41), with the HIP back end's resources
// beside them.  Host back ends: func_ptr is the entry point of a library opened from so_path (lib_handle).  HIP back
// end: jit_resource owns the launch plan and func_ptr is non-null exactly while that plan can be run, so
// IsReady() keeps its meaning; hip_modules are the run-time compiled modules whose kernels the plan launches.
// The destructor releases everything (dlclose, plan, modules), as the reference's does for its back ends
// (src/codegen/compiled_kernel.cc:21-39).
class CompiledKernelNode : public Object {
public:
    std::string kernel_name;
    CodeGenBackend backend{CodeGenBackend::kC};
    void* func_ptr{nullptr};
    void* jit_resource{nullptr};
    std::string so_path;
    void* lib_handle{nullptr};
    std::vector<tir::BufferInfo> param_buffers;      // signature of the packed arguments, in order
    // HIP back end
    std::vector<void*> hip_modules;                  // kxc_hip_module*
    int device_id{0};
    bool sync_after_run{true};                       // wait for the stream after enqueueing (callers read outputs at once)
    ~CompiledKernelNode() override;
};

class CompiledKernel : public Ref<CompiledKernelNode> {
public:
    CompiledKernel() = default;
    explicit CompiledKernel(std::shared_ptr<CompiledKernelNode> n) : Ref<CompiledKernelNode>(std::move(n)) {}
    // Calls the function with packed_args = inputs, constants, outputs.  Throws "CompiledKernel: not ready or
    // func_ptr is null", or "Kernel <name> returned error code N" (src/codegen/compiled_kernel.cc:41-55; the HIP back
    // end appends the library's message).  HIP: every pointer is a device pointer; the launches go to the calling
    // thread's current stream.
    void operator()(const std::vector<void*>& args) const;
    bool IsReady() const;
};

class CodeGenHIP {
public:
    // prefix: made part of every kernel symbol so several PrimFuncs can share one module
    HIPModuleSource Generate(const tir::PrimFunc& func, const std::string& prefix = "kxc");
};

}  // namespace codegen
}  // namespace kxc
