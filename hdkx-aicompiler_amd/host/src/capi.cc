// capi.cc -- a small C face of the host layer so that non-C++ callers (the benchmark, tests) can compile
// a graph for a target and run it with device pointers.  Errors are returned as codes; the message is
// kept per thread.
#include <cstring>
#include <memory>

#include "kxc/compiler.h"
#include "kxc/models.h"

namespace {
thread_local std::string g_error;
struct ModuleHandle {
    kxc::api::CompiledModule module;
    std::string symbols;     // newline-separated kernel symbols
    std::string plan_json;
    std::string constant_names;     // newline-separated, packed-argument order (graphs whose builder names its constants)
};
}  // namespace

extern "C" {

const char* kxc_host_last_error(void) { return g_error.c_str(); }

// target: "hip" or "cpu".  sync_after_run = 0 leaves synchronisation to the caller (benchmarks).
int kxc_host_compile_resnet18(const char* target, long long batch, long long hw, int use_handwritten, int fuse,
                              int sync_after_run, void** out_module) {
    try {
        const bool gpu = std::strcmp(target, "cpu") != 0;
        auto config = kxc::api::CompileConfig::AOT(kxc::BuildTarget(gpu ? kxc::kGPU : kxc::kCPU));
        config->hip_use_handwritten = use_handwritten != 0;
        config->hip_fuse = fuse != 0;
        config->sync_after_run = sync_after_run != 0;
        auto* h = new ModuleHandle();
        h->module = kxc::api::Compiler::Compile(kxc::models::BuildResNet18(batch, hw), config);
        for (const auto& e : h->module.GetKernelExecs()) h->symbols += e.op_name + " " + e.kernel_symbol + "\n";
        h->plan_json = h->module.ExecutionPlanJSON();
        *out_module = h;
        return 0;
    } catch (const std::exception& e) {
        g_error = e.what();
        return 1;
    }
}

// The quantised ResNet-18 (kxc::models::BuildQResNet18): res_mult = 8 residual multipliers, one per block.
// lanes: CompileConfigNode::hip_batch_lanes (0 = the back end decides).
// result: "" for the logits, or the name of an int8 activation to return instead (see BuildQResNet18).
int kxc_host_compile_qresnet18(const char* target, long long batch, long long hw, double input_scale, const double* res_mult,
                               double gap_mult, int lanes, int sync_after_run, const char* result, void** out_module) {
    try {
        const bool gpu = std::strcmp(target, "cpu") != 0;
        auto config = kxc::api::CompileConfig::AOT(kxc::BuildTarget(gpu ? kxc::kGPU : kxc::kCPU));
        config->sync_after_run = sync_after_run != 0;
        config->hip_batch_lanes = lanes;
        kxc::models::QResNet18Scales scales;
        scales.input_scale = input_scale;
        for (int i = 0; i < 8; ++i) scales.res_mult[i] = res_mult[i];
        scales.gap_mult = gap_mult;
        std::unique_ptr<ModuleHandle> h(new ModuleHandle());
        std::vector<kxc::runtime::NDArray> consts;
        std::vector<std::string> names;
        h->module = kxc::api::Compiler::Compile(kxc::models::BuildQResNet18(batch, hw, scales, &consts, &names, result ? result : ""), config);
        for (const auto& c : h->module.GetConstants())
            for (size_t i = 0; i < consts.size(); ++i)
                if (consts[i].get() == c.get()) h->constant_names += names[i] + "\n";
        for (const auto& e : h->module.GetKernelExecs()) h->symbols += e.op_name + " " + e.kernel_symbol + "\n";
        h->plan_json = h->module.ExecutionPlanJSON();
        *out_module = h.release();
        return 0;
    } catch (const std::exception& e) {
        g_error = e.what();
        return 1;
    }
}

int kxc_host_module_run(void* module, void** packed_args, int num_args) {
    try {
        static_cast<ModuleHandle*>(module)->module.Run(std::vector<void*>(packed_args, packed_args + num_args));
        return 0;
    } catch (const std::exception& e) {
        g_error = e.what();
        return 1;
    }
}

int kxc_host_module_enable_graph(void* module, int enable) {
    try {
        static_cast<ModuleHandle*>(module)->module.EnableGraphReplay(enable != 0);
        return 0;
    } catch (const std::exception& e) {
        g_error = e.what();
        return 1;
    }
}

int kxc_host_module_freeze_constants(void* module, int frozen) {
    try {
        static_cast<ModuleHandle*>(module)->module.FreezeConstants(frozen != 0);
        return 0;
    } catch (const std::exception& e) {
        g_error = e.what();
        return 1;
    }
}

int kxc_host_module_invalidate_constants(void* module) {
    try {
        static_cast<ModuleHandle*>(module)->module.InvalidateConstants();
        return 0;
    } catch (const std::exception& e) {
        g_error = e.what();
        return 1;
    }
}

// durations_ns[i] = duration of launch i (order of kxc_host_module_symbols); *count = number of launches.
int kxc_host_module_run_timed(void* module, void** packed_args, int num_args, long long* durations_ns, int capacity, int* count) {
    try {
        const std::vector<int64_t> d =
            static_cast<ModuleHandle*>(module)->module.RunTimed(std::vector<void*>(packed_args, packed_args + num_args));
        *count = static_cast<int>(d.size());
        if (capacity < *count) { g_error = "kxc_host_module_run_timed: capacity too small"; return 1; }
        for (size_t i = 0; i < d.size(); ++i) durations_ns[i] = d[i];
        return 0;
    } catch (const std::exception& e) {
        g_error = e.what();
        return 1;
    }
}

int kxc_host_module_is_ready(void* module) { return static_cast<ModuleHandle*>(module)->module.IsReady() ? 1 : 0; }
const char* kxc_host_module_status(void* module) {
    g_error = static_cast<ModuleHandle*>(module)->module.GetStatus();
    return g_error.c_str();
}
const char* kxc_host_module_symbols(void* module) { return static_cast<ModuleHandle*>(module)->symbols.c_str(); }
const char* kxc_host_module_constant_names(void* module) { return static_cast<ModuleHandle*>(module)->constant_names.c_str(); }
const char* kxc_host_module_plan_json(void* module) { return static_cast<ModuleHandle*>(module)->plan_json.c_str(); }
long long kxc_host_module_workspace_bytes(void* module) {
    return static_cast<long long>(static_cast<ModuleHandle*>(module)->module.workspace_bytes());
}
void kxc_host_module_free(void* module) { delete static_cast<ModuleHandle*>(module); }

}  // extern "C"
