// module.hip -- run-time compiled kernels: hipRTC compile for gfx950, hipModule load, launch.
// The loader a HIP CompiledKernelNode owns; mirrors the NVRTC + cuLaunchKernel sequence of the
// reference's only device-code launch site (test/cupti_smoke_test.cpp:143-205).
// Compilation is thread safe (hipRTC programs are independent objects; a mutex serialises the
// module load), because Compile may run on background worker threads
// (src/runtime/background_compiler.cc:52-92).
#include <hip/hiprtc.h>

#include <cstring>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include "common.h"

using namespace kxc_hip;

struct kxc_hip_module {
    hipModule_t module = nullptr;
    std::vector<char> code;
};

namespace {

std::mutex& LoadMutex() {
    static std::mutex m;
    return m;
}

std::unordered_map<hipFunction_t, std::string>& FunctionNames() {      // guarded by LoadMutex()
    static std::unordered_map<hipFunction_t, std::string> names;
    return names;
}

void CopyLog(const std::string& text, char* log, size_t cap) {
    if (!log || cap == 0) return;
    const size_t n = text.size() < cap - 1 ? text.size() : cap - 1;
    std::memcpy(log, text.data(), n);
    log[n] = '\0';
}

// Compile `source` to a gfx950 code object.  Strict fp32: no multiply-add contraction, so generated
// loop nests round exactly like the CPU backend's; packed fp32 instructions are disabled.
int32_t CompileToCode(const char* source, const char* name, std::vector<char>* code, char* log, size_t log_cap) {
    KXC_HIP_REQUIRE(source != nullptr, "kxc_hip_module_compile: source is NULL");
    hiprtcProgram prog = nullptr;
    hiprtcResult r = hiprtcCreateProgram(&prog, source, name ? name : "kxc_module.hip", 0, nullptr, nullptr);
    if (r != HIPRTC_SUCCESS) return Fail(KXC_HIP_ERR_COMPILE, "hiprtcCreateProgram failed: %s", hiprtcGetErrorString(r));
    const char* opts[] = {"--offload-arch=gfx950", "-O3", "-ffp-contract=off", "-std=c++17"};
    // The packed-fp32 switch is passed as a target feature where the front end accepts it; try the
    // feature form first and fall back to plain options if this hipRTC rejects it.
    const char* opts_feature[] = {"--offload-arch=gfx950", "-O3", "-ffp-contract=off", "-std=c++17",
                                  "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"};
    r = hiprtcCompileProgram(prog, 8, opts_feature);
    if (r != HIPRTC_SUCCESS) {
        std::string first_log;
        size_t n = 0;
        if (hiprtcGetProgramLogSize(prog, &n) == HIPRTC_SUCCESS && n > 1) {
            first_log.resize(n);
            hiprtcGetProgramLog(prog, &first_log[0]);
        }
        // Distinguish "option not understood" from a real compile error in the source.
        if (first_log.find("target-feature") != std::string::npos || first_log.find("Xclang") != std::string::npos ||
            first_log.find("unknown argument") != std::string::npos) {
            hiprtcDestroyProgram(&prog);
            prog = nullptr;
            r = hiprtcCreateProgram(&prog, source, name ? name : "kxc_module.hip", 0, nullptr, nullptr);
            if (r != HIPRTC_SUCCESS)
                return Fail(KXC_HIP_ERR_COMPILE, "hiprtcCreateProgram failed: %s", hiprtcGetErrorString(r));
            r = hiprtcCompileProgram(prog, 4, opts);
        }
    }
    std::string text;
    size_t log_size = 0;
    if (hiprtcGetProgramLogSize(prog, &log_size) == HIPRTC_SUCCESS && log_size > 1) {
        text.resize(log_size);
        hiprtcGetProgramLog(prog, &text[0]);
    }
    CopyLog(text, log, log_cap);
    if (r != HIPRTC_SUCCESS) {
        hiprtcDestroyProgram(&prog);
        return Fail(KXC_HIP_ERR_COMPILE, "hipRTC compilation failed: %s\n%s", hiprtcGetErrorString(r), text.c_str());
    }
    size_t code_size = 0;
    r = hiprtcGetCodeSize(prog, &code_size);
    if (r == HIPRTC_SUCCESS) {
        code->resize(code_size);
        r = hiprtcGetCode(prog, code->data());
    }
    hiprtcDestroyProgram(&prog);
    if (r != HIPRTC_SUCCESS) return Fail(KXC_HIP_ERR_COMPILE, "hiprtcGetCode failed: %s", hiprtcGetErrorString(r));
    return KXC_HIP_OK;
}

}  // namespace

extern "C" {

int32_t kxc_hip_module_compile_only(const char* source, const char* name, size_t* out_size, char* log,
                                    size_t log_capacity) {
    std::vector<char> code;
    if (int32_t rc = CompileToCode(source, name, &code, log, log_capacity)) return rc;
    if (out_size) *out_size = code.size();
    return KXC_HIP_OK;
}

int32_t kxc_hip_module_compile(const char* source, const char* name, kxc_hip_module** out, char* log,
                               size_t log_capacity) {
    KXC_HIP_REQUIRE(out != nullptr, "kxc_hip_module_compile: out is NULL");
    *out = nullptr;
    std::vector<char> code;
    if (int32_t rc = CompileToCode(source, name, &code, log, log_capacity)) return rc;
    kxc_hip_module* m = new kxc_hip_module();
    m->code.swap(code);
    {
        std::lock_guard<std::mutex> lock(LoadMutex());
        hipError_t e = hipModuleLoadData(&m->module, m->code.data());
        if (e != hipSuccess) {
            delete m;
            return Fail(KXC_HIP_ERR_RUNTIME, "hipModuleLoadData failed: %s", hipGetErrorString(e));
        }
    }
    *out = m;
    return KXC_HIP_OK;
}

int32_t kxc_hip_module_get_function(kxc_hip_module* module, const char* symbol, void** out_function) {
    KXC_HIP_REQUIRE(module && module->module && symbol && out_function, "kxc_hip_module_get_function: NULL argument");
    hipFunction_t f = nullptr;
    hipError_t e = hipModuleGetFunction(&f, module->module, symbol);
    if (e != hipSuccess)
        return Fail(KXC_HIP_ERR_RUNTIME, "hipModuleGetFunction(%s) failed: %s", symbol, hipGetErrorString(e));
    {
        std::lock_guard<std::mutex> lock(LoadMutex());
        FunctionNames()[f] = symbol;        // launch records name their kernel
    }
    *out_function = f;
    return KXC_HIP_OK;
}

int32_t kxc_hip_module_launch(void* function, const uint32_t grid[3], const uint32_t block[3], uint32_t shared_bytes,
                              void* stream, void** kernel_params) {
    KXC_HIP_REQUIRE(function && grid && block, "kxc_hip_module_launch: NULL argument");
    KXC_HIP_REQUIRE(grid[0] > 0 && grid[1] > 0 && grid[2] > 0 && block[0] > 0 && block[1] > 0 && block[2] > 0,
                    "kxc_hip_module_launch: empty grid or block");
    KXC_HIP_REQUIRE(static_cast<uint64_t>(block[0]) * block[1] * block[2] <= 1024,
                    "kxc_hip_module_launch: more than 1024 threads per block");
    NoteGrid(dim3(grid[0], grid[1], grid[2]));
    NoteBlock(dim3(block[0], block[1], block[2]));
    NoteLds(shared_bytes);
    hipStream_t s = ResolveStream(stream);
    hipError_t e = hipSuccess;
    if (ActivityOn()) {
        std::string name = "kxc_module_kernel";
        {
            std::lock_guard<std::mutex> lock(LoadMutex());
            auto it = FunctionNames().find(reinterpret_cast<hipFunction_t>(function));
            if (it != FunctionNames().end()) name = it->second;
        }
        ApiScope api("hipModuleLaunchKernel");
        DeviceScope dev(KXC_HIP_ACTIVITY_KERNEL, name.c_str(), s, api.correlation());
        for (int i = 0; i < 3; ++i) { dev.grid[i] = grid[i]; dev.block[i] = block[i]; }
        dev.dynamic_shared_memory = shared_bytes;
        e = hipModuleLaunchKernel(reinterpret_cast<hipFunction_t>(function), grid[0], grid[1], grid[2], block[0], block[1],
                                  block[2], shared_bytes, s, kernel_params, nullptr);
        api.SetResult(e);
    } else {
        e = hipModuleLaunchKernel(reinterpret_cast<hipFunction_t>(function), grid[0], grid[1], grid[2], block[0], block[1],
                                  block[2], shared_bytes, s, kernel_params, nullptr);
    }
    KXC_HIP_CALL(e, "hipModuleLaunchKernel");
    return KXC_HIP_OK;
}

int32_t kxc_hip_module_free(kxc_hip_module* module) {
    if (!module) return KXC_HIP_OK;
    hipError_t e = hipSuccess;
    if (module->module) {
        std::lock_guard<std::mutex> lock(LoadMutex());
        e = hipModuleUnload(module->module);
    }
    delete module;
    KXC_HIP_CALL(e, "hipModuleUnload");
    return KXC_HIP_OK;
}

}  // extern "C"
