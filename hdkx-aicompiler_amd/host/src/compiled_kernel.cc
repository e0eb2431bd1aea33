// compiled_kernel.cc -- CompiledKernelNode / CompiledKernel (see codegen.h).
#include <dlfcn.h>

#include <cstdio>

#include "kxc/codegen.h"
#include "kxc_hip.h"

namespace kxc {
namespace codegen {

CompiledKernelNode::~CompiledKernelNode() {
    if (backend == CodeGenBackend::kHIP) {
        if (jit_resource) kxc_hip_plan_destroy(static_cast<kxc_hip_plan*>(jit_resource));
        for (void* m : hip_modules) kxc_hip_module_free(static_cast<kxc_hip_module*>(m));
        jit_resource = nullptr;
    }
    if (lib_handle) {
        dlclose(lib_handle);
        lib_handle = nullptr;
    }
    if (!so_path.empty()) std::remove(so_path.c_str());      // the library was built for this kernel alone
    func_ptr = nullptr;
}

void CompiledKernel::operator()(const std::vector<void*>& args) const {
    const CompiledKernelNode* node = get();
    if (!node || !node->func_ptr) throw std::runtime_error("CompiledKernel: not ready or func_ptr is null");
    if (node->backend == CodeGenBackend::kHIP) {
        int32_t ret = kxc_hip_plan_run(static_cast<kxc_hip_plan*>(node->jit_resource), const_cast<void**>(args.data()), nullptr);
        if (ret == 0 && node->sync_after_run) ret = kxc_hip_stream_sync(node->device_id, nullptr);
        if (ret != 0)
            throw std::runtime_error("Kernel " + node->kernel_name + " returned error code " + std::to_string(ret) + ": " +
                                     kxc_hip_last_error());
        return;
    }
    using KernelFunc = int32_t (*)(void**);
    const int32_t ret = reinterpret_cast<KernelFunc>(node->func_ptr)(const_cast<void**>(args.data()));
    if (ret != 0) throw std::runtime_error("Kernel " + node->kernel_name + " returned error code " + std::to_string(ret));
}

bool CompiledKernel::IsReady() const { return get() != nullptr && get()->func_ptr != nullptr; }

}  // namespace codegen
}  // namespace kxc
