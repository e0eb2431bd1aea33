// packed_func.cc -- the global function registry and the functions registered in it (see packed_func.h).
#include "kxc/packed_func.h"

#include <fstream>
#include <mutex>
#include <sstream>

#include "kxc/compiler.h"
#include "kxc/relay.h"

namespace kxc {

namespace {
std::mutex& RegistryMutex() {
    static std::mutex mu;
    return mu;
}
}  // namespace

Registry& Registry::Global() {
    static Registry instance;
    return instance;
}

void Registry::Set(const std::string& name, PackedFunc func) {
    std::lock_guard<std::mutex> lock(RegistryMutex());
    if (functions_.count(name)) throw std::runtime_error("Function " + name + " is already registered.");
    functions_[name] = std::move(func);
}

PackedFunc Registry::Get(const std::string& name) const {
    std::lock_guard<std::mutex> lock(RegistryMutex());
    auto it = functions_.find(name);
    return it == functions_.end() ? PackedFunc() : it->second;
}

std::vector<std::string> Registry::ListNames() const {
    std::lock_guard<std::mutex> lock(RegistryMutex());
    std::vector<std::string> names;
    for (const auto& kv : functions_) names.push_back(kv.first);
    return names;
}

namespace {

template <typename T>
T Arg(const Args& args, int i) { return ArgConverter<T>::From(args[i], args.type_code(i)); }
void* Ptr(const Args& args, int i) { return reinterpret_cast<void*>(static_cast<uintptr_t>(Arg<int64_t>(args, i))); }
int64_t Int(const void* p) { return static_cast<int64_t>(reinterpret_cast<uintptr_t>(p)); }
DeviceAPI* ApiOf(const Device& d) { return DeviceAPIManager::Global()->GetAPI(d.device_type()); }
// a copy that touches the GPU is the GPU back end's (src/base/device_api.cc:499-504)
DeviceAPI* CopyApi(const Device& from, const Device& to) {
    return (from.device_type() == kCPU && to.device_type() != kCPU) ? ApiOf(to) : ApiOf(from);
}
using Body = PackedFunc::Body;

// Pointers and streams travel as integers, devices as objects; argument order as in src/base/device_api.cc:442-658.
KXC_REGISTER_GLOBAL("device_api.AllocDataSpace").set_body(PackedFunc(Body([](Args a, RetValue* rv) {
    const Device dev = Arg<Device>(a, 0);
    *rv = Int(ApiOf(dev)->AllocDataSpace(dev, static_cast<size_t>(Arg<int64_t>(a, 1)), static_cast<size_t>(Arg<int64_t>(a, 2))));
})));
KXC_REGISTER_GLOBAL("device_api.FreeDataSpace").set_body(PackedFunc(Body([](Args a, RetValue*) {
    const Device dev = Arg<Device>(a, 0);
    ApiOf(dev)->FreeDataSpace(dev, Ptr(a, 1));
})));
KXC_REGISTER_GLOBAL("device_api.AllocWorkspace").set_body(PackedFunc(Body([](Args a, RetValue* rv) {
    const Device dev = Arg<Device>(a, 0);
    *rv = Int(ApiOf(dev)->AllocWorkspace(dev, static_cast<size_t>(Arg<int64_t>(a, 1)), static_cast<size_t>(Arg<int64_t>(a, 2))));
})));
KXC_REGISTER_GLOBAL("device_api.FreeWorkspace").set_body(PackedFunc(Body([](Args a, RetValue*) {
    const Device dev = Arg<Device>(a, 0);
    ApiOf(dev)->FreeWorkspace(dev, Ptr(a, 1));
})));
KXC_REGISTER_GLOBAL("device_api.CopyDataFromTo").set_body(PackedFunc(Body([](Args a, RetValue*) {
    const Device from = Arg<Device>(a, 0), to = Arg<Device>(a, 2);
    CopyApi(from, to)->CopyDataFromTo(from, Ptr(a, 1), to, Ptr(a, 3), static_cast<size_t>(Arg<int64_t>(a, 4)));
})));
KXC_REGISTER_GLOBAL("device_api.CopyDataFromToEx").set_body(PackedFunc(Body([](Args a, RetValue*) {
    const Device from = Arg<Device>(a, 0), to = Arg<Device>(a, 3);
    CopyApi(from, to)->CopyDataFromTo(Ptr(a, 1), static_cast<size_t>(Arg<int64_t>(a, 2)), Ptr(a, 4),
                                      static_cast<size_t>(Arg<int64_t>(a, 5)), static_cast<size_t>(Arg<int64_t>(a, 6)), from, to,
                                      static_cast<StreamHandle>(Ptr(a, 7)));
})));
KXC_REGISTER_GLOBAL("device_api.GetAttr").set_body(PackedFunc(Body([](Args a, RetValue* rv) {
    GetDeviceAttr(Arg<Device>(a, 0), static_cast<DeviceAttrKind>(Arg<int>(a, 1)), rv);
})));
KXC_REGISTER_GLOBAL("device_api.CreateStream").set_body(PackedFunc(Body([](Args a, RetValue* rv) {
    const Device dev = Arg<Device>(a, 0);
    *rv = Int(ApiOf(dev)->CreateStream(dev));
})));
KXC_REGISTER_GLOBAL("device_api.FreeStream").set_body(PackedFunc(Body([](Args a, RetValue*) {
    const Device dev = Arg<Device>(a, 0);
    ApiOf(dev)->FreeStream(dev, static_cast<StreamHandle>(Ptr(a, 1)));
})));
KXC_REGISTER_GLOBAL("device_api.StreamSync").set_body(PackedFunc(Body([](Args a, RetValue*) {
    const Device dev = Arg<Device>(a, 0);
    ApiOf(dev)->StreamSync(dev, static_cast<StreamHandle>(Ptr(a, 1)));
})));
KXC_REGISTER_GLOBAL("device_api.SyncStreamFromTo").set_body(PackedFunc(Body([](Args a, RetValue*) {
    const Device dev = Arg<Device>(a, 0);
    ApiOf(dev)->SyncStreamFromTo(dev, static_cast<StreamHandle>(Ptr(a, 1)), static_cast<StreamHandle>(Ptr(a, 2)));
})));
KXC_REGISTER_GLOBAL("device_api.SetStream").set_body(PackedFunc(Body([](Args a, RetValue*) {
    const Device dev = Arg<Device>(a, 0);
    ApiOf(dev)->SetStream(dev, static_cast<StreamHandle>(Ptr(a, 1)));
})));
KXC_REGISTER_GLOBAL("device_api.GetCurrentStream").set_body(PackedFunc(Body([](Args a, RetValue* rv) {
    const Device dev = Arg<Device>(a, 0);
    *rv = Int(ApiOf(dev)->GetCurrentStream(dev));
})));
KXC_REGISTER_GLOBAL("device_api.NeedSetDevice").set_body(PackedFunc(Body([](Args a, RetValue* rv) {
    *rv = static_cast<int64_t>(DeviceAPI::NeedSetDevice(static_cast<DeviceTypeCode>(Arg<int>(a, 0))));
})));
KXC_REGISTER_GLOBAL("device_api.ListDevices").set_body(PackedFunc(Body([](Args, RetValue* rv) { *rv = ListDevicesJSON(); })));
KXC_REGISTER_GLOBAL("device_api.ListDevicesJSON").set_body(PackedFunc(Body([](Args, RetValue* rv) { *rv = ListDevicesJSON(); })));
KXC_REGISTER_GLOBAL("device_api.GetAllDeviceInfo").set_body(PackedFunc(Body([](Args, RetValue* rv) { *rv = GetAllDeviceInfoJSON(); })));
KXC_REGISTER_GLOBAL("device_api.GetAllDeviceInfoJSON").set_body(PackedFunc(Body([](Args, RetValue* rv) { *rv = GetAllDeviceInfoJSON(); })));
KXC_REGISTER_GLOBAL("device_api.GetTargetKind").set_body(PackedFunc(Body([](Args a, RetValue* rv) {
    const Device dev = Arg<Device>(a, 0);
    *rv = BuildTarget(dev.device_type(), dev.device_id())->kind;
})));
KXC_REGISTER_GLOBAL("device_api.GetTargetArch").set_body(PackedFunc(Body([](Args a, RetValue* rv) {
    const Device dev = Arg<Device>(a, 0);
    *rv = BuildTarget(dev.device_type(), dev.device_id())->attrs.arch;
})));
KXC_REGISTER_GLOBAL("target.Build").set_body(PackedFunc(Body([](Args a, RetValue* rv) {
    const Device dev = Arg<Device>(a, 0);
    *rv = ObjectRef(BuildTarget(dev.device_type(), dev.device_id()));
})));
KXC_REGISTER_GLOBAL("device.DetectAndRegister").set_body(PackedFunc(Body([](Args, RetValue*) { DetectAndRegisterDevices(); })));

// ---- a Relay function -> execution plan JSON (src/relay/transforms/multi_device.cc:524-539), compiled for the hip
// target, and the single-device runners of such a plan (the reference's runners take a multi-worker session,
// src/base/disco/executor.cc:284-322; one GPU needs none).
Function FunctionArg(const Args& a, int i) {
    const ObjectRef ref = Arg<ObjectRef>(a, i);
    auto node = std::dynamic_pointer_cast<FunctionNode>(ref.shared());
    if (!node) throw std::runtime_error("Type mismatch, expected ObjectRef");
    return Function(node->params, node->body);      // (a handle to an equal function: same parameters, same body)
}
std::string PlanJson(const Function& func) {
    auto config = api::CompileConfig::JIT(BuildTarget(kGPU, 0));
    return api::Compiler::Compile(func, config).ExecutionPlanJSON();
}
std::string ReadFile(const std::string& path) {
    std::ifstream in(path, std::ios::binary);
    if (!in) throw std::runtime_error("cannot open execution plan file: " + path);
    std::ostringstream os;
    os << in.rdbuf();
    return os.str();
}
// args: plan text, pointer to `count` packed argument pointers (inputs, constants, outputs), count
void RunPlanJson(const std::string& json, void* const* packed, int64_t count) {
    auto config = api::CompileConfig::JIT(BuildTarget(kGPU, 0));
    api::CompiledModule module = api::Compiler::LoadExecutionPlan(json, config);
    module.Run(std::vector<void*>(packed, packed + count));
}
KXC_REGISTER_GLOBAL("kxc.relay.transform.lower_to_exec_plan_json").set_body(PackedFunc(Body([](Args a, RetValue* rv) {
    *rv = PlanJson(FunctionArg(a, 0));
})));
KXC_REGISTER_GLOBAL("kxc.relay.transform.lower_to_exec_plan_json_file").set_body(PackedFunc(Body([](Args a, RetValue* rv) {
    const std::string path = Arg<std::string>(a, 1);
    std::ofstream out(path, std::ios::binary);
    if (!out) throw std::runtime_error("cannot write execution plan file: " + path);
    out << PlanJson(FunctionArg(a, 0));
    *rv = path;
})));
KXC_REGISTER_GLOBAL("kxc.hip.execute_plan_json").set_body(PackedFunc(Body([](Args a, RetValue* rv) {
    RunPlanJson(Arg<std::string>(a, 0), static_cast<void* const*>(Arg<void*>(a, 1)), Arg<int64_t>(a, 2));
    *rv = static_cast<int64_t>(0);
})));
KXC_REGISTER_GLOBAL("kxc.hip.execute_plan_json_file").set_body(PackedFunc(Body([](Args a, RetValue* rv) {
    RunPlanJson(ReadFile(Arg<std::string>(a, 0)), static_cast<void* const*>(Arg<void*>(a, 1)), Arg<int64_t>(a, 2));
    *rv = static_cast<int64_t>(0);
})));

}  // namespace

void DetectAndRegisterDevices() {
    static std::once_flag once;
    std::call_once(once, [] {
        for (const DeviceInfo& info : GetAllDeviceInfo()) {
            if (info.device_type != kGPU || !info.available) continue;
            const std::string prefix = "device_info.hip." + std::to_string(info.device_id);
            const std::string name = info.attrs.device_name, cap = info.attrs.compute_version;
            const int64_t memory = info.attrs.total_global_memory;
            Registry& reg = Registry::Global();
            reg.Set(prefix + ".name", PackedFunc(Body([name](Args, RetValue* rv) { *rv = name; })));
            reg.Set(prefix + ".memory", PackedFunc(Body([memory](Args, RetValue* rv) { *rv = memory; })));
            reg.Set(prefix + ".compute_capability", PackedFunc(Body([cap](Args, RetValue* rv) { *rv = cap; })));
        }
    });
}

}  // namespace kxc
