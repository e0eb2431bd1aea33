// device_api.cc -- CPUDeviceAPI, HIPDeviceAPI (over the C ABI), device enumeration, BuildTarget.
#include "kxc/device_api.h"
#include "kxc/profiling.h"

#include <cstdlib>
#include <cstring>
#include <sstream>

#include "kxc_hip.h"

namespace kxc {

// ------------------------------------------------------------------ defaults of optional calls
void DeviceAPI::CopyDataFromTo(const void* from_ptr, size_t from_offset, void* to_ptr, size_t to_offset, size_t nbytes,
                               const Device& from_dev, const Device& to_dev, StreamHandle) {
    CopyDataFromTo(from_dev, static_cast<const char*>(from_ptr) + from_offset, to_dev, static_cast<char*>(to_ptr) + to_offset,
                   nbytes);
}
StreamHandle DeviceAPI::CreateStream(const Device&) { return nullptr; }
void DeviceAPI::FreeStream(const Device&, StreamHandle) {}
void DeviceAPI::SetStream(const Device&, StreamHandle) {}
StreamHandle DeviceAPI::GetCurrentStream(const Device&) { return nullptr; }
void DeviceAPI::StreamSync(const Device&, StreamHandle) {}
void DeviceAPI::SyncStreamFromTo(const Device&, StreamHandle, StreamHandle) {}
void* DeviceAPI::AllocWorkspace(const Device& device, size_t nbytes, size_t alignment) {
    return AllocDataSpace(device, nbytes, alignment);
}
void DeviceAPI::FreeWorkspace(const Device& device, void* ptr) { FreeDataSpace(device, ptr); }

namespace {

// src/base/device/cpu_device_api.cc:80-171: posix_memalign + memcpy, target kind "llvm".
class CPUDeviceAPI : public DeviceAPI {
public:
    void SetDevice(const Device&) override {}
    void* AllocDataSpace(const Device&, size_t nbytes, size_t alignment) override {
        void* p = nullptr;
        if (alignment < sizeof(void*)) alignment = sizeof(void*);
        if (posix_memalign(&p, alignment, nbytes ? nbytes : 1) != 0) throw std::runtime_error("CPU AllocDataSpace failed");
        return p;
    }
    void FreeDataSpace(const Device&, void* ptr) override { std::free(ptr); }
    void CopyDataFromTo(const Device&, const void* from_ptr, const Device&, void* to_ptr, size_t nbytes) override {
        std::memcpy(to_ptr, from_ptr, nbytes);
    }
    DeviceAttributes GetDeviceAttributes(const Device&) override {
        DeviceAttributes a;
        a.exists = 1;
        a.device_name = "cpu";
        a.arch = "host";
        a.status = "ok";
        return a;
    }
    std::string GetTargetKind(const Device&) const override { return "llvm"; }
};

// Every device call is a "device_api" span with its byte count, as in the reference's CUDA device API
// (src/base/device/cuda_device_api.cc:90-157); without an active profiling context this is a no-op.
profiling::ScopedSpan ApiSpan(const char* event_type, const Device& d, double bytes = -1.0) {
    if (!profiling::CurrentContext()) return profiling::ScopedSpan();
    profiling::EventSpec e;
    e.component = "device_api";
    e.event_type = event_type;
    e.device = "hip:" + std::to_string(d.device_id());
    if (bytes >= 0.0) e.metrics["bytes"] = bytes;
    return profiling::CurrentSpan(e);
}

[[noreturn]] void ThrowHip(const char* what) {
    throw std::runtime_error(std::string("HIP ") + what + " failed: " + kxc_hip_last_error());
}

// Forwards one for one to the C-ABI device calls (include/kxc_hip.h, section 1).
class HIPDeviceAPI : public DeviceAPI {
public:
    void SetDevice(const Device& d) override {
        if (kxc_hip_set_device(d.device_id())) ThrowHip("SetDevice");
    }
    void* AllocDataSpace(const Device& d, size_t nbytes, size_t alignment) override {
        void* p = nullptr;
        profiling::ScopedSpan span = ApiSpan("alloc_data_space", d, static_cast<double>(nbytes));
        if (kxc_hip_alloc(d.device_id(), nbytes, alignment, &p)) ThrowHip("AllocDataSpace");
        return p;
    }
    void FreeDataSpace(const Device& d, void* ptr) override {
        profiling::ScopedSpan span = ApiSpan("free_data_space", d);
        if (kxc_hip_free(d.device_id(), ptr)) ThrowHip("FreeDataSpace");
    }
    void CopyDataFromTo(const Device& from_dev, const void* from_ptr, const Device& to_dev, void* to_ptr, size_t nbytes) override {
        CopyDataFromTo(from_ptr, 0, to_ptr, 0, nbytes, from_dev, to_dev, nullptr);
    }
    void CopyDataFromTo(const void* from_ptr, size_t from_offset, void* to_ptr, size_t to_offset, size_t nbytes,
                        const Device& from_dev, const Device& to_dev, StreamHandle stream) override {
        const bool fg = from_dev.device_type() == kGPU, tg = to_dev.device_type() == kGPU;
        const int kind = (!fg && tg) ? 0 : (fg && !tg) ? 1 : (fg && tg) ? 2 : 3;
        const int dev = tg ? to_dev.device_id() : from_dev.device_id();
        // event_type "copy" and the "from->to" device tag are what the reference records (cuda_device_api.cc:124-129),
        // and what its bundle analyser sums for the copy_dominance rule
        profiling::ScopedSpan span = ApiSpan("copy", tg ? to_dev : from_dev, static_cast<double>(nbytes));
        span.AddField("device_api.route", std::string(fg ? "hip:" : "cpu:") + std::to_string(from_dev.device_id()) + "->" +
                                              (tg ? "hip:" : "cpu:") + std::to_string(to_dev.device_id()));
        span.AddField("device_api.copy_kind", kind == 0 ? "host_to_device" : kind == 1 ? "device_to_host" : kind == 2 ? "device_to_device" : "host_to_host");
        if (kxc_hip_copy(from_ptr, from_offset, to_ptr, to_offset, nbytes, kind, dev, stream)) ThrowHip("CopyDataFromTo");
    }
    DeviceAttributes GetDeviceAttributes(const Device& d) override {
        kxc_hip_device_attrs a;
        kxc_hip_device_attributes(d.device_id(), &a);      // never fails: exists = 0 + status text
        DeviceAttributes out;
        out.exists = a.exists;
        out.max_threads_per_block = a.max_threads_per_block ? a.max_threads_per_block : 1;
        out.warp_size = a.warp_size;
        out.max_shared_memory_per_block = a.max_shared_memory_per_block;
        out.compute_version = std::to_string(a.compute_version_major) + "." + std::to_string(a.compute_version_minor);
        out.device_name = a.device_name;
        out.max_clock_rate_khz = a.max_clock_rate_khz;
        out.max_registers_per_block = a.max_registers_per_block;
        out.api_version = a.api_version;
        out.driver_version = a.driver_version;
        out.l2_cache_size_bytes = a.l2_cache_size_bytes;
        out.total_global_memory = a.total_global_memory;
        out.available_global_memory = a.available_global_memory;
        out.max_shared_memory_per_multiprocessor = a.max_shared_memory_per_multiprocessor;
        out.max_threads_per_multiprocessor = a.max_threads_per_multiprocessor;
        out.compute_version_major = a.compute_version_major;
        out.compute_version_minor = a.compute_version_minor;
        out.multi_processor_count = a.multi_processor_count ? a.multi_processor_count : 1;
        out.arch = a.arch;
        out.status = a.status;
        return out;
    }
    std::string GetTargetKind(const Device&) const override { return kxc_hip_target_kind(); }
    StreamHandle CreateStream(const Device& d) override {
        void* s = nullptr;
        if (kxc_hip_stream_create(d.device_id(), &s)) ThrowHip("StreamCreate");
        return s;
    }
    void FreeStream(const Device& d, StreamHandle s) override {
        if (kxc_hip_stream_destroy(d.device_id(), s)) ThrowHip("StreamDestroy");
    }
    void SetStream(const Device& d, StreamHandle s) override {
        if (kxc_hip_set_stream(d.device_id(), s)) ThrowHip("SetDevice");
    }
    StreamHandle GetCurrentStream(const Device& d) override {
        void* s = nullptr;
        kxc_hip_get_stream(d.device_id(), &s);
        return s;
    }
    void StreamSync(const Device& d, StreamHandle s) override {
        profiling::ScopedSpan span = ApiSpan("stream_sync", d);
        if (kxc_hip_stream_sync(d.device_id(), s)) ThrowHip("StreamSync");
    }
    void SyncStreamFromTo(const Device& d, StreamHandle src, StreamHandle dst) override {
        if (kxc_hip_stream_wait(d.device_id(), src, dst)) ThrowHip("SyncStreamFromTo");
    }
};

}  // namespace

DeviceAPI* GetCPUDeviceAPI() {
    static CPUDeviceAPI api;
    return &api;
}
DeviceAPI* GetHIPDeviceAPI() {
    static HIPDeviceAPI api;
    return &api;
}
DeviceAPIManager* DeviceAPIManager::Global() {
    static DeviceAPIManager instance;
    return &instance;
}
DeviceAPI* DeviceAPIManager::GetAPI(DeviceTypeCode type) {
    switch (type) {
        case kCPU: return GetCPUDeviceAPI();
        case kGPU: return GetHIPDeviceAPI();
        default: throw std::runtime_error("Device API not supported");
    }
}
DeviceAPI* GetDeviceAPI(DeviceTypeCode type) { return DeviceAPIManager::Global()->GetAPI(type); }

void DeviceAPI::GetAttr(const Device& device, DeviceAttrKind kind, RetValue* rv) {
    const DeviceAttributes a = GetDeviceAttributes(device);
    switch (kind) {
        case DeviceAttrKind::kExist: *rv = a.exists; return;
        case DeviceAttrKind::kMaxThreadsPerBlock: *rv = a.max_threads_per_block; return;
        case DeviceAttrKind::kWarpSize: *rv = a.warp_size; return;
        case DeviceAttrKind::kMaxSharedMemoryPerBlock: *rv = a.max_shared_memory_per_block; return;
        case DeviceAttrKind::kComputeVersion: *rv = a.compute_version; return;
        case DeviceAttrKind::kDeviceName: *rv = a.device_name; return;
        case DeviceAttrKind::kMaxClockRate: *rv = a.max_clock_rate_khz; return;
        case DeviceAttrKind::kMultiProcessorCount: *rv = a.multi_processor_count; return;
        case DeviceAttrKind::kMaxRegistersPerBlock: *rv = a.max_registers_per_block; return;
        case DeviceAttrKind::kApiVersion: *rv = a.api_version; return;
        case DeviceAttrKind::kDriverVersion: *rv = a.driver_version; return;
        case DeviceAttrKind::kL2CacheSizeBytes: *rv = a.l2_cache_size_bytes; return;
        case DeviceAttrKind::kTotalGlobalMemory: *rv = a.total_global_memory; return;
        case DeviceAttrKind::kAvailableGlobalMemory: *rv = a.available_global_memory; return;
        case DeviceAttrKind::kMaxSharedMemoryPerMultiprocessor: *rv = a.max_shared_memory_per_multiprocessor; return;
        case DeviceAttrKind::kMaxRegistersPerMultiprocessor: *rv = a.max_registers_per_block; return;
        case DeviceAttrKind::kMaxThreadsPerMultiprocessor: *rv = a.max_threads_per_multiprocessor; return;
        case DeviceAttrKind::kComputeVersionMajor: *rv = a.compute_version_major; return;
        case DeviceAttrKind::kComputeVersionMinor: *rv = a.compute_version_minor; return;
    }
    throw std::runtime_error("Unknown device attribute kind");
}
void GetDeviceAttr(const Device& device, DeviceAttrKind kind, RetValue* rv) {
    GetDeviceAPI(device.device_type())->GetAttr(device, kind, rv);
}
int64_t GetDeviceAttr(const Device& device, DeviceAttrKind kind) {
    RetValue rv;
    GetDeviceAttr(device, kind, &rv);
    return rv.v_int64;
}

std::vector<DeviceInfo> GetAllDeviceInfo() {
    std::vector<DeviceInfo> out;
    DeviceInfo cpu;
    cpu.device_type = kCPU; cpu.device_id = 0; cpu.device_type_name = "cpu"; cpu.target_kind = "llvm";
    cpu.available = true; cpu.status = "ok"; cpu.attrs = GetCPUDeviceAPI()->GetDeviceAttributes(Device(kCPU, 0));
    out.push_back(cpu);
    // the GPU entry is always listed, available or not (test/device_info_test.cpp:77-90)
    int32_t count = 0;
    kxc_hip_device_count(&count);
    const int n = count > 0 ? count : 1;
    for (int i = 0; i < n; ++i) {
        DeviceInfo g;
        g.device_type = kGPU; g.device_id = i; g.device_type_name = "hip"; g.target_kind = "hip";
        g.attrs = GetHIPDeviceAPI()->GetDeviceAttributes(Device(kGPU, i));
        g.available = g.attrs.exists != 0;
        g.status = g.attrs.status;
        out.push_back(g);
    }
    return out;
}

namespace {
std::string DeviceInfosToJSON(const std::vector<DeviceInfo>& infos);
}
std::string GetAllDeviceInfoJSON() { return DeviceInfosToJSON(GetAllDeviceInfo()); }

// Only the devices that can be used (src/base/device_api.cc:363-371).
std::string ListDevicesJSON() {
    std::vector<DeviceInfo> available;
    for (const auto& info : GetAllDeviceInfo())
        if (info.available) available.push_back(info);
    return DeviceInfosToJSON(available);
}

namespace {
std::string DeviceInfosToJSON(const std::vector<DeviceInfo>& infos) {
    std::ostringstream os;
    os << "[";
    bool first = true;
    for (const auto& d : infos) {
        os << (first ? "" : ",") << "{\"device_type\":" << static_cast<int>(d.device_type) << ",\"device_id\":" << d.device_id
           << ",\"device_type_name\":\"" << d.device_type_name << "\",\"target_kind\":\"" << d.target_kind
           << "\",\"available\":" << (d.available ? "true" : "false") << ",\"arch\":\"" << d.attrs.arch
           << "\",\"warp_size\":" << d.attrs.warp_size << ",\"multi_processor_count\":" << d.attrs.multi_processor_count << "}";
        first = false;
    }
    os << "]";
    return os.str();
}
}  // namespace

Target BuildTarget(DeviceTypeCode type, int device_id) {
    auto n = std::make_shared<TargetNode>();
    n->device = Device(type, device_id);
    DeviceAPI* api = GetDeviceAPI(type);
    n->kind = api->GetTargetKind(n->device);
    n->attrs = api->GetDeviceAttributes(n->device);
    return Target(n);
}

}  // namespace kxc
