// device_api.h -- Device, DeviceAPI (CPU and HIP), Target.
// Interface of the reference's include/base/device.h:20-62, include/base/device_api.h:42-151 and
// include/base/target.h:34-35.  kGPU is served by HIPDeviceAPI, a thin C++ face of the C-ABI
// library's device calls (the reference wires kGPU to its CUDA implementation,
// src/base/device_api.cc:164-178): target kind "hip", arch "gfx950", warp_size 64.
#pragma once

#include "kxc/base.h"

namespace kxc {

enum DeviceTypeCode { kCPU = 0, kGPU = 1, kOpenCL = 2, kMetal = 3, kUnknown = -1 };

class Device {
public:
    Device() = default;
    Device(DeviceTypeCode type, int id) : type_(type), id_(id) {}
    DeviceTypeCode device_type() const { return type_; }
    int device_id() const { return id_; }

private:
    DeviceTypeCode type_ = kCPU;
    int id_ = 0;
};

using StreamHandle = void*;

// Single-attribute query keys (include/base/device_api.h:19-39).
enum class DeviceAttrKind : int {
    kExist = 0, kMaxThreadsPerBlock = 1, kWarpSize = 2, kMaxSharedMemoryPerBlock = 3, kComputeVersion = 4, kDeviceName = 5,
    kMaxClockRate = 6, kMultiProcessorCount = 7, kMaxRegistersPerBlock = 8, kApiVersion = 9, kDriverVersion = 10,
    kL2CacheSizeBytes = 11, kTotalGlobalMemory = 12, kAvailableGlobalMemory = 13, kMaxSharedMemoryPerMultiprocessor = 14,
    kMaxRegistersPerMultiprocessor = 15, kMaxThreadsPerMultiprocessor = 16, kComputeVersionMajor = 17, kComputeVersionMinor = 18,
};
// What a packed function returns (include/base/packedfunc.h:110-230): nothing, an integer, a double, text or an object
// handle.  GetAttr gives an integer, or text for kComputeVersion / kDeviceName.
struct RetValue {
    int64_t v_int64{0};
    double v_float{0.0};
    std::string v_str;
    ObjectRef v_object;
    bool is_str{false}, is_float{false}, is_object{false}, is_set{false};
    RetValue& operator=(int64_t v) { Clear(); v_int64 = v; return *this; }
    RetValue& operator=(int v) { return *this = static_cast<int64_t>(v); }
    RetValue& operator=(bool v) { return *this = static_cast<int64_t>(v); }
    RetValue& operator=(double v) { Clear(); v_float = v; is_float = true; return *this; }
    RetValue& operator=(const std::string& s) { Clear(); v_str = s; is_str = true; return *this; }
    RetValue& operator=(const char* s) { return *this = std::string(s ? s : ""); }
    RetValue& operator=(const ObjectRef& o) { Clear(); v_object = o; is_object = true; return *this; }
    // conversions throw the reference's "Type mismatch: expected ..." when the held kind does not fit
    operator int64_t() const {
        if (is_float) return static_cast<int64_t>(v_float);
        if (is_str || is_object) throw std::runtime_error("Type mismatch: expected int");
        return v_int64;
    }
    operator double() const {
        if (is_float) return v_float;
        if (is_str || is_object) throw std::runtime_error("Type mismatch: expected double");
        return static_cast<double>(v_int64);
    }
    operator std::string() const {
        if (!is_str && is_set) throw std::runtime_error("Type mismatch: expected string");
        return v_str;
    }
    operator ObjectRef() const {
        if (!is_object && is_set) throw std::runtime_error("Type mismatch: expected ObjectRef");
        return v_object;
    }

private:
    void Clear() { v_int64 = 0; v_float = 0.0; v_str.clear(); v_object = ObjectRef(); is_str = is_float = is_object = false; is_set = true; }
};

struct DeviceAttributes {
    int exists{0};
    int64_t max_threads_per_block{1};
    int64_t warp_size{1};
    int64_t max_shared_memory_per_block{0};
    std::string compute_version{"0.0"};
    std::string device_name;
    int64_t max_clock_rate_khz{0};
    int64_t max_registers_per_block{0};
    int64_t api_version{0};
    int64_t driver_version{0};
    int64_t l2_cache_size_bytes{0};
    int64_t total_global_memory{0};
    int64_t available_global_memory{0};
    int64_t max_shared_memory_per_multiprocessor{0};
    int64_t max_threads_per_multiprocessor{0};
    int64_t compute_version_major{0};
    int64_t compute_version_minor{0};
    int64_t multi_processor_count{1};
    std::string arch;
    std::string status;
};

struct DeviceInfo {
    DeviceTypeCode device_type{kUnknown};
    int device_id{-1};
    std::string device_type_name;
    std::string target_kind;
    bool available{false};
    std::string status;
    DeviceAttributes attrs;
};

class DeviceAPI {
public:
    virtual ~DeviceAPI() = default;
    virtual void SetDevice(const Device& device) = 0;
    virtual void* AllocDataSpace(const Device& device, size_t nbytes, size_t alignment) = 0;
    virtual void FreeDataSpace(const Device& device, void* ptr) = 0;
    virtual void CopyDataFromTo(const Device& from_dev, const void* from_ptr, const Device& to_dev, void* to_ptr,
                                size_t nbytes) = 0;
    virtual void CopyDataFromTo(const void* from_ptr, size_t from_offset, void* to_ptr, size_t to_offset, size_t nbytes,
                                const Device& from_dev, const Device& to_dev, StreamHandle stream);
    virtual DeviceAttributes GetDeviceAttributes(const Device& device) = 0;
    virtual std::string GetTargetKind(const Device& device) const = 0;
    // One attribute of GetDeviceAttributes (src/base/device_api.cc:198-262); never throws for an absent device.
    virtual void GetAttr(const Device& device, DeviceAttrKind kind, RetValue* rv);
    virtual StreamHandle CreateStream(const Device& device);
    virtual void FreeStream(const Device& device, StreamHandle stream);
    virtual void SetStream(const Device& device, StreamHandle stream);
    virtual StreamHandle GetCurrentStream(const Device& device);
    virtual void StreamSync(const Device& device, StreamHandle stream);
    virtual void SyncStreamFromTo(const Device& device, StreamHandle src, StreamHandle dst);
    virtual void* AllocWorkspace(const Device& device, size_t nbytes, size_t alignment);
    virtual void FreeWorkspace(const Device& device, void* ptr);
    // Whether host code may do address arithmetic on this back end's device pointers (true for HIP and the CPU).
    virtual bool SupportsDevicePointerArithmeticsOnHost(const Device& device) const { return true; }
    // Whether SetDevice must be called before using a device of this type (src/base/device_api.cc:184-186).
    static bool NeedSetDevice(DeviceTypeCode type) { return type != kCPU; }
};

// Registry of the back ends by device type (include/base/device_api.h:126-135, src/base/device_api.cc:159-182): kCPU ->
// the host API, kGPU -> the HIP API; anything else throws "Device API not supported".
class DeviceAPIManager {
public:
    static DeviceAPIManager* Global();
    DeviceAPI* GetAPI(DeviceTypeCode type);

private:
    DeviceAPIManager() = default;
};
void GetDeviceAttr(const Device& device, DeviceAttrKind kind, RetValue* rv);
int64_t GetDeviceAttr(const Device& device, DeviceAttrKind kind);

DeviceAPI* GetCPUDeviceAPI();
DeviceAPI* GetHIPDeviceAPI();
DeviceAPI* GetDeviceAPI(DeviceTypeCode type);
std::vector<DeviceInfo> GetAllDeviceInfo();
std::string GetAllDeviceInfoJSON();
std::string ListDevicesJSON();      // the available ones only

struct TargetNode : Object {
    std::string kind;            // "llvm" for the CPU (the reference's name), "hip" for the GPU
    Device device;
    DeviceAttributes attrs;
};
class Target : public Ref<TargetNode> {
public:
    Target() = default;
    explicit Target(std::shared_ptr<TargetNode> n) : Ref<TargetNode>(std::move(n)) {}
};
// src/base/target.cc:34-51: kind and attributes come from the device API.
Target BuildTarget(DeviceTypeCode type, int device_id = 0);

}  // namespace kxc
