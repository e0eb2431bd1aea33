// device_api.hip -- HIP device API behind the C ABI (section 1 of kxc_hip.h).
// GPU counterpart of the reference's CUDADeviceAPI (src/base/device/cuda_device_api.cc:75-328):
// same call set, same conventions (thread-local current stream, NULL stream = synchronous copy /
// device-wide sync, attribute query that never fails).
#include <cstring>

#include <atomic>

#include "common.h"

namespace kxc_hip {
std::string& LastError() {
    static thread_local std::string msg;
    return msg;
}
LaunchNote& LastLaunch() {
    static thread_local LaunchNote note;
    return note;
}
hipStream_t& CurrentStream() {
    static thread_local hipStream_t s = nullptr;
    return s;
}
}  // namespace kxc_hip

using namespace kxc_hip;

namespace {
// One HIP runtime call, recorded as a RUNTIME_API activity while recording is on.
template <typename F>
hipError_t Api(const char* name, F&& call) {
    ApiScope scope(name);
    const hipError_t e = call();
    scope.SetResult(e);
    return e;
}
}  // namespace

namespace {
// Byte fill, 16 bytes per thread (whole aligned chunks as one store).
__global__ void __launch_bounds__(256) fill_bytes_kernel(uint8_t* __restrict__ p, uint8_t v, size_t n) {
    const size_t chunk = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    const size_t lo = chunk * 16;
    if (lo >= n) return;
    const size_t hi = lo + 16 < n ? lo + 16 : n;
    if (hi - lo == 16 && (reinterpret_cast<uintptr_t>(p + lo) & 15u) == 0) {
        const uint32_t w = 0x01010101u * v;
        *reinterpret_cast<uint4*>(p + lo) = make_uint4(w, w, w, w);
        return;
    }
    for (size_t i = lo; i < hi; ++i) p[i] = v;
}
std::atomic<int64_t> g_device_allocations{0};
}  // namespace

namespace kxc_hip {
void NoteDeviceAllocation() { g_device_allocations.fetch_add(1, std::memory_order_relaxed); }
}  // namespace kxc_hip

extern "C" {

int64_t kxc_hip_debug_device_allocations(void) { return g_device_allocations.load(std::memory_order_relaxed); }



const char* kxc_hip_last_error(void) { return LastError().c_str(); }
int32_t kxc_hip_abi_version(void) { return 1; }
const char* kxc_hip_target_kind(void) { return "hip"; }

int32_t kxc_hip_device_count(int32_t* count) {
    KXC_HIP_REQUIRE(count != nullptr, "kxc_hip_device_count: count is NULL");
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        n = 0;
    }
    *count = n;
    return KXC_HIP_OK;
}

int32_t kxc_hip_device_attributes(int32_t device_id, kxc_hip_device_attrs* out) {
    KXC_HIP_REQUIRE(out != nullptr, "kxc_hip_device_attributes: out is NULL");
    std::memset(out, 0, sizeof(*out));
    out->warp_size = 64;
    std::snprintf(out->arch, sizeof(out->arch), "gfx950");
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n <= 0) {
        (void)hipGetLastError();
        std::snprintf(out->status, sizeof(out->status), "no HIP device: %s",
                      e != hipSuccess ? hipGetErrorString(e) : "device count is 0");
        return KXC_HIP_OK;
    }
    if (device_id < 0 || device_id >= n) {
        std::snprintf(out->status, sizeof(out->status), "device id %d out of range [0,%d)", device_id, n);
        return KXC_HIP_OK;
    }
    hipDeviceProp_t p;
    e = hipGetDeviceProperties(&p, device_id);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        std::snprintf(out->status, sizeof(out->status), "hipGetDeviceProperties failed: %s", hipGetErrorString(e));
        return KXC_HIP_OK;
    }
    out->exists = 1;
    out->warp_size = p.warpSize;
    out->max_threads_per_block = p.maxThreadsPerBlock;
    out->max_shared_memory_per_block = static_cast<int64_t>(p.sharedMemPerBlock);
    out->max_shared_memory_per_multiprocessor = static_cast<int64_t>(p.maxSharedMemoryPerMultiProcessor);
    out->multi_processor_count = p.multiProcessorCount;
    out->max_clock_rate_khz = p.clockRate;
    out->max_registers_per_block = p.regsPerBlock;
    out->l2_cache_size_bytes = p.l2CacheSize;
    out->total_global_memory = static_cast<int64_t>(p.totalGlobalMem);
    out->max_threads_per_multiprocessor = p.maxThreadsPerMultiProcessor;
    out->compute_version_major = p.major;
    out->compute_version_minor = p.minor;
    std::snprintf(out->device_name, sizeof(out->device_name), "%s", p.name);
    // gcnArchName is "gfx950:sramecc+:xnack-"; keep the processor name only.
    std::snprintf(out->arch, sizeof(out->arch), "%s", p.gcnArchName);
    if (char* colon = std::strchr(out->arch, ':')) *colon = '\0';
    int v = 0;
    if (hipRuntimeGetVersion(&v) == hipSuccess) out->api_version = v;
    if (hipDriverGetVersion(&v) == hipSuccess) out->driver_version = v;
    size_t free_b = 0, total_b = 0;
    int cur = 0;
    if (hipGetDevice(&cur) == hipSuccess && hipSetDevice(device_id) == hipSuccess) {
        if (hipMemGetInfo(&free_b, &total_b) == hipSuccess) out->available_global_memory = static_cast<int64_t>(free_b);
        (void)hipSetDevice(cur);
    }
    (void)hipGetLastError();
    std::snprintf(out->status, sizeof(out->status), "ok");
    return KXC_HIP_OK;
}

int32_t kxc_hip_set_device(int32_t device_id) {
    KXC_HIP_CALL(hipSetDevice(device_id), "HIP SetDevice");
    return KXC_HIP_OK;
}

int32_t kxc_hip_alloc(int32_t device_id, size_t nbytes, size_t alignment, void** out_ptr) {
    KXC_HIP_REQUIRE(out_ptr != nullptr, "kxc_hip_alloc: out_ptr is NULL");
    KXC_HIP_REQUIRE(alignment <= 256, "kxc_hip_alloc: alignment %zu > 256 is not supported", alignment);
    *out_ptr = nullptr;
    KXC_HIP_CALL(hipSetDevice(device_id), "HIP SetDevice");
    KXC_HIP_CALL(Api("hipMalloc", [&] { return hipMalloc(out_ptr, nbytes ? nbytes : 1); }), "HIP AllocDataSpace");
    NoteDeviceAllocation();
    return KXC_HIP_OK;
}

int32_t kxc_hip_free(int32_t device_id, void* ptr) {
    if (!ptr) return KXC_HIP_OK;
    KXC_HIP_CALL(hipSetDevice(device_id), "HIP SetDevice");
    KXC_HIP_CALL(Api("hipFree", [&] { return hipFree(ptr); }), "HIP FreeDataSpace");
    return KXC_HIP_OK;
}

int32_t kxc_hip_copy(const void* from, size_t from_offset, void* to, size_t to_offset, size_t nbytes,
                     int32_t kind, int32_t device_id, void* stream) {
    KXC_HIP_REQUIRE(kind >= 0 && kind <= 3, "kxc_hip_copy: bad kind %d", kind);
    if (nbytes == 0) return KXC_HIP_OK;
    KXC_HIP_REQUIRE(from && to, "kxc_hip_copy: NULL pointer");
    static const hipMemcpyKind kinds[4] = {hipMemcpyHostToDevice, hipMemcpyDeviceToHost,
                                           hipMemcpyDeviceToDevice, hipMemcpyHostToHost};
    KXC_HIP_CALL(hipSetDevice(device_id), "HIP SetDevice");
    const uint8_t* src = static_cast<const uint8_t*>(from) + from_offset;
    uint8_t* dst = static_cast<uint8_t*>(to) + to_offset;
    hipStream_t s = ResolveStream(stream);
    hipError_t e = hipSuccess;
    {
        ApiScope api(s ? "hipMemcpyAsync" : "hipMemcpy");
        DeviceScope dev(KXC_HIP_ACTIVITY_MEMCPY, s ? "hipMemcpyAsync" : "hipMemcpy", s, api.correlation());
        dev.bytes = static_cast<int64_t>(nbytes);
        dev.copy_kind = kind;
        e = s ? hipMemcpyAsync(dst, src, nbytes, kinds[kind], s) : hipMemcpy(dst, src, nbytes, kinds[kind]);
        api.SetResult(e);
    }
    KXC_HIP_CALL(e, "HIP CopyDataFromTo");
    return KXC_HIP_OK;
}

int32_t kxc_hip_memset(void* ptr, int32_t value, size_t nbytes, int32_t device_id, void* stream) {
    if (nbytes == 0) return KXC_HIP_OK;
    KXC_HIP_REQUIRE(ptr != nullptr, "kxc_hip_memset: NULL pointer");
    KXC_HIP_CALL(hipSetDevice(device_id), "HIP SetDevice");
    hipStream_t s = ResolveStream(stream);
    hipError_t e = hipSuccess;
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    if (s != nullptr && hipStreamIsCapturing(s, &capture) == hipSuccess && capture == hipStreamCaptureStatusActive) {
        // a stream that is being captured records a kernel, never a memset node (replays of memset nodes have
        // produced wrong contents on this platform)
        const size_t chunks = (nbytes + 15) / 16;
        KXC_HIP_REQUIRE(chunks <= static_cast<size_t>(kMaxGridX) * 256, "kxc_hip_memset: region too large for one fill launch");
        fill_bytes_kernel<<<NoteGrid(static_cast<int>((chunks + 255) / 256)), NoteBlock(256), NoteLds(0), s>>>(
            static_cast<uint8_t*>(ptr), static_cast<uint8_t>(value & 0xff), nbytes);
        return CheckLaunch("fill_bytes_kernel");
    }
    {
        ApiScope api(s ? "hipMemsetAsync" : "hipMemset");
        DeviceScope dev(KXC_HIP_ACTIVITY_MEMSET, s ? "hipMemsetAsync" : "hipMemset", s, api.correlation());
        dev.bytes = static_cast<int64_t>(nbytes);
        dev.value = value & 0xff;
        e = s ? hipMemsetAsync(ptr, value, nbytes, s) : hipMemset(ptr, value, nbytes);
        api.SetResult(e);
    }
    KXC_HIP_CALL(e, "HIP Memset");
    return KXC_HIP_OK;
}

int32_t kxc_hip_stream_create(int32_t device_id, void** out_stream) {
    KXC_HIP_REQUIRE(out_stream != nullptr, "kxc_hip_stream_create: out_stream is NULL");
    KXC_HIP_CALL(hipSetDevice(device_id), "HIP SetDevice");
    hipStream_t s = nullptr;
    KXC_HIP_CALL(Api("hipStreamCreate", [&] { return hipStreamCreate(&s); }), "HIP StreamCreate");   // default priority only
    *out_stream = s;
    return KXC_HIP_OK;
}

int32_t kxc_hip_stream_destroy(int32_t device_id, void* stream) {
    if (!stream) return KXC_HIP_OK;
    KXC_HIP_CALL(hipSetDevice(device_id), "HIP SetDevice");
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    KXC_HIP_CALL(Api("hipStreamDestroy", [&] { return hipStreamDestroy(s); }), "HIP StreamDestroy");
    if (CurrentStream() == s) CurrentStream() = nullptr;
    return KXC_HIP_OK;
}

int32_t kxc_hip_set_stream(int32_t device_id, void* stream) {
    KXC_HIP_CALL(hipSetDevice(device_id), "HIP SetDevice");
    CurrentStream() = reinterpret_cast<hipStream_t>(stream);
    return KXC_HIP_OK;
}

int32_t kxc_hip_get_stream(int32_t device_id, void** out_stream) {
    KXC_HIP_REQUIRE(out_stream != nullptr, "kxc_hip_get_stream: out_stream is NULL");
    (void)device_id;
    *out_stream = CurrentStream();
    return KXC_HIP_OK;
}

int32_t kxc_hip_stream_sync(int32_t device_id, void* stream) {
    KXC_HIP_CALL(hipSetDevice(device_id), "HIP SetDevice");
    hipStream_t s = ResolveStream(stream);
    if (s == nullptr) {
        KXC_HIP_CALL(Api("hipDeviceSynchronize", [&] { return hipDeviceSynchronize(); }), "HIP StreamSync");
    } else {
        KXC_HIP_CALL(Api("hipStreamSynchronize", [&] { return hipStreamSynchronize(s); }), "HIP StreamSync");
    }
    return KXC_HIP_OK;
}

int32_t kxc_hip_stream_wait(int32_t device_id, void* src_stream, void* dst_stream) {
    KXC_HIP_CALL(hipSetDevice(device_id), "HIP SetDevice");
    hipEvent_t ev = nullptr;
    KXC_HIP_CALL(hipEventCreateWithFlags(&ev, hipEventDisableTiming), "HIP EventCreate");
    hipError_t e = hipEventRecord(ev, reinterpret_cast<hipStream_t>(src_stream));
    if (e == hipSuccess) e = hipStreamWaitEvent(reinterpret_cast<hipStream_t>(dst_stream), ev, 0);
    (void)hipEventDestroy(ev);
    KXC_HIP_CALL(e, "HIP SyncStreamFromTo");
    return KXC_HIP_OK;
}

}  // extern "C"
