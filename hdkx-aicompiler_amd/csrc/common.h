// common.h -- shared host-side helpers of libkxc_hip.so (error reporting, stream resolution).
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <string>

#include "kxc_hip.h"

namespace kxc_hip {

// Per-thread message of the last failure (returned by kxc_hip_last_error).
std::string& LastError();
// Per-thread current stream (DeviceAPI::SetStream semantics: thread local).
hipStream_t& CurrentStream();
// Counts every device allocation the library makes (kxc_hip_debug_device_allocations): call next to each hipMalloc.
void NoteDeviceAllocation();

inline int32_t Fail(int32_t code, const char* fmt, ...) {
    char buf[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    LastError() = buf;
    return code;
}

inline hipStream_t ResolveStream(void* stream) {
    return stream ? reinterpret_cast<hipStream_t>(stream) : CurrentStream();
}

// Launch-error check: hipGetLastError after a triple-chevron launch.
inline int32_t CheckLaunch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return Fail(KXC_HIP_ERR_RUNTIME, "%s launch failed: %s", what, hipGetErrorString(e));
    return KXC_HIP_OK;
}

// Geometry of the calling thread's most recent kernel launch, for the profiled plan run: the launch sites
// pass their grid, block and dynamic-LDS arguments through these.
struct LaunchNote {
    uint32_t grid[3] = {0, 0, 0};
    uint32_t block[3] = {0, 0, 0};
    uint32_t dynamic_lds = 0;
};
LaunchNote& LastLaunch();
inline dim3 NoteGrid(dim3 g) { LaunchNote& n = LastLaunch(); n.grid[0] = g.x; n.grid[1] = g.y; n.grid[2] = g.z; return g; }
inline dim3 NoteBlock(dim3 b) { LaunchNote& n = LastLaunch(); n.block[0] = b.x; n.block[1] = b.y; n.block[2] = b.z; return b; }
inline size_t NoteLds(size_t bytes) { LastLaunch().dynamic_lds = static_cast<uint32_t>(bytes); return bytes; }

// floor(x / d) for 0 <= x < 2^31 as a multiply and a shift: shift = 31 + ceil(log2 d), mul = floor(2^shift / d) + 1.
// The kernels' tile set-up divides by launch-invariant values about twenty times; an integer division without
// hardware support costs ~35 instructions, this costs three.
struct FastDiv {
    uint32_t mul, shift;
};
inline FastDiv MakeFastDiv(int32_t d) {
    FastDiv f{1u << 31, 31};
    if (d <= 0) return f;
    uint32_t s = 0;
    while ((1LL << s) < d) ++s;
    f.shift = 31 + s;
    f.mul = static_cast<uint32_t>((1ULL << f.shift) / static_cast<uint64_t>(d) + 1);
    return f;
}
__device__ __forceinline__ int fast_div(int x, FastDiv f) {
    return static_cast<int>((static_cast<uint64_t>(static_cast<uint32_t>(x)) * f.mul) >> f.shift);
}

// Reductions split over workgroups (both convolution kernels): every part writes raw partial outputs to
// partial[split][total]; SplitReduce adds them in split order (deterministic) and applies the layer's epilogue,
// y = relu(((p0 + p1) + ...) + bias[channel] + residual).
struct SplitReduceArgs {
    const float* partial;
    const float* bias;
    const float* res;
    float* y;
    int32_t gsplit, total, O;
    uint32_t flags;            // KXC_HIP_CONV_BIAS | _RESIDUAL | _RELU
    FastDiv div_ohw;
    // second output of a two-output launch (same shape; y2 == nullptr: none): its parts, bias and flags
    const float* partial2 = nullptr;
    const float* bias2 = nullptr;
    float* y2 = nullptr;
    uint32_t flags2 = 0;
};
// Scratch for the partial outputs: one grow-only buffer per (device, stream), so that launches on different
// streams never share one.  In steady state no call allocates.  The lease keeps other host threads that enqueue
// on the same stream out until the adding kernel has been enqueued behind the parts (release it after that).
struct SplitScratchLease {
    float* ptr = nullptr;
    uint32_t* counters = nullptr;      // kSplitCounters arrival counters, all zero between launches
    std::unique_lock<std::mutex> lock;
};
int32_t AcquireSplitScratch(hipStream_t stream, size_t bytes, SplitScratchLease* lease);
int32_t LaunchSplitReduce(hipStream_t stream, const SplitReduceArgs& a);

// A split reduction without the adding kernel: every part stores its raw partial outputs as before, then counts
// itself in at its tile's arrival counter; the part that arrives last adds all parts in split order (the same
// order, hence the same bits, as the adding kernel) and applies the epilogue.  The counters sit in front of the
// partial outputs, start at zero and are set back to zero by the last arrival, so a launch (or the replay of a
// captured one) leaves them as it found them.  Launches that share a scratch buffer are ordered by their stream.
constexpr int32_t kSplitCounters = 16384;
constexpr size_t kSplitCounterBytes = static_cast<size_t>(kSplitCounters) * sizeof(uint32_t);
// Largest number of parts the last arrival finishes itself (0: the adding kernel always does; see split_reduce.hip).
int32_t SplitFuseMaxParts();
// Number of equal launches expected to run beside this one on other streams (1: the launch has the GPU to itself).
// Variant selection sizes its fill rules for that many times the launch's workgroups.
int32_t SelectLanes();

#if defined(__HIPCC__)
// Cache policy of the parts' stores and of the last part's loads of partial outputs: device scope (sc1), i.e.
// written through to and read from the level all XCDs share.  With it no cache-wide write-back or invalidate is
// needed around the counter (a release fence at device scope writes back the whole L2 of the XCD: measured at about
// 20 us per launch of 200 workgroups).
constexpr int kDeviceScopeAux = 0x10;
// True for the workgroup that arrives last of `parts` at `counter`.  Every thread of the workgroup calls it after
// its device-scope stores of partial outputs; `flag` is a word of LDS nobody else uses until the call returns.
// The counter is bumped by a vector memory atomic at device scope once every wave's stores have been acknowledged.
__device__ __forceinline__ bool split_arrive_last(uint32_t* counter, int32_t parts, uint32_t* flag) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0) {
        const uint32_t prev = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const bool last = prev + 1u == static_cast<uint32_t>(parts);
        if (last) __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        *flag = last ? 1u : 0u;
    }
    __syncthreads();
    return *flag != 0u;
}
#endif

// A convolution launch resolved ahead of time (a launch plan's node): kernel, tile shape, grid, the split of the
// reduction and every environment switch are decided once, from the descriptor; a launch combines them with the
// operand pointers and the stream.  conv2d_f32.hip (implicit GEMM, one or two outputs) and conv2d_wino_f32.hip.
struct PreparedConv;
int32_t PrepareConv2d(const kxc_hip_conv2d_desc* desc, bool second_output, PreparedConv** out);
int32_t LaunchPreparedConv2d(const PreparedConv* p, const float* x, const float* w, const float* bias, const float* residual,
                             float* y, const float* w2, const float* bias2, float* y2, hipStream_t stream);
const char* PreparedConvName(const PreparedConv* p);
void FreePreparedConv(PreparedConv* p);
struct PreparedWinograd;
int32_t PrepareWinograd(const kxc_hip_conv2d_desc* desc, PreparedWinograd** out);
int32_t LaunchPreparedWinograd(const PreparedWinograd* p, const float* x, const float* u, const float* bias,
                               const float* residual, float* y, hipStream_t stream);
void FreePreparedWinograd(PreparedWinograd* p);

// The filter transforms of several Winograd layers in one launch (conv2d_wino_f32.hip).
struct WinoWeightJob {
    const kxc_hip_conv2d_desc* desc;
    const float* w;      // OIHW weights
    float* u;            // kxc_hip_conv2d_winograd_weight_bytes(desc) bytes
};
int32_t LaunchWinogradWeightTransforms(const WinoWeightJob* jobs, int32_t count, hipStream_t stream);

// The int8 weight tensors of several convolutions packed by one launch (qconv_c16_i8.hip); kind = KXC_HIP_QPACK_*.
struct QPackJob {
    int32_t kind;
    const kxc_hip_qconv2d_desc* desc;
    const int8_t* w;     // OIHW
    int8_t* wp;          // QPackedBytes(job) bytes
};
int32_t QPackedBytes(const QPackJob& job, size_t* out_bytes);
int32_t LaunchQWeightPacks(const QPackJob* jobs, int32_t count, hipStream_t stream);

// Activity recording (activity.hip).  ApiScope times one HIP runtime call on the host; DeviceScope brackets the
// copy / fill / kernel that call enqueues with two HIP events on its stream.  Both do nothing while recording is off.
bool ActivityOn();
struct ActivitySuppress {      // the calling thread records nothing while one of these lives (a profiled plan run
    ActivitySuppress();        // times its launches itself)
    ~ActivitySuppress();
};
class ApiScope {
public:
    explicit ApiScope(const char* name);
    ~ApiScope();
    void SetResult(hipError_t e) { result_ = static_cast<int32_t>(e); }
    uint64_t correlation() const { return correlation_; }
private:
    bool on_;
    const char* name_;
    uint64_t correlation_ = 0;
    int64_t start_ns_ = 0;
    int32_t result_ = 0;
};
class DeviceScope {
public:
    DeviceScope(int32_t kind, const char* name, hipStream_t stream, uint64_t correlation);
    ~DeviceScope();
    int64_t bytes = 0;
    int32_t value = 0, copy_kind = 0;
    uint32_t grid[3] = {0, 0, 0}, block[3] = {0, 0, 0}, dynamic_shared_memory = 0;
private:
    bool on_;
    int32_t kind_;
    const char* name_;
    hipStream_t stream_;
    uint64_t correlation_;
    int64_t host_start_ns_ = 0;
    hipEvent_t start_ = nullptr, stop_ = nullptr;
};

constexpr int64_t kMaxGridX = 2147483647LL;

inline int64_t CeilDiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

}  // namespace kxc_hip

#define KXC_HIP_CALL(expr, what)                                                              \
    do {                                                                                      \
        hipError_t _e = (expr);                                                               \
        if (_e != hipSuccess)                                                                 \
            return ::kxc_hip::Fail(KXC_HIP_ERR_RUNTIME, "%s failed: %s", what, hipGetErrorString(_e)); \
    } while (0)

#define KXC_HIP_REQUIRE(cond, ...)                                              \
    do {                                                                        \
        if (!(cond)) return ::kxc_hip::Fail(KXC_HIP_ERR_INVALID, __VA_ARGS__);  \
    } while (0)
