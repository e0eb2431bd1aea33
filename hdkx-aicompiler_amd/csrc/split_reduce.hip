// split_reduce.hip -- second half of a convolution whose reduction was split over workgroups, shared by the
// implicit-GEMM and the Winograd kernel: the partial outputs of the parts are added in split order and the
// layer's epilogue (bias, residual, ReLU) is applied; plus the scratch buffers the parts write to.
#include <cstdlib>
#include <memory>
#include <mutex>
#include <vector>

#include "common.h"

namespace kxc_hip {

namespace {

__device__ __forceinline__ float relu_sel(float v) { return (v > 0.0f) ? v : 0.0f; }

__global__ void __launch_bounds__(256) conv_split_reduce_kernel(const SplitReduceArgs a) {
    // XCD x (blockIdx % 8) takes the x-th eighth of the elements, like the kernels that wrote the parts
    const int32_t per_xcd = static_cast<int32_t>(gridDim.x >> 3);
    const int32_t block = static_cast<int32_t>(blockIdx.x & 7) * per_xcd + static_cast<int32_t>(blockIdx.x >> 3);
    int32_t e = block * 256 + static_cast<int32_t>(threadIdx.x);
    // elements total .. 2 * total - 1 are the second output of a two-output launch
    const bool second = a.y2 != nullptr && e >= a.total;
    if (second) e -= a.total;
    if (e >= a.total) return;
    const float* const p = (second ? a.partial2 : a.partial) + e;
    const uint32_t flags = second ? a.flags2 : a.flags;
    // every load of a batch of eight splits, the bias and the residual are in flight before the first addition
    float bias = 0.0f, res = 0.0f;
    if (flags & KXC_HIP_CONV_BIAS) { const int32_t plane = fast_div(e, a.div_ohw); bias = (second ? a.bias2 : a.bias)[plane % a.O]; }
    if (flags & KXC_HIP_CONV_RESIDUAL) res = a.res[e];
    float v = p[0];
    for (int32_t s0 = 1; s0 < a.gsplit; s0 += 8) {
        float t[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) t[i] = s0 + i < a.gsplit ? p[static_cast<int64_t>(s0 + i) * a.total] : 0.0f;
#pragma unroll
        for (int i = 0; i < 8; ++i) v = s0 + i < a.gsplit ? __fadd_rn(v, t[i]) : v;
    }
    if (flags & KXC_HIP_CONV_BIAS) v = __fadd_rn(v, bias);
    if (flags & KXC_HIP_CONV_RESIDUAL) v = __fadd_rn(v, res);
    if (flags & KXC_HIP_CONV_RELU) v = relu_sel(v);
    (second ? a.y2 : a.y)[e] = v;
}

__global__ void __launch_bounds__(256) split_counters_clear_kernel(uint32_t* counters, int32_t n) {
    const int32_t i = static_cast<int32_t>(blockIdx.x) * 256 + static_cast<int32_t>(threadIdx.x);
    if (i < n) counters[i] = 0u;
}

}  // namespace

// Off by default.  Measured on MI355X, ResNet-18 at batch 1 (13 split Winograd layers, graph replay): the last
// part's tail is three dependent round trips beyond the XCD's own L2 (stores acknowledged, counter, parts read back)
// and costs more than the adding kernel with its launch: 0.226 ms per image with the adding kernel everywhere,
// 0.240 with the four 4-part layers finished by the last part, 0.263 up to 8 parts, 0.309 up to 16, 0.373 up to 32.
// KXC_HIP_SPLIT_FUSE_MAX=<parts> turns it on for reductions split into at most that many parts.
int32_t SplitFuseMaxParts() {
    const char* e = std::getenv("KXC_HIP_SPLIT_FUSE_MAX");
    return e ? static_cast<int32_t>(std::atoi(e)) : 0;
}

// Set per thread (kxc_hip_set_select_lanes: a launch plan sets it while it resolves its launches, a graph builder
// while it asks which variant a shape would take); KXC_HIP_SELECT_LANES overrides it for measurements.
thread_local int32_t g_select_lanes = 1;
int32_t SelectLanes() {
    if (const char* e = std::getenv("KXC_HIP_SELECT_LANES")) {
        const int v = std::atoi(e);
        if (v >= 1 && v <= 16) return v;
    }
    return g_select_lanes;
}

// A buffer that has been handed out stays allocated until the process ends, also after a larger one replaced it:
// a captured graph may still hold its address.  Buffers double, so the retired ones add up to less than the
// current one.
int32_t AcquireSplitScratch(hipStream_t stream, size_t bytes, SplitScratchLease* lease) {
    struct Entry { int device; hipStream_t stream; float* ptr; uint32_t* counters; size_t bytes; std::mutex in_use; };
    static std::mutex mu;
    static std::vector<std::unique_ptr<Entry>> entries;      // entries are never removed: their addresses are stable
    int dev = 0;
    KXC_HIP_CALL(hipGetDevice(&dev), "hipGetDevice");
    Entry* e = nullptr;
    {
        std::lock_guard<std::mutex> lock(mu);
        for (auto& it : entries)
            if (it->device == dev && it->stream == stream) e = it.get();
        if (!e) {
            entries.emplace_back(new Entry{dev, stream, nullptr, nullptr, 0, {}});
            e = entries.back().get();
        }
    }
    std::unique_lock<std::mutex> in_use(e->in_use);
    if (e->bytes < bytes) {
        size_t want = e->bytes ? 2 * e->bytes : (static_cast<size_t>(1) << 20);
        while (want < bytes) want *= 2;
        char* fresh = nullptr;
        KXC_HIP_CALL(hipMalloc(reinterpret_cast<void**>(&fresh), kSplitCounterBytes + want), "hipMalloc(split scratch)");
        NoteDeviceAllocation();
        // the arrival counters in front start at zero: a fill kernel on the caller's stream, ahead of the first
        // launch that counts (under stream capture it becomes a node of the graph, which is harmless)
        split_counters_clear_kernel<<<kSplitCounters / 256, 256, 0, stream>>>(reinterpret_cast<uint32_t*>(fresh), kSplitCounters);
        if (int32_t rc = CheckLaunch("split_counters_clear")) { (void)hipFree(fresh); return rc; }
        e->counters = reinterpret_cast<uint32_t*>(fresh);
        e->ptr = reinterpret_cast<float*>(fresh + kSplitCounterBytes);          // the previous buffer is left allocated on purpose
        e->bytes = want;
    }
    lease->ptr = e->ptr;
    lease->counters = e->counters;
    lease->lock = std::move(in_use);
    return KXC_HIP_OK;
}

int32_t LaunchSplitReduce(hipStream_t stream, const SplitReduceArgs& a) {
    KXC_HIP_REQUIRE(a.gsplit >= 1 && a.total > 0 && a.O > 0 && a.partial && a.y, "split reduction: bad arguments");
    KXC_HIP_REQUIRE(!a.y2 || (a.partial2 && a.total < (1 << 30)), "split reduction: bad second output");
    const int64_t elems = static_cast<int64_t>(a.total) * (a.y2 ? 2 : 1);
    conv_split_reduce_kernel<<<NoteGrid(static_cast<int>(CeilDiv(CeilDiv(elems, 256), 8) * 8)), NoteBlock(256), NoteLds(0), stream>>>(a);
    return CheckLaunch("conv_split_reduce");
}

}  // namespace kxc_hip

extern "C" int32_t kxc_hip_set_select_lanes(int32_t lanes) {
    const int32_t prev = kxc_hip::g_select_lanes;
    kxc_hip::g_select_lanes = lanes < 1 ? 1 : (lanes > 16 ? 16 : lanes);
    return prev;
}
