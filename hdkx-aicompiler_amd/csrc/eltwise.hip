// eltwise.hip -- bandwidth-bound elementwise operators: nn_relu, broadcast add/sub/mul/div
// (optionally fused with a following ReLU), conv bias add, flatten copy, fp32 -> int8 quantise.
//
// All are pure streaming kernels: one 16-byte access per lane per tensor, consecutive lanes on
// consecutive addresses, enough workgroups to cover 256 CUs several times.  The arithmetic is a
// single correctly rounded fp32 operation per element, so results equal the CPU loop nests bit
// for bit (no multiply-add contraction can occur: no expression holds both a multiply and an add).
#include "common.h"

using namespace kxc_hip;

namespace {

constexpr int kBlock = 256;

// ReLU as the reference lowers Max(x, 0): an ordered compare and a select (NaN -> 0, -0 -> +0).
__device__ __forceinline__ float relu_sel(float v) { return (v > 0.0f) ? v : 0.0f; }

template <int OP>
__device__ __forceinline__ float binop(float a, float b) {
    if (OP == 0) return __fadd_rn(a, b);
    if (OP == 1) return __fsub_rn(a, b);
    if (OP == 2) return __fmul_rn(a, b);
    return __fdiv_rn(a, b);
}

__global__ void __launch_bounds__(kBlock) relu_kernel(const float* __restrict__ x, float* __restrict__ y,
                                                      int64_t n4, int64_t n) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlock;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; i < n4; i += stride) {
        float4 v = reinterpret_cast<const float4*>(x)[i];
        v.x = relu_sel(v.x); v.y = relu_sel(v.y); v.z = relu_sel(v.z); v.w = relu_sel(v.w);
        reinterpret_cast<float4*>(y)[i] = v;
    }
    // tail (n % 4 elements) by the first lanes of block 0
    const int64_t tail = n4 * 4 + static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (blockIdx.x == 0 && tail < n) y[tail] = relu_sel(x[tail]);
}

__global__ void __launch_bounds__(kBlock) relu_scalar_kernel(const float* __restrict__ x, float* __restrict__ y,
                                                             int64_t n) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlock;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; i < n; i += stride) y[i] = relu_sel(x[i]);
}

template <int OP, bool RELU>
__global__ void __launch_bounds__(kBlock) same_shape_kernel(const float* __restrict__ a, const float* __restrict__ b,
                                                            float* __restrict__ y, int64_t n4, int64_t n) {
    // two 16-byte vectors of each operand per thread and trip, all four loads issued before the first use.
    // (Non-temporal loads and stores were measured on the 77 MB add + ReLU: 16.2 -> 14.2 us with the operands in HBM,
    // 12.3 -> 11.4 us with them in the last-level cache -- but a kernel that reads the result next then fetches it
    // from HBM: the same hint on a pooling kernel's stores made the convolution behind it 9 us slower.  Not used.)
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlock;
    auto op4 = [](const float4& va, const float4& vb) {
        float4 r;
        r.x = binop<OP>(va.x, vb.x); r.y = binop<OP>(va.y, vb.y);
        r.z = binop<OP>(va.z, vb.z); r.w = binop<OP>(va.w, vb.w);
        if (RELU) { r.x = relu_sel(r.x); r.y = relu_sel(r.y); r.z = relu_sel(r.z); r.w = relu_sel(r.w); }
        return r;
    };
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; i < n4; i += 2 * stride) {
        const int64_t j = i + stride;
        const bool second = j < n4;
        const float4 va0 = reinterpret_cast<const float4*>(a)[i];
        const float4 vb0 = reinterpret_cast<const float4*>(b)[i];
        const float4 va1 = second ? reinterpret_cast<const float4*>(a)[j] : va0;
        const float4 vb1 = second ? reinterpret_cast<const float4*>(b)[j] : vb0;
        reinterpret_cast<float4*>(y)[i] = op4(va0, vb0);
        if (second) reinterpret_cast<float4*>(y)[j] = op4(va1, vb1);
    }
    const int64_t tail = n4 * 4 + static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (blockIdx.x == 0 && tail < n) {
        float r = binop<OP>(a[tail], b[tail]);
        y[tail] = RELU ? relu_sel(r) : r;
    }
}

struct BroadcastDims {
    int32_t ndim;
    int64_t out_shape[6];
    int64_t a_stride[6];   // 0 where the operand broadcasts
    int64_t b_stride[6];
};

template <int OP, bool RELU>
__global__ void __launch_bounds__(kBlock) broadcast_kernel(const float* __restrict__ a, const float* __restrict__ b,
                                                           float* __restrict__ y, BroadcastDims d, int64_t total) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlock;
    for (int64_t lin = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; lin < total; lin += stride) {
        int64_t rem = lin, ai = 0, bi = 0;
        for (int i = d.ndim - 1; i >= 0; --i) {
            const int64_t idx = rem % d.out_shape[i];
            rem /= d.out_shape[i];
            ai += idx * d.a_stride[i];
            bi += idx * d.b_stride[i];
        }
        float r = binop<OP>(a[ai], b[bi]);
        y[lin] = RELU ? relu_sel(r) : r;
    }
}

// y[n,o,:] = x[n,o,:] + bias[o]; one workgroup row per (n,o) plane chunk.
template <bool RELU>
__global__ void __launch_bounds__(kBlock) bias_add_kernel(const float* __restrict__ x, const float* __restrict__ bias,
                                                          float* __restrict__ y, int64_t o, int64_t hw, int64_t total) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlock;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; i < total; i += stride) {
        const int64_t ch = (i / hw) % o;
        float r = __fadd_rn(x[i], bias[ch]);
        y[i] = RELU ? relu_sel(r) : r;
    }
}

__global__ void __launch_bounds__(kBlock) copy_kernel(const float4* __restrict__ x, float4* __restrict__ y, int64_t n4,
                                                      const float* __restrict__ xs, float* __restrict__ ys, int64_t n) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlock;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; i < n4; i += stride) y[i] = x[i];
    const int64_t tail = n4 * 4 + static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (blockIdx.x == 0 && tail < n) ys[tail] = xs[tail];
}

// q = clamp(rint_half_even(v / scale), -127, 127); NaN -> 0.
__global__ void __launch_bounds__(kBlock) quantize_kernel(const float* __restrict__ x, int8_t* __restrict__ q,
                                                          int64_t n, float scale) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlock;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; i < n; i += stride) {
        const float v = __fdiv_rn(x[i], scale);
        float r = rintf(v);
        r = (v == v) ? r : 0.0f;
        r = fminf(fmaxf(r, -127.0f), 127.0f);
        q[i] = static_cast<int8_t>(static_cast<int32_t>(r));
    }
}

// max |x| over a tensor (NaN ignored): per-wave reduction, then one atomic per wave on the bit pattern
// (non-negative floats order like unsigned integers).  *out must be 0 on entry.
__global__ void __launch_bounds__(kBlock) absmax_kernel(const float* __restrict__ x, int64_t n, unsigned int* out) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlock;
    float m = 0.0f;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; i < n; i += stride) {
        const float v = fabsf(x[i]);
        m = (v > m) ? v : m;
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float o = __shfl_down(m, off, 64);
        m = (o > m) ? o : m;
    }
    if ((threadIdx.x & 63) == 0) atomicMax(out, __float_as_uint(m));
}

inline int GridFor(int64_t work_items) {
    // Enough workgroups for ~8 per CU at 256 CUs; grid-stride loops take the rest.
    int64_t g = CeilDiv(work_items, kBlock);
    if (g < 1) g = 1;
    if (g > 256 * 16) g = 256 * 16;
    return static_cast<int>(g);
}

inline bool Aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

template <int OP>
int32_t LaunchSameShape(const float* a, const float* b, float* y, int64_t n, bool relu, hipStream_t s) {
    const int64_t n4 = (Aligned16(a) && Aligned16(b) && Aligned16(y)) ? n / 4 : 0;
    const int grid = GridFor(n4 > 0 ? (n4 + 1) / 2 : n);      // the vector kernel takes two vectors per thread
    if (n4 == 0) {
        // unaligned: go through the generic kernel with a flat 1-d description
        BroadcastDims d{};
        d.ndim = 1; d.out_shape[0] = n; d.a_stride[0] = 1; d.b_stride[0] = 1;
        if (relu) broadcast_kernel<OP, true><<<NoteGrid(grid), NoteBlock(kBlock), NoteLds(0), s>>>(a, b, y, d, n);
        else broadcast_kernel<OP, false><<<NoteGrid(grid), NoteBlock(kBlock), NoteLds(0), s>>>(a, b, y, d, n);
    } else if (relu) {
        same_shape_kernel<OP, true><<<NoteGrid(grid), NoteBlock(kBlock), NoteLds(0), s>>>(a, b, y, n4, n);
    } else {
        same_shape_kernel<OP, false><<<NoteGrid(grid), NoteBlock(kBlock), NoteLds(0), s>>>(a, b, y, n4, n);
    }
    return CheckLaunch("broadcast_binary");
}

template <int OP>
int32_t LaunchBroadcast(const float* a, const float* b, float* y, const BroadcastDims& d, int64_t total, bool relu,
                        hipStream_t s) {
    const int grid = GridFor(total);
    if (relu) broadcast_kernel<OP, true><<<NoteGrid(grid), NoteBlock(kBlock), NoteLds(0), s>>>(a, b, y, d, total);
    else broadcast_kernel<OP, false><<<NoteGrid(grid), NoteBlock(kBlock), NoteLds(0), s>>>(a, b, y, d, total);
    return CheckLaunch("broadcast_binary");
}

}  // namespace

extern "C" {

int32_t kxc_hip_relu_f32(const float* x, float* y, int64_t n, void* stream) {
    KXC_HIP_REQUIRE(n >= 0, "kxc_hip_relu_f32: negative size");
    if (n == 0) return KXC_HIP_OK;
    KXC_HIP_REQUIRE(x && y, "kxc_hip_relu_f32: NULL pointer");
    hipStream_t s = ResolveStream(stream);
    if (Aligned16(x) && Aligned16(y) && n >= 4) {
        relu_kernel<<<NoteGrid(GridFor(n / 4)), NoteBlock(kBlock), NoteLds(0), s>>>(x, y, n / 4, n);
    } else {
        relu_scalar_kernel<<<NoteGrid(GridFor(n)), NoteBlock(kBlock), NoteLds(0), s>>>(x, y, n);
    }
    return CheckLaunch("relu");
}

int32_t kxc_hip_broadcast_binary_f32(int32_t op, const float* a, const int64_t* a_shape, int32_t a_ndim,
                                     const float* b, const int64_t* b_shape, int32_t b_ndim, float* y,
                                     int32_t relu, void* stream) {
    KXC_HIP_REQUIRE(op >= 0 && op <= 3, "kxc_hip_broadcast_binary_f32: bad op %d", op);
    KXC_HIP_REQUIRE(a_ndim >= 0 && a_ndim <= 6 && b_ndim >= 0 && b_ndim <= 6,
                    "kxc_hip_broadcast_binary_f32: rank above 6 is not supported");
    KXC_HIP_REQUIRE(a && b && y, "kxc_hip_broadcast_binary_f32: NULL pointer");
    const int ndim = a_ndim > b_ndim ? a_ndim : b_ndim;
    BroadcastDims d{};
    d.ndim = ndim > 0 ? ndim : 1;
    int64_t total = 1;
    bool same = (a_ndim == b_ndim);
    int64_t a_str = 1, b_str = 1;
    int64_t a_strides[6] = {0}, b_strides[6] = {0};
    for (int i = a_ndim - 1; i >= 0; --i) { a_strides[i] = a_str; a_str *= a_shape[i]; }
    for (int i = b_ndim - 1; i >= 0; --i) { b_strides[i] = b_str; b_str *= b_shape[i]; }
    if (ndim == 0) { d.out_shape[0] = 1; }
    for (int i = 0; i < ndim; ++i) {
        const int ai = i - (ndim - a_ndim), bi = i - (ndim - b_ndim);
        const int64_t da = ai >= 0 ? a_shape[ai] : 1;
        const int64_t db = bi >= 0 ? b_shape[bi] : 1;
        KXC_HIP_REQUIRE(da > 0 && db > 0, "kxc_hip_broadcast_binary_f32: non-positive dimension");
        KXC_HIP_REQUIRE(da == db || da == 1 || db == 1,
                        "kxc_hip_broadcast_binary_f32: shapes do not broadcast (%lld vs %lld at axis %d)",
                        static_cast<long long>(da), static_cast<long long>(db), i);
        d.out_shape[i] = da == 1 ? db : da;
        d.a_stride[i] = (ai >= 0 && da != 1) ? a_strides[ai] : 0;
        d.b_stride[i] = (bi >= 0 && db != 1) ? b_strides[bi] : 0;
        if (da != db) same = false;
        total *= d.out_shape[i];
    }
    hipStream_t s = ResolveStream(stream);
    if (same) {
        switch (op) {
            case 0: return LaunchSameShape<0>(a, b, y, total, relu != 0, s);
            case 1: return LaunchSameShape<1>(a, b, y, total, relu != 0, s);
            case 2: return LaunchSameShape<2>(a, b, y, total, relu != 0, s);
            default: return LaunchSameShape<3>(a, b, y, total, relu != 0, s);
        }
    }
    switch (op) {
        case 0: return LaunchBroadcast<0>(a, b, y, d, total, relu != 0, s);
        case 1: return LaunchBroadcast<1>(a, b, y, d, total, relu != 0, s);
        case 2: return LaunchBroadcast<2>(a, b, y, d, total, relu != 0, s);
        default: return LaunchBroadcast<3>(a, b, y, d, total, relu != 0, s);
    }
}

int32_t kxc_hip_bias_add_nchw_f32(const float* x, const float* bias, float* y, int64_t n, int64_t o, int64_t hw,
                                  int32_t relu, void* stream) {
    KXC_HIP_REQUIRE(n >= 0 && o >= 0 && hw >= 0, "kxc_hip_bias_add_nchw_f32: negative size");
    const int64_t total = n * o * hw;
    if (total == 0) return KXC_HIP_OK;
    KXC_HIP_REQUIRE(x && bias && y, "kxc_hip_bias_add_nchw_f32: NULL pointer");
    hipStream_t s = ResolveStream(stream);
    if (relu) bias_add_kernel<true><<<NoteGrid(GridFor(total)), NoteBlock(kBlock), NoteLds(0), s>>>(x, bias, y, o, hw, total);
    else bias_add_kernel<false><<<NoteGrid(GridFor(total)), NoteBlock(kBlock), NoteLds(0), s>>>(x, bias, y, o, hw, total);
    return CheckLaunch("bias_add");
}

int32_t kxc_hip_flatten_f32(const float* x, float* y, int64_t n, void* stream) {
    KXC_HIP_REQUIRE(n >= 0, "kxc_hip_flatten_f32: negative size");
    if (n == 0) return KXC_HIP_OK;
    KXC_HIP_REQUIRE(x && y, "kxc_hip_flatten_f32: NULL pointer");
    hipStream_t s = ResolveStream(stream);
    const int64_t n4 = (Aligned16(x) && Aligned16(y)) ? n / 4 : 0;
    if (n4 == 0) {
        KXC_HIP_CALL(hipMemcpyAsync(y, x, static_cast<size_t>(n) * sizeof(float), hipMemcpyDeviceToDevice, s),
                     "flatten copy");
        return KXC_HIP_OK;
    }
    copy_kernel<<<NoteGrid(GridFor(n4)), NoteBlock(kBlock), NoteLds(0), s>>>(reinterpret_cast<const float4*>(x), reinterpret_cast<float4*>(y), n4,
                                                x, y, n);
    return CheckLaunch("flatten");
}

int32_t kxc_hip_quantize_f32_i8(const float* x, int8_t* q, int64_t n, float scale, void* stream) {
    KXC_HIP_REQUIRE(n >= 0, "kxc_hip_quantize_f32_i8: negative size");
    if (n == 0) return KXC_HIP_OK;
    KXC_HIP_REQUIRE(x && q, "kxc_hip_quantize_f32_i8: NULL pointer");
    KXC_HIP_REQUIRE(scale > 0.0f, "kxc_hip_quantize_f32_i8: scale must be positive");
    quantize_kernel<<<NoteGrid(GridFor(n)), NoteBlock(kBlock), NoteLds(0), ResolveStream(stream)>>>(x, q, n, scale);
    return CheckLaunch("quantize");
}

int32_t kxc_hip_absmax_f32(const float* x, int64_t n, float* out, void* stream) {
    KXC_HIP_REQUIRE(n >= 0, "kxc_hip_absmax_f32: negative size");
    KXC_HIP_REQUIRE(out != nullptr, "kxc_hip_absmax_f32: NULL output");
    hipStream_t s = ResolveStream(stream);
    KXC_HIP_CALL(hipMemsetAsync(out, 0, sizeof(float), s), "hipMemsetAsync");
    if (n == 0) return KXC_HIP_OK;
    KXC_HIP_REQUIRE(x != nullptr, "kxc_hip_absmax_f32: NULL pointer");
    absmax_kernel<<<NoteGrid(GridFor(n)), NoteBlock(kBlock), NoteLds(0), s>>>(x, n, reinterpret_cast<unsigned int*>(out));
    return CheckLaunch("absmax");
}

}  // extern "C"
