// pool.hip -- nn_max_pool2d / nn_avg_pool2d / nn_global_avg_pool2d (fp32) and the int8 pools.
//
// All are HBM-bound.  Max pooling reproduces the reference's select chain exactly
// (start at -inf, taps in rh-major order, update old > src ? old : src, out-of-bounds taps
// contribute -1e30f), so results are bit-identical to the CPU loop nest, NaN and -0 included.
// Global average pooling sums each plane sequentially in row-major order from 0.0f and then
// performs a true IEEE division by (float)(H*W), which is the CPU loop nest's exact order too.
#include "common.h"

using namespace kxc_hip;

namespace {

constexpr int kBlock = 256;
constexpr float kPadValue = -1e30f;   // make_const(float32, -1e30), include/te/topi/nn.h:224

__device__ __forceinline__ float max_sel(float old, float src) { return (old > src) ? old : src; }

struct PoolDims {
    int32_t n, c, h, w, oh, ow;
    int32_t kh, kw, sh, sw, pt, pl;
};

// ---------------------------------------------------------------- generic: one thread per output
template <bool AVG>
__global__ void __launch_bounds__(kBlock) pool_generic_kernel(const float* __restrict__ x, float* __restrict__ y,
                                                              PoolDims d, int64_t total) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlock;
    const float denom = static_cast<float>(d.kh * d.kw);
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; i < total; i += stride) {
        const int32_t ow = static_cast<int32_t>(i % d.ow);
        const int64_t t = i / d.ow;
        const int32_t oh = static_cast<int32_t>(t % d.oh);
        const int64_t plane = t / d.oh;
        const float* xp = x + plane * d.h * d.w;
        float acc = AVG ? 0.0f : -INFINITY;
        for (int rh = 0; rh < d.kh; ++rh) {
            const int ih = oh * d.sh + rh - d.pt;
            for (int rw = 0; rw < d.kw; ++rw) {
                const int iw = ow * d.sw + rw - d.pl;
                const bool inb = ih >= 0 && ih < d.h && iw >= 0 && iw < d.w;
                if (AVG) {
                    acc = __fadd_rn(acc, inb ? xp[ih * d.w + iw] : 0.0f);
                } else {
                    acc = max_sel(acc, inb ? xp[ih * d.w + iw] : kPadValue);
                }
            }
        }
        y[i] = AVG ? __fdiv_rn(acc, denom) : acc;
    }
}

// ---------------------------------------------------------------- max 3x3 / stride 2 / pad 1
// Requirements (checked on the host): W % 8 == 0, OW == W/2, OH == H/2 (H even), 16-byte aligned
// planes.  One thread produces a 4-wide strip of ROWS consecutive output rows.  Per input row it
// issues two aligned 16-byte loads (columns 2*ow0 .. 2*ow0+7); the ninth value, column 2*ow0-1,
// is the left neighbour lane's last element, taken with a lane shuffle (a scalar reload only for
// the first lane of a wave).  Consecutive lanes read consecutive 32-byte pieces of a row, every
// input element is requested once per strip (plus the one shared row between vertical strips).
template <int ROWS>
__global__ void __launch_bounds__(kBlock) maxpool3x3s2_kernel(const float* __restrict__ x, float* __restrict__ y,
                                                              int32_t h, int32_t w, int32_t oh_total, int32_t ow_total,
                                                              int32_t col_groups, int32_t row_groups, int64_t total) {
    const int64_t tid = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    const bool active = tid < total;
    const int64_t t = active ? tid : total - 1;
    const int32_t cg = static_cast<int32_t>(t % col_groups);
    const int64_t t2 = t / col_groups;
    const int32_t rg = static_cast<int32_t>(t2 % row_groups);
    const int64_t plane = t2 / row_groups;
    const float* xp = x + plane * h * w;
    float* yp = y + plane * oh_total * ow_total;
    const int32_t oh0 = rg * ROWS;
    const int32_t iw0 = cg * 8;
    const int lane = threadIdx.x & 63;

    // Running state per output column: the chain for output row r is fed by input rows
    // 2r-1, 2r, 2r+1 in that order; row 2r+1 is also row 2(r+1)-1 of the next output row.
    float prev_row_vals[9];   // the shared row (2*oh-1 of the current output row)
    bool have_prev = false;

    auto load_row = [&](int32_t ih, float (&v)[9]) {
        if (ih < 0 || ih >= h) {
#pragma unroll
            for (int j = 0; j < 9; ++j) v[j] = kPadValue;
            return;
        }
        const float4 a = *reinterpret_cast<const float4*>(xp + static_cast<int64_t>(ih) * w + iw0);
        const float4 b = *reinterpret_cast<const float4*>(xp + static_cast<int64_t>(ih) * w + iw0 + 4);
        v[1] = a.x; v[2] = a.y; v[3] = a.z; v[4] = a.w;
        v[5] = b.x; v[6] = b.y; v[7] = b.z; v[8] = b.w;
        float left = __shfl_up(b.w, 1, 64);                      // neighbour lane's column iw0-1
        if (cg == 0) left = kPadValue;                           // column -1 is padding
        else if (lane == 0) left = xp[static_cast<int64_t>(ih) * w + iw0 - 1];
        v[0] = left;
    };

#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
        const int32_t oh = oh0 + r;
        float rows[3][9];
        if (have_prev) {
#pragma unroll
            for (int j = 0; j < 9; ++j) rows[0][j] = prev_row_vals[j];
        } else {
            load_row(2 * oh - 1, rows[0]);
        }
        load_row(2 * oh, rows[1]);
        load_row(2 * oh + 1, rows[2]);
        float out[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            float acc = -INFINITY;
#pragma unroll
            for (int rh = 0; rh < 3; ++rh) {
#pragma unroll
                for (int rw = 0; rw < 3; ++rw) acc = max_sel(acc, rows[rh][2 * k + rw]);
            }
            out[k] = acc;
        }
        if (active && oh < oh_total) {
            *reinterpret_cast<float4*>(yp + static_cast<int64_t>(oh) * ow_total + cg * 4) =
                make_float4(out[0], out[1], out[2], out[3]);
        }
#pragma unroll
        for (int j = 0; j < 9; ++j) prev_row_vals[j] = rows[2][j];
        have_prev = true;
    }
}

// Column max pool: window 3x1, stride (2,1), one row of padding above (and below when the height is even): the
// second half of a 3x3 / stride-2 max pool whose column maxima the convolution before it already took
// (KXC_HIP_CONV_HPOOL).  One thread produces a 4-wide strip of ROWS consecutive output rows from 2*ROWS + 1 aligned
// 16-byte loads; every input row is requested once per strip (plus the one row neighbouring strips share).
template <int ROWS>
__global__ void __launch_bounds__(kBlock) maxpool3x1s2_kernel(const float* __restrict__ x, float* __restrict__ y,
                                                              int32_t h, int32_t w, int32_t oh_total,
                                                              int32_t col_groups, int32_t row_groups, int64_t total) {
    const int64_t tid = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (tid >= total) return;
    const int32_t cg = static_cast<int32_t>(tid % col_groups);
    const int64_t t2 = tid / col_groups;
    const int32_t rg = static_cast<int32_t>(t2 % row_groups);
    const int64_t plane = t2 / row_groups;
    const float* xp = x + plane * h * w + cg * 4;
    float* yp = y + plane * oh_total * w + cg * 4;
    const int32_t oh0 = rg * ROWS;
    float4 rows[2 * ROWS + 1];
#pragma unroll
    for (int k = 0; k < 2 * ROWS + 1; ++k) {
        const int32_t ih = 2 * oh0 - 1 + k;
        rows[k] = (ih >= 0 && ih < h) ? *reinterpret_cast<const float4*>(xp + static_cast<int64_t>(ih) * w)
                                      : make_float4(kPadValue, kPadValue, kPadValue, kPadValue);
    }
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
        if (oh0 + r >= oh_total) break;
        float4 o;
        o.x = max_sel(max_sel(max_sel(-INFINITY, rows[2 * r].x), rows[2 * r + 1].x), rows[2 * r + 2].x);
        o.y = max_sel(max_sel(max_sel(-INFINITY, rows[2 * r].y), rows[2 * r + 1].y), rows[2 * r + 2].y);
        o.z = max_sel(max_sel(max_sel(-INFINITY, rows[2 * r].z), rows[2 * r + 1].z), rows[2 * r + 2].z);
        o.w = max_sel(max_sel(max_sel(-INFINITY, rows[2 * r].w), rows[2 * r + 1].w), rows[2 * r + 2].w);
        *reinterpret_cast<float4*>(yp + static_cast<int64_t>(oh0 + r) * w) = o;
    }
}

// ---------------------------------------------------------------- global average pool
// Small planes (HW <= 128): a workgroup of 256 threads takes 16 consecutive planes.  Their 16*HW contiguous
// floats are fetched with coalesced loads that are all in flight together and staged through LDS; one lane per
// plane then adds its plane up in row-major order, as the CPU loop does (LDS row stride is odd, so the lanes hit
// distinct banks).  16 planes per group keeps a batch-1 launch (512 planes) spread over 32 compute units.
constexpr int kGapPlanes = 16;       // planes per workgroup
constexpr int kGapThreads = 256;
constexpr int kGapMaxHw = 128;       // 16 planes x 128 elements = 8 loads per thread
__global__ void __launch_bounds__(kGapThreads) gap_lds_kernel(const float* __restrict__ x, float* __restrict__ y,
                                                              int64_t planes, int32_t hw, int32_t hw_pad, FastDiv div_hw) {
    extern __shared__ float tile[];
    const int64_t plane0 = static_cast<int64_t>(blockIdx.x) * kGapPlanes;
    const int64_t remaining = planes - plane0;
    const int32_t np = remaining < kGapPlanes ? static_cast<int32_t>(remaining) : kGapPlanes;
    const int32_t count = np * hw;
    const float* src = x + plane0 * hw;
    constexpr int kLoads = kGapPlanes * kGapMaxHw / kGapThreads;
    float v[kLoads];
    // every load is issued before the first value is used
#pragma unroll
    for (int k = 0; k < kLoads; ++k) {
        const int32_t e = static_cast<int32_t>(threadIdx.x) + k * kGapThreads;
        v[k] = e < count ? src[e] : 0.0f;
    }
#pragma unroll
    for (int k = 0; k < kLoads; ++k) {
        const int32_t e = static_cast<int32_t>(threadIdx.x) + k * kGapThreads;
        const int32_t p = fast_div(e, div_hw);
        if (e < count) tile[p * hw_pad + (e - p * hw)] = v[k];
    }
    __syncthreads();
    if (static_cast<int32_t>(threadIdx.x) < np) {
        float acc = 0.0f;
        const float* row = tile + threadIdx.x * hw_pad;
#pragma unroll 8
        for (int32_t i = 0; i < hw; ++i) acc = __fadd_rn(acc, row[i]);
        y[plane0 + threadIdx.x] = __fdiv_rn(acc, static_cast<float>(hw));
    }
}

// Large planes: one thread per plane would serialise; use one wave per plane with a strided
// partial sum and a wave reduction (order differs from the CPU loop; within fp32 tolerance).
__global__ void __launch_bounds__(64) gap_wave_kernel(const float* __restrict__ x, float* __restrict__ y,
                                                      int64_t planes, int64_t hw) {
    const int64_t plane = blockIdx.x;
    if (plane >= planes) return;
    const float* src = x + plane * hw;
    float acc = 0.0f;
    for (int64_t i = threadIdx.x; i < hw; i += 64) acc += src[i];
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) acc += __shfl_down(acc, off, 64);
    if (threadIdx.x == 0) y[plane] = __fdiv_rn(acc, static_cast<float>(hw));
}

// ---------------------------------------------------------------- int8
__global__ void __launch_bounds__(kBlock) maxpool_i8_kernel(const int8_t* __restrict__ x, int8_t* __restrict__ y,
                                                            PoolDims d, int64_t total) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlock;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; i < total; i += stride) {
        const int32_t ow = static_cast<int32_t>(i % d.ow);
        const int64_t t = i / d.ow;
        const int32_t oh = static_cast<int32_t>(t % d.oh);
        const int64_t plane = t / d.oh;
        const int8_t* xp = x + plane * d.h * d.w;
        int32_t m = -128;
        for (int rh = 0; rh < d.kh; ++rh) {
            const int ih = oh * d.sh + rh - d.pt;
            if (ih < 0 || ih >= d.h) continue;
            for (int rw = 0; rw < d.kw; ++rw) {
                const int iw = ow * d.sw + rw - d.pl;
                if (iw < 0 || iw >= d.w) continue;
                const int32_t v = xp[ih * d.w + iw];
                m = v > m ? v : m;
            }
        }
        y[i] = static_cast<int8_t>(m);
    }
}

__global__ void __launch_bounds__(kBlock) gap_i8_kernel(const int8_t* __restrict__ x, int8_t* __restrict__ y,
                                                        int64_t planes, int32_t hw, float mult) {
    const int64_t p = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (p >= planes) return;
    const int8_t* src = x + p * hw;
    int32_t s = 0;
    for (int32_t i = 0; i < hw; ++i) s += src[i];
    const float v = __fmul_rn(static_cast<float>(s), mult);
    float r = rintf(v);
    r = (v == v) ? r : 0.0f;
    r = fminf(fmaxf(r, -128.0f), 127.0f);
    y[p] = static_cast<int8_t>(static_cast<int32_t>(r));
}

int32_t FillDims(const kxc_hip_pool2d_desc* p, PoolDims* d, const char* who) {
    KXC_HIP_REQUIRE(p != nullptr, "%s: desc is NULL", who);
    KXC_HIP_REQUIRE(p->n >= 0 && p->c >= 0 && p->h > 0 && p->w > 0, "%s: bad input shape", who);
    KXC_HIP_REQUIRE(p->kh > 0 && p->kw > 0 && p->stride_h > 0 && p->stride_w > 0, "%s: bad window", who);
    KXC_HIP_REQUIRE(p->pad_top >= 0 && p->pad_left >= 0 && p->pad_bottom >= 0 && p->pad_right >= 0,
                    "%s: negative padding", who);
    const int hn = p->h + p->pad_top + p->pad_bottom - p->kh;
    const int wn = p->w + p->pad_left + p->pad_right - p->kw;
    // WindowOutputDim (src/relay/type_infer.cc:166-184)
    KXC_HIP_REQUIRE(hn >= 0 && wn >= 0, "%s: pool2d window is larger than input", who);
    d->n = p->n; d->c = p->c; d->h = p->h; d->w = p->w;
    d->oh = p->ceil_mode ? (hn + p->stride_h - 1) / p->stride_h + 1 : hn / p->stride_h + 1;
    d->ow = p->ceil_mode ? (wn + p->stride_w - 1) / p->stride_w + 1 : wn / p->stride_w + 1;
    d->kh = p->kh; d->kw = p->kw; d->sh = p->stride_h; d->sw = p->stride_w;
    d->pt = p->pad_top; d->pl = p->pad_left;
    return KXC_HIP_OK;
}

inline int GridFor(int64_t items) {
    int64_t g = CeilDiv(items, kBlock);
    if (g < 1) g = 1;
    if (g > 256 * 32) g = 256 * 32;
    return static_cast<int>(g);
}

}  // namespace

extern "C" {

int32_t kxc_hip_pool2d_f32(const kxc_hip_pool2d_desc* desc, const float* x, float* y, void* stream) {
    PoolDims d;
    if (int32_t rc = FillDims(desc, &d, "kxc_hip_pool2d_f32")) return rc;
    const int64_t planes = static_cast<int64_t>(d.n) * d.c;
    const int64_t total = planes * d.oh * d.ow;
    if (total == 0) return KXC_HIP_OK;
    KXC_HIP_REQUIRE(x && y, "kxc_hip_pool2d_f32: NULL pointer");
    hipStream_t s = ResolveStream(stream);
    const bool fast = !desc->is_avg && d.kh == 3 && d.kw == 3 && d.sh == 2 && d.sw == 2 && d.pt == 1 && d.pl == 1 &&
                      desc->pad_bottom == 1 && desc->pad_right == 1 && !desc->ceil_mode && (d.w % 8) == 0 &&
                      (d.h % 2) == 0 && d.ow == d.w / 2 && d.oh == d.h / 2 &&
                      (reinterpret_cast<uintptr_t>(x) & 15u) == 0 && (reinterpret_cast<uintptr_t>(y) & 15u) == 0;
    if (fast) {
        // four output rows per thread share input rows between them; a launch too small to give every compute
        // unit a workgroup that way (batch 1) takes one row per thread and four times the threads instead
        const int32_t col_groups = d.ow / 4;
        const bool small = planes * ((d.oh + 3) / 4) * col_groups < 256LL * kBlock;   // 256 compute units
        const int32_t rows = small ? 1 : 4;
        const int32_t row_groups = (d.oh + rows - 1) / rows;
        const int64_t threads = planes * row_groups * col_groups;
        const int64_t blocks = CeilDiv(threads, kBlock);
        KXC_HIP_REQUIRE(blocks <= kMaxGridX, "kxc_hip_pool2d_f32: tensor too large");
        if (small)
            maxpool3x3s2_kernel<1><<<NoteGrid(static_cast<int>(blocks)), NoteBlock(kBlock), NoteLds(0), s>>>(
                x, y, d.h, d.w, d.oh, d.ow, col_groups, row_groups, threads);
        else
            maxpool3x3s2_kernel<4><<<NoteGrid(static_cast<int>(blocks)), NoteBlock(kBlock), NoteLds(0), s>>>(
                x, y, d.h, d.w, d.oh, d.ow, col_groups, row_groups, threads);
        return CheckLaunch("maxpool3x3s2");
    }
    const bool columns = !desc->is_avg && d.kh == 3 && d.kw == 1 && d.sh == 2 && d.sw == 1 && d.pt == 1 && d.pl == 0 &&
                         desc->pad_right == 0 && desc->pad_bottom <= 1 && !desc->ceil_mode && (d.w % 4) == 0 &&
                         (reinterpret_cast<uintptr_t>(x) & 15u) == 0 && (reinterpret_cast<uintptr_t>(y) & 15u) == 0;
    if (columns) {
        const int32_t col_groups = d.w / 4;
        const bool small = planes * ((d.oh + 3) / 4) * col_groups < 256LL * kBlock;
        const int32_t rows = small ? 1 : 4;
        const int32_t row_groups = (d.oh + rows - 1) / rows;
        const int64_t threads = planes * row_groups * col_groups;
        const int64_t blocks = CeilDiv(threads, kBlock);
        KXC_HIP_REQUIRE(blocks <= kMaxGridX, "kxc_hip_pool2d_f32: tensor too large");
        if (small)
            maxpool3x1s2_kernel<1><<<NoteGrid(static_cast<int>(blocks)), NoteBlock(kBlock), NoteLds(0), s>>>(
                x, y, d.h, d.w, d.oh, col_groups, row_groups, threads);
        else
            maxpool3x1s2_kernel<4><<<NoteGrid(static_cast<int>(blocks)), NoteBlock(kBlock), NoteLds(0), s>>>(
                x, y, d.h, d.w, d.oh, col_groups, row_groups, threads);
        return CheckLaunch("maxpool3x1s2");
    }
    if (desc->is_avg) pool_generic_kernel<true><<<NoteGrid(GridFor(total)), NoteBlock(kBlock), NoteLds(0), s>>>(x, y, d, total);
    else pool_generic_kernel<false><<<NoteGrid(GridFor(total)), NoteBlock(kBlock), NoteLds(0), s>>>(x, y, d, total);
    return CheckLaunch("pool2d");
}

int32_t kxc_hip_global_avg_pool2d_f32(const float* x, float* y, int64_t n, int64_t c, int64_t h, int64_t w,
                                      void* stream) {
    KXC_HIP_REQUIRE(n >= 0 && c >= 0 && h > 0 && w > 0, "kxc_hip_global_avg_pool2d_f32: bad shape");
    const int64_t planes = n * c;
    if (planes == 0) return KXC_HIP_OK;
    KXC_HIP_REQUIRE(x && y, "kxc_hip_global_avg_pool2d_f32: NULL pointer");
    hipStream_t s = ResolveStream(stream);
    const int64_t hw = h * w;
    if (hw <= kGapMaxHw) {
        const int32_t hw_pad = static_cast<int32_t>(hw | 1);
        const int64_t blocks = CeilDiv(planes, kGapPlanes);
        KXC_HIP_REQUIRE(blocks <= kMaxGridX, "kxc_hip_global_avg_pool2d_f32: tensor too large");
        const size_t lds = static_cast<size_t>(kGapPlanes) * hw_pad * sizeof(float);   // <= 8.1 KiB
        gap_lds_kernel<<<NoteGrid(static_cast<int>(blocks)), NoteBlock(kGapThreads), NoteLds(lds), s>>>(
            x, y, planes, static_cast<int32_t>(hw), hw_pad, MakeFastDiv(static_cast<int32_t>(hw)));
        return CheckLaunch("global_avg_pool2d");
    }
    KXC_HIP_REQUIRE(planes <= kMaxGridX, "kxc_hip_global_avg_pool2d_f32: tensor too large");
    gap_wave_kernel<<<NoteGrid(static_cast<int>(planes)), NoteBlock(64), NoteLds(0), s>>>(x, y, planes, hw);
    return CheckLaunch("global_avg_pool2d");
}

int32_t kxc_hip_maxpool2d_i8(const kxc_hip_pool2d_desc* desc, const int8_t* x, int8_t* y, void* stream) {
    PoolDims d;
    if (int32_t rc = FillDims(desc, &d, "kxc_hip_maxpool2d_i8")) return rc;
    KXC_HIP_REQUIRE(!desc->is_avg, "kxc_hip_maxpool2d_i8: average pooling is not defined for int8");
    const int64_t total = static_cast<int64_t>(d.n) * d.c * d.oh * d.ow;
    if (total == 0) return KXC_HIP_OK;
    KXC_HIP_REQUIRE(x && y, "kxc_hip_maxpool2d_i8: NULL pointer");
    maxpool_i8_kernel<<<NoteGrid(GridFor(total)), NoteBlock(kBlock), NoteLds(0), ResolveStream(stream)>>>(x, y, d, total);
    return CheckLaunch("maxpool2d_i8");
}

int32_t kxc_hip_global_avg_pool2d_i8(const int8_t* x, int8_t* y, int64_t n, int64_t c, int64_t h, int64_t w,
                                     float mult, void* stream) {
    KXC_HIP_REQUIRE(n >= 0 && c >= 0 && h > 0 && w > 0, "kxc_hip_global_avg_pool2d_i8: bad shape");
    const int64_t planes = n * c;
    if (planes == 0) return KXC_HIP_OK;
    KXC_HIP_REQUIRE(x && y, "kxc_hip_global_avg_pool2d_i8: NULL pointer");
    KXC_HIP_REQUIRE(h * w <= 2147483647LL / 128, "kxc_hip_global_avg_pool2d_i8: plane too large for int32 sum");
    gap_i8_kernel<<<NoteGrid(static_cast<int>(CeilDiv(planes, kBlock))), NoteBlock(kBlock), NoteLds(0), ResolveStream(stream)>>>(
        x, y, planes, static_cast<int32_t>(h * w), mult);
    return CheckLaunch("global_avg_pool2d_i8");
}

}  // extern "C"
