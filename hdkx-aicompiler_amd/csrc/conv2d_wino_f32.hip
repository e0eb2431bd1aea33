// conv2d_wino_f32.hip -- nn_conv2d for 3x3 filters, stride 1, dilation 1 (NCHW, OIHW, fp32) as Winograd
// F(2x2, 3x3) on the fp32 matrix cores of gfx950.
//
//   Y = A^T [ (G g G^T) (.) (B^T d B) ] A      per 4x4 input patch d, 3x3 filter g, 2x2 output block Y
//
// 16 multiplies per 2x2 output block and channel instead of 36: the matrix work of a layer drops by 2.25x.  The
// sixteen element-wise products are sixteen independent matrix products  M_f[o][tile] = sum_c U_f[o][c] V_f[c][tile]
// (f = position in the 4x4 transform domain), which is what the matrix cores run.
//
//  * The filter transform U = G g G^T is done once per weight tensor by wino_weight_kernel into a packed buffer
//    whose blocks are byte-for-byte the LDS image the main kernel wants: [32 output channels][4 input channels]
//    as [c][o/16][f/4][o%16][f%4], 8 KiB per block, so that a workgroup fills its weight tile with 16-byte
//    loads that write straight to LDS, and a lane's four f values of one (o, c) are one 16-byte LDS read.
//  * The input transform V = B^T d B runs inside the main kernel: per step of 4 input channels every thread
//    loads 3 rows x 4 columns of one tile's patch into registers (two threads share a tile: rows 0-2 give
//    transform rows 0-1, rows 1-3 give rows 2-3), transforms them with 16 additions and writes two 16-byte
//    vectors to LDS.  Padding costs nothing: offsets of positions outside the image point beyond the buffer,
//    where a buffer load returns 0.  The loads for step s+2 are issued while step s multiplies.
//  * v_mfma_f32_16x16x4_f32: a wave owns 32 output channels x 16 tiles x all 16 f -- 32 accumulators of 4
//    registers.  Because every f of one (o, tile) lands in the same lane, the output transform A^T M A and the
//    epilogue (bias, residual, ReLU) run in registers and the 2x2 block is stored as two 8-byte runs; the 16
//    lanes of a quarter-wave hold consecutive tiles, i.e. 128 contiguous bytes of an output row.
//
// The sums are formed in a different order than the direct loop nest (and G introduces factors 1/2, 1/4), so
// results agree with the CPU backend within the fp32 tolerance of the operator (about 1e-6 relative on
// ResNet-sized reductions), not bit for bit.
#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <type_traits>
#include <utility>
#include <vector>

#include "common.h"

using namespace kxc_hip;

namespace {

typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx2 __attribute__((ext_vector_type(2)));
typedef uint32_t uintx2 __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) void* lds_ptr_t;

constexpr uint32_t kOob = 0x80000000u;     // beyond any buffer this kernel accepts (< 2 GiB): reads as 0

struct WinoArgs {
    const float* x;
    const float* u;
    const float* bias;
    const float* res;
    float* y;
    int32_t N, C, H, W, O, OH, OW, ph, pw;
    int32_t TW, TI, NT;              // tiles per output row, per image, in total
    int32_t HW, OHW;
    int32_t csteps;                  // C / 4
    int32_t t_groups, k_groups, num_units, units_per_xcd, k_fastest;
    uint32_t x_bytes, u_bytes, flags;
    // gsplit > 1: the input channels are split over gsplit workgroups per tile (steps_per_split steps each), which
    // write raw partial outputs to partial[split][N*O*OH*OW]; a second kernel adds them and applies the epilogue
    int32_t gsplit, steps_per_split;
    float* partial;
    uint32_t* counters;              // FUSE kernels: arrival counter of unit i at counters[i], zero between launches
    FastDiv div_ti, div_tw, div_kgroups, div_tgroups, div_gsplit;
};

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* p, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, static_cast<int>(bytes), 0x00020000);
}

// 16 bytes per lane from a buffer straight into LDS (lane l writes lds + 16*l).  The 16-byte form exists on
// gfx950 only; the host pass of the compiler does not know the target and rejects the size, so it sees an
// empty body.
__device__ __forceinline__ void load16_to_lds(__amdgpu_buffer_rsrc_t rsrc, lds_ptr_t lds, uint32_t voffset,
                                              uint32_t soffset) {
#if defined(__HIP_DEVICE_COMPILE__)
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, lds, 16, voffset, soffset, 0, 0);
#endif
}

__device__ __forceinline__ float load_f32(__amdgpu_buffer_rsrc_t rsrc, uint32_t voffset, uint32_t soffset) {
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc, voffset, soffset, 0));
}

// max(v, 0) with NaN -> 0, as (v > 0 ? v : 0) gives; one instruction instead of a compare and a select
__device__ __forceinline__ float relu_sel(float v) { return __builtin_fmaxf(v, 0.0f); }

// ------------------------------------------------------------------------------------------
// Filter transform, for o < 32*ceil(O/32) (absent output channels give zero blocks).
// packed index: ((o/32 * csteps + c/4) * 2048) + (((c%4)*2 + (o%32)/16)*4 + i)*64 + (o%16)*4 + j  for U[i][j]
// ------------------------------------------------------------------------------------------
// A workgroup of 256 threads transforms 32 output channels x 8 input channels: the 72 raw floats of every output
// channel are read as one run into LDS, then thread (c, o) = (tid / 32, tid % 32) transforms its filter and stores
// four float4 -- the 16 lanes of a quarter wave write 256 contiguous bytes, so every cache line is written whole
// (one thread per filter in (o, c) order wrote isolated 16-byte pieces: twice the bytes at the memory, 68 us for the
// thirteen layers of ResNet-18 against 20 us).
constexpr int kWeightTileC = 8;
__device__ __forceinline__ void wino_weight_tile(const float* __restrict__ w, float* __restrict__ u, int32_t O, int32_t C,
                                                 int tile, float* raw) {
    constexpr int RS = kWeightTileC * 9 + 1;      // odd row stride: lanes of different o hit different banks
    const int ctiles = (C + kWeightTileC - 1) / kWeightTileC;
    const int ob = tile / ctiles, cb = tile - ob * ctiles;
    const int o0 = ob * 32, c0 = cb * kWeightTileC;
    const int cn = min(kWeightTileC, C - c0);     // 4 or 8 (C is a multiple of 4)
    const int tid = threadIdx.x;
    for (int idx = tid; idx < 32 * kWeightTileC * 9; idx += 256) {
        const int ol = idx / (kWeightTileC * 9), r = idx - ol * (kWeightTileC * 9);
        const bool ok = o0 + ol < O && r < cn * 9;
        raw[ol * RS + r] = ok ? w[(static_cast<int64_t>(o0 + ol) * C + c0) * 9 + r] : 0.0f;
    }
    __syncthreads();
    const int cl = tid >> 5, ol = tid & 31;
    if (cl >= cn) return;
    float g[3][3];
#pragma unroll
    for (int i = 0; i < 3; ++i)
#pragma unroll
        for (int j = 0; j < 3; ++j) g[i][j] = raw[ol * RS + cl * 9 + i * 3 + j];
    float t[4][3];      // G g
#pragma unroll
    for (int j = 0; j < 3; ++j) {
        t[0][j] = g[0][j];
        t[1][j] = 0.5f * ((g[0][j] + g[2][j]) + g[1][j]);
        t[2][j] = 0.5f * ((g[0][j] + g[2][j]) - g[1][j]);
        t[3][j] = g[2][j];
    }
    const int csteps = C / 4;
    const int c = c0 + cl;
    float* const dst = u + (static_cast<int64_t>(ob) * csteps + c / 4) * 2048 + (((c % 4) * 2 + ol / 16) * 4) * 64 + (ol % 16) * 4;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        floatx4 v;
        v[0] = t[i][0];
        v[1] = 0.5f * ((t[i][0] + t[i][2]) + t[i][1]);
        v[2] = 0.5f * ((t[i][0] + t[i][2]) - t[i][1]);
        v[3] = t[i][2];
        *reinterpret_cast<floatx4*>(dst + i * 64) = v;
    }
}
inline int64_t WeightTiles(int64_t o_padded, int64_t C) { return (o_padded / 32) * ((C + kWeightTileC - 1) / kWeightTileC); }

__global__ void __launch_bounds__(256) wino_weight_kernel(const float* __restrict__ w, float* __restrict__ u, int32_t O,
                                                          int32_t C) {
    __shared__ float raw[32 * (kWeightTileC * 9 + 1)];
    wino_weight_tile(w, u, O, C, blockIdx.x, raw);
}

// The filter transforms of several layers in one launch (a launch plan transforms all its Winograd layers' weights
// at the start of a run): block b belongs to the job whose [first_block, next first_block) range holds it.
constexpr int kMaxWeightJobs = 32;
struct WinoWeightBatch {
    const float* w[kMaxWeightJobs];
    float* u[kMaxWeightJobs];
    int32_t O[kMaxWeightJobs], C[kMaxWeightJobs], first_block[kMaxWeightJobs + 1];
    int32_t count;
};
__global__ void __launch_bounds__(256) wino_weight_batch_kernel(const WinoWeightBatch b) {
    __shared__ float raw[32 * (kWeightTileC * 9 + 1)];
    int j = 0;
    while (j + 1 < b.count && static_cast<int32_t>(blockIdx.x) >= b.first_block[j + 1]) ++j;
    wino_weight_tile(b.w[j], b.u[j], b.O[j], b.C[j], static_cast<int>(blockIdx.x) - b.first_block[j], raw);
}

// ------------------------------------------------------------------------------------------
// Main kernel.  WK x WT waves; a wave owns 32 output channels x 16 tiles; the workgroup 32*WK x 16*WT.
// One step = 4 input channels.  LDS per buffer: U [WK][c4][o/16: 2][f/4: 4][o%16][f%4] and
// V [c4][WT][f/4: 4][tile%16][f%4]; two of each.
// ------------------------------------------------------------------------------------------
// FUSE: a reduction split over workgroups is finished by the part that arrives last (see split_arrive_last)
// instead of the adding kernel.
template <int WK, int WT, int KS, bool FUSE = false>
__global__ void __launch_bounds__(64 * WK * WT * KS) __attribute__((amdgpu_waves_per_eu(2)))
wino_kernel(const WinoArgs a) {
    static_assert(!FUSE || KS == 1, "the split over workgroups is never combined with the split over wave groups");
    constexpr int NW = WK * WT;                     // waves of one reduction group
    constexpr int NTH = 64 * NW;                    // threads of one reduction group
    constexpr int TT = 16 * WT;
    constexpr int U_FLOATS = 2048 * WK;
    constexpr int V_FLOATS = 1024 * WT;
    constexpr int ULOADS = U_FLOATS / 4 / NTH;     // 16-byte loads per thread and step
    constexpr int ITEMS = 2 / WK;                   // (tile, channel, half) items per thread and step
    static_assert(WK == 1 || WK == 2, "a thread transforms one or two input items per step");
    static_assert((U_FLOATS / 4) % NTH == 0, "weight tile must divide over the threads");
    static_assert(KS == 1 || KS == 2, "the input channels are split over at most two groups of waves");

    extern __shared__ float lds[];
    const int lane = threadIdx.x & 63;
    const int wave_all = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int kgroup = wave_all / NW;               // which share of the input channels this wave reduces
    const int wave = wave_all - kgroup * NW;
    const int tid = static_cast<int>(threadIdx.x) - kgroup * NTH;
    const int wave_k = wave / WT, wave_t = wave % WT;
    // Consecutive workgroups go to the 8 XCDs round-robin; each XCD (own L2) takes a contiguous run of units.
    const int slot = (blockIdx.x & 7) * a.units_per_xcd + (blockIdx.x >> 3);
    if (slot >= a.num_units * a.gsplit || static_cast<int>(blockIdx.x >> 3) >= a.units_per_xcd) return;
    const int unit = a.gsplit > 1 ? fast_div(slot, a.div_gsplit) : slot;
    const int split = slot - unit * a.gsplit;
    int kg, tg;
    if (a.k_fastest) { tg = fast_div(unit, a.div_kgroups); kg = unit - tg * a.k_groups; }
    else { kg = fast_div(unit, a.div_tgroups); tg = unit - kg * a.t_groups; }
    const int t0 = tg * TT;
    const __amdgpu_buffer_rsrc_t xr = make_rsrc(a.x, a.x_bytes);
    const __amdgpu_buffer_rsrc_t ur = make_rsrc(a.u, a.u_bytes);

    // ---- weight tile loads: 16-byte unit idx = j*NTH + tid of the tile; block h = idx / 512 is k32 group kg*WK + h
    uint32_t uoff[ULOADS];
#pragma unroll
    for (int j = 0; j < ULOADS; ++j) {
        const int idx = j * NTH + tid;
        const int h = idx / 512, within = idx - h * 512;
        uoff[j] = static_cast<uint32_t>((kg * WK + h) * a.csteps) * 8192u + static_cast<uint32_t>(within) * 16u;
    }

    float* const ub0 = lds + kgroup * 2 * (U_FLOATS + V_FLOATS);
    float* const ub1 = ub0 + U_FLOATS;
    float* const vb0 = ub0 + 2 * U_FLOATS;
    float* const vb1 = vb0 + V_FLOATS;
    // (the host never combines the split over workgroups with the split over wave groups)
    const int s_lo = a.gsplit > 1 ? split * a.steps_per_split : kgroup * (a.csteps / KS);
    const int s_hi = a.gsplit > 1 ? min(s_lo + a.steps_per_split, a.csteps) : s_lo + a.csteps / KS;
    const int last = s_hi - 1;

    auto issue_u = [&](int s, float* buf) {
#pragma unroll
        for (int j = 0; j < ULOADS; ++j)
            load16_to_lds(ur, (lds_ptr_t)(buf + (j * NTH + wave * 64) * 4), uoff[j], static_cast<uint32_t>(s) * 8192u);
    };
    // The first weight tile is requested before anything else is computed: at small batches it comes from beyond
    // the L2 and its latency then overlaps the gather offsets below.
    issue_u(s_lo, ub0);
    __builtin_amdgcn_sched_barrier(0);

    // ---- input items: item = tid + i*NTH -> tile = item % TT, channel = (item / TT) % 4, half = item / (4*TT)
    uint32_t goff[ITEMS][12];
    int vdst_a[ITEMS], vdst_b[ITEMS];
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
        const int item = tid + i * NTH;
        const int tile_l = item % TT, cl = (item / TT) % 4, half = item / (4 * TT);
        const int tile = t0 + tile_l;
        const int n = fast_div(tile, a.div_ti), rem = tile - n * a.TI;
        const int ty = fast_div(rem, a.div_tw), tx = rem - ty * a.TW;
        // (row and column validity are tested once each and combined per element: no per-element products)
        const int iw0 = 2 * tx - a.pw;
        uint32_t colmask[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) colmask[j] = (iw0 + j >= 0 && iw0 + j < a.W) ? 0u : kOob;
        const uint32_t plane = static_cast<uint32_t>((n * a.C + cl) * a.H);
#pragma unroll
        for (int r = 0; r < 3; ++r) {
            const int ih = 2 * ty - a.ph + half + r;
            const uint32_t rowmask = (tile < a.NT && ih >= 0 && ih < a.H) ? 0u : kOob;
            const uint32_t row = ((plane + static_cast<uint32_t>(ih)) * static_cast<uint32_t>(a.W) + static_cast<uint32_t>(iw0)) * 4u;
#pragma unroll
            // (an offset with the top bit set lies beyond the buffer whatever its other bits are)
            for (int j = 0; j < 4; ++j) goff[i][r * 4 + j] = (row + 4u * j) | rowmask | colmask[j];
        }
        // transform rows 2*half and 2*half + 1 of the tile; for half 1 the transform below produces them in the
        // order (3, 2)
        const int vrow = ((cl * WT + tile_l / 16) * 4 + 2 * half) * 64 + (tile_l % 16) * 4;
        vdst_a[i] = vrow + (half ? 64 : 0);
        vdst_b[i] = vrow + (half ? 0 : 64);
    }
    const int a_base = wave_k * 2048 + (lane >> 4) * 512 + (lane & 15) * 4;
    const int b_base = ((lane >> 4) * WT + wave_t) * 256 + (lane & 15) * 4;

    floatx4 acc[16][2];

    float d[ITEMS][12];
    auto load_raw = [&](int s) {
        const uint32_t soff = static_cast<uint32_t>(s) * static_cast<uint32_t>(a.HW) * 16u;   // 4 channels of HW floats
#pragma unroll
        for (int i = 0; i < ITEMS; ++i)
#pragma unroll
            for (int q = 0; q < 12; ++q) d[i][q] = load_f32(xr, goff[i][q], soff);
    };
    // On gfx950 the fp32 matrix instructions and the vector ALU share a datapath (measured: an independent v_add_f32
    // between two v_mfma_f32_16x16x4_f32 costs 4.3 cycles plus about 8 per change of kind; one issued by the other
    // wave of the SIMD costs 4.8), so every vector instruction of this kernel is paid for in matrix time.
    // Rows e0, e1, e2 of the patch are rows 0-2 (half 0) or 1-3 (half 1) of the 4x4 input patch d:
    //   half 0: t0 = d0 - d2 = e0 - e2,  t1 = d1 + d2 = e1 + e2
    //   half 1: t3 = d1 - d3 = e0 - e2,  t2 = d2 - d1 = e1 - e0
    // i.e. ta = e0 - e2 and tb = e1 + (half ? -e0 : e2): one select per column instead of both variants and two.
    // The half an item transforms is fixed for the whole kernel: with two items per thread item i is half i; with one, a
    // wave's threads all work on the half `wave_half`, and the main loop below exists once per half (one branch in
    // front of it), so that tb is one instruction per column instead of a select and an addition.
    auto transform = [&](float* buf, auto half_c) {
#pragma unroll
        for (int i = 0; i < ITEMS; ++i) {
            const bool half = ITEMS == 2 ? i == 1 : decltype(half_c)::value;
            float ta[4], tb[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float e0 = d[i][j], e1 = d[i][4 + j], e2 = d[i][8 + j];
                ta[j] = e0 - e2;
                tb[j] = half ? e1 - e0 : e1 + e2;
            }
            floatx4 va, vb;
            va[0] = ta[0] - ta[2]; va[1] = ta[1] + ta[2]; va[2] = ta[2] - ta[1]; va[3] = ta[1] - ta[3];
            vb[0] = tb[0] - tb[2]; vb[1] = tb[1] + tb[2]; vb[2] = tb[2] - tb[1]; vb[3] = tb[1] - tb[3];
            *reinterpret_cast<floatx4*>(buf + vdst_a[i]) = va;
            *reinterpret_cast<floatx4*>(buf + vdst_b[i]) = vb;
        }
    };
    // Operands of one group of four f values: two 16-byte reads of U (output-channel blocks 0 and 1) and one of V.
    // Two register sets: the reads for group fg+1 are issued before the matrix instructions of group fg.
    floatx4 ra[2][2], rb[2];
    auto fetch = [&](const float* ub, const float* vb, int fg, int set) {
        ra[set][0] = *reinterpret_cast<const floatx4*>(ub + a_base + fg * 64);
        ra[set][1] = *reinterpret_cast<const floatx4*>(ub + a_base + 256 + fg * 64);
        rb[set] = *reinterpret_cast<const floatx4*>(vb + b_base + fg * 64);
    };
    // first: the step that starts the accumulators -- C is a constant (0, or the bias for f = 5: m11 has the
    // coefficient +1 in all four outputs of A^T M A) instead of 128 registers cleared beforehand
    floatx4 bias4[2];
    auto mm = [&](int fg, int set, auto first) {
        constexpr bool FIRST = decltype(first)::value;
        const floatx4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int f = 0; f < 4; ++f) {
            const int ff = fg * 4 + f;
            acc[ff][0] = __builtin_amdgcn_mfma_f32_16x16x4f32(ra[set][0][f], rb[set][f], FIRST ? (ff == 5 ? bias4[0] : zero) : acc[ff][0], 0, 0, 0);
            acc[ff][1] = __builtin_amdgcn_mfma_f32_16x16x4f32(ra[set][1][f], rb[set][f], FIRST ? (ff == 5 ? bias4[1] : zero) : acc[ff][1], 0, 0, 0);
        }
    };

    // LDS: two weight tiles and two transformed-input tiles.  The compiler orders every barrier after the
    // LDS-writing loads issued before it, so a weight tile is requested at the top of the step before the one that
    // uses it and has that whole step to arrive; the raw input (registers) is requested two steps ahead.
    // KS == 2 (launches with too few units to give every SIMD two waves): the two groups of waves own their own
    // tiles and reduce one half of the input channels each, in lock step (the barriers are shared); their
    // accumulators are added through LDS after the loop.  The host passes a step count divisible by KS.
    // ---- prologue: weight tile and transformed input of the first step; raw input of the second in flight
    load_raw(s_lo);
    {
        // the bias enters through the accumulators (a part of a split reduction adds none: the descriptor is empty)
        // (of two groups of waves whose accumulators are added, the first brings it)
        const bool in_acc = a.gsplit == 1 && kgroup == 0 && (a.flags & KXC_HIP_CONV_BIAS) != 0;
        const __amdgpu_buffer_rsrc_t br = make_rsrc(in_acc ? a.bias : a.x, in_acc ? static_cast<uint32_t>(a.O) * 4u : 0u);
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int g = 0; g < 4; ++g)
                bias4[kb][g] = load_f32(br, static_cast<uint32_t>((kg * WK + wave_k) * 32 + kb * 16 + 4 * (lane >> 4) + g) * 4u, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
    auto main_loop = [&](auto half_c) {
    transform(vb0, half_c);
    load_raw(min(s_lo + 1, last));
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();

    // One step: the tiles of step s are multiplied while those of step s + 1 are made.  A scheduling barrier after
    // every fetch: left free, the compiler sinks one of the three reads below the matrix instructions of the group
    // before, to share its registers, and the wave then waits out that read's LDS latency at every change of group.
    // The transform runs in one block between two groups of matrix instructions (spreading it between them gains
    // nothing, see transform, and costs a change of kind per piece).
    auto step = [&](int s, const float* ucur, const float* vcur, float* unxt, float* vnxt, auto first) {
        // Steps past the end re-load the last step (never used), which keeps the step free of branches.
        issue_u(min(s + 1, last), unxt);
        fetch(ucur, vcur, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        fetch(ucur, vcur, 1, 1);
        __builtin_amdgcn_sched_barrier(0);
        mm(0, 0, first);
        __builtin_amdgcn_sched_barrier(0);
        fetch(ucur, vcur, 2, 0);
        __builtin_amdgcn_sched_barrier(0);
        transform(vnxt, half_c);       // raw input of step s + 1, requested one step ago
        __builtin_amdgcn_sched_barrier(0);
        mm(1, 1, first);
        __builtin_amdgcn_sched_barrier(0);
        fetch(ucur, vcur, 3, 1);
        __builtin_amdgcn_sched_barrier(0);
        mm(2, 0, first);
        load_raw(min(s + 2, last));
#pragma unroll
        for (int q = 0; q < 8; ++q) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);      // one matrix instruction
            __builtin_amdgcn_sched_group_barrier(0x020, 2, 0);      // two vector memory reads
        }
        __builtin_amdgcn_sched_barrier(0);
        mm(3, 1, first);
        __builtin_amdgcn_sched_barrier(0);
        __syncthreads();
    };
    step(s_lo, ub0, vb0, ub1, vb1, std::true_type{});
    // (two steps per trip, so that every call names its buffers: their per-lane addresses stay in registers)
    for (int s = s_lo + 1; s < s_hi; s += 2) {
        step(s, ub1, vb1, ub0, vb0, std::false_type{});
        if (s + 1 < s_hi) step(s + 1, ub0, vb0, ub1, vb1, std::false_type{});
    }
    };
    if (ITEMS == 2 || __builtin_amdgcn_readfirstlane(tid / (4 * TT)) == 0) main_loop(std::false_type{});
    else main_loop(std::true_type{});
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

    if (KS > 1) {
        // group 1 parks its accumulators in LDS (the tiles are dead after the loop's last barrier), one
        // output-channel block at a time ([f][g][thread]: 16 KiB per wave), group 0 adds them to its own
        float* const red = lds;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
            if (kgroup == 1) {
#pragma unroll
                for (int f = 0; f < 16; ++f)
#pragma unroll
                    for (int g = 0; g < 4; ++g) red[(f * 4 + g) * NTH + tid] = acc[f][kb][g];
            }
            __syncthreads();
            if (kgroup == 0) {
#pragma unroll
                for (int f = 0; f < 16; ++f)
#pragma unroll
                    for (int g = 0; g < 4; ++g) acc[f][kb][g] += red[(f * 4 + g) * NTH + tid];
            }
            __syncthreads();
        }
        if (kgroup != 0) return;
    }

    // ---- epilogue: accumulator register g of block kb holds output channel 16*kb + 4*(lane/16) + g, tile lane%16.
    // Everything goes through buffer descriptors: an offset beyond the buffer makes a load return 0 and drops a
    // store, so absent channels, tiles past the end and the odd last row / column need no branches, and all loads
    // (bias, residual) are issued before the first store -- a wait for a load would otherwise also wait for every
    // store issued before it.
    const int tile = t0 + wave_t * 16 + (lane & 15);
    const int tile_c = min(tile, a.NT - 1);
    const int n = fast_div(tile_c, a.div_ti), rem = tile_c - n * a.TI;
    const int ty = fast_div(rem, a.div_tw), tx = rem - ty * a.TW;
    const int oh = 2 * ty, ow = 2 * tx;
    const bool row1 = oh + 1 < a.OH, col1 = ow + 1 < a.OW;
    const bool vec2 = (a.OW & 1) == 0;
    const uint32_t y_bytes = static_cast<uint32_t>(a.N) * static_cast<uint32_t>(a.O) * static_cast<uint32_t>(a.OHW) * 4u;
    const uint32_t rowb = static_cast<uint32_t>(a.OW) * 4u;
    const uint32_t rowmask = row1 ? 0u : kOob, colmask = col1 ? 0u : kOob;   // OR-ed into an offset: beyond the buffer

    uint32_t off00[2][4], boff[2][4];
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int o = (kg * WK + wave_k) * 32 + kb * 16 + 4 * (lane >> 4) + g;
            const bool ok = tile < a.NT && o < a.O;
            off00[kb][g] = ok ? static_cast<uint32_t>(((n * a.O + o) * a.OH + oh) * a.OW + ow) * 4u : kOob;
            boff[kb][g] = ok ? static_cast<uint32_t>(o) * 4u : kOob;
        }
    // the four outputs of a tile from / to a tensor of the output's shape (also a part's raw outputs)
    // (aux: cache policy of the access, a compile-time constant passed as a type)
    auto load4 = [&](const __amdgpu_buffer_rsrc_t r, int kb, int g, float (&v)[4], auto aux) {
        constexpr int AUX = decltype(aux)::value;
        const uint32_t o0 = off00[kb][g], o1 = (o0 + rowb) | rowmask;
        auto ld = [&](uint32_t off) { return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, off, 0, AUX)); };
        // (two 4-byte loads per row: the 8-byte buffer-load builtin of this toolchain fetches only 4 bytes)
        v[0] = ld(o0);
        v[1] = ld((o0 + 4u) | colmask);      // (an even row length has no odd last column: the mask is 0)
        v[2] = ld(o1);
        v[3] = ld((o1 + 4u) | colmask);
    };
    using Cached = std::integral_constant<int, 0>;
    using DeviceScope = std::integral_constant<int, kDeviceScopeAux>;
    auto bits = [](float v) { return __builtin_bit_cast(uint32_t, v); };
    auto store_all = [&](const __amdgpu_buffer_rsrc_t yr, const float (&yv)[2][4][4], auto aux) {
        constexpr int AUX = decltype(aux)::value;
        if (vec2) {
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const uint32_t o0 = off00[kb][g], o1 = (o0 + rowb) | rowmask;
                    __builtin_amdgcn_raw_buffer_store_b64(uintx2{bits(yv[kb][g][0]), bits(yv[kb][g][1])}, yr, o0, 0, AUX);
                    __builtin_amdgcn_raw_buffer_store_b64(uintx2{bits(yv[kb][g][2]), bits(yv[kb][g][3])}, yr, o1, 0, AUX);
                }
        } else {
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const uint32_t o0 = off00[kb][g], o1 = (o0 + rowb) | rowmask;
                    __builtin_amdgcn_raw_buffer_store_b32(bits(yv[kb][g][0]), yr, o0, 0, AUX);
                    __builtin_amdgcn_raw_buffer_store_b32(bits(yv[kb][g][1]), yr, (o0 + 4u) | colmask, 0, AUX);
                    __builtin_amdgcn_raw_buffer_store_b32(bits(yv[kb][g][2]), yr, o1, 0, AUX);
                    __builtin_amdgcn_raw_buffer_store_b32(bits(yv[kb][g][3]), yr, (o1 + 4u) | colmask, 0, AUX);
                }
        }
    };
    // A^T M A with A^T = [1 1 1 0; 0 1 -1 -1]
    auto output_transform = [&](float (&yv)[2][4][4]) {
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                float r0[4], r1[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const float m0 = acc[j][kb][g], m1 = acc[4 + j][kb][g], m2 = acc[8 + j][kb][g], m3 = acc[12 + j][kb][g];
                    r0[j] = (m0 + m1) + m2;
                    r1[j] = (m1 - m2) - m3;
                }
                yv[kb][g][0] = (r0[0] + r0[1]) + r0[2]; yv[kb][g][1] = (r0[1] - r0[2]) - r0[3];
                yv[kb][g][2] = (r1[0] + r1[1]) + r1[2]; yv[kb][g][3] = (r1[1] - r1[2]) - r1[3];
            }
    };
    float bv[2][4];
    float q[2][4][4];
    // bias and residual of the layer's epilogue: issued early, used by finish()
    auto issue_epilogue_loads = [&](bool has_bias, bool has_res, const float* any) {
        const __amdgpu_buffer_rsrc_t rr = make_rsrc(has_res ? a.res : any, has_res ? y_bytes : 0u);
        const __amdgpu_buffer_rsrc_t br = make_rsrc(has_bias ? a.bias : any, has_bias ? static_cast<uint32_t>(a.O) * 4u : 0u);
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int g = 0; g < 4; ++g) bv[kb][g] = load_f32(br, boff[kb][g], 0);
        if (has_res) {
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int g = 0; g < 4; ++g) load4(rr, kb, g, q[kb][g], Cached{});
        }
    };
    auto finish = [&](float (&yv)[2][4][4], bool has_bias, bool has_res, bool do_relu) {
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int g = 0; g < 4; ++g)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float v = yv[kb][g][e];
                    if (has_bias) v = __fadd_rn(v, bv[kb][g]);
                    if (has_res) v = __fadd_rn(v, q[kb][g][e]);
                    if (do_relu) v = relu_sel(v);
                    yv[kb][g][e] = v;
                }
    };
    const bool has_bias = (a.flags & KXC_HIP_CONV_BIAS) != 0;
    const bool has_res = (a.flags & KXC_HIP_CONV_RESIDUAL) != 0;
    const bool do_relu = (a.flags & KXC_HIP_CONV_RELU) != 0;
    float yv[2][4][4];
    if (a.gsplit > 1) {
        // a part of a split reduction stores its raw output transform (the transform is linear)
        float* const part = a.partial + static_cast<int64_t>(split) * (y_bytes / 4u);
        output_transform(yv);
        if constexpr (FUSE) {
            // ... and the part that arrives last adds all of them in split order and finishes the layer; without
            // FUSE the adding kernel does.  Parts are stored and re-loaded at device scope (see kDeviceScopeAux).
            store_all(make_rsrc(part, y_bytes), yv, DeviceScope{});
            if (!split_arrive_last(a.counters + unit, a.gsplit, reinterpret_cast<uint32_t*>(lds))) return;
            issue_epilogue_loads(has_bias, has_res, a.y);
#pragma unroll 2
            for (int s = 0; s < a.gsplit; ++s) {
                const __amdgpu_buffer_rsrc_t pr = make_rsrc(a.partial + static_cast<int64_t>(s) * (y_bytes / 4u), y_bytes);
                float p[2][4][4];
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                    for (int g = 0; g < 4; ++g) load4(pr, kb, g, p[kb][g], DeviceScope{});
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                    for (int g = 0; g < 4; ++g)
#pragma unroll
                        for (int e = 0; e < 4; ++e) yv[kb][g][e] = s == 0 ? p[kb][g][e] : __fadd_rn(yv[kb][g][e], p[kb][g][e]);
            }
            finish(yv, has_bias, has_res, do_relu);
            store_all(make_rsrc(a.y, y_bytes), yv, Cached{});
        } else {
            store_all(make_rsrc(part, y_bytes), yv, Cached{});
        }
        return;
    }
    issue_epilogue_loads(false, has_res, a.y);          // (the bias came in through the accumulators)
    output_transform(yv);
    finish(yv, false, has_res, do_relu);
    store_all(make_rsrc(a.y, y_bytes), yv, Cached{});
}

struct WinoVariant {
    const char* name;
    int wk, wt, ks;
    void (*kernel)(const WinoArgs);
    void (*fuse_kernel)(const WinoArgs);      // the last part finishes a split reduction (nullptr: none)
};
#define KXC_WINO(WK, WT) {"winograd_f2k3_o" #WK "_t" #WT, WK, WT, 1, wino_kernel<WK, WT, 1>, wino_kernel<WK, WT, 1, true>}
#define KXC_WINO_KS2(WK, WT) {"winograd_f2k3_o" #WK "_t" #WT "_ks2", WK, WT, 2, wino_kernel<WK, WT, 2>, nullptr}
// name = winograd_f2k3_o<waves along output channels (32 each)>_t<waves along tiles (16 each)>[_ks2: input channels split over two groups of waves]
const WinoVariant kWino[] = {
    KXC_WINO(2, 2),   // 64 channels x 32 tiles, 4 waves, 48 KiB of LDS (default)
    KXC_WINO(2, 4),   // 64 x 64, 8 waves
    KXC_WINO(1, 4),   // 32 x 64, 4 waves
    KXC_WINO(2, 1),   // 64 x 16, 2 waves
    KXC_WINO(1, 2),   // 32 x 32, 2 waves
    KXC_WINO_KS2(2, 2),  // 64 x 32, input channels split over two groups of 4 waves (96 KiB of LDS)
    KXC_WINO_KS2(2, 1),  // 64 x 16, two groups of 2 waves
};
constexpr int kNumWino = sizeof(kWino) / sizeof(kWino[0]);

bool Supported(const kxc_hip_conv2d_desc* d) {
    if (!d || d->kh != 3 || d->kw != 3 || d->stride_h != 1 || d->stride_w != 1 || d->dil_h != 1 || d->dil_w != 1) return false;
    if (d->n <= 0 || d->c <= 0 || d->c % 4 != 0 || d->o <= 0 || d->h <= 0 || d->w <= 0) return false;
    if (d->flags & KXC_HIP_CONV_HPOOL) return false;      // the pooling epilogue exists in the direct-convolution kernels only
    // padding beyond the filter's reach only adds all-zero border tiles; cap it so the sizes below cannot overflow
    if (d->pad_h < 0 || d->pad_w < 0 || d->pad_h > (1 << 20) || d->pad_w > (1 << 20)) return false;
    const int64_t oh = static_cast<int64_t>(d->h) + 2 * d->pad_h - 2, ow = static_cast<int64_t>(d->w) + 2 * d->pad_w - 2;
    if (oh <= 0 || ow <= 0) return false;
    const int64_t x_bytes = static_cast<int64_t>(d->n) * d->c * d->h * d->w * 4;
    const int64_t y_elems = static_cast<int64_t>(d->n) * d->o * oh * ow;
    const int64_t u_bytes = CeilDiv(d->o, 32) * 32 * static_cast<int64_t>(d->c) * 64;
    const int64_t tiles = static_cast<int64_t>(d->n) * CeilDiv(oh, 2) * CeilDiv(ow, 2);
    return x_bytes < (1LL << 31) && y_elems * 4 < (1LL << 31) && u_bytes < (1LL << 31) && tiles < (1LL << 30);
}

int64_t Tiles(const kxc_hip_conv2d_desc* d) {
    const int64_t oh = static_cast<int64_t>(d->h) + 2 * d->pad_h - 2, ow = static_cast<int64_t>(d->w) + 2 * d->pad_w - 2;
    return static_cast<int64_t>(d->n) * CeilDiv(oh, 2) * CeilDiv(ow, 2);
}

// Launches that leave compute units idle split the input channels over workgroups: the number of parts for
// `units` 64 x 16 workgroups of `csteps` steps.  Two regimes, both measured on the ResNet-18 layers:
//  * tiny launches (batch 1-4): parts of at least four steps while all parts together stay below one workgroup
//    per compute unit (batch 1, 512 channels: 8 units -> 32 parts, 62.9 -> 14.7 us);
//  * up to 400 units (of the 512 workgroups the GPU holds at once) with a long reduction (64 steps and more; batch
//    8-32 of the 256- and 512-channel layers): parts of at least sixteen steps up to four workgroups per compute
//    unit, which is what fills every SIMD with two waves (batch 16, 512 channels: 128 units -> 8 parts, 55.7 -> 39.6
//    us; the split inside the workgroup: 66).  The bound was 256 units; 392 (the 256-channel layers at batch 64,
//    counting both shares of the batch) gain from two parts as well: ResNet-18 1.587 -> 1.574 ms at batch 64 in two
//    shares, 1.025 -> 1.014 at batch 32, no change in one share of 64 or at batch 128; a bound of 800 loses 4 %.
// The partial outputs (read back once by the adding kernel) stay below 16 MiB.
int GroupSplit(int64_t units, int csteps, int64_t out_elems) {
    int split = 1;
    while (split < 32) {
        const int next = split * 2;
        const int64_t groups = units * next;
        const int steps = csteps / next;
        const bool tiny = groups <= 256 && steps >= 4;
        const bool filling = units <= 400 && groups <= 1024 && csteps >= 64 && steps >= 16;
        if (!(tiny || filling)) break;
        if (out_elems * static_cast<int64_t>(sizeof(float)) * next > (16LL << 20)) break;
        split = next;
    }
    return split;
}

// Measured on MI355X: 64 x 32 workgroups (four waves) are the fastest shape once there is one per compute unit;
// smaller launches run faster as twice as many 64 x 16 workgroups of two waves.
const WinoVariant* SelectWino(const kxc_hip_conv2d_desc* d) {
    if (const char* e = std::getenv("KXC_HIP_WINOGRAD_VARIANT")) {
        for (int i = 0; i < kNumWino; ++i)
            if (std::strcmp(e, kWino[i].name) == 0 && (kWino[i].ks == 1 || (d->c / 4) % kWino[i].ks == 0)) return &kWino[i];
    }
    const int csteps = d->c / 4;
    const int64_t oh = static_cast<int64_t>(d->h) + 2 * d->pad_h - 2, ow = static_cast<int64_t>(d->w) + 2 * d->pad_w - 2;
    // Small launches (batch 1-8 of ResNet-18): 64 x 16 groups with the channels split over workgroups beat both
    // the split inside the workgroup and the implicit-GEMM kernel (batch 1, 512 channels: 14.7 against 62.9 and
    // 20.0 us).
    const int64_t lanes = SelectLanes();
    const int64_t units_t1 = CeilDiv(Tiles(d), 16) * CeilDiv(d->o, 64) * lanes;
    if (GroupSplit(units_t1, csteps, static_cast<int64_t>(d->n) * d->o * oh * ow) > 1) {
        for (int i = 0; i < kNumWino; ++i)
            if (kWino[i].wk == 2 && kWino[i].wt == 1 && kWino[i].ks == 1) return &kWino[i];
    }
    // 64 x 32 groups from one per compute unit on; below that twice as many 64 x 16 groups.  A launch that cannot
    // give every SIMD two waves (at most one 64 x 32 group per compute unit) and has a long reduction splits the
    // input channels over two groups of waves inside the workgroup instead.
    const int64_t units = CeilDiv(Tiles(d), 32) * CeilDiv(d->o, 64) * lanes;
    const int wt = units < 256 ? 1 : 2;
    const int ks = (units <= 256 && csteps % 2 == 0 && csteps >= 32) ? 2 : 1;
    for (int i = 0; i < kNumWino; ++i)
        if (kWino[i].wk == 2 && kWino[i].wt == wt && kWino[i].ks == ks) return &kWino[i];
    return &kWino[0];
}

// What the descriptor alone decides about a launch (variant, grid, the split over workgroups, the switches read
// from the environment): resolved once per call by the entry point, once per node by a launch plan.
struct WinoLaunch {
    const WinoVariant* v = nullptr;
    WinoArgs a;                 // without operand pointers, partial outputs and counters
    int64_t out_elems = 0;
    size_t scratch_bytes = 0;   // partial outputs of a split over workgroups (0: none)
    size_t lds_bytes = 0;
    bool fuse = false;          // the part that arrives last adds the parts: no adding kernel
};

int32_t WinoResolve(const kxc_hip_conv2d_desc* desc, WinoLaunch* L) {
    KXC_HIP_REQUIRE(desc && Supported(desc), "kxc_hip_conv2d_winograd_nchw_f32: unsupported shape");
    const WinoVariant* v = SelectWino(desc);
    L->v = v;
    WinoArgs& a = L->a;
    std::memset(&a, 0, sizeof(a));
    a.N = static_cast<int32_t>(desc->n); a.C = static_cast<int32_t>(desc->c); a.H = static_cast<int32_t>(desc->h);
    a.W = static_cast<int32_t>(desc->w); a.O = static_cast<int32_t>(desc->o);
    a.ph = static_cast<int32_t>(desc->pad_h); a.pw = static_cast<int32_t>(desc->pad_w);
    a.OH = a.H + 2 * a.ph - 2; a.OW = a.W + 2 * a.pw - 2;
    a.TW = (a.OW + 1) / 2;
    a.TI = ((a.OH + 1) / 2) * a.TW;
    a.NT = a.N * a.TI;
    a.HW = a.H * a.W; a.OHW = a.OH * a.OW;
    a.csteps = a.C / 4;
    a.x_bytes = static_cast<uint32_t>(static_cast<int64_t>(a.N) * a.C * a.HW * 4);
    a.u_bytes = static_cast<uint32_t>(CeilDiv(a.O, 32) * 32 * static_cast<int64_t>(a.C) * 64);
    a.flags = desc->flags;
    a.t_groups = static_cast<int32_t>(CeilDiv(a.NT, 16 * v->wt));
    a.k_groups = static_cast<int32_t>(CeilDiv(a.O, 32 * v->wk));
    a.num_units = a.t_groups * a.k_groups;
    // Small launches split the input channels over workgroups (GroupSplit): each part writes its raw output
    // transform (the transform is linear) to a scratch buffer, and a second kernel adds the parts in order and
    // applies the epilogue.
    a.gsplit = 1;
    a.steps_per_split = a.csteps;
    const int64_t out_elems = static_cast<int64_t>(a.N) * a.O * a.OHW;
    L->out_elems = out_elems;
    if (v->ks == 1) {
        int split = GroupSplit(static_cast<int64_t>(a.num_units) * SelectLanes(), a.csteps, out_elems);
        if (const char* e = std::getenv("KXC_HIP_WINOGRAD_GSPLIT")) {
            // (a forced split is honoured while its partial outputs stay below 256 MiB)
            const int f = std::atoi(e);
            if (f >= 1 && f <= a.csteps && out_elems * static_cast<int64_t>(sizeof(float)) * f <= (256LL << 20)) split = f;
        }
        if (split > 1) {
            a.steps_per_split = static_cast<int32_t>(CeilDiv(a.csteps, split));
            a.gsplit = static_cast<int32_t>(CeilDiv(a.csteps, a.steps_per_split));      // no empty part
            if (a.gsplit > 1) {
                L->scratch_bytes = static_cast<size_t>(a.gsplit) * out_elems * sizeof(float);
                L->fuse = v->fuse_kernel && a.gsplit <= SplitFuseMaxParts() && a.num_units <= kSplitCounters;
            } else {
                a.steps_per_split = a.csteps;
            }
        }
    }
    a.div_gsplit = MakeFastDiv(a.gsplit);
    a.units_per_xcd = static_cast<int32_t>(CeilDiv(static_cast<int64_t>(a.num_units) * a.gsplit, 8));
    // transformed weights of all output channels small next to an L2: neighbouring units share the input tile
    a.k_fastest = a.u_bytes <= (2u << 20) ? 1 : 0;
    if (const char* e = std::getenv("KXC_HIP_WINOGRAD_KFAST")) a.k_fastest = std::atoi(e);
    a.div_ti = MakeFastDiv(a.TI); a.div_tw = MakeFastDiv(a.TW);
    a.div_kgroups = MakeFastDiv(a.k_groups); a.div_tgroups = MakeFastDiv(a.t_groups);
    L->lds_bytes = v->ks * 2 * static_cast<size_t>(2048 * v->wk + 1024 * v->wt) * sizeof(float);
    return KXC_HIP_OK;
}

int32_t WinoRun(const WinoLaunch& L, const float* x, const float* u, const float* bias, const float* residual, float* y,
                hipStream_t s) {
    const WinoVariant* v = L.v;
    KXC_HIP_REQUIRE(x && u && y, "kxc_hip_conv2d_winograd_nchw_f32: NULL pointer");
    KXC_HIP_REQUIRE(!(L.a.flags & KXC_HIP_CONV_BIAS) || bias, "kxc_hip_conv2d_winograd_nchw_f32: bias flag without bias");
    KXC_HIP_REQUIRE(!(L.a.flags & KXC_HIP_CONV_RESIDUAL) || residual,
                    "kxc_hip_conv2d_winograd_nchw_f32: residual flag without residual");
    WinoArgs a = L.a;
    a.x = x; a.u = u; a.bias = bias; a.res = residual; a.y = y;
    SplitScratchLease lease;      // held until the adding kernel is enqueued
    if (L.scratch_bytes > 0) {
        if (int32_t rc = AcquireSplitScratch(s, L.scratch_bytes, &lease)) return rc;
        a.partial = lease.ptr;
        a.counters = lease.counters;
    }
    void (*const kernel)(const WinoArgs) = L.fuse ? v->fuse_kernel : v->kernel;
    if (L.lds_bytes > 64 * 1024) {
        // above the default 64 KiB the dynamic LDS size has to be granted per kernel and device (once)
        static std::mutex mu;
        static std::vector<std::pair<int, const void*>> granted;
        int dev = 0;
        KXC_HIP_CALL(hipGetDevice(&dev), "hipGetDevice");
        const void* fn = reinterpret_cast<const void*>(kernel);
        std::lock_guard<std::mutex> lock(mu);
        bool have = false;
        for (const auto& g : granted) have = have || (g.first == dev && g.second == fn);
        if (!have) {
            KXC_HIP_CALL(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(L.lds_bytes)),
                         "hipFuncSetAttribute(MaxDynamicSharedMemorySize)");
            granted.emplace_back(dev, fn);
        }
    }
    hipLaunchKernelGGL(kernel, NoteGrid(dim3(static_cast<unsigned>(a.units_per_xcd * 8))),
                       NoteBlock(dim3(64 * v->wk * v->wt * v->ks)), NoteLds(L.lds_bytes), s, a);
    if (int32_t rc = CheckLaunch(v->name)) return rc;
    if (a.gsplit > 1 && !L.fuse) {
        SplitReduceArgs r;
        r.partial = a.partial; r.bias = bias; r.res = residual; r.y = y;
        r.gsplit = a.gsplit; r.total = static_cast<int32_t>(L.out_elems); r.O = a.O; r.flags = a.flags;
        r.div_ohw = MakeFastDiv(a.OHW);
        return LaunchSplitReduce(s, r);
    }
    return KXC_HIP_OK;
}

}  // namespace

namespace kxc_hip {

struct PreparedWinograd {
    WinoLaunch launch;
};

int32_t PrepareWinograd(const kxc_hip_conv2d_desc* desc, PreparedWinograd** out) {
    PreparedWinograd* p = new PreparedWinograd;
    if (int32_t rc = WinoResolve(desc, &p->launch)) { delete p; return rc; }
    *out = p;
    return KXC_HIP_OK;
}

int32_t LaunchPreparedWinograd(const PreparedWinograd* p, const float* x, const float* u, const float* bias,
                               const float* residual, float* y, hipStream_t stream) {
    return WinoRun(p->launch, x, u, bias, residual, y, stream);
}

void FreePreparedWinograd(PreparedWinograd* p) { delete p; }

int32_t LaunchWinogradWeightTransforms(const WinoWeightJob* jobs, int32_t count, hipStream_t stream) {
    for (int32_t base = 0; base < count; base += kMaxWeightJobs) {
        WinoWeightBatch b;
        std::memset(&b, 0, sizeof(b));
        b.count = std::min<int32_t>(kMaxWeightJobs, count - base);
        int64_t blocks = 0;
        for (int32_t j = 0; j < b.count; ++j) {
            const WinoWeightJob& job = jobs[base + j];
            KXC_HIP_REQUIRE(job.desc && Supported(job.desc) && job.w && job.u, "winograd weight transform: bad job %d", base + j);
            b.w[j] = job.w; b.u[j] = job.u;
            b.O[j] = job.desc->o; b.C[j] = job.desc->c;
            b.first_block[j] = static_cast<int32_t>(blocks);
            blocks += WeightTiles(CeilDiv(job.desc->o, 32) * 32, job.desc->c);
            KXC_HIP_REQUIRE(blocks < kMaxGridX, "winograd weight transform: too many blocks");
        }
        b.first_block[b.count] = static_cast<int32_t>(blocks);
        wino_weight_batch_kernel<<<NoteGrid(static_cast<int>(blocks)), NoteBlock(256), NoteLds(0), stream>>>(b);
        if (int32_t rc = CheckLaunch("wino_weight_batch_kernel")) return rc;
    }
    return KXC_HIP_OK;
}

}  // namespace kxc_hip

extern "C" {

int32_t kxc_hip_conv2d_winograd_supported(const kxc_hip_conv2d_desc* desc) { return Supported(desc) ? 1 : 0; }

int32_t kxc_hip_conv2d_winograd_preferred(const kxc_hip_conv2d_desc* desc) {
    if (!Supported(desc)) return 0;
    // Measured against the implicit-GEMM kernel on the ResNet-18 layers from batch 1 to 64: faster or equal
    // everywhere once small launches split their channels over workgroups, so every supported shape takes it.
    // KXC_HIP_WINOGRAD_MIN_WORK = f restricts it to tiles * o >= f * c.
    int64_t factor = 0;
    if (const char* e = std::getenv("KXC_HIP_WINOGRAD_MIN_WORK")) factor = std::atoll(e);
    return Tiles(desc) * desc->o >= factor * desc->c ? 1 : 0;
}

const char* kxc_hip_conv2d_winograd_variant(const kxc_hip_conv2d_desc* desc) {
    return Supported(desc) ? SelectWino(desc)->name : "unsupported";
}

int32_t kxc_hip_conv2d_winograd_weight_bytes(const kxc_hip_conv2d_desc* desc, size_t* out_bytes) {
    KXC_HIP_REQUIRE(desc && out_bytes, "kxc_hip_conv2d_winograd_weight_bytes: NULL argument");
    KXC_HIP_REQUIRE(Supported(desc), "kxc_hip_conv2d_winograd_weight_bytes: shape is not a 3x3 stride-1 convolution with C %% 4 == 0");
    *out_bytes = static_cast<size_t>(CeilDiv(desc->o, 32)) * 32 * static_cast<size_t>(desc->c) * 16 * sizeof(float);
    return KXC_HIP_OK;
}

int32_t kxc_hip_conv2d_winograd_transform_weights(const kxc_hip_conv2d_desc* desc, const float* w, float* u, void* stream) {
    KXC_HIP_REQUIRE(desc && Supported(desc), "kxc_hip_conv2d_winograd_transform_weights: unsupported shape");
    KXC_HIP_REQUIRE(w && u, "kxc_hip_conv2d_winograd_transform_weights: NULL pointer");
    const int64_t tiles = WeightTiles(CeilDiv(desc->o, 32) * 32, desc->c);
    KXC_HIP_REQUIRE(tiles < kMaxGridX, "kxc_hip_conv2d_winograd_transform_weights: too many blocks");
    wino_weight_kernel<<<NoteGrid(static_cast<int>(tiles)), NoteBlock(256), NoteLds(0), ResolveStream(stream)>>>(
        w, u, static_cast<int32_t>(desc->o), static_cast<int32_t>(desc->c));
    return CheckLaunch("wino_weight_kernel");
}

int32_t kxc_hip_conv2d_winograd_nchw_f32(const kxc_hip_conv2d_desc* desc, const float* x, const float* u, const float* bias,
                                         const float* residual, float* y, void* stream) {
    WinoLaunch L;
    if (int32_t rc = WinoResolve(desc, &L)) return rc;
    return WinoRun(L, x, u, bias, residual, y, ResolveStream(stream));
}

}  // extern "C"
