// qconv_c16_i8.hip -- int8 convolution on the gfx950 int8 matrix cores (v_mfma_i32_32x32x32_i8), with the
// operators around it, on a channel-blocked activation layout.
//
// Layout "c16": an int8 activation of logical shape [N, C, H, W] is stored as [N][CB][H][W][16] with
// CB = ceil(C/16); element (n, c, h, w) lives at (((n*CB + c/16)*H + h)*W + w)*16 + c%16 and the bytes
// of channels >= C are zero.  One pixel's 16 channels are one 16-byte word: exactly the k-slice one lane
// feeds to the 32x32x32 matrix instruction, so a filter tap is ONE aligned ds_read_b128 per lane and no
// byte gather or transpose exists anywhere.  The reference compiler has no int8 operator, so there is no
// external layout to match; the NCHW entry points remain for interchange, with converters below.
//
// Arithmetic (identical to the NCHW kernel and the CPU definition):
//   acc = sum x*w in int32 (exact, order free) [+ bias[o]];  v = (float)acc * mult[o];
//   [v = v + (float)res * res_mult];  y = clamp(rint_half_even(v), relu ? 0 : -128, 127).
//
// Kernel structure: D[o][pixel] += W[o][k] * X[k][pixel]; pixels are flattened over (n, oh, ow).  A
// workgroup of WP waves owns 32*RO output channels by 32*WP consecutive pixels; every wave computes RO
// 32x32 blocks that share one pixel operand.  Per chunk of CBC channel blocks the workgroup stages in LDS
//   * the input rows its pixels touch, in "padded row space" Q = n*(H+2*pad) + ih + pad, as 16-byte
//     positions patch[cb][Q - Qmin][col + pad]  (zero padding comes from the buffer descriptor's
//     out-of-range rule, so it costs nothing), and
//   * the weights, which the host has pre-packed in exactly the order the lanes read them
//     ([o block][chunk][k-step][lane][16 bytes]), so the copy is linear.
// Both are written by LDS-direct buffer loads of 16 bytes per lane and double buffered.
// A k-step is 32 reduction values: lane half h takes linear index q = 2*step + h of the chunk's
// (tap, channel block) pairs, q = tap*CBC + cb_local; indices past the end carry zero weights.
#include <cstdlib>
#include <cstring>
#include <type_traits>
#include <vector>

#include "common.h"

using namespace kxc_hip;

namespace {

typedef int intx4 __attribute__((ext_vector_type(4)));
typedef int intx16 __attribute__((ext_vector_type(16)));
typedef __attribute__((address_space(3))) void* lds_ptr_t;

constexpr uint32_t kOob = 0x80000000u;
constexpr int kBlock = 256;

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

__device__ __forceinline__ int32_t requant_i32(int32_t acc, float mult, bool has_res, int32_t res, float res_mult,
                                               bool relu) {
    float v = __fmul_rn(static_cast<float>(acc), mult);
    if (has_res) v = __fadd_rn(v, __fmul_rn(static_cast<float>(res), res_mult));
    float r = rintf(v);
    r = (v == v) ? r : 0.0f;
    r = fminf(fmaxf(r, relu ? 0.0f : -128.0f), 127.0f);
    return static_cast<int32_t>(r);
}

struct QArgs {
    const int8_t* x;
    const int8_t* wp;
    const int32_t* bias;
    const float* mult;
    const int8_t* res;
    int8_t* y;
    int32_t N, CB, H, W, O, OH, OW;
    int32_t sh, sw, ph, pw;
    int32_t Hp, Wp, M, OHW;
    int32_t chs;          // 16-byte positions per channel block plane in LDS (multiple of 64)
    int32_t nchunks;
    uint32_t x_bytes, w_bytes;
    int32_t p_tiles, o_tiles, num_tiles, tiles_per_xcd;
    float res_mult;
    uint32_t flags;
    FastDiv div_wp, div_hp, div_ohw, div_ow, div_otiles;   // div_wp: positions per LDS row (pixels, or pixel quads on c4)
    // Second output of the DS kernels: a 1x1 convolution with the same strides and no padding on the same input
    // (a residual block's downsample beside the block's first 3x3 convolution).  Its operand x[n, c, oh*sh, ow*sw] is
    // the tap (rh, rw) = (pad_h, pad_w) of this convolution's window, which the staged patch already holds at byte
    // offset ds_off; wp2 is packed like wp with one tap ([o block][chunk][k-step][lane][16]); bias + requantise, no ReLU.
    const int8_t* wp2;
    const int32_t* bias2;
    const float* mult2;
    int8_t* y2;
    uint32_t w2_bytes;
    int32_t ds_off;
    // First layer with the 3x3 / stride-2 / padding-1 max pool behind it in the same kernel (qconv_k7s2_c4_pool_kernel):
    // pooled extents, pooled rows per workgroup, workgroups per image
    int32_t POH, PW, pool_rows, pool_tiles;
    FastDiv div_pool_tiles;
};

typedef unsigned int uintx2 __attribute__((ext_vector_type(2)));
typedef unsigned int uintx4 __attribute__((ext_vector_type(4)));

// v_permlane32_swap: a's lanes 32-63 change places with b's lanes 0-31 (gfx950).  The host pass of the compiler
// does not know the instruction and sees an empty body.
__device__ __forceinline__ void swap_halves(uint32_t& a, uint32_t& b) {
#if defined(__HIP_DEVICE_COMPILE__)
    const uintx2 r = __builtin_amdgcn_permlane32_swap(a, b, false, false);
    a = r[0]; b = r[1];
#endif
}

// Accumulator register g of a 32x32 block is output channel 8*(g/4) + 4*half + g%4 (within the block of 32) at the
// lane's pixel: registers 4j..4j+3 ("group j") are four consecutive channels = one dword of the pixel's c16 word.
// The accumulators START at the bias (int32 addition wraps the same way in any order), so the epilogue has no add.
template <int RO>
__device__ __forceinline__ void init_acc_with_bias(intx16 (&acc)[RO], const int32_t* bias, bool has_bias, int32_t O, int ob0, int half) {
#pragma unroll
    for (int i = 0; i < RO; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            int4 b = make_int4(0, 0, 0, 0);
            if (has_bias) b = *reinterpret_cast<const int4*>(bias + (ob0 + i) * 32 + 8 * j + 4 * half);
            acc[i][4 * j + 0] = b.x; acc[i][4 * j + 1] = b.y; acc[i][4 * j + 2] = b.z; acc[i][4 * j + 3] = b.w;
        }
}

// Epilogue shared by the matrix-core kernels: requantise RP x RO blocks whose accumulators already hold the bias.
// These kernels are bound by instruction issue around the (very fast) int8 matrix instructions, so it is kept short:
//  * rounding and conversion are one addition: v + 1.5*2^23 rounds v to an integer (ties to even) and leaves its two's
//    complement in the low mantissa bits, so after the clamp (one median instruction; with ReLU its lower bound 0 is
//    also what a NaN maps to, without ReLU a NaN is replaced by 0 first) the low byte of the sum IS the int8 result;
//  * four results are packed with three byte permutes, and two lane-half swaps per block turn the four packed dwords
//    of a lane (channel groups 0, 2, 4, 6 or 1, 3, 5, 7 of the block) into the 16 consecutive channels of one c16
//    word: lane r stores channels 0-15 and lane r + 32 channels 16-31 of pixel r with ONE 16-byte store each (and
//    reads the residual with one 16-byte load) instead of four 4-byte ones;
//  * the multipliers are loaded once for all pixel blocks of the wave, and every load is issued before the first
//    store (a wait for a load also waits for every store issued before it).
// ypix[j] = n*(O/16)*OHW + pixel index of the lane's pixel in block j, or -1 past the end.
template <int RO, int RP>
__device__ __forceinline__ void epilogue_c16(const intx16 (&acc)[RP][RO], const QArgs& a, const int (&ypix)[RP], int ob0, int half) {
    const bool has_res = (a.flags & KXC_HIP_CONV_RESIDUAL) != 0;
    const bool do_relu = (a.flags & KXC_HIP_CONV_RELU) != 0;
    // this lane's c16 word of block (i, j): channels (ob0 + i)*32 + 16*half .. + 15
    auto word = [&](int i, int j) {
        return (static_cast<int64_t>(ypix[j]) + static_cast<int64_t>((ob0 + i) * 2 + half) * a.OHW) * 16;
    };
    float4 mv[RO][4];
#pragma unroll
    for (int i = 0; i < RO; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            // (output channels are a multiple of 32: every block is whole)
            mv[i][j] = *reinterpret_cast<const float4*>(a.mult + (ob0 + i) * 32 + 8 * j + 4 * half);
        }
    // residual words, brought from "16 consecutive channels per lane" to the accumulators' channel groups
    uint32_t resw[RP][RO][4];
    if (has_res) {
#pragma unroll
        for (int j = 0; j < RP; ++j)
#pragma unroll
            for (int i = 0; i < RO; ++i) {
                uintx4 q = {0u, 0u, 0u, 0u};
                if (ypix[j] >= 0) q = *reinterpret_cast<const uintx4*>(a.res + word(i, j));
                uint32_t q0 = q[0], q1 = q[1], q2 = q[2], q3 = q[3];
                swap_halves(q0, q1);      // (the inverse of the stores' swaps below)
                swap_halves(q2, q3);
                resw[j][i][0] = q0; resw[j][i][2] = q1; resw[j][i][1] = q2; resw[j][i][3] = q3;
            }
    }
    auto finish = [&](auto relu_c, auto res_c) {
        constexpr bool kRelu = decltype(relu_c)::value, kRes = decltype(res_c)::value;
        constexpr float kMagic = 12582912.0f;      // 1.5 * 2^23
#pragma unroll
        for (int j = 0; j < RP; ++j)
#pragma unroll
            for (int i = 0; i < RO; ++i) {
                uint32_t w[4];
#pragma unroll
                for (int gq = 0; gq < 4; ++gq) {
                    const float ms[4] = {mv[i][gq].x, mv[i][gq].y, mv[i][gq].z, mv[i][gq].w};
                    uint32_t t[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        float v = __fmul_rn(static_cast<float>(acc[j][i][4 * gq + e]), ms[e]);
                        if (kRes) {
                            const int32_t rq = static_cast<int32_t>(static_cast<int8_t>((resw[j][i][gq] >> (8 * e)) & 0xff));
                            v = __fadd_rn(v, __fmul_rn(static_cast<float>(rq), a.res_mult));
                        }
                        if (!kRelu) v = (v == v) ? v : 0.0f;
                        v = __builtin_amdgcn_fmed3f(v, kRelu ? 0.0f : -128.0f, 127.0f);
                        t[e] = __builtin_bit_cast(uint32_t, __fadd_rn(v, kMagic));
                    }
                    const uint32_t lo = __builtin_amdgcn_perm(t[1], t[0], 0x0c0c0400u);
                    const uint32_t hi = __builtin_amdgcn_perm(t[3], t[2], 0x0c0c0400u);
                    w[gq] = __builtin_amdgcn_perm(hi, lo, 0x05040100u);
                }
                // lane half 0 holds channel groups 0, 2, 4, 6 (channels 0-3, 8-11, 16-19, 24-27), half 1 the odd ones:
                // after the swaps half 0 has channels 0-15 as (w0, w2, w1, w3) and half 1 channels 16-31 likewise
                swap_halves(w[0], w[2]);
                swap_halves(w[1], w[3]);
                if (ypix[j] >= 0) *reinterpret_cast<uintx4*>(a.y + word(i, j)) = uintx4{w[0], w[2], w[1], w[3]};
            }
    };
    using T = std::true_type;
    using F = std::false_type;
    if (do_relu) { if (has_res) finish(T{}, T{}); else finish(T{}, F{}); }
    else { if (has_res) finish(F{}, T{}); else finish(F{}, F{}); }
}

// RP: 32-pixel blocks per wave (a wave computes RO x RP blocks; a weight operand then feeds RP matrix
// instructions and a pixel operand RO of them).  These kernels are bound by the latency chain of a workgroup
// (set-up, first loads, one weight fetch per k-step, epilogue), not by the matrix pipe, so a launch runs fastest
// when all its waves are resident at once: larger per-wave tiles trade idle matrix cycles for fewer waves.
// WD: depth of the weight ring in k-steps (must divide the k-steps of a chunk).
// DS: the workgroup also produces the second output described in QArgs: per chunk (CBC + 1) / 2 more k-steps that read
// the window's tap at ds_off against the second packed weights, into a second set of accumulators.
template <int KH, int KW, int CBC, int WP, int RO, int PPT, int RP = 1, int WD = 0, bool DS = false>
__global__ void __launch_bounds__(64 * WP) __attribute__((amdgpu_waves_per_eu(2))) qconv_mfma_kernel(const QArgs a) {
    constexpr int KHW = KH * KW;
    constexpr int NS = (KHW * CBC + 1) / 2;          // matrix k-steps per chunk
    constexpr int NS2 = DS ? (CBC + 1) / 2 : 0;      // ... of the second output
    constexpr int TP = 32 * WP * RP;

    extern __shared__ __attribute__((aligned(16))) char lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int half = lane >> 5;
    const int r = lane & 31;

    const int xs_bytes = CBC * a.chs * 16;
    const int buf_bytes = xs_bytes;
    char* const buf0 = lds;
    char* const buf1 = lds + buf_bytes;              // present only when nchunks > 1

    // consecutive workgroups go to the 8 XCDs round-robin; give every XCD (own L2) a contiguous run of tiles
    const int tile = (blockIdx.x & 7) * a.tiles_per_xcd + (blockIdx.x >> 3);
    if (tile >= a.num_tiles || static_cast<int>(blockIdx.x >> 3) >= a.tiles_per_xcd) return;
    const int p_tile = fast_div(tile, a.div_otiles), o_tile = tile - p_tile * a.o_tiles;
    const int m0 = p_tile * TP;
    const int ob0 = o_tile * RO;                     // first 32-channel output block

    const int m_last = min(m0 + TP, a.M) - 1;
    int qmin, qlast;
    {
        const int n = fast_div(m0, a.div_ohw), rem = m0 - n * a.OHW;
        qmin = n * a.Hp + fast_div(rem, a.div_ow) * a.sh;
        const int n2 = fast_div(m_last, a.div_ohw), rem2 = m_last - n2 * a.OHW;
        qlast = n2 * a.Hp + fast_div(rem2, a.div_ow) * a.sh + (KH - 1);
    }
    const int P = (qlast - qmin + 1) * a.Wp;         // positions per plane (<= chs)
    const int xsegs = (P + 63) >> 6;
    const uint32_t plane_bytes = static_cast<uint32_t>(a.H) * a.W * 16u;

    const __amdgpu_buffer_rsrc_t xr = make_rsrc(a.x, a.x_bytes);
    const __amdgpu_buffer_rsrc_t wr = make_rsrc(a.wp, a.w_bytes);

    uint32_t goff[PPT];
#pragma unroll
    for (int i = 0; i < PPT; ++i) {
        const int pos = (wave + i * WP) * 64 + lane;
        const int q = fast_div(pos, a.div_wp), col = pos - q * a.Wp;
        const int Q = qmin + q;
        const int n = fast_div(Q, a.div_hp), ih = Q - n * a.Hp - a.ph, iw = col - a.pw;
        const bool ok = pos < P && n < a.N && ih >= 0 && ih < a.H && iw >= 0 && iw < a.W;
        goff[i] = ok ? (static_cast<uint32_t>(n) * a.CB * a.H * a.W + static_cast<uint32_t>(ih * a.W + iw)) * 16u : kOob;
    }

    // per-lane operand bases: byte address of each pixel's (tap 0, channel block 0) position
    int xbase[RP];
    int ypix[RP];        // position index (n*OB16*OHW + pixel) of this lane's output pixel for block 0, or -1
#pragma unroll
    for (int j = 0; j < RP; ++j) {
        const int m = m0 + (wave * RP + j) * 32 + r;
        const int mc = min(m, a.M - 1);
        const int n = fast_div(mc, a.div_ohw), rem = mc - n * a.OHW;
        const int oh = fast_div(rem, a.div_ow), ow = rem - oh * a.OW;
        xbase[j] = ((n * a.Hp + oh * a.sh - qmin) * a.Wp + ow * a.sw) * 16;
        if (CBC > 1) xbase[j] += half * a.chs * 16;
        ypix[j] = (m < a.M) ? n * (a.O >> 4) * a.OHW + rem : -1;
    }

    intx16 acc[RP][RO];
#pragma unroll
    for (int j = 0; j < RP; ++j) init_acc_with_bias<RO>(acc[j], a.bias, (a.flags & KXC_HIP_CONV_BIAS) != 0, a.O, ob0, half);

    auto issue_loads = [&](int chunk, char* buf) {
#pragma unroll
        for (int cl = 0; cl < CBC; ++cl) {
            const int cb = chunk * CBC + cl;
            if (cb < a.CB) {
                const uint32_t soff = static_cast<uint32_t>(cb) * plane_bytes;
#pragma unroll
                for (int i = 0; i < PPT; ++i) {
                    const int seg = wave + i * WP;
                    if (seg < xsegs)
                        load16_to_lds(xr, (lds_ptr_t)(buf + (cl * a.chs + seg * 64) * 16), goff[i], soff);
                }
            }   // a missing channel block keeps stale bytes; its packed weights are zero and integers have no NaN
        }
        __builtin_amdgcn_sched_barrier(0);
        asm volatile("" ::: "memory");      // the weight loads below stay behind these in program order
    };

    // Weights do not pass through LDS: the packed layout [o block][chunk][k-step][lane][16] makes a wave's
    // operand for linear step t = chunk*NS + step ONE contiguous 1 KiB load, shared by the workgroup's waves
    // through the vector cache.  A ring of D steps is kept in flight across chunk boundaries; loads past the
    // last step fall outside the buffer and return 0 without a branch.  With the weights out of LDS a workgroup
    // needs only the patch (12 KiB per buffer for a 56-wide map), which triples the resident workgroups per CU.
    constexpr int D = WD > 0 ? WD : ((NS % 3 == 0) ? 3 : (NS % 5 == 0 ? 5 : (NS % 2 == 0 ? 2 : 1)));
    static_assert(NS % D == 0, "the weight ring must divide the k-steps of a chunk");
    const uint32_t total_steps = static_cast<uint32_t>(a.nchunks) * NS;
    uint32_t wvoff[RO];
#pragma unroll
    for (int i = 0; i < RO; ++i) wvoff[i] = static_cast<uint32_t>(ob0 + i) * total_steps * 1024u + static_cast<uint32_t>(lane) * 16u;
    // (the step index is uniform: it goes into the instruction's scalar offset, clamped to the last step -- a ring
    // entry past the end is never used -- which costs two scalar instructions per load and no vector one)
    auto load_a = [&](int i, uint32_t t) -> intx4 {
        const uint32_t tc = t < total_steps ? t : total_steps - 1u;
        return __builtin_amdgcn_raw_buffer_load_b128(wr, wvoff[i], tc * 1024u, 0);
    };
    intx4 ring[D][RO];
    // second output: its few weight fragments of a chunk are requested at the top of the chunk
    const __amdgpu_buffer_rsrc_t wr2 = make_rsrc(DS ? a.wp2 : a.wp, DS ? a.w2_bytes : 0u);
    intx16 acc2[DS ? RP : 1][DS ? RO : 1];
    if constexpr (DS) {
#pragma unroll
        for (int j = 0; j < RP; ++j) init_acc_with_bias<RO>(acc2[j], a.bias2, a.bias2 != nullptr, a.O, ob0, half);
    }

    issue_loads(0, buf0);
#pragma unroll
    for (int d = 0; d < D; ++d)
#pragma unroll
        for (int i = 0; i < RO; ++i) ring[d][i] = load_a(i, d);
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(D * RO) : "memory");     // the patch has landed, the ring may still fly
    __syncthreads();

    for (int chunk = 0; chunk < a.nchunks; ++chunk) {
        const char* buf = (chunk & 1) ? buf1 : buf0;
        intx4 a2[DS ? NS2 : 1][RO];
        if constexpr (DS) {
#pragma unroll
            for (int s2 = 0; s2 < NS2; ++s2)
#pragma unroll
                for (int i = 0; i < RO; ++i)
                    a2[s2][i] = __builtin_amdgcn_raw_buffer_load_b128(
                        wr2, (static_cast<uint32_t>(ob0 + i) * static_cast<uint32_t>(a.nchunks) * NS2 + static_cast<uint32_t>(chunk) * NS2 + s2) * 1024u +
                                 static_cast<uint32_t>(lane) * 16u, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            asm volatile("" ::: "memory");      // ahead of the next patch's loads in program order
        }
        if (chunk + 1 < a.nchunks) issue_loads(chunk + 1, (chunk & 1) ? buf0 : buf1);
        auto tap_off = [&](int tap) {
            const int t = tap < KHW ? tap : KHW - 1;
            const int rh = t / KW, rw = t - rh * KW;
            return (rh * a.Wp + rw) * 16;
        };
        auto fetch_b = [&](int step, intx4 (&b)[RP]) {
            int off;
            if constexpr (CBC == 1) {
                off = half ? tap_off(2 * step + 1) : tap_off(2 * step);
            } else {
                constexpr int H2 = CBC / 2;
                off = tap_off(step / H2) + 2 * (step % H2) * a.chs * 16;
            }
#pragma unroll
            for (int j = 0; j < RP; ++j) b[j] = *reinterpret_cast<const intx4*>(buf + xbase[j] + off);
        };
        const uint32_t t0 = static_cast<uint32_t>(chunk) * NS;
        // Pixel operands are read DB k-steps ahead.  With several pixel blocks per wave every step ends in a scheduling
        // barrier: left free, the compiler gathers the LDS reads of many steps ahead of their matrix instructions and the
        // wave then waits for all of them at once (256 -> 256 channels at 14 x 14, batch 64: 12.4 -> 11.6 us; with one
        // pixel block per wave the barrier changes nothing or costs 1-2 %, so those variants stay as they were).
        constexpr int DB = RP >= 2 ? 2 : 1;
        intx4 bring[DB][RP];
#pragma unroll
        for (int s0 = 0; s0 < DB; ++s0) fetch_b(s0, bring[s0]);
#pragma unroll
        for (int step = 0; step < NS; ++step) {
#pragma unroll
            for (int j = 0; j < RP; ++j)
#pragma unroll
                for (int i = 0; i < RO; ++i)
                    acc[j][i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(ring[step % D][i], bring[step % DB][j], acc[j][i], 0, 0, 0);
#pragma unroll
            for (int i = 0; i < RO; ++i) ring[step % D][i] = load_a(i, t0 + step + D);
            if (step + DB < NS) fetch_b(step + DB, bring[step % DB]);
            if constexpr (RP >= 2) __builtin_amdgcn_sched_barrier(0);
        }
        if constexpr (DS) {
            // lane half h takes channel block 2*s2 + h of the chunk at the second output's tap
#pragma unroll
            for (int s2 = 0; s2 < NS2; ++s2) {
                const int off = a.ds_off + (CBC > 1 ? 2 * s2 * a.chs * 16 : 0);
#pragma unroll
                for (int j = 0; j < RP; ++j) {
                    const intx4 b2 = *reinterpret_cast<const intx4*>(buf + xbase[j] + off);
#pragma unroll
                    for (int i = 0; i < RO; ++i) acc2[j][i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a2[s2][i], b2, acc2[j][i], 0, 0, 0);
                }
            }
        }
        // every load older than the D*RO ring refills just issued has completed: that includes the next patch
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(D * RO) : "memory");
        __syncthreads();
    }

    epilogue_c16<RO, RP>(acc, a, ypix, ob0, half);
    if constexpr (DS) {
        QArgs second = a;
        second.mult = a.mult2; second.res = nullptr; second.y = a.y2;
        second.flags = 0u;      // (its bias is in the accumulators already; no residual, no ReLU)
        epilogue_c16<RO, RP>(acc2, second, ypix, ob0, half);
    }
}

// ------------------------------------------------------------------------------------------------
// The same convolution with the staged patch on a row pitch of P positions, P a power of two fixed at compile time
// (64: padded rows of 33 to 64 positions, the 56 x 56 layers of ResNet-18).
//  * A 64-lane LDS-direct load covers 64 / P whole rows, so a position's (row, column) is a shift and a mask of the
//    lane number instead of a division by the padded width, and for P = 64 the row -- hence the image, the input row
//    and its validity -- is uniform: scalar arithmetic, two vector instructions per load.  Every tap's LDS offset
//    (rh * P + rw) * 16 is an immediate of the ds_read, with the lane half's channel-block plane folded into the
//    lane's base address once; bias and multipliers need no clamped addresses (output channels are a multiple of 32).
// Measured on the ResNet-18 layers at batch 64 (one process, launches captured in a graph): 14.3 against 14.7-15.5 us
// for 64 -> 64 channels at 56 x 56, no difference for the stride-2 layer on the same input.  Pitches of 16 and 32
// positions for the narrower layers were built and were SLOWER than the general kernel (512 -> 512 at 7 x 7: 16.6
// against 14.1 us; rows 256 or 512 bytes apart put the same column of every row into the same LDS banks), so only
// the 64-position pitch is instantiated.  Also measured and not kept: splitting the input channels over two or four
// wave groups inside the workgroup (their accumulators added through LDS): 18.0-18.5 against 13.8 us for the 7 x 7
// layer, 12.6-19.5 against 11.9 for 14 x 14; and a ring of three or four patch buffers: vector-memory loads complete
// in order, so a wave that consumes a weight fragment has also waited for every patch load issued before it, and one
// chunk's patch in flight per wave is all a deeper ring can hold.
// Same tiles, accumulators, epilogue and second output as qconv_mfma_kernel; PPT = load slots per wave.
template <int KH, int KW, int CBC, int WP, int RO, int PPT, int RP, int P, bool DS = false>
__global__ void __launch_bounds__(64 * WP) __attribute__((amdgpu_waves_per_eu(2))) qconv_rows_kernel(const QArgs a) {
    constexpr int KHW = KH * KW;
    constexpr int NS = (KHW * CBC + 1) / 2;          // matrix k-steps per chunk
    constexpr int NS2 = DS ? (CBC + 1) / 2 : 0;      // ... of the second output
    constexpr int TP = 32 * WP * RP;
    constexpr int LOGP = P == 64 ? 6 : (P == 32 ? 5 : 4);
    static_assert(P == 16 || P == 32 || P == 64, "row pitch of 16, 32 or 64 positions");

    extern __shared__ __attribute__((aligned(16))) char lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int half = lane >> 5;
    const int r = lane & 31;

    const int plane = a.chs * 16;                    // LDS bytes per channel-block plane
    const int buf_bytes = CBC * plane;
    char* const buf0 = lds;
    char* const buf1 = lds + buf_bytes;              // present only when nchunks > 1

    const int tile = (blockIdx.x & 7) * a.tiles_per_xcd + (blockIdx.x >> 3);
    if (tile >= a.num_tiles || static_cast<int>(blockIdx.x >> 3) >= a.tiles_per_xcd) return;
    const int p_tile = fast_div(tile, a.div_otiles), o_tile = tile - p_tile * a.o_tiles;
    const int m0 = p_tile * TP;
    const int ob0 = o_tile * RO;

    const int m_last = min(m0 + TP, a.M) - 1;
    int qmin, qlast;
    {
        const int n = fast_div(m0, a.div_ohw), rem = m0 - n * a.OHW;
        qmin = n * a.Hp + fast_div(rem, a.div_ow) * a.sh;
        const int n2 = fast_div(m_last, a.div_ohw), rem2 = m_last - n2 * a.OHW;
        qlast = n2 * a.Hp + fast_div(rem2, a.div_ow) * a.sh + (KH - 1);
    }
    const int nslots = ((qlast - qmin + 1) * P + 63) >> 6;       // 64-position load slots per plane (<= chs / 64)
    const uint32_t plane_bytes = static_cast<uint32_t>(a.H) * a.W * 16u;

    const __amdgpu_buffer_rsrc_t xr = make_rsrc(a.x, a.x_bytes);
    const __amdgpu_buffer_rsrc_t wr = make_rsrc(a.wp, a.w_bytes);

    // slot s holds rows s * (64 / P) ...; lane -> (row within the slot, column)
    const int col = lane & (P - 1);
    const int iw = col - a.pw;
    const bool col_ok = iw >= 0 && iw < a.W;
    uint32_t goff[PPT];
#pragma unroll
    for (int i = 0; i < PPT; ++i) {
        const int slot = wave + i * WP;
        const int Q = qmin + ((slot << 6) >> LOGP) + (lane >> LOGP);
        const int n = fast_div(Q, a.div_hp), ih = Q - n * a.Hp - a.ph;
        const bool ok = col_ok && Q <= qlast && n < a.N && ih >= 0 && ih < a.H;
        goff[i] = ok ? (static_cast<uint32_t>(n) * a.CB * a.H * a.W + static_cast<uint32_t>(ih * a.W + iw)) * 16u : kOob;
    }

    int xbase[RP];
    int ypix[RP];
#pragma unroll
    for (int j = 0; j < RP; ++j) {
        const int m = m0 + (wave * RP + j) * 32 + r;
        const int mc = min(m, a.M - 1);
        const int n = fast_div(mc, a.div_ohw), rem = mc - n * a.OHW;
        const int oh = fast_div(rem, a.div_ow), ow = rem - oh * a.OW;
        xbase[j] = (((n * a.Hp + oh * a.sh - qmin) << LOGP) + ow * a.sw) * 16;
        if (CBC > 1) xbase[j] += half * plane;
        ypix[j] = (m < a.M) ? n * (a.O >> 4) * a.OHW + rem : -1;
    }

    // accumulators start at the bias
    intx16 acc[RP][RO];
    {
        const bool has_bias = (a.flags & KXC_HIP_CONV_BIAS) != 0;
#pragma unroll
        for (int i = 0; i < RO; ++i)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                int4 b = make_int4(0, 0, 0, 0);
                if (has_bias) b = *reinterpret_cast<const int4*>(a.bias + (ob0 + i) * 32 + 8 * g + 4 * half);
#pragma unroll
                for (int j = 0; j < RP; ++j) { acc[j][i][4 * g + 0] = b.x; acc[j][i][4 * g + 1] = b.y; acc[j][i][4 * g + 2] = b.z; acc[j][i][4 * g + 3] = b.w; }
            }
    }

    auto issue_loads = [&](int chunk, char* buf) {
#pragma unroll
        for (int cl = 0; cl < CBC; ++cl) {
            const int cb = chunk * CBC + cl;
            if (cb < a.CB) {
                const uint32_t soff = static_cast<uint32_t>(cb) * plane_bytes;
#pragma unroll
                for (int i = 0; i < PPT; ++i) {
                    const int slot = wave + i * WP;
                    if (slot < nslots)
                        load16_to_lds(xr, (lds_ptr_t)(buf + cl * plane + slot * 1024), goff[i], soff);
                }
            }   // a missing channel block keeps stale bytes; its packed weights are zero and integers have no NaN
        }
        __builtin_amdgcn_sched_barrier(0);
        asm volatile("" ::: "memory");      // the weight loads below stay behind these in program order
    };

    // weight ring: see qconv_mfma_kernel
    constexpr int D = (NS % 3 == 0) ? 3 : (NS % 5 == 0 ? 5 : (NS % 2 == 0 ? 2 : 1));
    static_assert(NS % D == 0, "the weight ring must divide the k-steps of a chunk");
    const uint32_t total_steps = static_cast<uint32_t>(a.nchunks) * NS;
    uint32_t wvoff[RO];
#pragma unroll
    for (int i = 0; i < RO; ++i) wvoff[i] = static_cast<uint32_t>(ob0 + i) * total_steps * 1024u + static_cast<uint32_t>(lane) * 16u;
    auto load_a = [&](int i, uint32_t t) -> intx4 {
        const uint32_t tc = t < total_steps ? t : total_steps - 1u;
        return __builtin_amdgcn_raw_buffer_load_b128(wr, wvoff[i], tc * 1024u, 0);
    };
    intx4 ring[D][RO];
    const __amdgpu_buffer_rsrc_t wr2 = make_rsrc(DS ? a.wp2 : a.wp, DS ? a.w2_bytes : 0u);
    intx16 acc2[DS ? RP : 1][DS ? RO : 1];
    if constexpr (DS) {
        const bool has_bias2 = a.bias2 != nullptr;
#pragma unroll
        for (int i = 0; i < RO; ++i)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                int4 b = make_int4(0, 0, 0, 0);
                if (has_bias2) b = *reinterpret_cast<const int4*>(a.bias2 + (ob0 + i) * 32 + 8 * g + 4 * half);
#pragma unroll
                for (int j = 0; j < RP; ++j) { acc2[j][i][4 * g + 0] = b.x; acc2[j][i][4 * g + 1] = b.y; acc2[j][i][4 * g + 2] = b.z; acc2[j][i][4 * g + 3] = b.w; }
            }
    }

    issue_loads(0, buf0);
#pragma unroll
    for (int d = 0; d < D; ++d)
#pragma unroll
        for (int i = 0; i < RO; ++i) ring[d][i] = load_a(i, d);
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(D * RO) : "memory");     // the patch has landed, the ring may still fly
    __syncthreads();

    for (int chunk = 0; chunk < a.nchunks; ++chunk) {
        const char* buf = (chunk & 1) ? buf1 : buf0;
        intx4 a2[DS ? NS2 : 1][RO];
        if constexpr (DS) {
#pragma unroll
            for (int s2 = 0; s2 < NS2; ++s2)
#pragma unroll
                for (int i = 0; i < RO; ++i)
                    a2[s2][i] = __builtin_amdgcn_raw_buffer_load_b128(
                        wr2,
                        (static_cast<uint32_t>(ob0 + i) * static_cast<uint32_t>(a.nchunks) * NS2 + static_cast<uint32_t>(chunk) * NS2 + s2) * 1024u +
                            static_cast<uint32_t>(lane) * 16u, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            asm volatile("" ::: "memory");      // ahead of the next patch's loads in program order
        }
        if (chunk + 1 < a.nchunks) issue_loads(chunk + 1, (chunk & 1) ? buf0 : buf1);
        {
            // this chunk's operand base per pixel block; the tap offsets below are compile-time constants
            const char* xb[RP];
#pragma unroll
            for (int j = 0; j < RP; ++j) xb[j] = buf + xbase[j];
            auto tap_imm = [](int tap) constexpr {
                const int t = tap < KHW ? tap : KHW - 1;
                return ((t / KW) * P + (t % KW)) * 16;
            };
            auto fetch_b = [&](int step, intx4 (&b)[RP]) {
                if constexpr (CBC == 1) {
                    const int off = half ? tap_imm(2 * step + 1) : tap_imm(2 * step);
#pragma unroll
                    for (int j = 0; j < RP; ++j) b[j] = *reinterpret_cast<const intx4*>(xb[j] + off);
                } else {
                    constexpr int H2 = CBC / 2;
                    const int pl = 2 * (step % H2) * plane;          // 0 when a chunk is two channel blocks
#pragma unroll
                    for (int j = 0; j < RP; ++j) b[j] = *reinterpret_cast<const intx4*>(xb[j] + pl + tap_imm(step / H2));
                }
            };
            const uint32_t t0 = static_cast<uint32_t>(chunk) * NS;
            // (pixel operands two k-steps ahead and a scheduling barrier per step for several pixel blocks per wave: see
            // qconv_mfma_kernel; 64 -> 64 channels at 56 x 56, batch 64: 13.2-13.7 -> 12.9 us)
            constexpr int DB = RP >= 2 ? 2 : 1;
            intx4 bring[DB][RP];
#pragma unroll
            for (int s0 = 0; s0 < DB; ++s0) fetch_b(s0, bring[s0]);
#pragma unroll
            for (int step = 0; step < NS; ++step) {
#pragma unroll
                for (int j = 0; j < RP; ++j)
#pragma unroll
                    for (int i = 0; i < RO; ++i)
                        acc[j][i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(ring[step % D][i], bring[step % DB][j], acc[j][i], 0, 0, 0);
#pragma unroll
                for (int i = 0; i < RO; ++i) ring[step % D][i] = load_a(i, t0 + step + D);
                if (step + DB < NS) fetch_b(step + DB, bring[step % DB]);
                if constexpr (RP >= 2) __builtin_amdgcn_sched_barrier(0);
            }
            if constexpr (DS) {
#pragma unroll
                for (int s2 = 0; s2 < NS2; ++s2) {
                    const int off = a.ds_off + (CBC > 1 ? 2 * s2 * plane : 0);
#pragma unroll
                    for (int j = 0; j < RP; ++j) {
                        const intx4 b2 = *reinterpret_cast<const intx4*>(xb[j] + off);
#pragma unroll
                        for (int i = 0; i < RO; ++i) acc2[j][i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a2[s2][i], b2, acc2[j][i], 0, 0, 0);
                    }
                }
            }
        }
        // every load older than the ring refills just issued has completed: that includes the next patch
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(D * RO) : "memory");
        __syncthreads();
    }

    epilogue_c16<RO, RP>(acc, a, ypix, ob0, half);
    if constexpr (DS) {
        QArgs second = a;
        second.mult = a.mult2; second.res = nullptr; second.y = a.y2;
        second.flags = 0u;
        epilogue_c16<RO, RP>(acc2, second, ypix, ob0, half);
    }
}

// ------------------------------------------------------------------------------------------------
// First layer: 7x7, stride 2, padding 3, at most 4 input channels, on the "c4" input layout
// [N][H][W][4] (4 bytes per pixel, channels >= C zero).  A 16-byte k-slice is four horizontally adjacent
// pixels x 4 channels, so a k-step (32 values) is ONE filter row: lane half h covers the taps
// kw = 4h-1 .. 4h+2 (the window is widened by one tap on the left, with zero weight, so that it starts on
// an 8-byte boundary).  7 k-steps per 32x32 block instead of the 25 that padding 3 channels to a 16-channel
// block costs, and a quarter of the input bytes.  LDS rows hold [4 zero pixels][W pixels][4 zero pixels]
// as 16-byte positions; a tile's rows are loaded once (single chunk).  Output is c16.
template <int WP, int RO, int PPT>
__global__ void __launch_bounds__(64 * WP) __attribute__((amdgpu_waves_per_eu(2))) qconv_k7s2_c4_kernel(const QArgs a) {
    constexpr int KH = 7;
    constexpr int TP = 32 * WP;
    constexpr int WSEG = RO * KH;
    constexpr int WPT = (WSEG + WP - 1) / WP;
    extern __shared__ __attribute__((aligned(16))) char lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int half = lane >> 5;
    const int r = lane & 31;
    const int W4 = (a.W >> 2) + 2;                  // 16-byte positions per LDS row
    const int xs_bytes = a.chs * 16;

    const int tile = (blockIdx.x & 7) * a.tiles_per_xcd + (blockIdx.x >> 3);
    if (tile >= a.num_tiles || static_cast<int>(blockIdx.x >> 3) >= a.tiles_per_xcd) return;
    const int p_tile = fast_div(tile, a.div_otiles), o_tile = tile - p_tile * a.o_tiles;
    const int m0 = p_tile * TP;
    const int ob0 = o_tile * RO;
    const int m_last = min(m0 + TP, a.M) - 1;
    int qmin, qlast;
    {
        const int n = fast_div(m0, a.div_ohw), rem = m0 - n * a.OHW;
        qmin = n * a.Hp + fast_div(rem, a.div_ow) * 2;
        const int n2 = fast_div(m_last, a.div_ohw), rem2 = m_last - n2 * a.OHW;
        qlast = n2 * a.Hp + fast_div(rem2, a.div_ow) * 2 + (KH - 1);
    }
    const int P = (qlast - qmin + 1) * W4;
    const int xsegs = (P + 63) >> 6;
    const __amdgpu_buffer_rsrc_t xr = make_rsrc(a.x, a.x_bytes);
    const __amdgpu_buffer_rsrc_t wr = make_rsrc(a.wp, a.w_bytes);
#pragma unroll
    for (int i = 0; i < PPT; ++i) {
        const int seg = wave + i * WP;
        if (seg < xsegs) {
            const int pos = seg * 64 + lane;
            const int q = fast_div(pos, a.div_wp), c4 = pos - q * W4;
            const int Q = qmin + q;
            const int n = fast_div(Q, a.div_hp), ih = Q - n * a.Hp - 3;
            const bool ok = pos < P && n < a.N && ih >= 0 && ih < a.H && c4 >= 1 && c4 <= (a.W >> 2);
            const uint32_t off = ok ? static_cast<uint32_t>((n * a.H + ih) * a.W + (c4 - 1) * 4) * 4u : kOob;
            load16_to_lds(xr, (lds_ptr_t)(lds + seg * 1024), off, 0);
        }
    }
#pragma unroll
    for (int i = 0; i < WPT; ++i) {
        const int seg = wave + i * WP;
        if (seg < WSEG) {
            const int ro = seg / KH, st = seg - ro * KH;
            load16_to_lds(wr, (lds_ptr_t)(lds + xs_bytes + seg * 1024), static_cast<uint32_t>(lane) * 16u,
                          (static_cast<uint32_t>(ob0 + ro) * KH + st) * 1024u);
        }
    }
    const int m = m0 + wave * 32 + r;
    int xbase;
    int ypix[1];
    {
        const int mc = min(m, a.M - 1);
        const int n = fast_div(mc, a.div_ohw), rem = mc - n * a.OHW;
        const int oh = fast_div(rem, a.div_ow), ow = rem - oh * a.OW;
        xbase = (n * a.Hp + oh * 2 - qmin) * W4 * 16 + ow * 8 + half * 16;
        ypix[0] = (m < a.M) ? n * (a.O >> 4) * a.OHW + rem : -1;
    }
    intx16 acc[1][RO];
    init_acc_with_bias<RO>(acc[0], a.bias, (a.flags & KXC_HIP_CONV_BIAS) != 0, a.O, ob0, half);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    const char* ws = lds + xs_bytes + lane * 16;
#pragma unroll
    for (int kh = 0; kh < KH; ++kh) {
        const int2 lo = *reinterpret_cast<const int2*>(lds + xbase + kh * W4 * 16);        // 8-byte aligned
        const int2 hi = *reinterpret_cast<const int2*>(lds + xbase + kh * W4 * 16 + 8);
        intx4 b;
        b[0] = lo.x; b[1] = lo.y; b[2] = hi.x; b[3] = hi.y;
#pragma unroll
        for (int i = 0; i < RO; ++i) {
            const intx4 wv = *reinterpret_cast<const intx4*>(ws + (i * KH + kh) * 1024);
            acc[0][i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wv, b, acc[0][i], 0, 0, 0);
        }
    }
    epilogue_c16<RO, 1>(acc, a, ypix, ob0, half);
}


// ------------------------------------------------------------------------------------------
// First layer AND the max pool behind it (3x3, stride 2, padding 1) in one kernel: int8 c4 input -> the pooled
// feature map in c16.  The unpooled map (51 MB at batch 64, written once and read once) never exists.
//
// A workgroup of four waves owns `pool_rows` pooled rows of one image for RO blocks of 32 output channels and walks
// the 2*pool_rows + 1 convolution rows they need, top to bottom (neighbouring workgroups compute the row they share
// twice: 1/(2*pool_rows) more matrix and requantisation work).  Wave w computes convolution columns 30w-1 .. 30w+30
// of every row -- 32 columns for the 15 pooling windows centred on columns 30w, 30w+2, ..., 30w+28, so that all
// three columns of a window lie in one wave and no value crosses waves (neighbouring waves overlap by two columns).
// Per row: seven matrix instructions per channel block, the usual requantisation up to the clamp -- kept as a float
// because rounding is monotonic: the maximum of the rounded values is the rounded maximum -- the maximum over lanes
// r-1, r, r+1 (two DPP operands), and the running maximum over rows in registers; after a window's third row the
// odd lanes round, pack and store their pooled pixel.  Columns and rows outside the convolution's output count as
// -128, the pooling pad candidate of int8 (the lowest value: it never wins against a real one): a missing column
// through per-lane clamp bounds, a missing row by not being computed.
// ------------------------------------------------------------------------------------------
template <int RO, bool RELU>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) qconv_k7s2_c4_pool_kernel(const QArgs a) {
    constexpr int KH = 7;
    constexpr int WP = 4;
    constexpr int WSEG = RO * KH;
    extern __shared__ __attribute__((aligned(16))) char lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int half = lane >> 5;
    const int r = lane & 31;
    const int W4 = (a.W >> 2) + 2;                  // 16-byte positions per LDS row
    const int row_bytes = W4 * 16;
    const int xs_bytes = a.chs * 16;

    const int tile = (blockIdx.x & 7) * a.tiles_per_xcd + (blockIdx.x >> 3);
    if (tile >= a.num_tiles || static_cast<int>(blockIdx.x >> 3) >= a.tiles_per_xcd) return;
    const int p_tile = fast_div(tile, a.div_otiles), o_tile = tile - p_tile * a.o_tiles;
    const int n = fast_div(p_tile, a.div_pool_tiles), pt = p_tile - n * a.pool_tiles;
    const int ob0 = o_tile * RO;
    const int p0 = pt * a.pool_rows, p1 = min(p0 + a.pool_rows, a.POH);       // pooled rows [p0, p1)
    const int c_lo = max(2 * p0 - 1, 0), c_hi = min(2 * (p1 - 1) + 1, a.OH - 1);   // convolution rows needed
    const int nrows = 2 * (c_hi - c_lo) + KH;                                 // padded input rows staged
    const int P = nrows * W4;
    const int xsegs = (P + 63) >> 6;
    const __amdgpu_buffer_rsrc_t xr = make_rsrc(a.x, a.x_bytes);
    const __amdgpu_buffer_rsrc_t wr = make_rsrc(a.wp, a.w_bytes);
    for (int seg = wave; seg < xsegs; seg += WP) {
        const int pos = seg * 64 + lane;
        const int q = fast_div(pos, a.div_wp), c4 = pos - q * W4;
        const int ih = 2 * c_lo + q - 3;
        const bool ok = pos < P && ih >= 0 && ih < a.H && c4 >= 1 && c4 <= (a.W >> 2);
        const uint32_t off = ok ? static_cast<uint32_t>((n * a.H + ih) * a.W + (c4 - 1) * 4) * 4u : kOob;
        load16_to_lds(xr, (lds_ptr_t)(lds + seg * 1024), off, 0);
    }
    for (int seg = wave; seg < WSEG; seg += WP) {
        const int ro = seg / KH, st = seg - ro * KH;
        load16_to_lds(wr, (lds_ptr_t)(lds + xs_bytes + seg * 1024), static_cast<uint32_t>(lane) * 16u,
                      (static_cast<uint32_t>(ob0 + ro) * KH + st) * 1024u);
    }
    // this lane's column, its place in an LDS row, and the pooled pixel an odd lane owns
    const int col = 30 * wave - 1 + r;
    const bool col_ok = col >= 0 && col < a.OW;
    const int xcol = min(max(col, 0), a.OW - 1) * 8 + half * 16;
    const int pw = 15 * wave + (r >> 1);
    const bool owner = (r & 1) && r <= 29 && pw < a.PW;
    const bool has_bias = (a.flags & KXC_HIP_CONV_BIAS) != 0;
    constexpr float kPad = -128.0f;
    // the clamp's bounds are per lane: a column outside the map clamps to [-128, -128] and so becomes the pad candidate
    const float lower = col_ok ? (RELU ? 0.0f : -128.0f) : kPad;
    const float upper = col_ok ? 127.0f : kPad;
    intx16 bv[RO];
    float4 mv[RO][4];
#pragma unroll
    for (int i = 0; i < RO; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int4 b4 = has_bias ? *reinterpret_cast<const int4*>(a.bias + (ob0 + i) * 32 + 8 * j + 4 * half) : make_int4(0, 0, 0, 0);
            bv[i][4 * j + 0] = b4.x; bv[i][4 * j + 1] = b4.y; bv[i][4 * j + 2] = b4.z; bv[i][4 * j + 3] = b4.w;
            mv[i][j] = *reinterpret_cast<const float4*>(a.mult + (ob0 + i) * 32 + 8 * j + 4 * half);
        }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    const char* ws = lds + xs_bytes + lane * 16;

    // One convolution row: for every accumulator register the requantised value before rounding, already the maximum
    // over the lane's column and its two neighbours, handed to sink(i, g, value).
    auto conv_row = [&](int c, auto&& sink) {
        intx16 acc[RO];
        const char* xrow = lds + 2 * (c - c_lo) * row_bytes + xcol;
#pragma unroll
        for (int kh = 0; kh < KH; ++kh) {
            const int2 lo = *reinterpret_cast<const int2*>(xrow + kh * row_bytes);        // 8-byte aligned
            const int2 hi = *reinterpret_cast<const int2*>(xrow + kh * row_bytes + 8);
            intx4 b;
            b[0] = lo.x; b[1] = lo.y; b[2] = hi.x; b[3] = hi.y;
#pragma unroll
            for (int i = 0; i < RO; ++i) {
                const intx4 wv = *reinterpret_cast<const intx4*>(ws + (i * KH + kh) * 1024);
                // (the sum starts at the bias: the first instruction takes it as its addend)
                acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wv, b, kh == 0 ? bv[i] : acc[i], 0, 0, 0);
            }
        }
#pragma unroll
        for (int i = 0; i < RO; ++i)
#pragma unroll
            for (int gq = 0; gq < 4; ++gq) {
                const float ms[4] = {mv[i][gq].x, mv[i][gq].y, mv[i][gq].z, mv[i][gq].w};
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    // (the requantisation of epilogue_c16 up to the clamp)
                    float v = __fmul_rn(static_cast<float>(acc[i][4 * gq + e]), ms[e]);
                    if (!RELU) v = (v == v) ? v : 0.0f;
                    v = __builtin_amdgcn_fmed3f(v, lower, upper);
                    const int bits = __builtin_bit_cast(int, v);
                    constexpr int kLowest = static_cast<int>(0xff800000u);      // -inf: what a lane without a neighbour reads
                    // lane l reads lane l-1 (0x138: whole-wave shift right by one) and lane l+1 (0x130)
                    const float left = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(kLowest, bits, 0x138, 0xf, 0xf, false));
                    const float right = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(kLowest, bits, 0x130, 0xf, 0xf, false));
                    sink(i, 4 * gq + e, fmaxf(fmaxf(v, left), right));
                }
            }
    };

    // carry = the row above the next window (row 2p - 1), which is the previous window's last row
    float carry[RO][16];
    if (2 * p0 - 1 >= 0) {
        conv_row(2 * p0 - 1, [&](int i, int g, float v) { carry[i][g] = v; });
    } else {
#pragma unroll
        for (int i = 0; i < RO; ++i)
#pragma unroll
            for (int g = 0; g < 16; ++g) carry[i][g] = kPad;
    }
    for (int p = p0; p < p1; ++p) {
        float best[RO][16];
        conv_row(2 * p, [&](int i, int g, float v) { best[i][g] = fmaxf(carry[i][g], v); });      // (row 2p always exists)
        if (2 * p + 1 < a.OH)
            conv_row(2 * p + 1, [&](int i, int g, float v) { best[i][g] = fmaxf(best[i][g], v); carry[i][g] = v; });
        constexpr float kMagic = 12582912.0f;      // 1.5 * 2^23: the sum's low byte is the rounded value
#pragma unroll
        for (int i = 0; i < RO; ++i) {
            uint32_t w[4];
#pragma unroll
            for (int gq = 0; gq < 4; ++gq) {
                uint32_t t[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) t[e] = __builtin_bit_cast(uint32_t, __fadd_rn(best[i][4 * gq + e], kMagic));
                const uint32_t lo = __builtin_amdgcn_perm(t[1], t[0], 0x0c0c0400u);
                const uint32_t hi = __builtin_amdgcn_perm(t[3], t[2], 0x0c0c0400u);
                w[gq] = __builtin_amdgcn_perm(hi, lo, 0x05040100u);
            }
            swap_halves(w[0], w[2]);      // (as in epilogue_c16: half 0 ends up with channels 0-15, half 1 with 16-31)
            swap_halves(w[1], w[3]);
            if (owner) {
                const int64_t word = (static_cast<int64_t>((n * (a.O >> 4) + (ob0 + i) * 2 + half) * a.POH + p) * a.PW + pw) * 16;
                *reinterpret_cast<uintx4*>(a.y + word) = uintx4{w[0], w[2], w[1], w[3]};
            }
        }
    }
}

// Weights of the first-layer kernel: [o block][kh][lane][16]; lane (o, half), byte j = pixel j/4, channel j%4,
// tap kw = 4*half + j/4 - 1.
__device__ __forceinline__ void pack_k7_c4_slot(const int8_t* __restrict__ w, int8_t* __restrict__ wp, int32_t O, int32_t C, int64_t s) {
    const int lane = static_cast<int>(s & 63);
    const int64_t t = s >> 6;
    const int kh = static_cast<int>(t % 7);
    const int ob = static_cast<int>(t / 7);
    const int o = ob * 32 + (lane & 31), h = lane >> 5;
    int8_t out[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) {
        const int kw = 4 * h + (j >> 2) - 1, c = j & 3;
        out[j] = (kw >= 0 && kw < 7 && c < C && o < O) ? w[((static_cast<int64_t>(o) * C + c) * 7 + kh) * 7 + kw] : 0;
    }
    *reinterpret_cast<int4*>(wp + s * 16) = *reinterpret_cast<const int4*>(out);
}

__global__ void __launch_bounds__(kBlock) pack_weights_k7_c4_kernel(const int8_t* __restrict__ w, int8_t* __restrict__ wp,
                                                                    int32_t O, int32_t C, int64_t total_slots) {
    const int64_t s = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (s >= total_slots) return;
    pack_k7_c4_slot(w, wp, O, C, s);
}

// fp32 NCHW -> int8 c4 ([N][H][W][4]); one thread per pixel.
__global__ void __launch_bounds__(kBlock) quantize_to_c4_kernel(const float* __restrict__ x, int8_t* __restrict__ y,
                                                                int32_t C, int64_t HW, int64_t total, float scale) {
    const int64_t s = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (s >= total) return;
    const int64_t p = s % HW, n = s / HW;
    uint32_t word = 0;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        int32_t q = 0;
        if (c < C) {
            const float v = __fdiv_rn(x[(n * C + c) * HW + p], scale);
            float rr = rintf(v);
            rr = (v == v) ? rr : 0.0f;
            rr = fminf(fmaxf(rr, -127.0f), 127.0f);
            q = static_cast<int32_t>(rr);
        }
        word |= (static_cast<uint32_t>(q) & 0xffu) << (8 * c);
    }
    reinterpret_cast<uint32_t*>(y)[s] = word;
}

// The same for four consecutive pixels per thread (plane size a multiple of 4, 16-byte aligned tensors): one 16-byte
// load per channel, one 16-byte store, a quarter of the index arithmetic.  Same arithmetic per element.
__global__ void __launch_bounds__(kBlock) quantize_to_c4_x4_kernel(const float* __restrict__ x, int8_t* __restrict__ y,
                                                                   int32_t C, int32_t HW4, int64_t total4, float scale) {
    const int64_t s = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (s >= total4) return;
    const int64_t n = s / HW4;
    const int32_t p4 = static_cast<int32_t>(s - n * HW4);
    uint32_t word[4] = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        if (c < C) {
            const float4 v4 = reinterpret_cast<const float4*>(x)[(n * C + c) * HW4 + p4];
            const float e[4] = {v4.x, v4.y, v4.z, v4.w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float v = __fdiv_rn(e[i], scale);
                float rr = rintf(v);
                rr = (v == v) ? rr : 0.0f;
                rr = fminf(fmaxf(rr, -127.0f), 127.0f);
                word[i] |= (static_cast<uint32_t>(static_cast<int32_t>(rr)) & 0xffu) << (8 * c);
            }
        }
    }
    reinterpret_cast<uint4*>(y)[s] = make_uint4(word[0], word[1], word[2], word[3]);
}

// ------------------------------------------------------------------ weight packing
struct PackArgs {
    const int8_t* w;      // OIHW
    int8_t* wp;
    int32_t O, C, KHW, CBC, NS, nchunks, oblocks;
};

__device__ __forceinline__ void pack_slot(const PackArgs& a, int64_t s) {
    const int lane = static_cast<int>(s & 63);
    int64_t t = s >> 6;
    const int step = static_cast<int>(t % a.NS); t /= a.NS;
    const int chunk = static_cast<int>(t % a.nchunks);
    const int ob = static_cast<int>(t / a.nchunks);
    const int o = ob * 32 + (lane & 31), h = lane >> 5;
    const int q = 2 * step + h;
    const int tap = q / a.CBC, cbl = q - tap * a.CBC;
    const int cb = chunk * a.CBC + cbl;
    int8_t out[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) {
        const int c = cb * 16 + j;
        out[j] = (tap < a.KHW && c < a.C && o < a.O) ? a.w[(static_cast<int64_t>(o) * a.C + c) * a.KHW + tap] : 0;
    }
    *reinterpret_cast<int4*>(a.wp + s * 16) = *reinterpret_cast<const int4*>(out);
}

__global__ void __launch_bounds__(kBlock) pack_weights_kernel(const PackArgs a, int64_t total_slots) {
    const int64_t s = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (s >= total_slots) return;
    pack_slot(a, s);
}

// The weight tensors of several layers in one launch (a launch plan packs the constants of a whole network at the
// start of a run).  Job j owns the blocks first_block[j] .. first_block[j + 1] - 1.  A block of a job with
// staged != 0 packs one (output block of 32 channels, chunk) unit: the unit's 32 rows of OIHW bytes -- each a
// contiguous run of CBC*16*KHW bytes -- are read once, coalesced, into LDS, and its NS*64 slots, which are
// contiguous in the packed tensor, are written from there (one thread per slot gathers bytes KHW apart: from
// memory that costs a cache line per byte).  Other jobs (the first-layer order, NS == 0; windows too large for the
// LDS array) take one thread per slot straight from memory.
constexpr int kMaxPackJobs = 24;
constexpr int kPackRowBytes = 800;           // room per staged row: CBC*16*KHW bytes + 4
struct PackBatch {
    PackArgs job[kMaxPackJobs];
    int64_t slots[kMaxPackJobs];
    int32_t first_block[kMaxPackJobs + 1];
    int32_t staged[kMaxPackJobs];
    int32_t count;
};
__global__ void __launch_bounds__(kBlock) pack_weights_batch_kernel(const PackBatch b) {
    __shared__ __attribute__((aligned(16))) uint8_t raw[32 * kPackRowBytes];
    int j = 0;
    while (j + 1 < b.count && static_cast<int32_t>(blockIdx.x) >= b.first_block[j + 1]) ++j;
    const PackArgs& a = b.job[j];
    const int32_t local = static_cast<int32_t>(blockIdx.x) - b.first_block[j];
    if (!b.staged[j]) {
        const int64_t s = static_cast<int64_t>(local) * kBlock + threadIdx.x;
        if (s >= b.slots[j]) return;
        if (a.NS == 0) pack_k7_c4_slot(a.w, a.wp, a.O, a.C, s);
        else pack_slot(a, s);
        return;
    }
    const int ob = local / a.nchunks, chunk = local - ob * a.nchunks;
    const int c0 = chunk * a.CBC * 16;
    const int nch = min(a.CBC * 16, a.C - c0);               // channels of this chunk that exist
    const int row_bytes = nch * a.KHW;                        // contiguous bytes per output channel
    const int pitch = ((a.CBC * 16 * a.KHW + 3) & ~3) + 4;    // LDS bytes per row: an odd number of words
    const bool words = ((static_cast<int64_t>(a.C) * a.KHW) & 3) == 0 && (row_bytes & 3) == 0 && ((c0 * a.KHW) & 3) == 0 &&
                       (reinterpret_cast<uintptr_t>(a.w) & 3u) == 0;
    if (words) {
        const int row_words = row_bytes >> 2;
        for (int e = threadIdx.x; e < 32 * row_words; e += kBlock) {
            const int r = e / row_words, k = e - r * row_words;
            const int o = ob * 32 + r;
            uint32_t v = 0;
            if (o < a.O) v = reinterpret_cast<const uint32_t*>(a.w + (static_cast<int64_t>(o) * a.C + c0) * a.KHW)[k];
            *reinterpret_cast<uint32_t*>(raw + r * pitch + 4 * k) = v;
        }
    } else {
        for (int e = threadIdx.x; e < 32 * row_bytes; e += kBlock) {
            const int r = e / row_bytes, k = e - r * row_bytes;
            const int o = ob * 32 + r;
            raw[r * pitch + k] = o < a.O ? static_cast<uint8_t>(a.w[(static_cast<int64_t>(o) * a.C + c0) * a.KHW + k]) : uint8_t{0};
        }
    }
    __syncthreads();
    int8_t* const out = a.wp + (static_cast<int64_t>(ob) * a.nchunks + chunk) * a.NS * 1024;
    for (int s = threadIdx.x; s < a.NS * 64; s += kBlock) {
        const int lane = s & 63, step = s >> 6;
        const int r = lane & 31, h = lane >> 5;
        const int q = 2 * step + h;
        const int tap = q / a.CBC, cbl = q - tap * a.CBC;
        uint32_t word[4] = {0u, 0u, 0u, 0u};
        if (tap < a.KHW) {
#pragma unroll
            for (int jj = 0; jj < 16; ++jj) {
                const int cl = cbl * 16 + jj;
                const uint32_t v = cl < nch ? raw[r * pitch + cl * a.KHW + tap] : 0u;
                word[jj >> 2] |= v << (8 * (jj & 3));
            }
        }
        *reinterpret_cast<uint4*>(out + s * 16) = make_uint4(word[0], word[1], word[2], word[3]);
    }
}

// ------------------------------------------------------------------ layout conversion and quantisation
// One thread per 16-byte position of the c16 tensor.
__global__ void __launch_bounds__(kBlock) nchw_to_c16_kernel(const int8_t* __restrict__ x, int8_t* __restrict__ y,
                                                             int32_t C, int32_t CB, int64_t HW, int64_t total) {
    const int64_t s = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (s >= total) return;
    const int64_t p = s % HW;
    const int64_t t = s / HW;
    const int cb = static_cast<int>(t % CB);
    const int64_t n = t / CB;
    int8_t out[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) {
        const int c = cb * 16 + j;
        out[j] = c < C ? x[(n * C + c) * HW + p] : 0;
    }
    *reinterpret_cast<int4*>(y + s * 16) = *reinterpret_cast<const int4*>(out);
}

__global__ void __launch_bounds__(kBlock) c16_to_nchw_kernel(const int8_t* __restrict__ x, int8_t* __restrict__ y,
                                                             int32_t C, int32_t CB, int64_t HW, int64_t total) {
    const int64_t e = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;   // NCHW element
    if (e >= total) return;
    const int64_t p = e % HW;
    const int64_t t = e / HW;
    const int c = static_cast<int>(t % C);
    const int64_t n = t / C;
    y[e] = x[((n * CB + (c >> 4)) * HW + p) * 16 + (c & 15)];
}

__global__ void __launch_bounds__(kBlock) quantize_to_c16_kernel(const float* __restrict__ x, int8_t* __restrict__ y,
                                                                 int32_t C, int32_t CB, int64_t HW, int64_t total,
                                                                 float scale) {
    const int64_t s = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (s >= total) return;
    const int64_t p = s % HW;
    const int64_t t = s / HW;
    const int cb = static_cast<int>(t % CB);
    const int64_t n = t / CB;
    int8_t out[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) {
        const int c = cb * 16 + j;
        int32_t q = 0;
        if (c < C) {
            const float v = __fdiv_rn(x[(n * C + c) * HW + p], scale);
            float rr = rintf(v);
            rr = (v == v) ? rr : 0.0f;
            rr = fminf(fmaxf(rr, -127.0f), 127.0f);
            q = static_cast<int32_t>(rr);
        }
        out[j] = static_cast<int8_t>(q);
    }
    *reinterpret_cast<int4*>(y + s * 16) = *reinterpret_cast<const int4*>(out);
}

// ------------------------------------------------------------------ pooling on c16
struct PoolArgs {
    int32_t N, CB, H, W, OH, OW, KH, KW, sh, sw, pt, pl;
};

// One thread per output position (16 channels): byte-wise signed max over the window.
__global__ void __launch_bounds__(kBlock) maxpool_c16_kernel(const int8_t* __restrict__ x, int8_t* __restrict__ y,
                                                             const PoolArgs d, int64_t total) {
    const int64_t s = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (s >= total) return;
    const int ow = static_cast<int>(s % d.OW);
    int64_t t = s / d.OW;
    const int oh = static_cast<int>(t % d.OH);
    const int64_t plane = t / d.OH;                  // n*CB + cb
    const int8_t* xp = x + plane * d.H * d.W * 16;
    int32_t m[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) m[j] = -128;
    for (int rh = 0; rh < d.KH; ++rh) {
        const int ih = oh * d.sh + rh - d.pt;
        if (ih < 0 || ih >= d.H) continue;
        for (int rw = 0; rw < d.KW; ++rw) {
            const int iw = ow * d.sw + rw - d.pl;
            if (iw < 0 || iw >= d.W) continue;
            const int4 v = *reinterpret_cast<const int4*>(xp + (static_cast<int64_t>(ih) * d.W + iw) * 16);
            const int vw[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                const int32_t b = static_cast<int32_t>(static_cast<int8_t>((vw[j >> 2] >> (8 * (j & 3))) & 0xff));
                m[j] = b > m[j] ? b : m[j];
            }
        }
    }
    uint32_t o[4] = {0, 0, 0, 0};
#pragma unroll
    for (int j = 0; j < 16; ++j) o[j >> 2] |= (static_cast<uint32_t>(m[j]) & 0xffu) << (8 * (j & 3));
    *reinterpret_cast<int4*>(y + s * 16) = make_int4(o[0], o[1], o[2], o[3]);
}

// The same for a compile-time window every one of whose placements meets the input (the host checks): a tap
// outside the input re-reads the nearest row / column inside it, which lies in the same window and cannot change the
// maximum, so all KH*KW loads are issued at once, without branches.  The signed byte maxima are taken two at a time:
// bytes 0 and 2 of a dword are moved to the high bytes of its 16-bit halves, bytes 1 and 3 are there already, and a
// packed 16-bit signed max of such halves orders them like the bytes.
typedef short shortx2 __attribute__((ext_vector_type(2)));
template <int KH, int KW>
__global__ void __launch_bounds__(kBlock) maxpool_c16_window_kernel(const int8_t* __restrict__ x, int8_t* __restrict__ y,
                                                                    const PoolArgs d, int32_t total) {
    const int32_t s = static_cast<int32_t>(blockIdx.x) * kBlock + static_cast<int32_t>(threadIdx.x);
    if (s >= total) return;
    const int32_t t = s / d.OW;
    const int ow = s - t * d.OW;
    const int32_t plane = t / d.OH;                  // n*CB + cb
    const int oh = t - plane * d.OH;
    const int4* xp = reinterpret_cast<const int4*>(x) + static_cast<int64_t>(plane) * d.H * d.W;
    int4 v[KH][KW];
#pragma unroll
    for (int rh = 0; rh < KH; ++rh) {
        const int ih = min(max(oh * d.sh + rh - d.pt, 0), d.H - 1);
#pragma unroll
        for (int rw = 0; rw < KW; ++rw) {
            const int iw = min(max(ow * d.sw + rw - d.pl, 0), d.W - 1);
            v[rh][rw] = xp[ih * d.W + iw];
        }
    }
    uint32_t even[4], odd[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) even[j] = odd[j] = 0x80008000u;
    auto pk_max = [](uint32_t a, uint32_t b) {
        return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(shortx2, a), __builtin_bit_cast(shortx2, b)));
    };
#pragma unroll
    for (int rh = 0; rh < KH; ++rh)
#pragma unroll
        for (int rw = 0; rw < KW; ++rw) {
            const uint32_t w[4] = {static_cast<uint32_t>(v[rh][rw].x), static_cast<uint32_t>(v[rh][rw].y),
                                   static_cast<uint32_t>(v[rh][rw].z), static_cast<uint32_t>(v[rh][rw].w)};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                even[j] = pk_max(even[j], (w[j] << 8) & 0xff00ff00u);
                odd[j] = pk_max(odd[j], w[j] & 0xff00ff00u);
            }
        }
    uint32_t o[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) o[j] = ((even[j] >> 8) & 0x00ff00ffu) | (odd[j] & 0xff00ff00u);
    reinterpret_cast<int4*>(y)[s] = make_int4(static_cast<int>(o[0]), static_cast<int>(o[1]), static_cast<int>(o[2]), static_cast<int>(o[3]));
}

// Four threads per (n, channel block) plane, each summing one dword (4 channels) of every position; output
// [N][CB*16] (= c16 with H = W = 1).
__global__ void __launch_bounds__(kBlock) gap_c16_kernel(const int8_t* __restrict__ x, int8_t* __restrict__ y,
                                                         int64_t planes, int32_t hw, float mult) {
    const int64_t t = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (t >= planes * 4) return;
    const uint32_t* src = reinterpret_cast<const uint32_t*>(x) + (t >> 2) * hw * 4 + (t & 3);
    int32_t sum[4] = {0, 0, 0, 0};
#pragma unroll 7
    for (int i = 0; i < hw; ++i) {
        const uint32_t v = src[static_cast<int64_t>(i) * 4];
#pragma unroll
        for (int j = 0; j < 4; ++j) sum[j] += static_cast<int32_t>(static_cast<int8_t>((v >> (8 * j)) & 0xff));
    }
    uint32_t o = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j)
        o |= (static_cast<uint32_t>(requant_i32(sum[j], mult, false, 0, 0.0f, false)) & 0xffu) << (8 * j);
    reinterpret_cast<uint32_t*>(y)[t] = o;
}

// ------------------------------------------------------------------ host side
struct QVariant {
    const char* name;
    int kh, kw, cbc, wp, ro, ppt, rp;
    void (*kernel)(const QArgs);
    void (*ds_kernel)(const QArgs);     // with the second output (nullptr: none)
};

#define KXC_QV(KH, KW, CBC, WP, RO, PPT)                                                             \
    { "qmfma_k" #KH "x" #KW "_cb" #CBC "_p" #WP "_o" #RO, KH, KW, CBC, WP, RO, PPT, 1,                   \
      qconv_mfma_kernel<KH, KW, CBC, WP, RO, PPT>, nullptr }
#define KXC_QV_DS(KH, KW, CBC, WP, RO, PPT)                                                          \
    { "qmfma_k" #KH "x" #KW "_cb" #CBC "_p" #WP "_o" #RO, KH, KW, CBC, WP, RO, PPT, 1,                   \
      qconv_mfma_kernel<KH, KW, CBC, WP, RO, PPT>, qconv_mfma_kernel<KH, KW, CBC, WP, RO, PPT, 1, 0, true> }
// (RP pixel blocks per wave, weight ring of WD k-steps)
#define KXC_QV2(KH, KW, CBC, WP, RO, PPT, RP, WD)                                                    \
    { "qmfma_k" #KH "x" #KW "_cb" #CBC "_p" #WP "x" #RP "_o" #RO "_d" #WD, KH, KW, CBC, WP, RO, PPT, RP,  \
      qconv_mfma_kernel<KH, KW, CBC, WP, RO, PPT, RP, WD>, nullptr }

const QVariant kQVariants[] = {
    KXC_QV_DS(3, 3, 2, 4, 2, 4),
    KXC_QV_DS(3, 3, 2, 4, 1, 4),
    KXC_QV_DS(3, 3, 2, 2, 1, 4),
    KXC_QV(1, 1, 4, 4, 2, 6),
    KXC_QV(1, 1, 4, 4, 1, 6),
    KXC_QV(1, 1, 4, 2, 1, 6),
    KXC_QV_DS(3, 3, 1, 4, 1, 4),      // at most 16 input channels: k-steps pair filter taps
    KXC_QV_DS(3, 3, 1, 2, 1, 4),
    KXC_QV(1, 1, 1, 4, 1, 6),
    KXC_QV(1, 1, 1, 2, 1, 6),
    KXC_QV(7, 7, 1, 4, 2, 12),
    KXC_QV(7, 7, 1, 2, 2, 12),
    // two pixel blocks per wave (chosen by the shape rules in PrepareUncached, or by name); a deeper weight ring (nine
    // k-steps, a whole chunk, instead of three) was measured twice on all seven ResNet-18 layer shapes and was never
    // faster (e.g. 512 -> 512 channels at 7 x 7: 14.1 against 13.2 us)
    KXC_QV2(3, 3, 2, 4, 2, 8, 2, 3),
    KXC_QV2(3, 3, 2, 4, 1, 8, 2, 3),
    KXC_QV2(3, 3, 2, 2, 2, 8, 2, 3),
    KXC_QV2(3, 3, 2, 2, 1, 8, 2, 3),
    // 64 channels x 128 pixels per wave (128 accumulator registers): the largest maps only
    KXC_QV2(3, 3, 2, 4, 2, 8, 4, 3),
};

// The same tiles on a compile-time row pitch of 64 positions (qconv_rows_kernel): chosen in place of the variant above
// with the same (window, chunk, waves, blocks per wave) for stride-1 layers whose padded rows take 33 to 64 positions.
struct QRowVariant {
    const char* name;
    int kh, kw, cbc, wp, ro, ppt, rp, p;
    void (*kernel)(const QArgs);
    void (*ds_kernel)(const QArgs);
};
#define KXC_QR(KH, KW, CBC, WP, RO, PPT, RP, P)                                                                    \
    { "qrows_k" #KH "x" #KW "_cb" #CBC "_p" #WP "x" #RP "_o" #RO "_w" #P, KH, KW, CBC, WP, RO, PPT, RP, P,              \
      qconv_rows_kernel<KH, KW, CBC, WP, RO, PPT, RP, P>, nullptr }
#define KXC_QR_DS(KH, KW, CBC, WP, RO, PPT, RP, P)                                                                 \
    { "qrows_k" #KH "x" #KW "_cb" #CBC "_p" #WP "x" #RP "_o" #RO "_w" #P, KH, KW, CBC, WP, RO, PPT, RP, P,              \
      qconv_rows_kernel<KH, KW, CBC, WP, RO, PPT, RP, P>, qconv_rows_kernel<KH, KW, CBC, WP, RO, PPT, RP, P, true> }
const QRowVariant kQRowVariants[] = {
    KXC_QR_DS(3, 3, 2, 4, 2, 4, 1, 64),
    KXC_QR_DS(3, 3, 2, 4, 1, 4, 1, 64),
    KXC_QR_DS(3, 3, 2, 2, 1, 8, 1, 64),
    KXC_QR(3, 3, 2, 4, 2, 4, 2, 64),
    KXC_QR(3, 3, 2, 4, 1, 4, 2, 64),
    KXC_QR(3, 3, 2, 2, 2, 8, 2, 64),
    KXC_QR(3, 3, 2, 2, 1, 8, 2, 64),
    KXC_QR(3, 3, 2, 4, 2, 4, 4, 64),
};

// Channel blocks (of 16 channels) per LDS chunk.  Larger chunks (64 or 128 channels) were measured on the ResNet-18
// layers at batch 64 and were slower everywhere (512 -> 512 channels at 7 x 7: 14.3 -> 15-20 us; 256 -> 512 with
// stride 2: 11 -> 23 us): with few chunks the first, large patch load is exposed and nothing overlaps it.
int CbcFor(int c, int kh, int kw) {
    const int cb = (c + 15) / 16;
    if (cb == 1) return 1;
    if (kh == 1 && kw == 1) return 4;
    return 2;
}

struct QLaunch {
    const QVariant* v = nullptr;
    QArgs args;
    int grid = 0;
    size_t lds_bytes = 0;
    // what is launched: the variant's kernels, or those of the row-pitch variant that replaced it
    const char* name = "";
    void (*kernel)(const QArgs) = nullptr;
    void (*ds_kernel)(const QArgs) = nullptr;
    int threads = 0;
};

// Largest number of patch rows any pixel tile of TP pixels touches.
int MaxRows(const QArgs& a, int KH, int TP) {
    int best = 0;
    for (int m0 = 0; m0 < a.M; m0 += TP) {
        const int ml = (m0 + TP < a.M ? m0 + TP : a.M) - 1;
        const int n = m0 / a.OHW, rem = m0 - n * a.OHW;
        const int n2 = ml / a.OHW, rem2 = ml - n2 * a.OHW;
        const int qmin = n * a.Hp + (rem / a.OW) * a.sh;
        const int qlast = n2 * a.Hp + (rem2 / a.OW) * a.sh + KH - 1;
        if (qlast - qmin + 1 > best) best = qlast - qmin + 1;
    }
    return best;
}

int32_t PrepareUncached(const kxc_hip_qconv2d_desc* d, QLaunch* L, const char* who);

// The selection walks every pixel tile once; a forward pass repeats the same few descriptors, so the last
// results are kept per thread (pointers are filled in by the caller afterwards).
int32_t Prepare(const kxc_hip_qconv2d_desc* d, QLaunch* L, const char* who) {
    KXC_HIP_REQUIRE(d != nullptr, "%s: desc is NULL", who);
    struct Entry { kxc_hip_qconv2d_desc desc; QLaunch launch; };
    thread_local std::vector<Entry> cache;
    if (const char* f = std::getenv("KXC_HIP_QCONV_VARIANT"))
        if (*f) return PrepareUncached(d, L, who);          // forced variants are not cached
    if (std::getenv("KXC_HIP_QCONV_ROWS") || std::getenv("KXC_HIP_QCONV_BIG_TILE")) return PrepareUncached(d, L, who);
    for (const Entry& e : cache)
        if (std::memcmp(&e.desc, d, sizeof(*d)) == 0) { *L = e.launch; return KXC_HIP_OK; }
    if (int32_t rc = PrepareUncached(d, L, who)) return rc;
    if (cache.size() >= 128) cache.clear();
    Entry e;
    std::memcpy(&e.desc, d, sizeof(*d));
    e.launch = *L;
    cache.push_back(e);
    return KXC_HIP_OK;
}

int32_t PrepareUncached(const kxc_hip_qconv2d_desc* d, QLaunch* L, const char* who) {
    KXC_HIP_REQUIRE(d->n >= 0 && d->c > 0 && d->h > 0 && d->w > 0 && d->o > 0 && d->kh > 0 && d->kw > 0,
                    "%s: bad shape", who);
    KXC_HIP_REQUIRE(d->stride_h > 0 && d->stride_w > 0 && d->pad_h >= 0 && d->pad_w >= 0, "%s: bad stride or padding", who);
    const int64_t nh = static_cast<int64_t>(d->h) + 2 * d->pad_h - d->kh;
    const int64_t nw = static_cast<int64_t>(d->w) + 2 * d->pad_w - d->kw;
    KXC_HIP_REQUIRE(nh >= 0 && nw >= 0, "%s: window is larger than input", who);
    KXC_HIP_REQUIRE(d->o % 32 == 0, "%s: output channels must be a multiple of 32 (got %d)", who, d->o);
    KXC_HIP_REQUIRE(static_cast<int64_t>(d->c) * d->kh * d->kw <= 2147483647LL / (128 * 128),
                    "%s: reduction too long for int32 accumulation", who);
    QArgs& a = L->args;
    std::memset(&a, 0, sizeof(a));
    a.N = d->n; a.CB = (d->c + 15) / 16; a.H = d->h; a.W = d->w; a.O = d->o;
    a.OH = static_cast<int32_t>(nh / d->stride_h + 1);
    a.OW = static_cast<int32_t>(nw / d->stride_w + 1);
    a.sh = d->stride_h; a.sw = d->stride_w; a.ph = d->pad_h; a.pw = d->pad_w;
    a.Hp = a.H + 2 * a.ph; a.Wp = a.W + 2 * a.pw;
    a.OHW = a.OH * a.OW;
    const int64_t M = static_cast<int64_t>(a.N) * a.OHW;
    const int64_t xb = static_cast<int64_t>(a.N) * a.CB * a.H * a.W * 16;
    KXC_HIP_REQUIRE(M < (1LL << 30) && xb < (1LL << 31) && M * (a.O / 16) * 16 < (1LL << 31) &&
                    static_cast<int64_t>(a.N + 1) * a.Hp * a.Wp < (1LL << 30),
                    "%s: tensor too large for 32-bit addressing", who);
    a.M = static_cast<int32_t>(M);
    a.x_bytes = static_cast<uint32_t>(xb);
    a.res_mult = d->res_mult;
    a.flags = d->flags;
    const int cbc = CbcFor(d->c, d->kh, d->kw);
    a.nchunks = (a.CB + cbc - 1) / cbc;
    if (M == 0) return KXC_HIP_OK;
    // pick the first variant that fits, preferring enough workgroups to fill 256 CUs a few times over
    const QVariant* best = nullptr;
    int best_chs = 0;
    const char* forced = std::getenv("KXC_HIP_QCONV_VARIANT");        // a variant by name (kernel experiments, tests)
    // Shape rules, from a sweep of every 3x3 variant over the ResNet-18 layers at batch 64 (the kernels are bound by
    // instruction issue around the matrix instructions, so fewer, larger per-wave tiles win while there are enough
    // pixels): stride 1 with at least 8192 output pixels takes two pixel blocks per wave (64 -> 64 channels at 56 x 56:
    // 21.4 -> 17.7 us; 128 at 28 x 28: 17.8 -> 13.6; 256 at 14 x 14: 15.4 -> 12.4), stride 2 two output-channel
    // blocks per wave (128 -> 256 at 28 -> 14: 11.7 -> 10.2 us); the small 7 x 7 maps keep one block per wave.
    if (!(forced && *forced) && d->kh == 3 && d->kw == 3 && cbc == 2) {
        // (a wave that takes 64 channels x 128 pixels feeds four matrix instructions from every weight fragment and two
        // from every pixel fragment, but at 210 registers only two such workgroups fit a compute unit: it wins where its
        // tiles fill those 512 places well -- 64 -> 64 channels at 56 x 56: 14.2 -> 13.8 us at batch 64 (392 tiles) and
        // 26.7 -> 26.3 at batch 128 (784), the quantised ResNet-18 0.2993 -> 0.2924 ms per batch of 64 -- and loses where
        // they do not: 8.6 -> 9.4 us at batch 32 (196 tiles), 20.4 -> 21.1 at batch 96 (588); on the 28 x 28 and
        // smaller maps it is 10-60 % slower than two pixel blocks of one channel block)
        if (d->stride_h == 1 && d->stride_w == 1 && M >= 8192) {
            const char* big = std::getenv("KXC_HIP_QCONV_BIG_TILE");       // 0: never the 64 x 128 tile, 1: from 100 000 pixels on
            bool big_ok = M >= 100000 && (a.O / 32) % 2 == 0 && !(big && big[0] == '0');
            if (big_ok && !(big && big[0] == '1')) {
                const int64_t tiles = CeilDiv(M, 512) * (a.O / 64), rounds = CeilDiv(tiles, 512);
                big_ok = 10 * tiles >= 7 * rounds * 512;
            }
            forced = M >= 100000 ? (big_ok ? "qmfma_k3x3_cb2_p4x4_o2_d3" : "qmfma_k3x3_cb2_p4x2_o1_d3") : "qmfma_k3x3_cb2_p2x2_o1_d3";
        }
        else if (d->stride_h == 2 && d->stride_w == 2 && (a.O / 32) % 2 == 0 && M >= 2048) forced = "qmfma_k3x3_cb2_p4_o2";
    }
    const bool by_rule = forced && *forced && !(std::getenv("KXC_HIP_QCONV_VARIANT") && *std::getenv("KXC_HIP_QCONV_VARIANT"));
    for (int pass = 0; pass < 2 && best == nullptr; ++pass) {
    if (pass == 1) {
        if (!by_rule) break;
        forced = nullptr;           // the rule's variant does not hold this shape's patch: walk the table
    }
    for (const QVariant& v : kQVariants) {
        if (v.kh != d->kh || v.kw != d->kw || v.cbc != cbc) continue;
        if ((a.O / 32) % v.ro != 0) continue;
        if (forced && *forced ? std::strcmp(forced, v.name) != 0 : v.rp != 1 || std::strstr(v.name, "_d") != nullptr) continue;
        const int TP = 32 * v.wp * v.rp;
        const int rows = MaxRows(a, v.kh, TP);
        const int positions = rows * a.Wp;
        const int segs = (positions + 63) / 64;
        if (segs > v.ppt * v.wp) continue;
        const int chs = segs * 64;
        const size_t buf = static_cast<size_t>(cbc) * chs * 16;      // the patch only; weights stream from memory
        const size_t lds = buf * (a.nchunks > 1 ? 2 : 1);
        if (lds > 160 * 1024) continue;
        const int64_t tiles = CeilDiv(M, TP) * ((a.O / 32) / v.ro);
        if (best == nullptr) { best = &v; best_chs = chs; L->lds_bytes = lds; }
        if (tiles >= 2 * 256 || (forced && *forced)) { best = &v; best_chs = chs; L->lds_bytes = lds; break; }
    }
    }
    KXC_HIP_REQUIRE(best != nullptr, "%s: no matrix-core variant for a %dx%d filter on this shape", who, d->kh, d->kw);
    a.chs = best_chs;
    a.p_tiles = static_cast<int32_t>(CeilDiv(M, 32 * best->wp * best->rp));
    a.o_tiles = (a.O / 32) / best->ro;
    a.num_tiles = a.p_tiles * a.o_tiles;
    a.tiles_per_xcd = (a.num_tiles + 7) / 8;
    a.div_wp = MakeFastDiv(a.Wp); a.div_hp = MakeFastDiv(a.Hp); a.div_ohw = MakeFastDiv(a.OHW);
    a.div_ow = MakeFastDiv(a.OW); a.div_otiles = MakeFastDiv(a.o_tiles);
    L->grid = a.tiles_per_xcd * 8;
    L->v = best;
    L->name = best->name; L->kernel = best->kernel; L->ds_kernel = best->ds_kernel; L->threads = 64 * best->wp;
    const int NS = (best->kh * best->kw * cbc + 1) / 2;
    a.w_bytes = static_cast<uint32_t>(static_cast<int64_t>(a.O / 32) * a.nchunks * NS * 1024);
    // the same tile on a compile-time row pitch for stride-1 layers whose padded rows take 33 to 64 positions
    // (KXC_HIP_QCONV_ROWS=0: never)
    const char* rows_env = std::getenv("KXC_HIP_QCONV_ROWS");
    const int pitch = a.Wp > 32 && a.Wp <= 64 && d->stride_h == 1 && d->stride_w == 1 ? 64 : 0;
    if (pitch != 0 && !(rows_env && rows_env[0] == '0')) {
        for (const QRowVariant& rv : kQRowVariants) {
            if (rv.kh != best->kh || rv.kw != best->kw || rv.cbc != cbc || rv.wp != best->wp || rv.ro != best->ro ||
                rv.rp != best->rp || rv.p != pitch)
                continue;
            if (best->ds_kernel != nullptr && rv.ds_kernel == nullptr) continue;      // keep the second output available
            const int rows = MaxRows(a, rv.kh, 32 * rv.wp * rv.rp);
            const int nslots = (rows * pitch + 63) / 64;
            if (nslots > rv.ppt * rv.wp) continue;
            const size_t lds = static_cast<size_t>(cbc) * nslots * 1024 * (a.nchunks > 1 ? 2 : 1);
            if (lds > 160 * 1024) continue;
            a.chs = nslots * 64;
            L->lds_bytes = lds;
            L->name = rv.name; L->kernel = rv.kernel; L->ds_kernel = rv.ds_kernel; L->threads = 64 * rv.wp;
            break;
        }
    }
    return KXC_HIP_OK;
}

}  // namespace

extern "C" {

int32_t kxc_hip_qconv2d_c16_packed_bytes(const kxc_hip_qconv2d_desc* d, size_t* out_bytes) {
    KXC_HIP_REQUIRE(d != nullptr && out_bytes != nullptr, "kxc_hip_qconv2d_c16_packed_bytes: NULL argument");
    KXC_HIP_REQUIRE(d->c > 0 && d->o > 0 && d->kh > 0 && d->kw > 0 && d->o % 32 == 0,
                    "kxc_hip_qconv2d_c16_packed_bytes: bad shape (output channels must be a multiple of 32)");
    const int cbc = CbcFor(d->c, d->kh, d->kw);
    const int cb = (d->c + 15) / 16;
    const int64_t nchunks = (cb + cbc - 1) / cbc;
    const int64_t NS = (static_cast<int64_t>(d->kh) * d->kw * cbc + 1) / 2;
    *out_bytes = static_cast<size_t>((d->o / 32) * nchunks * NS * 1024);
    return KXC_HIP_OK;
}

int32_t kxc_hip_qconv2d_c16_pack_weights(const kxc_hip_qconv2d_desc* d, const int8_t* w_oihw, int8_t* packed,
                                         void* stream) {
    size_t bytes = 0;
    if (int32_t rc = kxc_hip_qconv2d_c16_packed_bytes(d, &bytes)) return rc;
    KXC_HIP_REQUIRE(w_oihw && packed, "kxc_hip_qconv2d_c16_pack_weights: NULL pointer");
    PackArgs p;
    p.w = w_oihw; p.wp = packed; p.O = d->o; p.C = d->c; p.KHW = d->kh * d->kw;
    p.CBC = CbcFor(d->c, d->kh, d->kw);
    p.NS = (p.KHW * p.CBC + 1) / 2;
    p.nchunks = ((d->c + 15) / 16 + p.CBC - 1) / p.CBC;
    p.oblocks = d->o / 32;
    const int64_t slots = static_cast<int64_t>(bytes / 16);
    pack_weights_kernel<<<NoteGrid(static_cast<int>(CeilDiv(slots, kBlock))), NoteBlock(kBlock), NoteLds(0), ResolveStream(stream)>>>(p, slots);
    return CheckLaunch("qconv2d_c16_pack_weights");
}

const char* kxc_hip_qconv2d_c16_variant(const kxc_hip_qconv2d_desc* d) {
    QLaunch L;
    if (Prepare(d, &L, "kxc_hip_qconv2d_c16_variant") != KXC_HIP_OK) return "none";
    return L.v ? L.name : "empty";
}

int32_t kxc_hip_qconv2d_c16_i8(const kxc_hip_qconv2d_desc* d, const int8_t* x, const int8_t* w_packed,
                               const int32_t* bias, const float* mult, const int8_t* residual, int8_t* y,
                               void* stream) {
    QLaunch L;
    if (int32_t rc = Prepare(d, &L, "kxc_hip_qconv2d_c16_i8")) return rc;
    if (L.args.M == 0) return KXC_HIP_OK;
    KXC_HIP_REQUIRE(x && w_packed && mult && y, "kxc_hip_qconv2d_c16_i8: NULL pointer");
    KXC_HIP_REQUIRE(!(d->flags & KXC_HIP_CONV_BIAS) || bias, "kxc_hip_qconv2d_c16_i8: bias flag without bias");
    KXC_HIP_REQUIRE(!(d->flags & KXC_HIP_CONV_RESIDUAL) || residual, "kxc_hip_qconv2d_c16_i8: residual flag without residual");
    QArgs& a = L.args;
    a.x = x; a.wp = w_packed; a.bias = bias; a.mult = mult; a.res = residual; a.y = y;
    if (L.lds_bytes > 64 * 1024) {
        KXC_HIP_CALL(hipFuncSetAttribute(reinterpret_cast<const void*>(L.kernel),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(L.lds_bytes)),
                     "hipFuncSetAttribute");
    }
    hipLaunchKernelGGL(L.kernel, NoteGrid(dim3(L.grid)), NoteBlock(dim3(L.threads)), NoteLds(L.lds_bytes), ResolveStream(stream), a);
    return CheckLaunch(L.name);
}

// ---- two outputs from one launch: the convolution and a 1x1 convolution with the same strides, no padding
// The second output's operand must be a tap of the window (pad < filter size) and the unpadded 1x1 convolution must
// have this convolution's output extent (true for "same" padding, 2*pad = k-1).
static bool PairGeometry(const kxc_hip_qconv2d_desc* d) {
    if (!d || d->pad_h >= d->kh || d->pad_w >= d->kw || d->stride_h <= 0 || d->stride_w <= 0) return false;
    const int64_t oh = (static_cast<int64_t>(d->h) + 2 * d->pad_h - d->kh) / d->stride_h + 1;
    const int64_t ow = (static_cast<int64_t>(d->w) + 2 * d->pad_w - d->kw) / d->stride_w + 1;
    return oh == (d->h - 1) / d->stride_h + 1 && ow == (d->w - 1) / d->stride_w + 1;
}

int32_t kxc_hip_qconv2d_c16_pair_supported(const kxc_hip_qconv2d_desc* d) {
    QLaunch L;
    if (!PairGeometry(d)) return 0;
    if (Prepare(d, &L, "kxc_hip_qconv2d_c16_pair_supported") != KXC_HIP_OK) { LastError().clear(); return 0; }
    return (L.v && L.ds_kernel) ? 1 : 0;
}

int32_t kxc_hip_qconv2d_c16_pair_packed_bytes(const kxc_hip_qconv2d_desc* d, size_t* out_bytes) {
    KXC_HIP_REQUIRE(d != nullptr && out_bytes != nullptr, "kxc_hip_qconv2d_c16_pair_packed_bytes: NULL argument");
    KXC_HIP_REQUIRE(d->c > 0 && d->o > 0 && d->kh > 0 && d->kw > 0 && d->o % 32 == 0,
                    "kxc_hip_qconv2d_c16_pair_packed_bytes: bad shape (output channels must be a multiple of 32)");
    const int cbc = CbcFor(d->c, d->kh, d->kw);
    const int64_t nchunks = ((d->c + 15) / 16 + cbc - 1) / cbc;
    *out_bytes = static_cast<size_t>((d->o / 32) * nchunks * ((cbc + 1) / 2) * 1024);
    return KXC_HIP_OK;
}

// w2_oihw: [o, c, 1, 1] int8; packed in the chunking of the convolution `d` describes
int32_t kxc_hip_qconv2d_c16_pair_pack_weights(const kxc_hip_qconv2d_desc* d, const int8_t* w2_oihw, int8_t* packed, void* stream) {
    size_t bytes = 0;
    if (int32_t rc = kxc_hip_qconv2d_c16_pair_packed_bytes(d, &bytes)) return rc;
    KXC_HIP_REQUIRE(w2_oihw && packed, "kxc_hip_qconv2d_c16_pair_pack_weights: NULL pointer");
    PackArgs p;
    p.w = w2_oihw; p.wp = packed; p.O = d->o; p.C = d->c; p.KHW = 1;
    p.CBC = CbcFor(d->c, d->kh, d->kw);
    p.NS = (p.CBC + 1) / 2;
    p.nchunks = ((d->c + 15) / 16 + p.CBC - 1) / p.CBC;
    p.oblocks = d->o / 32;
    const int64_t slots = static_cast<int64_t>(bytes / 16);
    pack_weights_kernel<<<NoteGrid(static_cast<int>(CeilDiv(slots, kBlock))), NoteBlock(kBlock), NoteLds(0), ResolveStream(stream)>>>(p, slots);
    return CheckLaunch("qconv2d_c16_pair_pack_weights");
}

int32_t kxc_hip_qconv2d_c16_pair_i8(const kxc_hip_qconv2d_desc* d, const int8_t* x, const int8_t* w_packed, const int32_t* bias,
                                    const float* mult, const int8_t* residual, int8_t* y, const int8_t* w2_packed,
                                    const int32_t* bias2, const float* mult2, int8_t* y2, void* stream) {
    const char* who = "kxc_hip_qconv2d_c16_pair_i8";
    QLaunch L;
    if (int32_t rc = Prepare(d, &L, who)) return rc;
    KXC_HIP_REQUIRE(L.v && L.ds_kernel && PairGeometry(d), "%s: no kernel with a second output covers this shape", who);
    if (L.args.M == 0) return KXC_HIP_OK;
    KXC_HIP_REQUIRE(x && w_packed && mult && y && w2_packed && mult2 && y2, "%s: NULL pointer", who);
    KXC_HIP_REQUIRE(!(d->flags & KXC_HIP_CONV_BIAS) || bias, "%s: bias flag without bias", who);
    KXC_HIP_REQUIRE(!(d->flags & KXC_HIP_CONV_RESIDUAL) || residual, "%s: residual flag without residual", who);
    QArgs& a = L.args;
    a.x = x; a.wp = w_packed; a.bias = bias; a.mult = mult; a.res = residual; a.y = y;
    a.wp2 = w2_packed; a.bias2 = bias2; a.mult2 = mult2; a.y2 = y2;
    a.w2_bytes = static_cast<uint32_t>(static_cast<int64_t>(a.O / 32) * a.nchunks * ((L.v->cbc + 1) / 2) * 1024);
    // the second output's tap in the staged patch: rows are Wp positions apart, or the row pitch of a qrows variant
    int row_positions = a.Wp;
    if (std::strncmp(L.name, "qrows", 5) == 0) row_positions = 64;
    a.ds_off = (d->pad_h * row_positions + d->pad_w) * 16;
    if (L.lds_bytes > 64 * 1024) {
        KXC_HIP_CALL(hipFuncSetAttribute(reinterpret_cast<const void*>(L.ds_kernel),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(L.lds_bytes)),
                     "hipFuncSetAttribute");
    }
    hipLaunchKernelGGL(L.ds_kernel, NoteGrid(dim3(L.grid)), NoteBlock(dim3(L.threads)), NoteLds(L.lds_bytes), ResolveStream(stream), a);
    return CheckLaunch(L.name);
}

int32_t kxc_hip_i8_nchw_to_c16(const int8_t* x, int8_t* y, int64_t n, int64_t c, int64_t hw, void* stream) {
    KXC_HIP_REQUIRE(n >= 0 && c > 0 && hw >= 0, "kxc_hip_i8_nchw_to_c16: bad shape");
    const int64_t cb = (c + 15) / 16, total = n * cb * hw;
    if (total == 0) return KXC_HIP_OK;
    KXC_HIP_REQUIRE(x && y, "kxc_hip_i8_nchw_to_c16: NULL pointer");
    KXC_HIP_REQUIRE(CeilDiv(total, kBlock) <= kMaxGridX, "kxc_hip_i8_nchw_to_c16: tensor too large");
    nchw_to_c16_kernel<<<NoteGrid(static_cast<int>(CeilDiv(total, kBlock))), NoteBlock(kBlock), NoteLds(0), ResolveStream(stream)>>>(
        x, y, static_cast<int32_t>(c), static_cast<int32_t>(cb), hw, total);
    return CheckLaunch("i8_nchw_to_c16");
}

int32_t kxc_hip_i8_c16_to_nchw(const int8_t* x, int8_t* y, int64_t n, int64_t c, int64_t hw, void* stream) {
    KXC_HIP_REQUIRE(n >= 0 && c > 0 && hw >= 0, "kxc_hip_i8_c16_to_nchw: bad shape");
    const int64_t cb = (c + 15) / 16, total = n * c * hw;
    if (total == 0) return KXC_HIP_OK;
    KXC_HIP_REQUIRE(x && y, "kxc_hip_i8_c16_to_nchw: NULL pointer");
    KXC_HIP_REQUIRE(CeilDiv(total, kBlock) <= kMaxGridX, "kxc_hip_i8_c16_to_nchw: tensor too large");
    c16_to_nchw_kernel<<<NoteGrid(static_cast<int>(CeilDiv(total, kBlock))), NoteBlock(kBlock), NoteLds(0), ResolveStream(stream)>>>(
        x, y, static_cast<int32_t>(c), static_cast<int32_t>(cb), hw, total);
    return CheckLaunch("i8_c16_to_nchw");
}

int32_t kxc_hip_quantize_f32_nchw_to_c16_i8(const float* x, int8_t* y, int64_t n, int64_t c, int64_t hw, float scale,
                                            void* stream) {
    KXC_HIP_REQUIRE(n >= 0 && c > 0 && hw >= 0, "kxc_hip_quantize_f32_nchw_to_c16_i8: bad shape");
    KXC_HIP_REQUIRE(scale > 0.0f, "kxc_hip_quantize_f32_nchw_to_c16_i8: scale must be positive");
    const int64_t cb = (c + 15) / 16, total = n * cb * hw;
    if (total == 0) return KXC_HIP_OK;
    KXC_HIP_REQUIRE(x && y, "kxc_hip_quantize_f32_nchw_to_c16_i8: NULL pointer");
    KXC_HIP_REQUIRE(CeilDiv(total, kBlock) <= kMaxGridX, "kxc_hip_quantize_f32_nchw_to_c16_i8: tensor too large");
    quantize_to_c16_kernel<<<NoteGrid(static_cast<int>(CeilDiv(total, kBlock))), NoteBlock(kBlock), NoteLds(0), ResolveStream(stream)>>>(
        x, y, static_cast<int32_t>(c), static_cast<int32_t>(cb), hw, total, scale);
    return CheckLaunch("quantize_f32_nchw_to_c16_i8");
}

int32_t kxc_hip_maxpool2d_c16_i8(const kxc_hip_pool2d_desc* p, const int8_t* x, int8_t* y, void* stream) {
    KXC_HIP_REQUIRE(p != nullptr, "kxc_hip_maxpool2d_c16_i8: desc is NULL");
    KXC_HIP_REQUIRE(p->n >= 0 && p->c > 0 && p->h > 0 && p->w > 0, "kxc_hip_maxpool2d_c16_i8: bad input shape");
    KXC_HIP_REQUIRE(p->kh > 0 && p->kw > 0 && p->stride_h > 0 && p->stride_w > 0, "kxc_hip_maxpool2d_c16_i8: bad window");
    KXC_HIP_REQUIRE(p->pad_top >= 0 && p->pad_left >= 0 && p->pad_bottom >= 0 && p->pad_right >= 0,
                    "kxc_hip_maxpool2d_c16_i8: negative padding");
    KXC_HIP_REQUIRE(!p->is_avg, "kxc_hip_maxpool2d_c16_i8: average pooling is not defined for int8");
    const int hn = p->h + p->pad_top + p->pad_bottom - p->kh;
    const int wn = p->w + p->pad_left + p->pad_right - p->kw;
    KXC_HIP_REQUIRE(hn >= 0 && wn >= 0, "kxc_hip_maxpool2d_c16_i8: pool2d window is larger than input");
    PoolArgs d;
    d.N = p->n; d.CB = (p->c + 15) / 16; d.H = p->h; d.W = p->w;
    d.OH = p->ceil_mode ? (hn + p->stride_h - 1) / p->stride_h + 1 : hn / p->stride_h + 1;
    d.OW = p->ceil_mode ? (wn + p->stride_w - 1) / p->stride_w + 1 : wn / p->stride_w + 1;
    d.KH = p->kh; d.KW = p->kw; d.sh = p->stride_h; d.sw = p->stride_w; d.pt = p->pad_top; d.pl = p->pad_left;
    const int64_t total = static_cast<int64_t>(d.N) * d.CB * d.OH * d.OW;
    if (total == 0) return KXC_HIP_OK;
    KXC_HIP_REQUIRE(x && y, "kxc_hip_maxpool2d_c16_i8: NULL pointer");
    KXC_HIP_REQUIRE(CeilDiv(total, kBlock) <= kMaxGridX, "kxc_hip_maxpool2d_c16_i8: tensor too large");
    // every placement of a 3x3 window meets the input (first window's last row / column, last window's first)
    const bool meets = d.pt <= d.KH - 1 && d.pl <= d.KW - 1 && (d.OH - 1) * d.sh - d.pt <= d.H - 1 && (d.OW - 1) * d.sw - d.pl <= d.W - 1;
    const int64_t in_words = static_cast<int64_t>(d.N) * d.CB * d.H * d.W;
    if (d.KH == 3 && d.KW == 3 && meets && total < (1LL << 31) && in_words < (1LL << 31) &&
        ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) & 15u) == 0) {
        maxpool_c16_window_kernel<3, 3><<<NoteGrid(static_cast<int>(CeilDiv(total, kBlock))), NoteBlock(kBlock), NoteLds(0), ResolveStream(stream)>>>(
            x, y, d, static_cast<int32_t>(total));
        return CheckLaunch("maxpool2d_c16_i8");
    }
    maxpool_c16_kernel<<<NoteGrid(static_cast<int>(CeilDiv(total, kBlock))), NoteBlock(kBlock), NoteLds(0), ResolveStream(stream)>>>(x, y, d, total);
    return CheckLaunch("maxpool2d_c16_i8");
}

int32_t kxc_hip_global_avg_pool2d_c16_i8(const int8_t* x, int8_t* y, int64_t n, int64_t c, int64_t h, int64_t w,
                                         float mult, void* stream) {
    KXC_HIP_REQUIRE(n >= 0 && c > 0 && h > 0 && w > 0, "kxc_hip_global_avg_pool2d_c16_i8: bad shape");
    KXC_HIP_REQUIRE(h * w <= 2147483647LL / 128, "kxc_hip_global_avg_pool2d_c16_i8: plane too large for int32 sum");
    const int64_t planes = n * ((c + 15) / 16);
    if (planes == 0) return KXC_HIP_OK;
    KXC_HIP_REQUIRE(x && y, "kxc_hip_global_avg_pool2d_c16_i8: NULL pointer");
    gap_c16_kernel<<<NoteGrid(static_cast<int>(CeilDiv(planes * 4, kBlock))), NoteBlock(kBlock), NoteLds(0), ResolveStream(stream)>>>(
        x, y, planes, static_cast<int32_t>(h * w), mult);
    return CheckLaunch("global_avg_pool2d_c16_i8");
}

}  // extern "C"

// ---- first layer on the c4 layout
namespace {

struct K7Variant { const char* name; int wp, ro, ppt; void (*kernel)(const QArgs); };
const K7Variant kK7Variants[] = {
    {"qmfma_k7x7s2_c4_p4_o2", 4, 2, 4, qconv_k7s2_c4_kernel<4, 2, 4>},
    {"qmfma_k7x7s2_c4_p4_o1", 4, 1, 4, qconv_k7s2_c4_kernel<4, 1, 4>},
    {"qmfma_k7x7s2_c4_p2_o1", 2, 1, 8, qconv_k7s2_c4_kernel<2, 1, 8>},
};

// select_variant = false: only the geometry (the kernel with the pool has its own tiling)
int32_t PrepareK7(const kxc_hip_qconv2d_desc* d, QLaunch* L, const K7Variant** out, const char* who, bool select_variant = true) {
    KXC_HIP_REQUIRE(d != nullptr, "%s: desc is NULL", who);
    KXC_HIP_REQUIRE(d->kh == 7 && d->kw == 7 && d->stride_h == 2 && d->stride_w == 2 && d->pad_h == 3 && d->pad_w == 3,
                    "%s: only a 7x7 filter with stride 2 and padding 3 runs on the c4 layout", who);
    KXC_HIP_REQUIRE(d->c >= 1 && d->c <= 4, "%s: at most 4 input channels (got %d)", who, d->c);
    KXC_HIP_REQUIRE(d->n >= 0 && d->h >= 1 && d->w >= 4 && d->w % 4 == 0, "%s: width must be a positive multiple of 4", who);
    KXC_HIP_REQUIRE(d->o > 0 && d->o % 32 == 0, "%s: output channels must be a multiple of 32 (got %d)", who, d->o);
    KXC_HIP_REQUIRE(!(d->flags & KXC_HIP_CONV_RESIDUAL), "%s: no residual operand on the first layer", who);
    QArgs& a = L->args;
    std::memset(&a, 0, sizeof(a));
    a.N = d->n; a.CB = 1; a.H = d->h; a.W = d->w; a.O = d->o;
    a.OH = (d->h + 6 - 7) / 2 + 1;
    a.OW = (d->w + 6 - 7) / 2 + 1;
    a.sh = a.sw = 2; a.ph = a.pw = 3;
    a.Hp = a.H + 6; a.Wp = a.W + 6;
    a.OHW = a.OH * a.OW;
    const int64_t M = static_cast<int64_t>(a.N) * a.OHW;
    const int64_t xb = static_cast<int64_t>(a.N) * a.H * a.W * 4;
    KXC_HIP_REQUIRE(M < (1LL << 30) && xb < (1LL << 31) && M * a.O < (1LL << 31) &&
                    static_cast<int64_t>(a.N + 1) * a.Hp * (a.W / 4 + 2) < (1LL << 26),
                    "%s: tensor too large for 32-bit addressing", who);
    a.M = static_cast<int32_t>(M);
    a.x_bytes = static_cast<uint32_t>(xb);
    a.flags = d->flags;
    a.nchunks = 1;
    a.w_bytes = static_cast<uint32_t>((a.O / 32) * 7 * 1024);
    *out = nullptr;
    if (M == 0) return KXC_HIP_OK;
    const int W4 = a.W / 4 + 2;
    a.div_wp = MakeFastDiv(W4); a.div_hp = MakeFastDiv(a.Hp); a.div_ohw = MakeFastDiv(a.OHW);
    a.div_ow = MakeFastDiv(a.OW);
    if (!select_variant) return KXC_HIP_OK;
    for (const K7Variant& v : kK7Variants) {
        if ((a.O / 32) % v.ro != 0) continue;
        const int rows = MaxRows(a, 7, 32 * v.wp);
        const int segs = (rows * W4 + 63) / 64;
        if (segs > v.ppt * v.wp) continue;
        const size_t lds = static_cast<size_t>(segs) * 1024 + static_cast<size_t>(v.ro) * 7 * 1024;
        if (lds > 160 * 1024) continue;
        const int64_t tiles = CeilDiv(M, 32 * v.wp) * ((a.O / 32) / v.ro);
        if (*out == nullptr || tiles >= 2 * 256) {
            *out = &v; a.chs = segs * 64; L->lds_bytes = lds;
            if (tiles >= 2 * 256) break;
        }
    }
    KXC_HIP_REQUIRE(*out != nullptr, "%s: image rows too wide for the first-layer kernel (width %d)", who, d->w);
    a.p_tiles = static_cast<int32_t>(CeilDiv(M, 32 * (*out)->wp));
    a.o_tiles = (a.O / 32) / (*out)->ro;
    a.num_tiles = a.p_tiles * a.o_tiles;
    a.tiles_per_xcd = (a.num_tiles + 7) / 8;
    a.div_otiles = MakeFastDiv(a.o_tiles);
    L->grid = a.tiles_per_xcd * 8;
    return KXC_HIP_OK;
}

// The first layer with the max pool in the same kernel: the first-layer conditions, a pooled width the four waves
// cover (15 windows each), and rows per workgroup chosen so that the launch has about two workgroups per compute
// unit (KXC_HIP_QPOOL_ROWS forces it).
struct K7PoolLaunch {
    QArgs args;
    void (*kernel)(const QArgs) = nullptr;
    const char* name = "";
    int grid = 0;
    size_t lds_bytes = 0;
};

int32_t PrepareK7Pool(const kxc_hip_qconv2d_desc* d, K7PoolLaunch* L, const char* who) {
    QLaunch base;
    const K7Variant* unused = nullptr;
    if (int32_t rc = PrepareK7(d, &base, &unused, who, false)) return rc;
    QArgs& a = L->args;
    a = base.args;
    a.POH = (a.OH - 1) / 2 + 1;       // (OH + 2*1 - 3) / 2 + 1
    a.PW = (a.OW - 1) / 2 + 1;
    KXC_HIP_REQUIRE(a.PW <= 60, "%s: the pooled map is %d columns wide, the kernel covers 60", who, a.PW);
    KXC_HIP_REQUIRE(static_cast<int64_t>(a.N) * a.O * a.POH * a.PW < (1LL << 31), "%s: tensor too large for 32-bit addressing", who);
    if (a.M == 0) return KXC_HIP_OK;
    const int ro = (a.O / 32) % 2 == 0 ? 2 : 1;
    a.o_tiles = (a.O / 32) / ro;
    const int W4 = a.W / 4 + 2;
    // measured on the 224 x 224 first layer (us, rows 2 / 3 / 4 / 5 / 7 / 8): batch 16 10.8 / 13.7 / 11.5 / 13.2 / 17.2 /
    // 19.1, batch 32 19.0 / 19.8 / 17.0 / 20.0 / 17.6 / 19.4, batch 64 30.9 / 30.1 / 30.4 / 29.4 / 27.1 / 29.9, batch 128
    // 59.1 / 55.9 / 51.2 / 53.8 / 49.8 / 55.3: as many rows as leave about two workgroups per compute unit, at most 7
    int rows = 1;
    for (int r = 7; r >= 1; --r) {
        rows = r;
        if (static_cast<int64_t>(a.N) * CeilDiv(a.POH, r) * a.o_tiles >= 448) break;
    }
    if (const char* e = std::getenv("KXC_HIP_QPOOL_ROWS")) {
        const int f = std::atoi(e);
        if (f >= 1 && f <= 16) rows = f;
    }
    if (rows > a.POH) rows = a.POH;
    size_t lds = 0;
    for (;; --rows) {
        const int segs = ((4 * rows + 7) * W4 + 63) / 64;
        lds = static_cast<size_t>(segs) * 1024 + static_cast<size_t>(ro) * 7 * 1024;
        a.chs = segs * 64;
        if (lds <= 64 * 1024 || rows == 1) break;
    }
    KXC_HIP_REQUIRE(lds <= 64 * 1024, "%s: image rows too wide for the first-layer kernel (width %d)", who, d->w);
    a.pool_rows = rows;
    a.pool_tiles = static_cast<int32_t>(CeilDiv(a.POH, rows));
    a.div_pool_tiles = MakeFastDiv(a.pool_tiles);
    a.p_tiles = a.N * a.pool_tiles;
    a.num_tiles = a.p_tiles * a.o_tiles;
    a.tiles_per_xcd = (a.num_tiles + 7) / 8;
    a.div_otiles = MakeFastDiv(a.o_tiles);
    const bool relu = (a.flags & KXC_HIP_CONV_RELU) != 0;
    L->kernel = ro == 2 ? (relu ? qconv_k7s2_c4_pool_kernel<2, true> : qconv_k7s2_c4_pool_kernel<2, false>)
                        : (relu ? qconv_k7s2_c4_pool_kernel<1, true> : qconv_k7s2_c4_pool_kernel<1, false>);
    L->name = ro == 2 ? "qmfma_k7x7s2_c4_o2_maxpool3x3s2" : "qmfma_k7x7s2_c4_o1_maxpool3x3s2";
    L->grid = a.tiles_per_xcd * 8;
    L->lds_bytes = lds;
    return KXC_HIP_OK;
}

}  // namespace

extern "C" {

int32_t kxc_hip_qconv2d_c4_maxpool_supported(const kxc_hip_qconv2d_desc* d) {
    if (!d) return 0;
    K7PoolLaunch L;
    if (PrepareK7Pool(d, &L, "kxc_hip_qconv2d_c4_maxpool_supported") != KXC_HIP_OK) { LastError().clear(); return 0; }
    return 1;
}

int32_t kxc_hip_qconv2d_c4_maxpool_i8(const kxc_hip_qconv2d_desc* d, const int8_t* x_c4, const int8_t* w_packed,
                                      const int32_t* bias, const float* mult, int8_t* y_c16, void* stream) {
    K7PoolLaunch L;
    if (int32_t rc = PrepareK7Pool(d, &L, "kxc_hip_qconv2d_c4_maxpool_i8")) return rc;
    if (L.args.M == 0) return KXC_HIP_OK;
    KXC_HIP_REQUIRE(x_c4 && w_packed && mult && y_c16, "kxc_hip_qconv2d_c4_maxpool_i8: NULL pointer");
    KXC_HIP_REQUIRE(!(d->flags & KXC_HIP_CONV_BIAS) || bias, "kxc_hip_qconv2d_c4_maxpool_i8: bias flag without bias");
    QArgs& a = L.args;
    a.x = x_c4; a.wp = w_packed; a.bias = bias; a.mult = mult; a.res = nullptr; a.y = y_c16;
    hipLaunchKernelGGL(L.kernel, NoteGrid(dim3(L.grid)), NoteBlock(dim3(256)), NoteLds(L.lds_bytes), ResolveStream(stream), a);
    return CheckLaunch(L.name);
}

int32_t kxc_hip_qconv2d_c4_packed_bytes(const kxc_hip_qconv2d_desc* d, size_t* out_bytes) {
    KXC_HIP_REQUIRE(d != nullptr && out_bytes != nullptr, "kxc_hip_qconv2d_c4_packed_bytes: NULL argument");
    KXC_HIP_REQUIRE(d->kh == 7 && d->kw == 7 && d->c >= 1 && d->c <= 4 && d->o > 0 && d->o % 32 == 0,
                    "kxc_hip_qconv2d_c4_packed_bytes: needs a 7x7 filter, at most 4 input channels, output channels a multiple of 32");
    *out_bytes = static_cast<size_t>(d->o / 32) * 7 * 1024;
    return KXC_HIP_OK;
}

int32_t kxc_hip_qconv2d_c4_pack_weights(const kxc_hip_qconv2d_desc* d, const int8_t* w_oihw, int8_t* packed, void* stream) {
    size_t bytes = 0;
    if (int32_t rc = kxc_hip_qconv2d_c4_packed_bytes(d, &bytes)) return rc;
    KXC_HIP_REQUIRE(w_oihw && packed, "kxc_hip_qconv2d_c4_pack_weights: NULL pointer");
    const int64_t slots = static_cast<int64_t>(bytes / 16);
    pack_weights_k7_c4_kernel<<<NoteGrid(static_cast<int>(CeilDiv(slots, kBlock))), NoteBlock(kBlock), NoteLds(0),
                                ResolveStream(stream)>>>(w_oihw, packed, d->o, d->c, slots);
    return CheckLaunch("qconv2d_c4_pack_weights");
}

int32_t kxc_hip_qconv2d_c4_i8(const kxc_hip_qconv2d_desc* d, const int8_t* x_c4, const int8_t* w_packed,
                              const int32_t* bias, const float* mult, int8_t* y_c16, void* stream) {
    QLaunch L;
    const K7Variant* v = nullptr;
    if (int32_t rc = PrepareK7(d, &L, &v, "kxc_hip_qconv2d_c4_i8")) return rc;
    if (L.args.M == 0) return KXC_HIP_OK;
    KXC_HIP_REQUIRE(x_c4 && w_packed && mult && y_c16, "kxc_hip_qconv2d_c4_i8: NULL pointer");
    KXC_HIP_REQUIRE(!(d->flags & KXC_HIP_CONV_BIAS) || bias, "kxc_hip_qconv2d_c4_i8: bias flag without bias");
    QArgs& a = L.args;
    a.x = x_c4; a.wp = w_packed; a.bias = bias; a.mult = mult; a.res = nullptr; a.y = y_c16;
    if (L.lds_bytes > 64 * 1024) {
        KXC_HIP_CALL(hipFuncSetAttribute(reinterpret_cast<const void*>(v->kernel),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(L.lds_bytes)),
                     "hipFuncSetAttribute");
    }
    hipLaunchKernelGGL(v->kernel, NoteGrid(dim3(L.grid)), NoteBlock(dim3(64 * v->wp)), NoteLds(L.lds_bytes),
                       ResolveStream(stream), a);
    return CheckLaunch(v->name);
}

int32_t kxc_hip_quantize_f32_nchw_to_c4_i8(const float* x, int8_t* y, int64_t n, int64_t c, int64_t hw, float scale,
                                           void* stream) {
    KXC_HIP_REQUIRE(n >= 0 && c >= 1 && c <= 4 && hw >= 0, "kxc_hip_quantize_f32_nchw_to_c4_i8: needs 1..4 channels");
    KXC_HIP_REQUIRE(scale > 0.0f, "kxc_hip_quantize_f32_nchw_to_c4_i8: scale must be positive");
    const int64_t total = n * hw;
    if (total == 0) return KXC_HIP_OK;
    KXC_HIP_REQUIRE(x && y, "kxc_hip_quantize_f32_nchw_to_c4_i8: NULL pointer");
    KXC_HIP_REQUIRE(CeilDiv(total, kBlock) <= kMaxGridX, "kxc_hip_quantize_f32_nchw_to_c4_i8: tensor too large");
    if (hw % 4 == 0 && hw / 4 < (1LL << 31) && ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) & 15u) == 0) {
        quantize_to_c4_x4_kernel<<<NoteGrid(static_cast<int>(CeilDiv(total / 4, kBlock))), NoteBlock(kBlock), NoteLds(0),
                                   ResolveStream(stream)>>>(x, y, static_cast<int32_t>(c), static_cast<int32_t>(hw / 4), total / 4, scale);
        return CheckLaunch("quantize_f32_nchw_to_c4_i8");
    }
    quantize_to_c4_kernel<<<NoteGrid(static_cast<int>(CeilDiv(total, kBlock))), NoteBlock(kBlock), NoteLds(0),
                            ResolveStream(stream)>>>(x, y, static_cast<int32_t>(c), hw, total, scale);
    return CheckLaunch("quantize_f32_nchw_to_c4_i8");
}

}  // extern "C"

// ---- the weight tensors of several layers packed by one launch
namespace kxc_hip {

int32_t QPackedBytes(const QPackJob& job, size_t* out_bytes) {
    KXC_HIP_REQUIRE(job.desc != nullptr, "weight pack: desc is NULL");
    switch (job.kind) {
        case KXC_HIP_QPACK_C16: return kxc_hip_qconv2d_c16_packed_bytes(job.desc, out_bytes);
        case KXC_HIP_QPACK_C4: return kxc_hip_qconv2d_c4_packed_bytes(job.desc, out_bytes);
        case KXC_HIP_QPACK_C16_PAIR: return kxc_hip_qconv2d_c16_pair_packed_bytes(job.desc, out_bytes);
        default: return Fail(KXC_HIP_ERR_INVALID, "weight pack: unknown kind %d", job.kind);
    }
}

int32_t LaunchQWeightPacks(const QPackJob* jobs, int32_t count, hipStream_t stream) {
    for (int32_t base = 0; base < count; base += kMaxPackJobs) {
        PackBatch b;
        std::memset(&b, 0, sizeof(b));
        b.count = std::min<int32_t>(kMaxPackJobs, count - base);
        int64_t blocks = 0;
        for (int32_t j = 0; j < b.count; ++j) {
            const QPackJob& job = jobs[base + j];
            size_t bytes = 0;
            if (int32_t rc = QPackedBytes(job, &bytes)) return rc;
            KXC_HIP_REQUIRE(job.w && job.wp, "weight pack: NULL pointer in job %d", base + j);
            const kxc_hip_qconv2d_desc* d = job.desc;
            PackArgs& p = b.job[j];
            p.w = job.w; p.wp = job.wp; p.O = d->o; p.C = d->c;
            if (job.kind == KXC_HIP_QPACK_C4) {
                p.NS = 0;                                   // first-layer order
            } else {
                const bool pair = job.kind == KXC_HIP_QPACK_C16_PAIR;
                p.KHW = pair ? 1 : d->kh * d->kw;
                p.CBC = CbcFor(d->c, d->kh, d->kw);
                p.NS = pair ? (p.CBC + 1) / 2 : (p.KHW * p.CBC + 1) / 2;
                p.nchunks = ((d->c + 15) / 16 + p.CBC - 1) / p.CBC;
                p.oblocks = d->o / 32;
            }
            b.slots[j] = static_cast<int64_t>(bytes / 16);
            b.first_block[j] = static_cast<int32_t>(blocks);
            b.staged[j] = p.NS != 0 && ((p.CBC * 16 * p.KHW + 3) & ~3) + 4 <= kPackRowBytes ? 1 : 0;
            blocks += b.staged[j] ? static_cast<int64_t>(p.oblocks) * p.nchunks : CeilDiv(b.slots[j], kBlock);
            KXC_HIP_REQUIRE(blocks < kMaxGridX, "weight pack: too many blocks");
        }
        b.first_block[b.count] = static_cast<int32_t>(blocks);
        if (blocks == 0) continue;
        pack_weights_batch_kernel<<<NoteGrid(static_cast<int>(blocks)), NoteBlock(kBlock), NoteLds(0), stream>>>(b);
        if (int32_t rc = CheckLaunch("pack_weights_batch_kernel")) return rc;
    }
    return KXC_HIP_OK;
}

}  // namespace kxc_hip

extern "C" {

int32_t kxc_hip_qconv2d_c4_supported(const kxc_hip_qconv2d_desc* d) {
    QLaunch L;
    const K7Variant* v = nullptr;
    if (PrepareK7(d, &L, &v, "kxc_hip_qconv2d_c4_supported") != KXC_HIP_OK) { LastError().clear(); return 0; }
    return 1;
}

int32_t kxc_hip_qconv2d_c16_supported(const kxc_hip_qconv2d_desc* d) {
    QLaunch L;
    if (Prepare(d, &L, "kxc_hip_qconv2d_c16_supported") != KXC_HIP_OK) { LastError().clear(); return 0; }
    return 1;
}

}  // extern "C"
