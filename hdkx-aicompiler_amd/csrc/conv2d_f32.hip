// conv2d_f32.hip -- nn_conv2d (NCHW data, OIHW weights, fp32) for gfx950.
//
// Two kernels behind one entry point:
//
//  * conv_mfma_kernel: implicit GEMM on the fp32 matrix cores (v_mfma_f32_32x32x2_f32),
//    D[o][pixel] += W[o][k] * X[k][pixel], k = (channel, rh, rw).
//      - Output pixels are flattened over (n, oh, ow); a workgroup owns TO output channels by TP
//        consecutive pixels.  The weights are the MFMA "A" operand and the pixels the "B"
//        operand, so the 32 lanes of a half-wave hold 32 consecutive pixels of ONE output
//        channel: NCHW stores (and residual loads) are 128-byte contiguous runs.
//      - The input is NOT expanded to an im2col matrix.  For each chunk of CC input channels the
//        workgroup stages the raw input rows its pixels touch (with the zero padding
//        materialised) in LDS as patch[channel][padded_row][padded_col]; the operand for tap
//        (rh, rw) is the same patch read at a shifted address, so every input element is
//        fetched from memory once per workgroup instead of KH*KW times.  Rows are addressed in
//        "padded row space" Q = n*(H+2*pad_h) + ih + pad_h, which makes a tile that crosses
//        image boundaries (7x7 and 14x14 feature maps) just a longer run of rows.
//      - One MFMA consumes two k values, one per half-wave.  They are chosen as the SAME tap of
//        two adjacent channels, so a lane's LDS address is (per-lane base) + (uniform offset)
//        for both operands; the reduction order differs from the CPU loop only in that way and
//        in the blocking of channels, which is what the 1e-3 tolerance is for.
//      - Chunks are double buffered: the next chunk's global loads are issued before the MFMA
//        loop over the current one and written to the other LDS buffer after it.
//      - The epilogue adds bias, the residual operand, and applies ReLU, each as one rounded
//        fp32 operation in the order of the unfused operator chain.
//
//  * conv_direct_kernel: one thread per output element, the CPU loop nest's exact order
//    (rc, rh, rw ascending from 0.0f, multiply and add rounded separately, padded taps add
//    0.0f * w).  Bit-identical to the CPU backend; used for shapes the MFMA tiling does not
//    cover (output channels not a multiple of 32, very wide rows) and on request.
#include <cstdlib>
#include <cstring>
#include <memory>
#include <type_traits>
#include <mutex>
#include <string>
#include <utility>
#include <vector>

#include "common.h"

using namespace kxc_hip;

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

struct ConvArgs {
    const float* x;
    const float* w;
    const float* bias;
    const float* res;
    float* y;
    int32_t N, C, H, W, O, OH, OW;
    int32_t sh, sw, ph, pw, dh, dw;
    int32_t Hp, Wp;      // padded input extent: H + 2*ph, W + 2*pw
    int32_t Hv, row_step;   // rows the matrix kernel sees and their distance in input rows (see RowView)
    // reduction split over workgroups: workgroup (tile, split) reduces chunks [split*cps, min((split+1)*cps, nchunks))
    // and writes raw partial sums to partial[split][N*O*OH*OW]; a second kernel adds them up (gsplit == 1: off)
    float* partial;
    int32_t gsplit, cps;
    int64_t out_elems;
    int32_t M;           // N*OH*OW output pixels
    int32_t OHW;
    int32_t chs;         // LDS floats per patch channel (>= rows*Wp, padded)
    int32_t nchunks;     // ceil(C / CC)
    uint32_t x_bytes, w_bytes;
    int32_t p_tiles, o_tiles, num_tiles, tiles_per_xcd, o_fastest;
    uint32_t flags;
    FastDiv div_wp, div_hp, div_ohw, div_ow, div_otiles, div_ptiles, div_gsplit;
    // Second output of the DS kernels: a 1x1 convolution with the same strides and no padding on the same input,
    // y2[n,o,oh,ow] = sum_c x[n,c,oh*sh,ow*sw] * w2[o,c] (+ bias2[o]).  Its operand is one tap of this
    // convolution's window (the centre tap of a 3x3 window with padding 1), which the staged patch already holds;
    // ds_off is that tap's offset inside a channel's patch.
    const float* w2;
    const float* bias2;
    float* y2;
    uint32_t w2_bytes;
    int32_t ds_off;
    // Stride 2 in both directions (phase != 0): a channel's patch is kept as four phase planes -- (row parity,
    // column parity) of the padded position, plane (2*rp + cp) at cp_plane*(2*rp + cp), row pitch Wp/2 -- so that
    // the 32 pixels a half-wave reads for one tap are neighbours in LDS (dense banks) instead of every other float
    // of every other row.  plane = ceil(rows/2) * Wp/2 floats for the tallest tile of the launch; needs Hp, Wp even.
    int32_t phase, plane, halfw;
    FastDiv div_plane, div_halfw;
    // HP kernels (KXC_HIP_CONV_HPOOL): width of the pooled output, OW / 2
    int32_t PW;
};

__device__ __forceinline__ float relu_sel(float v) { return (v > 0.0f) ? v : 0.0f; }

// ------------------------------------------------------------------------------------------
// MFMA kernel.  KH,KW: filter; CC: channels per LDS chunk (even); WO x WP waves, each wave
// RO x RP blocks of 32x32; PPT: 64-float patch segments per wave per channel (upper bound,
// checked on the host).
//
// Both LDS tiles are filled by buffer loads that write straight to LDS (buffer_load_dword ... lds):
// lane l of a wave writes LDS float (segment base + l), its global byte offset comes from a
// per-thread table computed once, and the chunk's channel offset is the instruction's scalar
// offset.  Table entries for padding / out-of-tile positions hold an offset beyond the buffer,
// for which the hardware returns 0 -- zero padding costs no branch and no select, and the loads
// need no staging registers: they run while the matrix cores work on the other LDS buffer.
// ------------------------------------------------------------------------------------------
constexpr uint32_t kOobOffset = 0x80000000u;   // beyond any buffer this kernel accepts (< 2 GiB)

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* p, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, static_cast<int>(bytes), 0x00020000);
}

typedef __attribute__((address_space(3))) void* lds_ptr_t;

// KS: split of the reduction inside the workgroup.  The waves form KS groups; group g owns its own pair of
// LDS tiles and works on chunks g, g+KS, ...; the partial accumulators are added through LDS in group
// order at the end (deterministic).  It multiplies the waves per output block for launches that have too
// few 32x32 blocks to occupy 1024 SIMDs (7x7 feature maps, batch 1).
//
// TPAIR: how the two k values of one matrix instruction are chosen.  false: the same filter tap of two adjacent
// channels (CC even).  true: two consecutive taps of ONE channel (an odd tap count gets a zero-weight partner):
// for a 3-channel 7x7 first layer that is 75 k-steps instead of the 98 that pairing channels 2 and "3" costs.
//
// DS: the workgroup also produces the second output described in ConvArgs (a residual block's 1x1 downsample next
// to the block's first 3x3 convolution): per chunk CC/2 more k-steps that read the window's centre tap and a
// second, small weight tile [2 planes][TO][CC/2], into a second set of accumulators.
//
// HP: the result leaves the kernel max-pooled along W (window 3, stride 2, one column of padding on the left; see the
// epilogue): the first half of a 3x3 / stride-2 max pool that follows the convolution, done while the row is still
// in registers, so that only half the feature map is written.
template <int KH, int KW, int CC, int WO, int WP, int RO, int RP, int PPT, int KS, bool TPAIR = false, bool DS = false,
          bool HP = false>
__global__ void __launch_bounds__(64 * WO * WP * KS) __attribute__((amdgpu_waves_per_eu(2)))
conv_mfma_kernel(const ConvArgs a) {
    static_assert(!(DS && TPAIR), "the second output pairs channels");
    static_assert(!HP || (KS == 1 && !DS), "the pooling epilogue handles one reduction group and one output");
    constexpr int NW = WO * WP;                               // waves per reduction group
    constexpr int TO = 32 * RO * WO;
    constexpr int TP = 32 * RP * WP;
    constexpr int KHW = KH * KW;
    constexpr int TPS = (KHW + 1) / 2;                        // tap pairs per channel (TPAIR)
    constexpr int NS = TPAIR ? CC * TPS : (CC / 2) * KHW;     // matrix k-steps per chunk
    constexpr int KS2 = NS | 1;                               // odd row stride of one weight plane
    constexpr int PL = (TO * KS2 + 63) / 64 * 64 + 32;        // plane stride: 32 mod 64
    constexpr int WSZ = 2 * PL;                               // floats in the weight tile (multiple of 64)
    constexpr int WSEG = WSZ / 64;                            // 64-float segments of the weight tile
    constexpr int WPT = (WSEG + NW - 1) / NW;                 // weight segments per wave
    constexpr int PF = (RO * RP >= 4) ? 1 : (RO * RP == 2 ? 2 : 3);   // operand prefetch distance in k-steps
    // second weight tile (DS): element L = plane*PLB + row*KS2B + pair, channel = 2*pair + plane
    constexpr int NS2 = DS ? CC / 2 : 0;                      // k-steps of the second output per chunk
    constexpr int KS2B = (CC / 2) | 1;
    constexpr int PLB = (TO * KS2B + 63) / 64 * 64 + 32;
    constexpr int WSZB = DS ? 2 * PLB : 0;
    constexpr int WSEGB = WSZB / 64;
    constexpr int WPTB = (WSEGB + NW - 1) / NW;
    constexpr int NST = NS + NS2;                             // all k-steps of a chunk

    extern __shared__ float lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave_all = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int kgroup = wave_all / NW;
    const int wave = wave_all - kgroup * NW;
    const int xs_size = (CC * a.chs + 31) & ~31;              // rounded so that every tile starts 128-byte aligned
    // Workgroup -> (tile, split).  The dispatcher hands consecutive workgroups to the 8 XCDs round-robin and every
    // XCD has its own L2, so workgroup L works on logical unit (L % 8) * units_per_xcd + L / 8: each XCD owns a
    // contiguous run of tiles and the halo rows / weight slices neighbouring tiles share are fetched into one L2
    // instead of eight.  Within the run the output-channel tile or the pixel tile varies fastest (host's choice:
    // whichever operand is larger stays put).
    const int unit = (blockIdx.x & 7) * a.tiles_per_xcd + (blockIdx.x >> 3);
    if (unit >= a.num_tiles * a.gsplit || static_cast<int>(blockIdx.x >> 3) >= a.tiles_per_xcd) return;
    const int tile = a.gsplit > 1 ? fast_div(unit, a.div_gsplit) : unit;
    const int split = unit - tile * a.gsplit;
    const int c_lo = split * a.cps;                           // this workgroup's chunks: [c_lo, c_hi)
    const int c_hi = min(a.nchunks, c_lo + a.cps);
    const int iters = (c_hi - c_lo + KS - 1) / KS;            // chunk steps of every reduction group
    // per group: [xs0][ws0][vs0][xs1][ws1][vs1] (vs: the second output's weight tile); the second set exists only
    // when a group has more than one chunk
    float* const xs0 = lds + kgroup * (iters > 1 ? 2 : 1) * (xs_size + WSZ + WSZB);
    float* const ws0 = xs0 + xs_size;                 // (vs0 = ws0 + WSZ)
    float* const xs1 = ws0 + WSZ + WSZB;
    float* const ws1 = xs1 + xs_size;

    const int wave_o = wave / WP;
    const int wave_p = wave % WP;
    const int half = lane >> 5;
    const int r = lane & 31;

    int p_tile, o_tile;
    if (a.o_fastest) { p_tile = fast_div(tile, a.div_otiles); o_tile = tile - p_tile * a.o_tiles; }
    else { o_tile = fast_div(tile, a.div_ptiles); p_tile = tile - o_tile * a.p_tiles; }
    const int m0 = p_tile * TP;
    const int o0 = o_tile * TO;

    // ---- geometry of this tile in padded row space
    const int m_last = min(m0 + TP, a.M) - 1;
    int qmin, qlast;
    {
        const int n = fast_div(m0, a.div_ohw), rem = m0 - n * a.OHW;
        qmin = n * a.Hp + fast_div(rem, a.div_ow) * a.sh;
        const int n2 = fast_div(m_last, a.div_ohw), rem2 = m_last - n2 * a.OHW;
        qlast = n2 * a.Hp + fast_div(rem2, a.div_ow) * a.sh + (KH - 1) * a.dh;
    }
    const int P = (qlast - qmin + 1) * a.Wp;      // patch positions per channel (<= chs - 32)
    const int xsegs = ((a.phase ? 4 * a.plane : P) + 63) >> 6;              // 64-float segments per channel
    const int HW = a.H * a.W;

    const __amdgpu_buffer_rsrc_t xr = make_rsrc(a.x, a.x_bytes);
    const __amdgpu_buffer_rsrc_t wr = make_rsrc(a.w, a.w_bytes);
    const __amdgpu_buffer_rsrc_t w2r = make_rsrc(DS ? a.w2 : a.w, DS ? a.w2_bytes : 0u);

    // ---- per-thread load tables (byte offsets; kOobOffset reads as 0)
    uint32_t goff[PPT];
#pragma unroll
    for (int i = 0; i < PPT; ++i) {
        const int pos = (wave + i * NW) * 64 + lane;
        int q, col;
        if (a.phase) {
            // LDS position -> plane, row and column inside the plane -> padded row and column
            const int pl = fast_div(pos, a.div_plane), rem = pos - pl * a.plane;
            const int qr = fast_div(rem, a.div_halfw), qc = rem - qr * a.halfw;
            q = 2 * qr + (pl >> 1); col = 2 * qc + (pl & 1);
        } else {
            q = fast_div(pos, a.div_wp); col = pos - q * a.Wp;
        }
        const int Q = qmin + q;
        const int n = fast_div(Q, a.div_hp), ih = Q - n * a.Hp - a.ph, iw = col - a.pw;
        const bool ok = (a.phase ? (pos < 4 * a.plane && Q <= qlast) : pos < P) && n < a.N && ih >= 0 && ih < a.Hv && iw >= 0 && iw < a.W;
        goff[i] = ok ? static_cast<uint32_t>(((n * a.C) * a.H + ih * a.row_step) * a.W + iw) * 4u : kOobOffset;
    }
    // weight tile element L = plane*PL + row*KS2 + col; col = pair*KHW + tap with channel = 2*pair + plane, or
    // (TPAIR) col = channel*TPS + s with tap = 2*s + plane
    uint32_t woff[WPT];
    uint32_t woff2[WPTB > 0 ? WPTB : 1];
    auto weight_table = [&](int channels_left) {
        if (DS) {
#pragma unroll
            for (int i = 0; i < WPTB; ++i) {
                const int L = (wave + i * NW) * 64 + lane;
                const int plane = L >= PLB ? 1 : 0;
                const int rem = L - plane * PLB;
                const int row = rem / KS2B, pair = rem - row * KS2B;
                const int cl = 2 * pair + plane;
                const bool ok = L < WSZB && row < TO && pair < NS2 && (o0 + row) < a.O && cl < channels_left;
                woff2[i] = ok ? static_cast<uint32_t>((o0 + row) * a.C + cl) * 4u : kOobOffset;
            }
        }
#pragma unroll
        for (int i = 0; i < WPT; ++i) {
            const int L = (wave + i * NW) * 64 + lane;
            const int plane = L >= PL ? 1 : 0;
            const int rem = L - plane * PL;
            const int row = rem / KS2, col = rem - row * KS2;
            int cl, tap;
            if (TPAIR) { cl = col / TPS; tap = 2 * (col - cl * TPS) + plane; }
            else { const int pair = col / KHW; tap = col - pair * KHW; cl = 2 * pair + plane; }
            const bool ok = L < WSZ && row < TO && col < NS && tap < KHW && (o0 + row) < a.O && cl < channels_left;
            woff[i] = ok ? static_cast<uint32_t>(((o0 + row) * a.C + cl) * KHW + tap) * 4u : kOobOffset;
        }
    };
    weight_table(min(CC, a.C - (c_lo + kgroup) * CC));

    // ---- per-lane operand bases
    int xbase[RP];
    int ybase[RP];      // offset of (n, o=0, oh, ow) in y, or -1 when the pixel is past the end
#pragma unroll
    for (int j = 0; j < RP; ++j) {
        const int m = m0 + (wave_p * RP + j) * 32 + r;
        const int mc = min(m, a.M - 1);
        const int n = fast_div(mc, a.div_ohw), rem = mc - n * a.OHW;
        const int oh = fast_div(rem, a.div_ow), ow = rem - oh * a.OW;
        // (phase planes: the window's first row is an even row of the patch, its first column an even column)
        xbase[j] = a.phase ? ((n * a.Hp + oh * 2 - qmin) >> 1) * a.halfw + ow + (TPAIR ? 0 : half * a.chs)
                           : (n * a.Hp + oh * a.sh - qmin) * a.Wp + ow * a.sw + (TPAIR ? 0 : half * a.chs);
        ybase[j] = (m < a.M) ? n * a.O * a.OHW + rem : -1;
    }
    int wbase[RO];
    int wbase2[RO];
#pragma unroll
    for (int i = 0; i < RO; ++i) {
        wbase[i] = half * PL + ((wave_o * RO + i) * 32 + r) * KS2;
        wbase2[i] = half * PLB + ((wave_o * RO + i) * 32 + r) * KS2B;
    }

    // offset of filter tap (rh, rw) from the window's first element inside a channel's patch
    int toff[KHW];
#pragma unroll
    for (int t = 0; t < KHW; ++t) {
        const int rh = t / KW, rw = t % KW;
        toff[t] = a.phase ? ((rh & 1) * 2 + (rw & 1)) * a.plane + (rh >> 1) * a.halfw + (rw >> 1)
                          : rh * a.dh * a.Wp + rw * a.dw;
    }

    floatx16 acc[RO][RP];
    floatx16 acc2[DS ? RO : 1][DS ? RP : 1];
#pragma unroll
    for (int i = 0; i < RO; ++i)
#pragma unroll
        for (int j = 0; j < RP; ++j)
#pragma unroll
            for (int g = 0; g < 16; ++g) {
                acc[i][j][g] = 0.0f;
                if constexpr (DS) acc2[i][j][g] = 0.0f;
            }

    // The loads of one chunk as NOPS separate operations (CC*PPT patch segments, then WPT weight segments), so
    // that the main loop can issue them a few at a time between matrix instructions instead of in one burst
    // during which the wave feeds nothing to the matrix pipe.
    constexpr int NOPS = CC * PPT + WPT + WPTB;
    auto issue_op = [&](int j, int chunk, float* xs, float* ws) {
        const int c0 = chunk * CC;
        if (DS && j >= CC * PPT + WPT) {
            const int i = j - CC * PPT - WPT;
            const int seg = wave + i * NW;
            if (seg < WSEGB)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(w2r, (lds_ptr_t)(ws + WSZ + seg * 64), 4, woff2[i < WPTB ? i : 0],
                                                         static_cast<uint32_t>(c0) * 4u, 0, 0);
        } else if (j < CC * PPT) {
            const int cl = j / PPT, i = j - cl * PPT;
            const int seg = wave + i * NW;
            if (seg < xsegs) {
                if (c0 + cl < a.C) {
                    const uint32_t soff = static_cast<uint32_t>(c0 + cl) * static_cast<uint32_t>(HW) * 4u;
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(xr, (lds_ptr_t)(xs + cl * a.chs + seg * 64), 4, goff[i], soff, 0, 0);
                } else {
                    // channel beyond C: zero plane (the matching weights are zero too, keep the product exact)
                    xs[cl * a.chs + seg * 64 + lane] = 0.0f;
                }
            }
        } else {
            const int i = j - CC * PPT;
            const int seg = wave + i * NW;
            if (seg < WSEG) {
                const uint32_t wsoff = static_cast<uint32_t>(c0) * KHW * 4u;
                __builtin_amdgcn_raw_ptr_buffer_load_lds(wr, (lds_ptr_t)(ws + seg * 64), 4, woff[i], wsoff, 0, 0);
            }
        }
    };
    auto issue_loads = [&](int chunk, float* xs, float* ws) {
        if (chunk * CC + CC > a.C && chunk >= c_lo + KS) weight_table(a.C - chunk * CC);   // partial last chunk (rare)
#pragma unroll
        for (int j = 0; j < NOPS; ++j) issue_op(j, chunk, xs, ws);
    };

    if (c_lo + kgroup < c_hi) issue_loads(c_lo + kgroup, xs0, ws0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();

    for (int it = 0; it < iters; ++it) {
        const int chunk = c_lo + it * KS + kgroup;
        const float* xs = (it & 1) ? xs1 : xs0;
        const float* ws = (it & 1) ? ws1 : ws0;
        const bool has_next = chunk + KS < c_hi;
        float* const nxs = (it & 1) ? xs0 : xs1;
        float* const nws = (it & 1) ? ws0 : ws1;
        if (has_next && (chunk + KS) * CC + CC > a.C) weight_table(a.C - (chunk + KS) * CC);   // partial last chunk (rare)
        if (chunk < c_hi) {
        constexpr int OPS_PER_STEP = (NOPS + NST - 1) / NST;

        // k-steps of this chunk: step = pair * KHW + tap.  Operands are fetched from LDS PF steps ahead of
        // the matrix instruction that consumes them (rotating register sets; all indices are compile-time
        // after unrolling), so the LDS latency is covered by the PF matrix instructions in between.
        auto fetch = [&](int step, float (&av)[RO], float (&bv)[RP]) {
            int koff_x, koff_w;
            if (DS && step >= NS) {
                // second output: the window's centre tap of channel pair step - NS, weights from the second tile
                const int cp = step - NS;
                koff_x = (2 * cp) * a.chs + a.ds_off;
#pragma unroll
                for (int i = 0; i < RO; ++i) av[i] = ws[WSZ + wbase2[i] + cp];
#pragma unroll
                for (int j = 0; j < RP; ++j) bv[j] = xs[xbase[j] + koff_x];
                return;
            }
            if (TPAIR) {
                // lane half h reads tap 2*s + h of channel c; a tap past the end (zero weight) re-reads the last one
                const int c = step / TPS, s2 = 2 * (step - c * TPS);
                const int t0 = s2, t1 = s2 + 1 < KHW ? s2 + 1 : KHW - 1;
                const int off0 = toff[t0], off1 = toff[t1];
                koff_x = c * a.chs + (half ? off1 : off0);
                koff_w = step;
            } else {
                const int cp = step / KHW, tap = step - cp * KHW;
                koff_x = (2 * cp) * a.chs + toff[tap];
                koff_w = cp * KHW + tap;
            }
#pragma unroll
            for (int i = 0; i < RO; ++i) av[i] = ws[wbase[i] + koff_w];
#pragma unroll
            for (int j = 0; j < RP; ++j) bv[j] = xs[xbase[j] + koff_x];
        };
        float av[PF + 1][RO], bv[PF + 1][RP];
#pragma unroll
        for (int p = 0; p < PF; ++p)
            if (p < NST) fetch(p, av[p % (PF + 1)], bv[p % (PF + 1)]);
#pragma unroll
        for (int step = 0; step < NST; ++step) {
            if (step + PF < NST) fetch(step + PF, av[(step + PF) % (PF + 1)], bv[(step + PF) % (PF + 1)]);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < RO; ++i)
#pragma unroll
                for (int j = 0; j < RP; ++j) {
                    if constexpr (DS) {
                        if (step >= NS) {
                            acc2[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[step % (PF + 1)][i], bv[step % (PF + 1)][j],
                                                                              acc2[i][j], 0, 0, 0);
                            continue;
                        }
                    }
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[step % (PF + 1)][i], bv[step % (PF + 1)][j],
                                                                     acc[i][j], 0, 0, 0);
                }
            __builtin_amdgcn_sched_barrier(0);
            // next chunk's loads, a few per k-step, issued while this step's matrix instructions execute
            if (has_next) {
#pragma unroll
                for (int u = 0; u < OPS_PER_STEP; ++u)
                    if (step * OPS_PER_STEP + u < NOPS) issue_op(step * OPS_PER_STEP + u, chunk + KS, nxs, nws);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        }

        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
    }

    // ---- combine the reduction groups: groups 1.. park their accumulators in LDS (the tiles are dead after
    // the loop's last barrier), group 0 adds them in group order; the second output's accumulators follow in a
    // second round through the same LDS
    if (KS > 1) {
        float* const red = lds;
        auto combine = [&](auto& accs) {
            if (kgroup > 0) {
#pragma unroll
                for (int i = 0; i < RO; ++i)
#pragma unroll
                    for (int j = 0; j < RP; ++j)
#pragma unroll
                        for (int g = 0; g < 16; ++g)
                            red[((((kgroup - 1) * NW + wave) * RO * RP + i * RP + j) * 16 + g) * 64 + lane] = accs[i][j][g];
            }
            __syncthreads();
            if (kgroup == 0) {
#pragma unroll
                for (int kg = 1; kg < KS; ++kg)
#pragma unroll
                    for (int i = 0; i < RO; ++i)
#pragma unroll
                        for (int j = 0; j < RP; ++j)
#pragma unroll
                            for (int g = 0; g < 16; ++g)
                                accs[i][j][g] += red[((((kg - 1) * NW + wave) * RO * RP + i * RP + j) * 16 + g) * 64 + lane];
            }
        };
        combine(acc);
        if constexpr (DS) {
            __syncthreads();
            combine(acc2);
        }
        if (kgroup > 0) return;
    }

    // ---- epilogue: accumulator register g of a block holds row 8*(g/4) + 4*half + g%4, column r
    if constexpr (HP) {
        // y[n,o,oh,pw] = max over columns 2pw-1 .. 2pw+1 of the (bias, ReLU) result; column -1 does not exist.  The host
        // guarantees that OW is even, that a tile is a whole number of output rows and that every tile is full, so a
        // lane's column has the parity of r and the even lanes own the windows: lane r needs lanes r-1 and r+1 of its
        // half-wave.  The left neighbour of a block's lane 0 is lane 31 of the wave before it (one float per
        // accumulator register, handed over through LDS -- the tiles are dead after the loop's last barrier); the
        // first window of a row has no left neighbour.  With ReLU the values are >= +0 and never NaN, so the order
        // of the comparisons does not matter and a padding candidate would never win.
        // The vector ALU shares its datapath with the fp32 matrix instructions, and with 16 x RO x RP values per lane this
        // epilogue is a tenth of the kernel: the neighbours come through the LDS crossbar (ds_bpermute, no vector-ALU
        // instruction; a row's first column names itself as its left neighbour), the one float from the block before
        // is read by every lane and selected, ReLU is one maximum (NaN -> 0 as (v > 0 ? v : 0) gives; the host only
        // offers this epilogue with ReLU), and the channel part of a store's address rides in its scalar offset.
        const bool has_bias = (a.flags & KXC_HIP_CONV_BIAS) != 0;
        const __amdgpu_buffer_rsrc_t br = make_rsrc(has_bias ? a.bias : a.y, has_bias ? static_cast<uint32_t>(a.O) * 4u : 0u);
        // (the host guarantees O % 8 == 0: the eight channels of a register group's two lane halves are all there or all absent)
        const int ch0 = o0 + wave_o * RO * 32;                 // uniform: channel of (i, g) = ch0 + 32 i + 8 (g / 4) + g % 4 + 4 half
        float bv[RO][16];                                      // (no bias: the descriptor is empty, loads give 0; v + 0 then ReLU = ReLU(v))
#pragma unroll
        for (int i = 0; i < RO; ++i)
#pragma unroll
            for (int g = 0; g < 16; ++g) {
                const int o = ch0 + 32 * i + 8 * (g / 4) + (g % 4) + 4 * half;
                bv[i][g] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(br, o < a.O ? static_cast<uint32_t>(o) * 4u : kOobOffset, 0, 0));
            }
        // edge[block][half][RO][16], block = the wave's 32-pixel blocks in tile order per output-channel group
        float* const edge = lds;
        auto edge_at = [&](int block, int i, int g) { return (((wave_o * WP * RP + block) * 2 + half) * RO + i) * 16 + g; };
#pragma unroll
        for (int i = 0; i < RO; ++i)
#pragma unroll
            for (int j = 0; j < RP; ++j)
#pragma unroll
                for (int g = 0; g < 16; ++g) acc[i][j][g] = __builtin_fmaxf(__fadd_rn(acc[i][j][g], bv[i][g]), 0.0f);
        if (r == 31) {
#pragma unroll
            for (int i = 0; i < RO; ++i)
#pragma unroll
                for (int j = 0; j < RP; ++j)
#pragma unroll
                    for (int g = 0; g < 16; ++g) edge[edge_at(wave_p * RP + j, i, g)] = acc[i][j][g];
        }
        __syncthreads();
        const uint32_t y_bytes = static_cast<uint32_t>(a.out_elems) * 4u;
        const uint32_t plane = static_cast<uint32_t>(a.OH * a.PW) * 4u;
        const __amdgpu_buffer_rsrc_t yr = make_rsrc(a.y, y_bytes);
        const int right_addr = ((lane + 1) & 63) * 4;        // (lane 31 / 63 reads a lane of the other half: an odd column, never stored)
#pragma unroll
        for (int j = 0; j < RP; ++j) {
            const int block = wave_p * RP + j;
            const int m = m0 + block * 32 + r;                        // < M: every tile is full
            const int n = fast_div(m, a.div_ohw), rem = m - n * a.OHW;
            const int oh = fast_div(rem, a.div_ow), ow = rem - oh * a.OW;
            const bool row_start = ow == 0;
            const bool from_edge = r == 0 && !row_start;              // (then block > 0: a tile starts a row)
            const int left_addr = (row_start || r == 0 ? lane : lane - 1) * 4;
            // even columns own the windows; the lane half's four channels per register group are part of the lane's offset
            const uint32_t yb = (r & 1) ? kOobOffset
                                        : static_cast<uint32_t>((n * a.O * a.OH + oh) * a.PW + (ow >> 1)) * 4u + static_cast<uint32_t>(4 * half) * plane;
            const int prev = block > 0 ? block - 1 : 0;
#pragma unroll
            for (int i = 0; i < RO; ++i)
#pragma unroll
                for (int gq = 0; gq < 4; ++gq) {
                    const int cg = ch0 + 32 * i + 8 * gq;              // uniform; its channels are cg .. cg + 7
                    const uint32_t yv = cg + 8 <= a.O ? yb : kOobOffset;
#pragma unroll
                    for (int ge = 0; ge < 4; ++ge) {
                        const int g = 4 * gq + ge;
                        const float v = acc[i][j][g];
                        const int bits = __builtin_bit_cast(int, v);
                        float left = __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(left_addr, bits));
                        const float right = __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(right_addr, bits));
                        const float before = edge[edge_at(prev, i, g)];
                        left = from_edge ? before : left;
                        const float pooled = fmaxf(v, fmaxf(left, right));
                        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, pooled), yr, yv,
                                                              static_cast<uint32_t>(cg + ge) * plane, 0);
                    }
                }
        }
        return;
    }
    if (a.gsplit > 1) {
        // raw partial sums of this split; conv_split_reduce_kernel finishes the layer.  The parts of a second output
        // follow those of the first: partial[gsplit + split][...].
        float* const part = a.partial + static_cast<int64_t>(split) * a.out_elems;
        if (KS == 1 || kgroup == 0) {
#pragma unroll
            for (int i = 0; i < RO; ++i)
#pragma unroll
                for (int g = 0; g < 16; ++g) {
                    const int o = o0 + (wave_o * RO + i) * 32 + 8 * (g / 4) + 4 * half + (g % 4);
                    if (o >= a.O) continue;
#pragma unroll
                    for (int j = 0; j < RP; ++j)
                        if (ybase[j] >= 0) {
                            part[ybase[j] + o * a.OHW] = acc[i][j][g];
                            if constexpr (DS) part[static_cast<int64_t>(a.gsplit) * a.out_elems + ybase[j] + o * a.OHW] = acc2[i][j][g];
                        }
                }
        }
        return;
    }
    // Bias, residual and output go through buffer descriptors: an offset beyond the buffer makes a load return 0
    // and drops a store, so absent channels and pixels past the end need no branches, and every load is issued
    // before the first store (a wait for a load also waits for all stores issued before it: with loads and stores
    // interleaved each of the 16 rows would cost a full memory round trip).
    const uint32_t y_bytes = static_cast<uint32_t>(a.out_elems) * 4u;
    const uint32_t plane = static_cast<uint32_t>(a.OHW) * 4u;
    uint32_t yb[RP];
#pragma unroll
    for (int j = 0; j < RP; ++j) yb[j] = ybase[j] >= 0 ? static_cast<uint32_t>(ybase[j]) * 4u : kOobOffset;
    auto channel = [&](int i, int g) { return o0 + (wave_o * RO + i) * 32 + 8 * (g / 4) + 4 * half + (g % 4); };
    auto out_off = [&](int i, int g, int j) {
        const int o = channel(i, g);
        return o < a.O ? yb[j] + static_cast<uint32_t>(o) * plane : kOobOffset;
    };
    auto load_bias = [&](float (&bv)[RO][16], const float* bias, bool has_bias) {
        const __amdgpu_buffer_rsrc_t br = make_rsrc(has_bias ? bias : a.y, has_bias ? static_cast<uint32_t>(a.O) * 4u : 0u);
#pragma unroll
        for (int i = 0; i < RO; ++i)
#pragma unroll
            for (int g = 0; g < 16; ++g) {
                const int o = channel(i, g);
                bv[i][g] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(br, o < a.O ? static_cast<uint32_t>(o) * 4u : kOobOffset, 0, 0));
            }
    };
    auto finish = [&](auto& accs, const float (&bv)[RO][16], bool has_bias, const float* res, bool has_res, bool do_relu, float* y) {
        const __amdgpu_buffer_rsrc_t yr = make_rsrc(y, y_bytes);
        const __amdgpu_buffer_rsrc_t rr = make_rsrc(has_res ? res : y, has_res ? y_bytes : 0u);
        // rows (accumulator registers) per batch of residual loads: the whole block when one block per wave, fewer
        // for register-blocked tiles so that the staged residual never needs more than 16 registers
        constexpr int GC = 16 / (RO * RP) < 4 ? 4 : 16 / (RO * RP);
#pragma unroll
        for (int gc = 0; gc < 16; gc += GC) {
            float q[RO][RP][GC];
            if (has_res) {
#pragma unroll
                for (int i = 0; i < RO; ++i)
#pragma unroll
                    for (int g = 0; g < GC; ++g)
#pragma unroll
                        for (int j = 0; j < RP; ++j)
                            q[i][j][g] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rr, out_off(i, gc + g, j), 0, 0));
            }
#pragma unroll
            for (int i = 0; i < RO; ++i) {
#pragma unroll
                for (int g = 0; g < GC; ++g) {
#pragma unroll
                    for (int j = 0; j < RP; ++j) {
                        float v = accs[i][j][gc + g];
                        if (has_bias) v = __fadd_rn(v, bv[i][gc + g]);
                        if (has_res) v = __fadd_rn(v, q[i][j][g]);
                        if (do_relu) v = relu_sel(v);
                        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, v), yr, out_off(i, gc + g, j), 0, 0);
                    }
                }
            }
        }
    };
    // both outputs' bias values are loaded before anything is stored; the second output has no other loads, so its
    // stores simply follow the main output's
    const bool has_bias = (a.flags & KXC_HIP_CONV_BIAS) != 0;
    float bias_main[RO][16];
    float bias_second[DS ? RO : 1][16];
    load_bias(bias_main, a.bias, has_bias);
    if constexpr (DS) load_bias(bias_second, a.bias2, a.bias2 != nullptr);
    finish(acc, bias_main, has_bias, a.res, (a.flags & KXC_HIP_CONV_RESIDUAL) != 0, (a.flags & KXC_HIP_CONV_RELU) != 0, a.y);
    if constexpr (DS) finish(acc2, bias_second, a.bias2 != nullptr, nullptr, false, false, a.y2);
}

// ------------------------------------------------------------------------------------------
// 1x1 filters on small launches (the downsample convolutions at batch 1-4): the general kernel's set-up and its
// chunked LDS pipeline cost about 10 us however little work there is.  Here a workgroup owns 32 output channels
// x 32 pixels; its four (eight from 256 channels on) waves split the input channels and each feeds v_mfma_f32_32x32x2f32 straight from memory
// (A = one weight per lane, B = one input value per lane, gathered with the convolution's stride), then the four
// waves' partial tiles are added through LDS in wave order and the usual epilogue follows.  Requires C % 8 == 0, no
// padding.
// ------------------------------------------------------------------------------------------
template <int NWAVES>
__global__ void __launch_bounds__(64 * NWAVES) conv1x1_small_kernel(const ConvArgs a) {
    __shared__ float part[NWAVES][32 * 33];
    const int wave = threadIdx.x >> 6;
    const int lane = threadIdx.x & 63;
    const int half = lane >> 5;
    const int r = lane & 31;
    // consecutive workgroups go to the 8 XCDs round-robin; every XCD (own L2) gets a contiguous run of pixel tiles with
    // all their output-channel tiles, so an input tile is fetched into one L2 instead of eight (measured: 16 x the
    // input bytes fetched for the 14 x 14 / 512-channel downsample with the output-channel tile as blockIdx.x)
    const int unit = (blockIdx.x & 7) * a.tiles_per_xcd + (blockIdx.x >> 3);
    if (unit >= a.num_tiles || static_cast<int>(blockIdx.x >> 3) >= a.tiles_per_xcd) return;
    const int p_tile = fast_div(unit, a.div_otiles), o_tile = unit - p_tile * a.o_tiles;
    const int o0 = o_tile * 32, p0 = p_tile * 32;
    const int o = min(o0 + r, a.O - 1);                 // clamped rows / pixels are computed and never stored
    const int px = min(p0 + r, a.M - 1);
    const int n = fast_div(px, a.div_ohw), rem = px - n * a.OHW;
    const int oh = fast_div(rem, a.div_ow), ow = rem - oh * a.OW;
    const int HW = a.H * a.W;
    const int kw = a.C / NWAVES;                        // input channels of this wave (even)
    const float* wp = a.w + static_cast<int64_t>(o) * a.C + wave * kw + half;
    const float* xp = a.x + (static_cast<int64_t>(n) * a.C + wave * kw + half) * HW + (oh * a.sh) * a.W + ow * a.sw;
    floatx16 acc = {0};
    // D[i][j] += A[i][k] * B[k][j]: i = output channel (lane % 32), j = pixel (lane % 32), k = lane / 32.
    // The loop is latency-bound: 32 loads (16 k-steps) are in flight before the first matrix instruction of a
    // batch uses one; shorter batches take what is left.
    int k = 0;
    auto batch = [&](auto steps) {
        constexpr int U = decltype(steps)::value;
        float wa[U], xb[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            wa[u] = wp[k + 2 * u];
            xb[u] = xp[static_cast<int64_t>(k + 2 * u) * HW];
        }
#pragma unroll
        for (int u = 0; u < U; ++u) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(wa[u], xb[u], acc, 0, 0, 0);
        k += 2 * U;
    };
    while (k + 32 <= kw) batch(std::integral_constant<int, 16>{});
    while (k + 8 <= kw) batch(std::integral_constant<int, 4>{});
    while (k < kw) batch(std::integral_constant<int, 1>{});
    // accumulator register g holds D[i][j] with j = lane % 32, i = 8*(g/4) + 4*(lane/32) + g%4
#pragma unroll
    for (int g = 0; g < 16; ++g) part[wave][(8 * (g / 4) + 4 * half + (g % 4)) * 33 + r] = acc[g];
    __syncthreads();
    const bool has_bias = (a.flags & KXC_HIP_CONV_BIAS) != 0;
    const bool has_res = (a.flags & KXC_HIP_CONV_RESIDUAL) != 0;
    const bool do_relu = (a.flags & KXC_HIP_CONV_RELU) != 0;
    // 1024 outputs: consecutive threads on consecutive pixels, the waves' parts added in wave order
    for (int e = threadIdx.x; e < 1024; e += 64 * NWAVES) {
        const int i = e >> 5, j = e & 31;
        float v = part[0][i * 33 + j];
#pragma unroll
        for (int q = 1; q < NWAVES; ++q) v = __fadd_rn(v, part[q][i * 33 + j]);
        const int oc = o0 + i, pj = p0 + j;
        if (oc >= a.O || pj >= a.M) continue;
        const int nj = fast_div(pj, a.div_ohw);
        const int64_t idx = (static_cast<int64_t>(nj) * a.O + oc) * a.OHW + (pj - nj * a.OHW);
        if (has_bias) v = __fadd_rn(v, a.bias[oc]);
        if (has_res) v = __fadd_rn(v, a.res[idx]);
        if (do_relu) v = relu_sel(v);
        a.y[idx] = v;
    }
}

// ------------------------------------------------------------------------------------------
// Direct kernel: the CPU loop nest, one thread per output element.
// ------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(256) conv_direct_kernel(const ConvArgs a, int32_t KH, int32_t KW, int64_t total) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * 256;
    const bool has_bias = (a.flags & KXC_HIP_CONV_BIAS) != 0;
    const bool has_res = (a.flags & KXC_HIP_CONV_RESIDUAL) != 0;
    const bool do_relu = (a.flags & KXC_HIP_CONV_RELU) != 0;
    for (int64_t e = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; e < total; e += stride) {
        const int32_t ow = static_cast<int32_t>(e % a.OW);
        int64_t t = e / a.OW;
        const int32_t oh = static_cast<int32_t>(t % a.OH);
        t /= a.OH;
        const int32_t o = static_cast<int32_t>(t % a.O);
        const int64_t n = t / a.O;
        const float* xn = a.x + n * a.C * a.H * a.W;
        const float* wo = a.w + static_cast<int64_t>(o) * a.C * KH * KW;
        float acc = 0.0f;
        for (int32_t rc = 0; rc < a.C; ++rc)
            for (int32_t rh = 0; rh < KH; ++rh) {
                const int32_t ih = oh * a.sh + rh * a.dh - a.ph;
                for (int32_t rw = 0; rw < KW; ++rw) {
                    const int32_t iw = ow * a.sw + rw * a.dw - a.pw;
                    const bool inb = ih >= 0 && ih < a.H && iw >= 0 && iw < a.W;
                    const float v = inb ? xn[(static_cast<int64_t>(rc) * a.H + ih) * a.W + iw] : 0.0f;
                    acc = __fadd_rn(acc, __fmul_rn(v, wo[(rc * KH + rh) * KW + rw]));
                }
            }
        if (has_bias) acc = __fadd_rn(acc, a.bias[o]);
        if (has_res) acc = __fadd_rn(acc, a.res[e]);
        if (do_relu) acc = relu_sel(acc);
        a.y[e] = acc;
    }
}

// ------------------------------------------------------------------------------------------
// Host side: variant table and selection.
// ------------------------------------------------------------------------------------------
struct Variant {
    const char* name;
    int kh, kw, cc, to, tp, nw, ppt, ks, tpair;
    void (*kernel)(const ConvArgs);
    void (*ds_kernel)(const ConvArgs);      // the same tile with the second (1x1 downsample) output, or nullptr
    void (*hp_kernel)(const ConvArgs);      // the same tile with the pooling epilogue (KXC_HIP_CONV_HPOOL), or nullptr
};

#define KXC_VARIANT(KH, KW, CC, WO, WP, RO, RP, PPT)                                                   \
    {"mfma_k" #KH "x" #KW "_c" #CC "_o" #WO "x" #RO "_p" #WP "x" #RP, KH, KW, CC, 32 * RO * WO, 32 * RP * WP, \
     WO * WP, PPT, 1, 0, conv_mfma_kernel<KH, KW, CC, WO, WP, RO, RP, PPT, 1>, nullptr}
#define KXC_VARIANT_KS(KH, KW, CC, WO, WP, RO, RP, PPT, KS)                                            \
    {"mfma_k" #KH "x" #KW "_c" #CC "_o" #WO "x" #RO "_p" #WP "x" #RP "_ks" #KS, KH, KW, CC, 32 * RO * WO,   \
     32 * RP * WP, WO * WP, PPT, KS, 0, conv_mfma_kernel<KH, KW, CC, WO, WP, RO, RP, PPT, KS>, nullptr}
#define KXC_VARIANT_TP(KH, KW, CC, WO, WP, RO, RP, PPT)                                                \
    {"mfma_k" #KH "x" #KW "_t" #CC "_o" #WO "x" #RO "_p" #WP "x" #RP, KH, KW, CC, 32 * RO * WO, 32 * RP * WP, \
     WO * WP, PPT, 1, 1, conv_mfma_kernel<KH, KW, CC, WO, WP, RO, RP, PPT, 1, true>, nullptr}
#define KXC_VARIANT_TP_HP(KH, KW, CC, WO, WP, RO, RP, PPT)                                             \
    {"mfma_k" #KH "x" #KW "_t" #CC "_o" #WO "x" #RO "_p" #WP "x" #RP, KH, KW, CC, 32 * RO * WO, 32 * RP * WP, \
     WO * WP, PPT, 1, 1, conv_mfma_kernel<KH, KW, CC, WO, WP, RO, RP, PPT, 1, true>, nullptr,              \
     conv_mfma_kernel<KH, KW, CC, WO, WP, RO, RP, PPT, 1, true, false, true>}
// (tiles that also exist with the second output)
#define KXC_VARIANT_DS(KH, KW, CC, WO, WP, RO, RP, PPT)                                                \
    {"mfma_k" #KH "x" #KW "_c" #CC "_o" #WO "x" #RO "_p" #WP "x" #RP, KH, KW, CC, 32 * RO * WO, 32 * RP * WP, \
     WO * WP, PPT, 1, 0, conv_mfma_kernel<KH, KW, CC, WO, WP, RO, RP, PPT, 1>,                          \
     conv_mfma_kernel<KH, KW, CC, WO, WP, RO, RP, PPT, 1, false, true>}
#define KXC_VARIANT_KS_DS(KH, KW, CC, WO, WP, RO, RP, PPT, KS)                                         \
    {"mfma_k" #KH "x" #KW "_c" #CC "_o" #WO "x" #RO "_p" #WP "x" #RP "_ks" #KS, KH, KW, CC, 32 * RO * WO,   \
     32 * RP * WP, WO * WP, PPT, KS, 0, conv_mfma_kernel<KH, KW, CC, WO, WP, RO, RP, PPT, KS>,          \
     conv_mfma_kernel<KH, KW, CC, WO, WP, RO, RP, PPT, KS, false, true>}

// name = mfma_k<filter>_c<channels per chunk>_o<waves x blocks along output channels>_p<waves x blocks
// along pixels>; tile = 32*blocks*waves in each direction.
//
// Measured on MI355X (batch 64 ResNet-18 layers): one 32x32 block per wave with many waves per SIMD
// beats larger register tiles -- the matrix pipe is kept busy by wave-level parallelism, and small
// workgroups (32 output channels x 128 pixels, 28 KiB of LDS) fit five to a CU and balance the
// 256 CUs well.  Per filter size the table is in order of preference; Select() takes the first
// entry that fits the shape, except that launches too small to fill the GPU take the entry with
// the most workgroups.
//
// Register-blocked tiles for the three 3x3 stride-2 launches with a second output (a wave keeps 32 channels x 64 to
// 224 pixels of both outputs), forced one layer at a time inside the batch-64 network: every one slower than the
// table's choice (64 x 128 in four waves of 32 x 64: the 28 x 28 layer's pass 1.567 -> 1.609 ms; 64 x 256 in eight
// waves of 32 x 64 on the 56 x 56 layer: 1.567 -> 1.579 ms; 32 x 224 per wave: four to ten times slower, the two
// accumulator sets no longer fit the registers).  Only the 3-channel first layer gains from blocking (see below).
const Variant kVariants[] = {
    KXC_VARIANT_DS(3, 3, 4, 1, 4, 1, 1, 4),   // 32 x 128, 4 waves            (default)
    KXC_VARIANT_DS(3, 3, 4, 1, 8, 1, 1, 2),   // 32 x 256, 8 waves            (14x14 maps: fewer weight refills)
    KXC_VARIANT_DS(3, 3, 2, 1, 4, 1, 1, 4),   // 32 x 128, 2-channel chunks   (stride-2 56->28: smaller patch)
    KXC_VARIANT_DS(3, 3, 4, 1, 2, 1, 1, 8),   // 32 x 64, 2 waves             (small launches)
    KXC_VARIANT(3, 3, 4, 2, 4, 1, 1, 4),   // 64 x 128, 8 waves
    KXC_VARIANT_DS(3, 3, 4, 2, 8, 1, 1, 2),   // 64 x 256, 16 waves
    KXC_VARIANT_DS(3, 3, 4, 2, 7, 1, 1, 2),   // 64 x 224, 14 waves
    KXC_VARIANT(3, 3, 4, 1, 4, 2, 1, 4),   // 64 x 128, 4 waves of 64x32
    KXC_VARIANT(3, 3, 4, 1, 4, 2, 2, 4),   // 64 x 256, 4 waves of 64x64
    KXC_VARIANT(3, 3, 8, 1, 8, 1, 1, 2),   // 8-channel chunks
    KXC_VARIANT_KS_DS(3, 3, 4, 1, 4, 1, 1, 4, 2),   // 32 x 128, reduction split 2 ways (8 waves)
    KXC_VARIANT_KS_DS(3, 3, 4, 1, 7, 1, 1, 4, 2),   // 32 x 224, split 2 ways (14 waves)
    KXC_VARIANT_KS_DS(3, 3, 4, 1, 2, 1, 1, 8, 4),   // 32 x 64, split 4 ways (8 waves)
    KXC_VARIANT_KS_DS(3, 3, 4, 1, 2, 1, 1, 8, 8),   // 32 x 64, split 8 ways (16 waves)
    KXC_VARIANT(1, 1, 8, 1, 4, 2, 1, 4),   // 64 x 128
    KXC_VARIANT(1, 1, 8, 1, 4, 2, 2, 6),   // 64 x 256
    KXC_VARIANT(1, 1, 8, 2, 2, 1, 1, 6),   // 64 x 64
    KXC_VARIANT(1, 1, 8, 1, 4, 1, 1, 4),   // 32 x 128
    KXC_VARIANT(1, 1, 16, 2, 2, 1, 1, 6),
    KXC_VARIANT_KS(1, 1, 8, 1, 4, 1, 1, 4, 2),   // reduction split inside the workgroup for small launches
    KXC_VARIANT_KS(1, 1, 8, 1, 4, 1, 1, 4, 4),
    KXC_VARIANT_KS(1, 1, 8, 1, 2, 1, 1, 8, 8),
    KXC_VARIANT_TP(7, 7, 1, 1, 8, 2, 1, 8),   // 64 x 256, taps paired, one channel per chunk (double buffered): RGB first layer
    KXC_VARIANT_TP(7, 7, 1, 1, 8, 1, 1, 8),   // 32 x 256, one channel per chunk
    KXC_VARIANT_TP(7, 7, 1, 1, 4, 1, 1, 12),  // 32 x 128, one channel per chunk
    KXC_VARIANT_TP(7, 7, 3, 1, 8, 1, 1, 8),   // 32 x 256, all three channels in one chunk
    KXC_VARIANT_TP(7, 7, 3, 1, 4, 1, 1, 12),  // 32 x 128
    KXC_VARIANT_TP(7, 7, 3, 1, 8, 2, 1, 8),   // 64 x 256
    // tiles that are whole rows of a 112-wide map, which the pooling epilogue needs.  Seven 32-pixel blocks per
    // row pair do not divide over eight waves: seven waves of one block each leave a SIMD short (227 us for the
    // batch-64 first layer against 194 us for the 64 x 256 tile), 14 waves of one block 255 us; four waves that
    // each keep 32 channels x 224 pixels (seven blocks) in registers reach 192 us.
    KXC_VARIANT_TP_HP(7, 7, 1, 2, 2, 1, 7, 12),  // 64 x 448, 4 waves of 32 x 224
    KXC_VARIANT_TP_HP(7, 7, 1, 1, 7, 2, 1, 8),   // 64 x 224, 7 waves of 64 x 32
    KXC_VARIANT(7, 7, 2, 1, 8, 1, 1, 8),   // 32 x 256; 2-channel chunks: two chunks for RGB, loads overlap compute
    KXC_VARIANT(7, 7, 2, 1, 7, 1, 1, 8),   // 32 x 224: two full output rows of a 112-wide map
    KXC_VARIANT(7, 7, 4, 1, 8, 1, 1, 8),   // 32 x 256, one chunk (3 input channels padded to 4)
    KXC_VARIANT(7, 7, 2, 1, 4, 1, 1, 12),  // 32 x 128
    KXC_VARIANT(7, 7, 4, 1, 4, 1, 1, 12),
};
constexpr int kNumVariants = sizeof(kVariants) / sizeof(kVariants[0]);

struct Choice {
    const Variant* v = nullptr;
    int32_t chs = 0;
    int32_t plane = 0;      // > 0: phase-plane patch layout with planes of this many floats (see ConvArgs)
    size_t lds_bytes = 0;
};

// Stride 2 both ways, no dilation, even padded extents: the patch can be staged as four phase planes
// (KXC_HIP_CONV_PHASE=1; 2: also for the tap-pairing 7x7 kernels).  Off by default.  Measured on MI355X, batch 64,
// the three 3x3/2 + 1x1/2 launches of ResNet-18: SQ_LDS_BANK_CONFLICT drops from 7.5M / 4.5M / 16.1M cycles per
// launch to 4.0M each, and the launch times do not move (98 / 95 / 108 us; the 56 -> 28 layer gets 3 % slower
// because its planes round up to one more 64-float segment per channel): LDS bank conflicts are not what limits
// these kernels -- how evenly the workgroups fill the compute units is (see Select()).
bool UsePhasePlanes(const ConvArgs& a, const Variant& v) {
    if (a.sh != 2 || a.sw != 2 || a.dh != 1 || a.dw != 1 || (a.Hp & 1) || (a.Wp & 1)) return false;
    const char* e = std::getenv("KXC_HIP_CONV_PHASE");
    const int mode = e ? std::atoi(e) : 0;
    return mode == 2 || (mode == 1 && !v.tpair);
}

// Largest padded-row span any pixel tile of size tp touches.
int32_t MaxTileRows(const ConvArgs& a, int kh, int tp) {
    int32_t best = 0;
    for (int64_t m0 = 0; m0 < a.M; m0 += tp) {
        const int64_t ml = (m0 + tp < a.M ? m0 + tp : a.M) - 1;
        const int32_t n = static_cast<int32_t>(m0 / a.OHW), rem = static_cast<int32_t>(m0 - static_cast<int64_t>(n) * a.OHW);
        const int32_t n2 = static_cast<int32_t>(ml / a.OHW), rem2 = static_cast<int32_t>(ml - static_cast<int64_t>(n2) * a.OHW);
        const int32_t qmin = n * a.Hp + (rem / a.OW) * a.sh;
        const int32_t qlast = n2 * a.Hp + (rem2 / a.OW) * a.sh + (kh - 1) * a.dh;
        if (qlast - qmin + 1 > best) best = qlast - qmin + 1;
    }
    return best;
}

constexpr size_t kMaxLdsBytes = 160 * 1024;  // LDS of one gfx950 compute unit
constexpr int kNumCUs = 256;

bool Fits(const Variant& v, const ConvArgs& a, Choice* out, bool ds = false) {
    if (ds && !v.ds_kernel) return false;
    const int32_t rows = MaxTileRows(a, v.kh, v.tp);
    const bool phase = UsePhasePlanes(a, v);
    const int64_t plane = phase ? static_cast<int64_t>((rows + 1) / 2) * (a.Wp / 2) : 0;
    const int64_t P = phase ? 4 * plane : static_cast<int64_t>(rows) * a.Wp;
    const int64_t segs = (P + 63) / 64;
    if (segs > static_cast<int64_t>(v.ppt) * v.nw) return false;
    // Channel stride: a multiple of 64 floats plus 32, so the two half-waves (which read channels
    // c and c+1 at the same position) fall into different halves of the LDS banks.
    // With a horizontal stride of 2 the lanes of a half-wave already use every other bank, so the second
    // half-wave is skewed by one more float to land on the odd banks.
    // (Phase planes are read densely: no skew.)
    const int32_t chs = static_cast<int32_t>(segs * 64 + 32) + ((a.sw % 2 == 0 && !v.tpair && !phase) ? 1 : 0);
    const int khw = v.kh * v.kw;
    if (v.tpair && a.C % 2 == 0) return false;     // pairing taps pays when channels cannot be paired evenly
    const int ks2 = (v.tpair ? v.cc * ((khw + 1) / 2) : (v.cc / 2) * khw) | 1;
    const int pl = (v.to * ks2 + 63) / 64 * 64 + 32;
    const int nchunks = (a.C + v.cc - 1) / v.cc;
    if (v.ks > 1 && nchunks < 2 * v.ks) return false;          // not enough reduction to split
    const int buffers = (nchunks + v.ks - 1) / v.ks > 1 ? 2 : 1;   // a single chunk step needs no second buffer
    const size_t xs_size = (static_cast<size_t>(v.cc) * chs + 31) & ~static_cast<size_t>(31);
    const int plb = (v.to * ((v.cc / 2) | 1) + 63) / 64 * 64 + 32;                 // second output's weight planes
    size_t lds = static_cast<size_t>(v.ks) * buffers * (xs_size + 2 * static_cast<size_t>(pl) + (ds ? 2 * static_cast<size_t>(plb) : 0)) * sizeof(float);
    const size_t red = static_cast<size_t>(v.ks - 1) * v.to * v.tp * sizeof(float);   // partial accumulators
    if (red > lds) lds = red;
    if (lds > kMaxLdsBytes) return false;
    out->v = &v;
    out->chs = chs;
    out->plane = static_cast<int32_t>(plane);
    out->lds_bytes = lds;
    return true;
}

// Picks the MFMA variant for a shape, or leaves choice.v == nullptr for the direct kernel.
void Select(const ConvArgs& real, int kh, int kw, Choice* choice, bool ds = false) {
    choice->v = nullptr;
    if (real.O < 32 || real.M < 32) return;
    // the rules below see the pixels of all launches expected to run side by side
    ConvArgs a = real;
    if (static_cast<int64_t>(a.M) * SelectLanes() < (1LL << 31)) a.M *= SelectLanes();
    // 32-bit byte offsets inside the kernel
    const int64_t x_bytes = static_cast<int64_t>(a.N) * a.C * a.H * a.W * 4;
    const int64_t y_elems = static_cast<int64_t>(a.N) * a.O * a.OHW;
    const int64_t w_bytes = static_cast<int64_t>(a.O) * a.C * kh * kw * 4;
    const int64_t q_rows = static_cast<int64_t>(a.N + 1) * a.Hp + kh * a.dh;
    if (x_bytes >= (1LL << 31) || y_elems * 4 >= (1LL << 31) || w_bytes >= (1LL << 31) || q_rows * a.Wp >= (1LL << 31)) return;
    const char* forced = std::getenv("KXC_HIP_CONV_VARIANT");
    // Shape rules on top of the table order (measured, see the table's comment).
    const char* preferred = nullptr;
    if (kh == 3 && a.OW <= 14 && a.M >= 8192) preferred = "mfma_k3x3_c4_o1x1_p8x1";
    if (kh == 3 && a.sh == 2 && a.W >= 56) preferred = "mfma_k3x3_c2_o1x1_p4x1";
    if (kh == 3 && a.sh == 2 && a.W >= 28 && a.W < 56 && a.O % 64 == 0 && a.M >= 8192) preferred = "mfma_k3x3_c4_o2x1_p8x1";
    if (kh == 3 && a.sh == 1 && a.W >= 56 && a.O % 64 == 0 && a.M >= 65536) preferred = "mfma_k3x3_c4_o1x2_p4x1";
    if (kh == 7 && kw == 7) {
        // first layer at small batch: fewer than 128 of the 64 x 256 tiles leave half the compute units idle
        // (batch 1: 17.5 us; 32 x 128 tiles 10.8 us; batch 2: 18.1 us; 32 x 256 tiles 12.9 us; equal from batch 4 on)
        const int64_t big_tiles = CeilDiv(a.M, 256) * CeilDiv(a.O, 64);
        if (big_tiles < 64) preferred = "mfma_k7x7_t1_o1x1_p4x1";
        else if (big_tiles < 128) preferred = "mfma_k7x7_t1_o1x1_p8x1";
    }
    // Pass 0 takes the rule's variant (or the forced one).  Pass 1 takes the first table entry that fits,
    // unless that launch would leave most SIMDs idle (fewer than three waves per SIMD): then the reduction is
    // split inside the workgroup -- two ways on the 32x128 tile if that is enough, else four or eight ways on
    // the 32x64 tile (measured: layer4 43% -> 53% of peak, batch-1 layers 1.6x faster).
    constexpr int64_t kEnoughWaves = 3 * 4 * kNumCUs;
    static const char* const kSplitOrder3x3[] = {"mfma_k3x3_c4_o1x1_p4x1_ks2", "mfma_k3x3_c4_o1x1_p2x1_ks4",
                                                 "mfma_k3x3_c4_o1x1_p2x1_ks8"};
    static const char* const kSplitOrder1x1[] = {"mfma_k1x1_c8_o1x1_p4x1_ks2", "mfma_k1x1_c8_o1x1_p4x1_ks4",
                                                 "mfma_k1x1_c8_o1x1_p2x1_ks8"};
    const char* const* kSplitOrder = kh == 1 ? kSplitOrder1x1 : kSplitOrder3x3;
    Choice first_fit;
    int64_t first_waves = 0;
    Choice split[3];
    int64_t split_waves[3] = {0, 0, 0};
    for (int pass = 0; pass < 2 && !choice->v; ++pass) {
        for (int i = 0; i < kNumVariants; ++i) {
            const Variant& v = kVariants[i];
            if (v.kh != kh || v.kw != kw) continue;
            if (forced && *forced && std::strcmp(forced, v.name) != 0) continue;
            if (pass == 0 && !(forced && *forced) && (!preferred || std::strcmp(preferred, v.name) != 0)) continue;
            if (v.to > a.O && v.to > 32) continue;    // do not spend matrix work on absent output channels
            Choice c;
            if (!Fits(v, a, &c, ds)) continue;
            if (pass == 0 || (forced && *forced)) { *choice = c; return; }
            const int64_t waves = CeilDiv(a.M, v.tp) * CeilDiv(a.O, v.to) * v.nw * v.ks;
            if (!first_fit.v && v.ks == 1) { first_fit = c; first_waves = waves; }
            for (int k = 0; k < 3; ++k)
                if (std::strcmp(v.name, kSplitOrder[k]) == 0) { split[k] = c; split_waves[k] = waves; }
        }
        if (pass == 1) {
            *choice = first_fit;
            // (a 1x1 filter's reduction is only as long as its input channels: splitting 64 or 128 of them costs more
            // than the idle SIMDs -- batch 32, 64 -> 128 channels at 56 x 56, stride 2: 26.6 us split two ways, 21.4 whole)
            if (first_fit.v && first_waves < kEnoughWaves && !(kh == 1 && a.C < 256)) {
                for (int k = 0; k < 3; ++k) {
                    if (!split[k].v) continue;
                    *choice = split[k];
                    if (split_waves[k] >= 2560) break;      // enough waves: stop splitting further
                    // 3x3: two wave groups on the 32 x 128 tile plus the split over workgroups beat the deeper
                    // splits on 32 x 64 tiles from batch 1 to 16, at stride 2 (batch 8, 128 -> 256 channels at
                    // 28 x 28: 20.5 against 31.5 us) and at stride 1 (batch 1, 256 channels at 14 x 14: 12.6
                    // against 19.8 us with the adding kernel; batch 4, 512 channels at 7 x 7: 23.8 against 37.9)
                    if (kh == 3) break;
                }
            }
            // Every workgroup of a launch does the same work, so the launch takes as long as the compute unit with
            // the most workgroups: 400 of the 32 x 128 two-group tiles (batch 64, 256 -> 512 channels at 14 x 14,
            // stride 2) are two on 144 compute units and one on the rest (measured: 256 tiles 77 us, 400 tiles 109,
            // 512 tiles 116).  The 32 x 224 tile makes 224 workgroups of 14 waves, one per compute unit: 106 us
            // against 118 in the same process.  Taken when it fills the compute units better.
            if (kh == 3 && choice->v && std::strcmp(choice->v->name, "mfma_k3x3_c4_o1x1_p4x1_ks2") == 0 && a.M >= 2048) {
                auto fill = [&](const Variant& v) {
                    const int64_t wgs = CeilDiv(a.M, v.tp) * CeilDiv(a.O, v.to);
                    return static_cast<double>(wgs) / static_cast<double>(CeilDiv(wgs, kNumCUs) * kNumCUs);
                };
                for (int i = 0; i < kNumVariants; ++i) {
                    const Variant& v = kVariants[i];
                    Choice c;
                    if (std::strcmp(v.name, "mfma_k3x3_c4_o1x1_p7x1_ks2") != 0 || !Fits(v, a, &c, ds)) continue;
                    if (CeilDiv(a.M, v.tp) * CeilDiv(a.O, v.to) <= kNumCUs && fill(v) > fill(*choice->v) + 0.05) *choice = c;
                }
            }
        }
    }
}

// The variant whose pooling epilogue (KXC_HIP_CONV_HPOOL) covers a shape: ReLU and no residual, an even output
// width, tiles that are whole output rows and all full.  `a` is the shape after FillArgs.
bool HpoolChoice(const kxc_hip_conv2d_desc* desc, const ConvArgs& a, Choice* choice) {
    choice->v = nullptr;
    if (!(desc->flags & KXC_HIP_CONV_RELU) || (desc->flags & (KXC_HIP_CONV_RESIDUAL | KXC_HIP_CONV_FORCE_DIRECT))) return false;
    if (a.M <= 0 || a.OW < 2 || (a.OW & 1)) return false;
    if (a.O % 8 != 0) return false;      // the epilogue masks absent channels eight at a time
    const int64_t x_bytes = static_cast<int64_t>(a.N) * a.C * a.H * a.W * 4;
    const int64_t y_elems = static_cast<int64_t>(a.N) * a.O * a.OHW;
    const int64_t w_bytes = static_cast<int64_t>(a.O) * a.C * desc->kh * desc->kw * 4;
    const int64_t q_rows = static_cast<int64_t>(a.N + 1) * a.Hp + desc->kh * a.dh;
    if (x_bytes >= (1LL << 31) || y_elems * 4 >= (1LL << 31) || w_bytes >= (1LL << 31) || q_rows * a.Wp >= (1LL << 31)) return false;
    const char* forced = std::getenv("KXC_HIP_CONV_HPOOL_VARIANT");
    for (int i = 0; i < kNumVariants; ++i) {
        const Variant& v = kVariants[i];
        if (!v.hp_kernel || v.kh != desc->kh || v.kw != desc->kw) continue;
        if (forced && *forced && std::strcmp(forced, v.name) != 0) continue;
        if (v.tp % a.OW != 0 || a.M % v.tp != 0) continue;
        Choice c;
        if (!Fits(v, a, &c)) continue;
        *choice = c;
        return true;
    }
    return false;
}

int32_t FillArgs(const kxc_hip_conv2d_desc* d, ConvArgs* a, const char* who) {
    KXC_HIP_REQUIRE(d != nullptr, "%s: desc is NULL", who);
    KXC_HIP_REQUIRE(d->n >= 0 && d->c > 0 && d->h > 0 && d->w > 0 && d->o > 0 && d->kh > 0 && d->kw > 0,
                    "%s: bad shape", who);
    KXC_HIP_REQUIRE(d->stride_h > 0 && d->stride_w > 0 && d->dil_h > 0 && d->dil_w > 0,
                    "%s: nn_conv2d stride and dilation must be positive", who);
    KXC_HIP_REQUIRE(d->pad_h >= 0 && d->pad_w >= 0, "%s: negative padding", who);
    // WindowOutputDim (src/relay/type_infer.cc:166-184)
    const int64_t nh = static_cast<int64_t>(d->h) + 2 * d->pad_h - (static_cast<int64_t>(d->dil_h) * (d->kh - 1) + 1);
    const int64_t nw = static_cast<int64_t>(d->w) + 2 * d->pad_w - (static_cast<int64_t>(d->dil_w) * (d->kw - 1) + 1);
    KXC_HIP_REQUIRE(nh >= 0 && nw >= 0, "%s: nn_conv2d window is larger than input", who);
    std::memset(a, 0, sizeof(*a));
    a->N = d->n; a->C = d->c; a->H = d->h; a->W = d->w; a->O = d->o;
    a->OH = static_cast<int32_t>(nh / d->stride_h + 1);
    a->OW = static_cast<int32_t>(nw / d->stride_w + 1);
    a->sh = d->stride_h; a->sw = d->stride_w; a->ph = d->pad_h; a->pw = d->pad_w; a->dh = d->dil_h; a->dw = d->dil_w;
    a->Hp = d->h + 2 * d->pad_h; a->Wp = d->w + 2 * d->pad_w;
    a->Hv = d->h; a->row_step = 1;
    a->OHW = a->OH * a->OW;
    const int64_t M = static_cast<int64_t>(d->n) * a->OHW;
    a->M = M < (1LL << 31) ? static_cast<int32_t>(M) : 0;
    a->flags = d->flags;
    return KXC_HIP_OK;
}

void ApplyRowView(ConvArgs* a, int kh) {
    if (kh == 1 && a->ph == 0 && a->sh > 1) {
        a->Hv = a->OH; a->Hp = a->OH; a->row_step = a->sh; a->sh = 1;
    }
}

// The small-launch 1x1 kernel takes unpadded 1x1 filters with C % 8 == 0 while the whole launch has at most 2^21
// outputs (pixels x channels).  Measured on the three ResNet-18 downsamples: 5.3 / 6.1 / 7.9 us against 10.0 / 12.0 / 15.6 us
// for the general kernel at batch 1, still ahead at batch 16 (14.1 / 13.3 / 13.2 against 17.6 / 20.9 / 18.3) and, for
// the two deeper ones, at batch 32 (1.6 M outputs each: 22.4 / 24.2 against 29.5 / 26.2); behind from 3.2 M outputs
// on (batch 64, 128 -> 256 channels at 28 x 28: 43.4 against 35.2 us for the 64 x 128 tile; batch 32, 64 -> 128 at
// 56 x 56: 25.7 against 21.3).
bool UseSmall1x1(const kxc_hip_conv2d_desc* d, const ConvArgs& a) {
    if (d->kh != 1 || d->kw != 1 || d->pad_h != 0 || d->pad_w != 0 || a.C % 8 != 0 || a.M <= 0) return false;
    if (d->flags & KXC_HIP_CONV_FORCE_DIRECT) return false;
    const int64_t x_elems = static_cast<int64_t>(a.N) * a.C * a.H * a.W, y_elems = static_cast<int64_t>(a.N) * a.O * a.OHW;
    if (x_elems >= (1LL << 31) || y_elems >= (1LL << 31) || CeilDiv(a.M, 32) > 65535) return false;
    if (const char* e = std::getenv("KXC_HIP_CONV_VARIANT")) return std::strcmp(e, "mfma_k1x1_small") == 0;
    return a.M <= 16384 && static_cast<int64_t>(a.M) * a.O <= (1LL << 21);
}

// Launches that still leave most SIMDs idle (batch 1, deep layers: a handful of tiles, a long reduction) split
// the reduction over workgroups as well; every workgroup keeps at least two chunks per wave group, and the partial
// sums stay small next to the caches (the split re-reads them once): at most 8 MiB.
void SplitOverWorkgroups(const Choice& c, int32_t nchunks, int64_t tiles, int64_t total, int* out_split) {
    const int64_t waves = tiles * SelectLanes() * c.v->nw * c.v->ks;      // of all launches expected side by side
    int split = 1;
    while (split < 16 && waves * split < 2048 && nchunks / (split * 2) >= 2 * c.v->ks &&
           total * static_cast<int64_t>(sizeof(float)) * split * 2 <= (8LL << 20))
        split *= 2;
    if (const char* e = std::getenv("KXC_HIP_CONV_GSPLIT")) {
        // (a forced split is honoured while its partial sums stay below 256 MiB)
        const int f = std::atoi(e);
        if (f >= 1 && f <= nchunks && total * static_cast<int64_t>(sizeof(float)) * f <= (256LL << 20)) split = f;
    }
    *out_split = split;
}

// ------------------------------------------------------------------------------------------
// Scratch of the entry point that allocates nothing (kxc_hip_conv2d_nchw_f32_noalloc): the raw partial sums of a
// reduction split over workgroups live in this file-scope device array instead of a hipMalloc'ed buffer.  Every
// GPU the library runs on holds its own copy (8 MiB) until the process ends.  The array's name is only a host-side
// handle; its device address is asked for once per device (with that device current) and kernels get that address.
// ------------------------------------------------------------------------------------------
constexpr size_t kNoAllocScratchBytes = static_cast<size_t>(8) << 20;
static __device__ __align__(256) float scratch[kNoAllocScratchBytes / sizeof(float)];

constexpr int kMaxDevices = 64;
int32_t NoAllocScratch(float** out) {
    static std::mutex mu;
    static float* addr[kMaxDevices] = {};
    int dev = 0;
    KXC_HIP_CALL(hipGetDevice(&dev), "hipGetDevice");
    KXC_HIP_REQUIRE(dev >= 0 && dev < kMaxDevices, "kxc_hip_conv2d_nchw_f32_noalloc: device %d out of range", dev);
    std::lock_guard<std::mutex> lock(mu);
    if (!addr[dev]) {
        float* p = nullptr;
        KXC_HIP_CALL(hipGetSymbolAddress(reinterpret_cast<void**>(&p), HIP_SYMBOL(scratch)), "hipGetSymbolAddress(scratch)");
        KXC_HIP_REQUIRE(p != nullptr, "kxc_hip_conv2d_nchw_f32_noalloc: no device address for the scratch array");
        addr[dev] = p;
    }
    *out = addr[dev];
    return KXC_HIP_OK;
}

// Whether a convolution can carry the second output: the 1x1 convolution's operand x[n,c,oh*sh,ow*sw] must be a tap
// of this window, i.e. the padding is a multiple of the dilation and lies inside the filter.
bool PairTap(const kxc_hip_conv2d_desc* d, int* rh, int* rw) {
    if (d->pad_h % d->dil_h != 0 || d->pad_w % d->dil_w != 0) return false;
    *rh = d->pad_h / d->dil_h; *rw = d->pad_w / d->dil_w;
    if (*rh >= d->kh || *rw >= d->kw) return false;
    // ... and the unpadded 1x1 convolution must have this convolution's output extent (true for "same" padding,
    // 2*pad = dil*(k-1)): otherwise the second output would have rows or columns the 1x1 convolution does not have
    const int64_t oh = (static_cast<int64_t>(d->h) + 2 * d->pad_h - (static_cast<int64_t>(d->dil_h) * (d->kh - 1) + 1)) / d->stride_h + 1;
    const int64_t ow = (static_cast<int64_t>(d->w) + 2 * d->pad_w - (static_cast<int64_t>(d->dil_w) * (d->kw - 1) + 1)) / d->stride_w + 1;
    return oh == (d->h - 1) / d->stride_h + 1 && ow == (d->w - 1) / d->stride_w + 1;
}

// Everything about a launch that the descriptor alone decides (kernel, tile shape, grid, the split of the reduction,
// the switches read from the environment): resolved once per call by the entry points, once per node by a launch
// plan (kxc_hip::PreparedConv), and combined with the operand pointers and the stream at launch time.
struct ConvLaunch {
    enum Path { kEmpty, kSmall1x1, kMfma, kDirect };
    Path path = kEmpty;
    ConvArgs a;                     // without operand pointers and partial-sum buffer
    ConvArgs direct_args;
    void (*kernel)(const ConvArgs) = nullptr;
    const char* name = "";
    dim3 grid, block;
    size_t lds_bytes = 0;
    size_t scratch_bytes = 0;       // partial sums of a reduction split over workgroups (0: none)
    int32_t kh = 0, kw = 0;
    int64_t total = 0;
    bool second = false;
};

int32_t Conv2dResolve(const kxc_hip_conv2d_desc* desc, bool second, const char* who, ConvLaunch* L) {
    ConvArgs& a = L->a;
    if (int32_t rc = FillArgs(desc, &a, who)) return rc;
    L->second = second;
    L->kh = desc->kh; L->kw = desc->kw;
    L->total = static_cast<int64_t>(a.N) * a.O * a.OHW;
    if (L->total == 0) { L->path = ConvLaunch::kEmpty; return KXC_HIP_OK; }
    const int64_t total = L->total;
    a.x_bytes = static_cast<uint32_t>(static_cast<int64_t>(a.N) * a.C * a.H * a.W * 4);       // < 2 GiB on the MFMA path
    a.w_bytes = static_cast<uint32_t>(static_cast<int64_t>(a.O) * a.C * desc->kh * desc->kw * 4);

    // A filter one row high with a vertical stride touches only every stride-th input row (the 1x1/2
    // downsample convolutions): the matrix kernel then sees an image of OH rows that are stride rows apart, so
    // the skipped rows are neither loaded nor staged.
    const bool hpool = (desc->flags & KXC_HIP_CONV_HPOOL) != 0;
    if (!second && !hpool && UseSmall1x1(desc, a)) {
        a.div_ohw = MakeFastDiv(a.OHW); a.div_ow = MakeFastDiv(a.OW);
        L->path = ConvLaunch::kSmall1x1;
        a.o_tiles = static_cast<int32_t>(CeilDiv(a.O, 32));
        a.p_tiles = static_cast<int32_t>(CeilDiv(a.M, 32));
        a.num_tiles = a.o_tiles * a.p_tiles;
        a.tiles_per_xcd = (a.num_tiles + 7) / 8;
        a.div_otiles = MakeFastDiv(a.o_tiles);
        L->grid = dim3(static_cast<unsigned>(a.tiles_per_xcd * 8));
        // eight waves split a long reduction (each keeps an even number of channels)
        const bool eight = a.C >= 256 && a.C % 16 == 0;
        L->kernel = eight ? conv1x1_small_kernel<8> : conv1x1_small_kernel<4>;
        L->block = dim3(eight ? 512 : 256);
        L->name = "mfma_k1x1_small";
        return KXC_HIP_OK;
    }
    L->direct_args = a;
    ApplyRowView(&a, desc->kh);
    Choice c;
    if (hpool) {
        KXC_HIP_REQUIRE(!second && HpoolChoice(desc, a, &c), "%s: no kernel with the pooling epilogue covers this shape", who);
        a.PW = a.OW / 2;
    } else if (!(desc->flags & KXC_HIP_CONV_FORCE_DIRECT) && a.M > 0) {
        Select(a, desc->kh, desc->kw, &c, second);
    }
    if (second) {
        int rh = 0, rw = 0;
        KXC_HIP_REQUIRE(c.v && c.v->ds_kernel && PairTap(desc, &rh, &rw), "%s: no kernel with a second output covers this shape", who);
        a.w2_bytes = static_cast<uint32_t>(static_cast<int64_t>(a.O) * a.C * 4);
        a.ds_off = c.plane > 0 ? ((rh & 1) * 2 + (rw & 1)) * c.plane + (rh >> 1) * (a.Wp / 2) + (rw >> 1)
                               : rh * a.dh * a.Wp + rw * a.dw;
    }
    if (!c.v) {
        int64_t g = CeilDiv(total, 256);
        if (g > 256 * 64) g = 256 * 64;
        L->path = ConvLaunch::kDirect;
        L->grid = dim3(static_cast<unsigned>(g));
        L->block = dim3(256);
        L->name = "conv_direct";
        return KXC_HIP_OK;
    }
    a.chs = c.chs;
    a.phase = c.plane > 0 ? 1 : 0;
    a.plane = c.plane;
    a.halfw = a.Wp / 2;
    a.div_plane = MakeFastDiv(a.plane);
    a.div_halfw = MakeFastDiv(a.halfw);
    a.nchunks = (a.C + c.v->cc - 1) / c.v->cc;
    a.p_tiles = static_cast<int32_t>(CeilDiv(a.M, c.v->tp));
    a.o_tiles = static_cast<int32_t>(CeilDiv(a.O, c.v->to));
    const int64_t tiles = static_cast<int64_t>(a.p_tiles) * a.o_tiles;
    KXC_HIP_REQUIRE(tiles < (1LL << 30), "%s: too many tiles", who);
    a.num_tiles = static_cast<int32_t>(tiles);
    // Launches that still leave most SIMDs idle (batch 1, deep layers: a handful of tiles, a long reduction)
    // split the reduction over workgroups as well; every workgroup keeps at least two chunks per wave group.
    a.gsplit = 1;
    a.cps = a.nchunks;
    a.out_elems = hpool ? static_cast<int64_t>(a.N) * a.O * a.OH * a.PW : total;
    int split = 1;
    // (a second output has parts of its own; the pooling epilogue needs the whole sum in one workgroup)
    if (!hpool) SplitOverWorkgroups(c, a.nchunks, tiles, total * (second ? 2 : 1), &split);
    if (split > 1) {
        a.cps = static_cast<int32_t>(CeilDiv(a.nchunks, split));
        a.gsplit = static_cast<int32_t>(CeilDiv(a.nchunks, a.cps));      // no empty split
        if (a.gsplit > 1) L->scratch_bytes = static_cast<size_t>(a.gsplit) * total * sizeof(float) * (second ? 2 : 1);
        else a.cps = a.nchunks;
    }
    a.div_gsplit = MakeFastDiv(a.gsplit);
    a.tiles_per_xcd = static_cast<int32_t>(CeilDiv(tiles * a.gsplit, 8));
    a.div_wp = MakeFastDiv(a.Wp); a.div_hp = MakeFastDiv(a.Hp); a.div_ohw = MakeFastDiv(a.OHW);
    a.div_ow = MakeFastDiv(a.OW); a.div_otiles = MakeFastDiv(a.o_tiles); a.div_ptiles = MakeFastDiv(a.p_tiles);
    // weights of one output-channel tile: to * C * kh * kw * 4 bytes; keep the larger operand resident
    const int64_t w_tile_bytes = static_cast<int64_t>(c.v->to) * a.C * desc->kh * desc->kw * 4;
    a.o_fastest = w_tile_bytes * a.o_tiles <= (2 << 20) ? 1 : 0;
    if (const char* e = std::getenv("KXC_HIP_CONV_OFAST")) a.o_fastest = std::atoi(e);
    L->path = ConvLaunch::kMfma;
    L->kernel = second ? c.v->ds_kernel : hpool ? c.v->hp_kernel : c.v->kernel;
    L->name = c.v->name;
    L->grid = dim3(static_cast<unsigned>(a.tiles_per_xcd * 8));
    L->block = dim3(64 * c.v->nw * c.v->ks);
    L->lds_bytes = c.lds_bytes;
    return KXC_HIP_OK;
}

// Above the default 64 KiB the dynamic LDS size has to be granted per kernel and device (once).
int32_t GrantLds(void (*kernel)(const ConvArgs), size_t lds_bytes) {
    static std::mutex mu;
    static std::vector<std::pair<int, const void*>> granted;
    int dev = 0;
    KXC_HIP_CALL(hipGetDevice(&dev), "hipGetDevice");
    const void* fn = reinterpret_cast<const void*>(kernel);
    std::lock_guard<std::mutex> lock(mu);
    for (const auto& g : granted)
        if (g.first == dev && g.second == fn) return KXC_HIP_OK;
    KXC_HIP_CALL(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(kMaxLdsBytes)),
                 "hipFuncSetAttribute(MaxDynamicSharedMemorySize)");
    granted.emplace_back(dev, fn);
    return KXC_HIP_OK;
}

// The second output of kxc_hip_conv2d_pair_nchw_f32 (see ConvArgs).
struct SecondOutput {
    const float* w2 = nullptr;
    const float* bias2 = nullptr;
    float* y2 = nullptr;
};

// no_alloc: the partial sums of a split reduction go to the file-scope scratch array instead of the grow-only
// per-stream buffer, and a launch that would need more is refused.
int32_t Conv2dLaunch(const ConvLaunch& L, const char* who, const float* x, const float* w, const float* bias,
                     const float* residual, float* y, void* stream, bool no_alloc, const SecondOutput* second) {
    if (L.path == ConvLaunch::kEmpty) return KXC_HIP_OK;
    KXC_HIP_REQUIRE(x && w && y, "%s: NULL pointer", who);
    KXC_HIP_REQUIRE(!(L.a.flags & KXC_HIP_CONV_BIAS) || bias, "%s: bias flag without bias", who);
    KXC_HIP_REQUIRE(!(L.a.flags & KXC_HIP_CONV_RESIDUAL) || residual, "%s: residual flag without residual", who);
    KXC_HIP_REQUIRE(L.second == (second != nullptr), "%s: launch resolved for a different number of outputs", who);
    hipStream_t s = ResolveStream(stream);
    if (L.path == ConvLaunch::kDirect) {
        ConvArgs d = L.direct_args;
        d.x = x; d.w = w; d.bias = bias; d.res = residual; d.y = y;
        conv_direct_kernel<<<NoteGrid(L.grid), NoteBlock(L.block), NoteLds(0), s>>>(d, L.kh, L.kw, L.total);
        return CheckLaunch("conv_direct");
    }
    ConvArgs a = L.a;
    a.x = x; a.w = w; a.bias = bias; a.res = residual; a.y = y;
    if (L.path == ConvLaunch::kSmall1x1) {
        hipLaunchKernelGGL(L.kernel, NoteGrid(L.grid), NoteBlock(L.block), NoteLds(0), s, a);
        return CheckLaunch(L.name);
    }
    if (second) {
        KXC_HIP_REQUIRE(second->w2 && second->y2, "%s: NULL pointer", who);
        a.w2 = second->w2; a.bias2 = second->bias2; a.y2 = second->y2;
    }
    SplitScratchLease lease;      // held until the adding kernel is enqueued
    if (L.scratch_bytes > 0) {
        if (no_alloc) {
            // every kernel of the pair overwrites what it reads later, nothing has to start at zero
            KXC_HIP_REQUIRE(L.scratch_bytes <= kNoAllocScratchBytes,
                            "%s: the split reduction needs %zu bytes of scratch, the built-in array holds %zu",
                            who, L.scratch_bytes, kNoAllocScratchBytes);
            if (int32_t rc = NoAllocScratch(&a.partial)) return rc;
        } else {
            if (int32_t rc = AcquireSplitScratch(s, L.scratch_bytes, &lease)) return rc;
            a.partial = lease.ptr;
        }
    }
    if (L.lds_bytes > 64 * 1024)
        if (int32_t rc = GrantLds(L.kernel, L.lds_bytes)) return rc;
    hipLaunchKernelGGL(L.kernel, NoteGrid(L.grid), NoteBlock(L.block), NoteLds(L.lds_bytes), s, a);
    if (int32_t rc = CheckLaunch(L.name)) return rc;
    if (a.gsplit > 1) {
        SplitReduceArgs r;
        r.partial = a.partial; r.bias = a.bias; r.res = a.res; r.y = a.y;
        r.gsplit = a.gsplit; r.total = static_cast<int32_t>(L.total); r.O = a.O; r.flags = a.flags; r.div_ohw = a.div_ohw;
        if (second) {
            r.partial2 = a.partial + static_cast<int64_t>(a.gsplit) * L.total;
            r.bias2 = a.bias2; r.y2 = a.y2; r.flags2 = a.bias2 ? KXC_HIP_CONV_BIAS : 0u;
        }
        return LaunchSplitReduce(s, r);
    }
    return KXC_HIP_OK;
}

int32_t Conv2dRun(const kxc_hip_conv2d_desc* desc, const float* x, const float* w, const float* bias,
                  const float* residual, float* y, void* stream, bool no_alloc, const SecondOutput* second = nullptr) {
    const char* const who = second ? "kxc_hip_conv2d_pair_nchw_f32" : no_alloc ? "kxc_hip_conv2d_nchw_f32_noalloc" : "kxc_hip_conv2d_nchw_f32";
    ConvLaunch L;
    if (int32_t rc = Conv2dResolve(desc, second != nullptr, who, &L)) return rc;
    return Conv2dLaunch(L, who, x, w, bias, residual, y, stream, no_alloc, second);
}

}  // namespace

namespace kxc_hip {

struct PreparedConv {
    ConvLaunch launch;
    std::string who;
};

int32_t PrepareConv2d(const kxc_hip_conv2d_desc* desc, bool second_output, PreparedConv** out) {
    std::unique_ptr<PreparedConv> p(new PreparedConv);
    p->who = second_output ? "kxc_hip_conv2d_pair_nchw_f32 (plan node)" : "kxc_hip_conv2d_nchw_f32 (plan node)";
    if (int32_t rc = Conv2dResolve(desc, second_output, p->who.c_str(), &p->launch)) return rc;
    *out = p.release();
    return KXC_HIP_OK;
}

int32_t LaunchPreparedConv2d(const PreparedConv* p, const float* x, const float* w, const float* bias, const float* residual,
                             float* y, const float* w2, const float* bias2, float* y2, hipStream_t stream) {
    SecondOutput second;
    second.w2 = w2; second.bias2 = bias2; second.y2 = y2;
    return Conv2dLaunch(p->launch, p->who.c_str(), x, w, bias, residual, y, stream, false, p->launch.second ? &second : nullptr);
}

const char* PreparedConvName(const PreparedConv* p) { return p->launch.name; }

void FreePreparedConv(PreparedConv* p) { delete p; }

}  // namespace kxc_hip

extern "C" {

const char* kxc_hip_conv2d_variant(const kxc_hip_conv2d_desc* desc) {
    ConvArgs a;
    if (FillArgs(desc, &a, "kxc_hip_conv2d_variant") != KXC_HIP_OK) return "invalid";
    if (desc->flags & KXC_HIP_CONV_HPOOL) {
        Choice hp;
        return HpoolChoice(desc, a, &hp) ? hp.v->name : "unsupported";
    }
    if (desc->flags & KXC_HIP_CONV_FORCE_DIRECT) return "direct";
    if (UseSmall1x1(desc, a)) return "mfma_k1x1_small";
    ApplyRowView(&a, desc->kh);
    Choice c;
    Select(a, desc->kh, desc->kw, &c);
    return c.v ? c.v->name : "direct";
}

int32_t kxc_hip_conv2d_nchw_f32(const kxc_hip_conv2d_desc* desc, const float* x, const float* w, const float* bias,
                                const float* residual, float* y, void* stream) {
    return Conv2dRun(desc, x, w, bias, residual, y, stream, false);
}

int32_t kxc_hip_conv2d_nchw_f32_noalloc(const kxc_hip_conv2d_desc* desc, const float* x, const float* w, const float* bias,
                                        const float* residual, float* y, void* stream) {
    return Conv2dRun(desc, x, w, bias, residual, y, stream, true);
}

size_t kxc_hip_conv2d_noalloc_scratch_bytes(void) { return kNoAllocScratchBytes; }

// Variant of the pair kernel for a shape, or nullptr.
static const Variant* PairVariant(const kxc_hip_conv2d_desc* desc) {
    ConvArgs a;
    if (!desc || FillArgs(desc, &a, "kxc_hip_conv2d_pair_supported") != KXC_HIP_OK) return nullptr;
    int rh = 0, rw = 0;
    if ((desc->flags & (KXC_HIP_CONV_FORCE_DIRECT | KXC_HIP_CONV_HPOOL)) || a.M <= 0 || !PairTap(desc, &rh, &rw)) return nullptr;
    if (desc->kh == 1 && desc->kw == 1) return nullptr;
    Choice c;
    Select(a, desc->kh, desc->kw, &c, true);
    if (!c.v || !c.v->ds_kernel) return nullptr;
    // KXC_HIP_PAIR_SPLIT=0: a launch small enough to split its reduction over workgroups (batch 1-4 of the deep
    // layers) keeps two launches instead of a two-output launch whose outputs both have parts.
    const char* ps = std::getenv("KXC_HIP_PAIR_SPLIT");
    if (ps && std::atoi(ps) == 0 && !std::getenv("KXC_HIP_CONV_VARIANT")) {
        const int32_t nchunks = (a.C + c.v->cc - 1) / c.v->cc;
        int split = 1;
        SplitOverWorkgroups(c, nchunks, CeilDiv(a.M, c.v->tp) * CeilDiv(a.O, c.v->to), static_cast<int64_t>(a.N) * a.O * a.OHW, &split);
        if (split > 1) return nullptr;
    }
    return c.v;
}

int32_t kxc_hip_conv2d_pair_supported(const kxc_hip_conv2d_desc* desc) { return PairVariant(desc) ? 1 : 0; }

int32_t kxc_hip_conv2d_hpool_supported(const kxc_hip_conv2d_desc* desc) {
    ConvArgs a;
    if (!desc || FillArgs(desc, &a, "kxc_hip_conv2d_hpool_supported") != KXC_HIP_OK) return 0;
    Choice c;
    return HpoolChoice(desc, a, &c) ? 1 : 0;
}

// Measured on MI355X, 3 -> 64 channels, 7x7 / 2 on 224 x 224, inside the network (launch + pool, us): batch 64
// 192 + 27 against 194 + 51, batch 32 114 + 17 against 109 + 26, batch 16 63 + 12 against 65 + 17, batch 8 46 + 8
// against 37 + 13, batch 4 44 + 7 against 25 + 8: the 64 x 448 tile needs 448 workgroups (16 images) to fill the
// compute units; below that the smaller tiles of the unpooled kernel win.
int32_t kxc_hip_conv2d_hpool_preferred(const kxc_hip_conv2d_desc* desc) {
    ConvArgs a;
    if (!desc || FillArgs(desc, &a, "kxc_hip_conv2d_hpool_preferred") != KXC_HIP_OK) return 0;
    Choice c;
    if (!HpoolChoice(desc, a, &c)) return 0;
    if (const char* e = std::getenv("KXC_HIP_CONV_HPOOL")) return std::atoi(e) != 0 ? 1 : 0;
    return CeilDiv(a.M, c.v->tp) * CeilDiv(a.O, c.v->to) >= 448 ? 1 : 0;
}

const char* kxc_hip_conv2d_pair_variant(const kxc_hip_conv2d_desc* desc) {
    // static storage: one name per table entry
    static std::once_flag once;
    static std::vector<std::string> names;
    std::call_once(once, [] { for (int i = 0; i < kNumVariants; ++i) names.push_back(std::string(kVariants[i].name) + "_ds"); });
    const Variant* v = PairVariant(desc);
    return v ? names[static_cast<size_t>(v - kVariants)].c_str() : "unsupported";
}

int32_t kxc_hip_conv2d_pair_nchw_f32(const kxc_hip_conv2d_desc* desc, const float* x, const float* w, const float* bias,
                                     const float* residual, float* y, const float* w2, const float* bias2, float* y2,
                                     void* stream) {
    SecondOutput second;
    second.w2 = w2; second.bias2 = bias2; second.y2 = y2;
    return Conv2dRun(desc, x, w, bias, residual, y, stream, false, &second);
}

int32_t kxc_hip_conv2d_scratch_needed(const kxc_hip_conv2d_desc* desc, size_t* out_bytes) {
    KXC_HIP_REQUIRE(out_bytes != nullptr, "kxc_hip_conv2d_scratch_needed: out_bytes is NULL");
    *out_bytes = 0;
    ConvArgs a;
    if (int32_t rc = FillArgs(desc, &a, "kxc_hip_conv2d_scratch_needed")) return rc;
    const int64_t total = static_cast<int64_t>(a.N) * a.O * a.OHW;
    if (total == 0 || (desc->flags & (KXC_HIP_CONV_FORCE_DIRECT | KXC_HIP_CONV_HPOOL)) || UseSmall1x1(desc, a) || a.M <= 0) return KXC_HIP_OK;
    ApplyRowView(&a, desc->kh);
    Choice c;
    Select(a, desc->kh, desc->kw, &c);
    if (!c.v) return KXC_HIP_OK;
    const int32_t nchunks = (a.C + c.v->cc - 1) / c.v->cc;
    int split = 1;
    SplitOverWorkgroups(c, nchunks, CeilDiv(a.M, c.v->tp) * CeilDiv(a.O, c.v->to), total, &split);
    if (split > 1) {
        const int64_t parts = CeilDiv(nchunks, CeilDiv(nchunks, split));
        if (parts > 1) *out_bytes = static_cast<size_t>(parts) * total * sizeof(float);
    }
    return KXC_HIP_OK;
}

}  // extern "C"
