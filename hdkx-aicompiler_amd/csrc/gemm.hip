// gemm.hip -- nn_dense / nn_gemm on the fp32 matrix cores.
//
//   y[m,n] = alpha * sum_k a[m,k] * b[n,k]  (+ beta * c[n])          (transB = 1, the ResNet FC layer)
//
// MFMA kernel (v_mfma_f32_32x32x2_f32): one workgroup of four waves owns a 32x32 output tile; the
// waves split K four ways and, inside a wave, the two half-waves take the lower and upper half of
// the wave's K range, so every lane walks ONE contiguous run of its own row of `a` and of `b`
// with 16-byte loads straight into the MFMA operand registers (no LDS staging, no shuffles: the
// matrix instruction only needs the two half-waves to hold different k, not adjacent k).  The four
// partial tiles are combined through LDS in a fixed order, so results are deterministic.
// The FC layer of ResNet-18 (64x512 by 1000x512) is launch-latency/weight-read bound: 64 tiles of
// four waves each keep 64 CUs busy for a few microseconds.
//
// Everything else (transB = 0, K not a multiple of 32, unaligned rows) goes to a one-thread-per-
// output kernel that adds in the CPU loop's exact order (k ascending, separate multiply and add).
#include "common.h"

using namespace kxc_hip;

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

__device__ __forceinline__ float epilogue(float acc, float alpha, float beta, const float* c, int64_t j, int64_t c_len,
                                          bool scale_a, bool scale_c) {
    float v = acc;
    if (scale_a) v = __fmul_rn(v, alpha);
    if (c != nullptr) {
        float cb = c[c_len == 1 ? 0 : j];
        if (scale_c) cb = __fmul_rn(cb, beta);
        v = __fadd_rn(v, cb);
    }
    return v;
}

__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) gemm_nt_mfma_kernel(const float* __restrict__ a, const float* __restrict__ b,
                                                           const float* __restrict__ c, float* __restrict__ y,
                                                           int32_t M, int32_t N, int32_t K, float alpha, float beta,
                                                           int64_t c_len, int scale_a, int scale_c) {
    __shared__ float part[4][32 * 33];
    const int wave = threadIdx.x >> 6;
    const int lane = threadIdx.x & 63;
    const int half = lane >> 5;
    const int r = lane & 31;
    const int m0 = blockIdx.y * 32, n0 = blockIdx.x * 32;
    const int arow = min(m0 + r, M - 1);       // clamped rows are computed and never stored
    const int brow = min(n0 + r, N - 1);
    const int kw = K / 4;                      // K range of this wave
    const int kh = kw / 2;                     // K range of this half-wave (multiple of 4)
    const float* ap = a + static_cast<int64_t>(arow) * K + wave * kw + half * kh;
    const float* bp = b + static_cast<int64_t>(brow) * K + wave * kw + half * kh;
    floatx16 acc = {0};
    for (int k = 0; k < kh; k += 4) {
        const float4 va = *reinterpret_cast<const float4*>(ap + k);
        const float4 vb = *reinterpret_cast<const float4*>(bp + k);
        // D[i][j] += A[i][k] * B[k][j]: operand A from rows of a (i = m), operand B from rows of b (j = n)
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(va.x, vb.x, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(va.y, vb.y, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(va.z, vb.z, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(va.w, vb.w, acc, 0, 0, 0);
    }
    // accumulator register g holds D[i][j] with j = lane % 32, i = 8*(g/4) + 4*(lane/32) + g%4
#pragma unroll
    for (int g = 0; g < 16; ++g) {
        const int i = 8 * (g / 4) + 4 * half + (g % 4);
        part[wave][i * 33 + r] = acc[g];
    }
    __syncthreads();
    // 1024 outputs, 256 threads: 4 each, consecutive threads on consecutive n
    for (int e = threadIdx.x; e < 1024; e += 256) {
        const int i = e >> 5, j = e & 31;
        float s = part[0][i * 33 + j];
        s = __fadd_rn(s, part[1][i * 33 + j]);
        s = __fadd_rn(s, part[2][i * 33 + j]);
        s = __fadd_rn(s, part[3][i * 33 + j]);
        const int m = m0 + i, n = n0 + j;
        if (m < M && n < N)
            y[static_cast<int64_t>(m) * N + n] = epilogue(s, alpha, beta, c, n, c_len, scale_a != 0, scale_c != 0);
    }
}

// A handful of rows (batch 1-4 of a classifier layer): the matrix-core tile above would be 32 rows of which at
// most 4 are real, and its k loop is a chain of dependent load latencies.  Here a wave owns four output columns for
// every row; its lanes split k (a lane takes 4 consecutive floats of every 256), all loads of a 256-chunk are in
// flight together, and the lanes' sums are added across the wave at the end (a tree: not the CPU order, within the
// fp32 tolerance like the matrix-core kernel).  Measured on MI355X inside ResNet-18 (FC 512 -> 1000): batch 1
// 0.2068 -> 0.2040 ms per pass, batch 2 0.2511 -> 0.2480, batch 4 equal, batch 8 slower (0.4643 -> 0.4728).
constexpr int kGemvRows = 4;
constexpr int kGemvCols = 4;
template <int ROWS>
__global__ void __launch_bounds__(256) gemv_nt_kernel(const float* __restrict__ a, const float* __restrict__ b,
                                                      const float* __restrict__ c, float* __restrict__ y,
                                                      int32_t N, int32_t K, float alpha, float beta, int64_t c_len,
                                                      int scale_a, int scale_c) {
    const int lane = threadIdx.x & 63;
    const int n0 = (static_cast<int>(blockIdx.x) * 4 + static_cast<int>(threadIdx.x >> 6)) * kGemvCols;
    if (n0 >= N) return;
    float acc[ROWS][kGemvCols];
#pragma unroll
    for (int i = 0; i < ROWS; ++i)
#pragma unroll
        for (int j = 0; j < kGemvCols; ++j) acc[i][j] = 0.0f;
    for (int k0 = lane * 4; k0 < K; k0 += 256) {
        float4 vb[kGemvCols], va[ROWS];
#pragma unroll
        for (int j = 0; j < kGemvCols; ++j)
            vb[j] = *reinterpret_cast<const float4*>(b + static_cast<int64_t>(min(n0 + j, N - 1)) * K + k0);
#pragma unroll
        for (int i = 0; i < ROWS; ++i) va[i] = *reinterpret_cast<const float4*>(a + static_cast<int64_t>(i) * K + k0);
#pragma unroll
        for (int i = 0; i < ROWS; ++i)
#pragma unroll
            for (int j = 0; j < kGemvCols; ++j) {
                acc[i][j] = fmaf(va[i].x, vb[j].x, acc[i][j]);
                acc[i][j] = fmaf(va[i].y, vb[j].y, acc[i][j]);
                acc[i][j] = fmaf(va[i].z, vb[j].z, acc[i][j]);
                acc[i][j] = fmaf(va[i].w, vb[j].w, acc[i][j]);
            }
    }
#pragma unroll
    for (int i = 0; i < ROWS; ++i)
#pragma unroll
        for (int j = 0; j < kGemvCols; ++j) {
            float v = acc[i][j];
#pragma unroll
            for (int d = 32; d >= 1; d >>= 1) v += __shfl_xor(v, d, 64);
            if (lane == 0 && n0 + j < N)
                y[static_cast<int64_t>(i) * N + n0 + j] = epilogue(v, alpha, beta, c, n0 + j, c_len, scale_a != 0, scale_c != 0);
        }
}

// Reference-order kernel: k ascending from 0.0f, multiply and add rounded separately.
template <bool TRANS_B>
__global__ void __launch_bounds__(256) gemm_direct_kernel(const float* __restrict__ a, const float* __restrict__ b,
                                                          const float* __restrict__ c, float* __restrict__ y,
                                                          int64_t M, int64_t N, int64_t K, float alpha, float beta,
                                                          int64_t c_len, int scale_a, int scale_c) {
    const int64_t total = M * N;
    const int64_t stride = static_cast<int64_t>(gridDim.x) * 256;
    for (int64_t e = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; e < total; e += stride) {
        const int64_t i = e / N, j = e - i * N;
        float acc = 0.0f;
        for (int64_t k = 0; k < K; ++k) {
            const float bv = TRANS_B ? b[j * K + k] : b[k * N + j];
            acc = __fadd_rn(acc, __fmul_rn(a[i * K + k], bv));
        }
        y[e] = epilogue(acc, alpha, beta, c, j, c_len, scale_a != 0, scale_c != 0);
    }
}

// int8 dense: acc int32 exact, y = (float)(acc + bias[n]) * mult[n].
__global__ void __launch_bounds__(256) qdense_kernel(const int8_t* __restrict__ a, const int8_t* __restrict__ b,
                                                     const int32_t* __restrict__ bias, const float* __restrict__ mult,
                                                     float* __restrict__ y, int64_t M, int64_t N, int64_t K) {
    const int64_t total = M * N;
    const int64_t stride = static_cast<int64_t>(gridDim.x) * 256;
    for (int64_t e = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; e < total; e += stride) {
        const int64_t i = e / N, j = e - i * N;
        const int8_t* ar = a + i * K;
        const int8_t* br = b + j * K;
        int32_t acc = 0;
        int64_t k = 0;
        if (((reinterpret_cast<uintptr_t>(ar) | reinterpret_cast<uintptr_t>(br)) & 3u) == 0) {
            for (; k + 4 <= K; k += 4) {
                const int32_t va = *reinterpret_cast<const int32_t*>(ar + k);
                const int32_t vb = *reinterpret_cast<const int32_t*>(br + k);
                acc = __builtin_amdgcn_sdot4(va, vb, acc, false);
            }
        }
        for (; k < K; ++k) acc += static_cast<int32_t>(ar[k]) * static_cast<int32_t>(br[k]);
        if (bias) acc += bias[j];
        y[e] = __fmul_rn(static_cast<float>(acc), mult[j]);
    }
}

// int8 dense, one wave per output column j and 64 rows at a time.  Lane l owns bytes [16l, 16l+16) of every
// 1 KiB slice of K: the weight row is read once, every activation row as one coalesced 16-byte load per lane,
// products go through the 4-way int8 dot instruction, and the 64 per-lane partial sums of the 64 rows are
// combined with a transposing butterfly (63 exchanges instead of 64 x 6) that leaves row r's total in lane r.
__global__ void __launch_bounds__(256) qdense_wave_kernel(const int8_t* __restrict__ a, const int8_t* __restrict__ b,
                                                          const int32_t* __restrict__ bias, const float* __restrict__ mult,
                                                          float* __restrict__ y, int32_t M, int32_t N, int32_t K) {
    const int lane = threadIdx.x & 63;
    const int j = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (j >= N) return;
    const int32_t bj = bias ? bias[j] : 0;
    const float mj = mult[j];
    for (int i0 = 0; i0 < M; i0 += 64) {
        int32_t acc[64];
#pragma unroll
        for (int r = 0; r < 64; ++r) acc[r] = 0;
        for (int k0 = 0; k0 < K; k0 += 1024) {
            const int kk = k0 + lane * 16;
            if (kk < K) {
                const int4 vb = *reinterpret_cast<const int4*>(b + static_cast<int64_t>(j) * K + kk);
#pragma unroll
                for (int r = 0; r < 64; ++r) {
                    if (i0 + r < M) {
                        const int4 va = *reinterpret_cast<const int4*>(a + static_cast<int64_t>(i0 + r) * K + kk);
                        int32_t t = acc[r];
                        t = __builtin_amdgcn_sdot4(va.x, vb.x, t, false);
                        t = __builtin_amdgcn_sdot4(va.y, vb.y, t, false);
                        t = __builtin_amdgcn_sdot4(va.z, vb.z, t, false);
                        t = __builtin_amdgcn_sdot4(va.w, vb.w, t, false);
                        acc[r] = t;
                    }
                }
            }
        }
#pragma unroll
        for (int s = 32; s >= 1; s >>= 1) {
            const bool upper = (lane & s) != 0;
#pragma unroll
            for (int t = 0; t < s; ++t) {
                const int32_t send = upper ? acc[t] : acc[t + s];
                const int32_t keep = upper ? acc[t + s] : acc[t];
                acc[t] = keep + __shfl_xor(send, s, 64);
            }
        }
        const int row = i0 + lane;
        if (row < M) y[static_cast<int64_t>(row) * N + j] = __fmul_rn(static_cast<float>(acc[0] + bj), mj);
    }
}

// int8 dense on the int8 matrix cores: one wave per 32x32 block of y, D[i][j] += A[i][k] * B[j][k].  Both
// operands are k-contiguous in memory, so a lane's 16-byte k-slice of the 32x32x32 instruction is one global
// load each (no LDS): lane (r, half) reads a[i0+r][32*step + 16*half ..] and b[j0+r][same].  Rows / columns
// past the end are clamped for the loads and skipped at the store.
typedef int intx4_t __attribute__((ext_vector_type(4)));
typedef int intx16_t __attribute__((ext_vector_type(16)));
__global__ void __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(2))) qdense_mfma_kernel(const int8_t* __restrict__ a, const int8_t* __restrict__ b,
                                                         const int32_t* __restrict__ bias, const float* __restrict__ mult,
                                                         float* __restrict__ y, int32_t M, int32_t N, int32_t K,
                                                         int32_t col_blocks) {
    const int lane = threadIdx.x;
    const int r = lane & 31, half = lane >> 5;
    const int ib = blockIdx.x / col_blocks, jb = blockIdx.x - ib * col_blocks;
    const int i0 = ib * 32, j0 = jb * 32;
    const int8_t* ap = a + static_cast<int64_t>(min(i0 + r, M - 1)) * K + 16 * half;
    const int8_t* bp = b + static_cast<int64_t>(min(j0 + r, N - 1)) * K + 16 * half;
    intx16_t acc;
#pragma unroll
    for (int g = 0; g < 16; ++g) acc[g] = 0;
    const int steps = K >> 5;
    int s = 0;
    for (; s + 4 <= steps; s += 4) {
        intx4_t av[4], bv[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            av[u] = *reinterpret_cast<const intx4_t*>(ap + (s + u) * 32);
            bv[u] = *reinterpret_cast<const intx4_t*>(bp + (s + u) * 32);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(av[u], bv[u], acc, 0, 0, 0);
    }
    for (; s < steps; ++s) {
        const intx4_t av = *reinterpret_cast<const intx4_t*>(ap + s * 32);
        const intx4_t bv = *reinterpret_cast<const intx4_t*>(bp + s * 32);
        acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(av, bv, acc, 0, 0, 0);
    }
    const int j = j0 + r;
    if (j >= N) return;
    const int32_t bj = bias ? bias[j] : 0;
    const float mj = mult[j];
#pragma unroll
    for (int g = 0; g < 16; ++g) {
        const int i = i0 + 8 * (g / 4) + 4 * half + (g % 4);
        if (i < M) y[static_cast<int64_t>(i) * N + j] = __fmul_rn(static_cast<float>(acc[g] + bj), mj);
    }
}

}  // namespace

extern "C" {

int32_t kxc_hip_gemm_f32(const float* a, const float* b, const float* c, float* y, int64_t m, int64_t n, int64_t k,
                         float alpha, float beta, int32_t transB, int64_t c_len, void* stream) {
    KXC_HIP_REQUIRE(m >= 0 && n >= 0 && k >= 0, "kxc_hip_gemm_f32: negative dimension");
    if (m == 0 || n == 0) return KXC_HIP_OK;
    KXC_HIP_REQUIRE(a && b && y, "kxc_hip_gemm_f32: NULL pointer");
    KXC_HIP_REQUIRE(c == nullptr || c_len == n || c_len == 1, "kxc_hip_gemm_f32: bias length %lld is neither %lld nor 1",
                    static_cast<long long>(c_len), static_cast<long long>(n));
    hipStream_t s = ResolveStream(stream);
    const int scale_a = (static_cast<double>(alpha) != 1.0) ? 1 : 0;   // ScaleTensor, src/relay/op/nn/dense.cc:17-24
    const int scale_c = (static_cast<double>(beta) != 1.0) ? 1 : 0;
    const bool aligned = ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b)) & 15u) == 0;
    // (the same shapes as the matrix-core kernel below: whatever took the reference-order kernel still does)
    if (transB && k > 0 && (k % 32) == 0 && aligned && m <= kGemvRows && n < (1 << 20) && k < (1 << 30)) {
        const unsigned grid = static_cast<unsigned>(CeilDiv(n, 4 * kGemvCols));
        const int32_t n32 = static_cast<int32_t>(n), k32 = static_cast<int32_t>(k);
#define KXC_GEMV(R) gemv_nt_kernel<R><<<NoteGrid(grid), NoteBlock(256), NoteLds(0), s>>>(a, b, c, y, n32, k32, alpha, beta, c_len, scale_a, scale_c)
        switch (m) {
            case 1: KXC_GEMV(1); break;
            case 2: KXC_GEMV(2); break;
            case 3: KXC_GEMV(3); break;
            default: KXC_GEMV(4); break;
        }
#undef KXC_GEMV
        return CheckLaunch("gemv_nt");
    }
    if (transB && k > 0 && (k % 32) == 0 && aligned && m < (1 << 20) && n < (1 << 20) && k < (1 << 30)) {
        dim3 grid(static_cast<unsigned>(CeilDiv(n, 32)), static_cast<unsigned>(CeilDiv(m, 32)));
        KXC_HIP_REQUIRE(grid.y <= 65535u, "kxc_hip_gemm_f32: m too large");
        gemm_nt_mfma_kernel<<<NoteGrid(grid), NoteBlock(256), NoteLds(0), s>>>(a, b, c, y, static_cast<int32_t>(m), static_cast<int32_t>(n),
                                                  static_cast<int32_t>(k), alpha, beta, c_len, scale_a, scale_c);
        return CheckLaunch("gemm_nt_mfma");
    }
    int64_t g = CeilDiv(m * n, 256);
    if (g > 256 * 32) g = 256 * 32;
    if (transB) gemm_direct_kernel<true><<<NoteGrid(static_cast<int>(g)), NoteBlock(256), NoteLds(0), s>>>(a, b, c, y, m, n, k, alpha, beta, c_len, scale_a, scale_c);
    else gemm_direct_kernel<false><<<NoteGrid(static_cast<int>(g)), NoteBlock(256), NoteLds(0), s>>>(a, b, c, y, m, n, k, alpha, beta, c_len, scale_a, scale_c);
    return CheckLaunch("gemm_direct");
}

int32_t kxc_hip_qdense_i8(const int8_t* a, const int8_t* b, const int32_t* bias, const float* mult, float* y,
                          int64_t m, int64_t n, int64_t k, void* stream) {
    KXC_HIP_REQUIRE(m >= 0 && n >= 0 && k >= 0, "kxc_hip_qdense_i8: negative dimension");
    if (m == 0 || n == 0) return KXC_HIP_OK;
    KXC_HIP_REQUIRE(a && b && mult && y, "kxc_hip_qdense_i8: NULL pointer");
    KXC_HIP_REQUIRE(k <= 2147483647LL / (128 * 128), "kxc_hip_qdense_i8: k too large for int32 accumulation");
    const bool aligned16 = ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b)) & 15u) == 0;
    if (k % 32 == 0 && k > 0 && aligned16 && m < (1LL << 30) && n < (1LL << 30) &&
        CeilDiv(m, 32) * CeilDiv(n, 32) <= kMaxGridX) {
        const int32_t col_blocks = static_cast<int32_t>(CeilDiv(n, 32));
        qdense_mfma_kernel<<<NoteGrid(static_cast<int>(CeilDiv(m, 32) * col_blocks)), NoteBlock(64), NoteLds(0),
                             ResolveStream(stream)>>>(a, b, bias, mult, y, static_cast<int32_t>(m),
                                                      static_cast<int32_t>(n), static_cast<int32_t>(k), col_blocks);
        return CheckLaunch("qdense_mfma");
    }
    if (k % 16 == 0 && m < (1LL << 31) && n < (1LL << 31) && CeilDiv(n, 4) <= kMaxGridX &&
        ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b)) & 15u) == 0) {
        qdense_wave_kernel<<<NoteGrid(static_cast<int>(CeilDiv(n, 4))), NoteBlock(256), NoteLds(0), ResolveStream(stream)>>>(
            a, b, bias, mult, y, static_cast<int32_t>(m), static_cast<int32_t>(n), static_cast<int32_t>(k));
        return CheckLaunch("qdense_wave");
    }
    int64_t g = CeilDiv(m * n, 256);
    if (g > 256 * 32) g = 256 * 32;
    qdense_kernel<<<NoteGrid(static_cast<int>(g)), NoteBlock(256), NoteLds(0), ResolveStream(stream)>>>(a, b, bias, mult, y, m, n, k);
    return CheckLaunch("qdense");
}

}  // extern "C"
