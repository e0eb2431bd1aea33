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

__global__ void __launch_bounds__(256) gemm_nt_mfma_kernel(const float* __restrict__ a, const float* __restrict__ b,
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
    int64_t g = CeilDiv(m * n, 256);
    if (g > 256 * 32) g = 256 * 32;
    qdense_kernel<<<NoteGrid(static_cast<int>(g)), NoteBlock(256), NoteLds(0), ResolveStream(stream)>>>(a, b, bias, mult, y, m, n, k);
    return CheckLaunch("qdense");
}

}  // extern "C"
