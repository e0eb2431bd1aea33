/*
 * kxc_oracle.h -- CPU restatement of the reference compiler's lowered-operator
 * semantics (what its LLVM CPU backend computes for each operator).
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  It is the checker the GPU
 * results are compared with, and the single-core CPU baseline a benchmark may
 * time.  Nothing on the product path links, loads or calls it.
 *
 * Every function is a scalar, single-threaded, FMA-free loop nest in the
 * reference's own loop and rounding order (build with -ffp-contract=off and
 * without fast-math, see the Makefile next to this file).  Reference
 * citations are relative to the reference checkout.
 *
 * Pinning status (what independent evidence each function is checked against
 * in tests/test_oracle_*.py):
 *   conv2d / bias_add / relu / add / pool2d / global_avg_pool2d / dense /
 *   matmul / gemm / flatten : the literal known answers of the reference's
 *       test/op_numeric_llvm_test.cpp, closed forms, float64 brute force,
 *       torch CPU cross-checks, and (where it builds) the reference's own
 *       lowering + C code generator in oracle/_ref.
 *   qconv2d / qdense / quantize / requant : PARITY UNPINNED by the reference
 *       (it has no int8 operator).  Defined here; pinned only by closed forms
 *       and int64 brute force.
 */
#ifndef KXC_ORACLE_H_
#define KXC_ORACLE_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* include/te/topi/nn.h:107-158 (conv2d_nchw), src/relay/backend/lower.cc:416-444
 * (init store 0, then out = out + src with rc outermost, rw innermost). */
void kxc_oracle_conv2d_nchw_f32(const float* x, const float* w, float* y,
                                int64_t N, int64_t C, int64_t H, int64_t W,
                                int64_t O, int64_t KH, int64_t KW,
                                int stride_h, int stride_w, int pad_h, int pad_w,
                                int dil_h, int dil_w);

/* src/relay/op/nn/convolution.cc:72-74 (T_conv2d_bias_add = T_conv2d + bias[o]). */
void kxc_oracle_bias_add_nchw_f32(const float* x, const float* bias, float* y,
                                  int64_t N, int64_t O, int64_t HW);

/* include/te/topi/nn.h:19-30 with Max lowered as (x > 0) ? x : 0
 * (src/codegen/codegen_llvm.cc:326-333). */
void kxc_oracle_relu_f32(const float* x, float* y, int64_t n);

/* include/te/topi/broadcast.h:18-113; op: 0 add, 1 subtract, 2 multiply, 3 divide.
 * Shapes are right-aligned, a dim of 1 broadcasts.  ndim <= 8. */
void kxc_oracle_broadcast_binary_f32(int op, const float* a, const int64_t* a_shape, int a_ndim,
                                     const float* b, const int64_t* b_shape, int b_ndim,
                                     float* y, const int64_t* y_shape, int y_ndim);

/* include/te/topi/nn.h:161-258 (pool2d); is_avg 0 = max, 1 = avg.
 * Padding top,left,bottom,right.  Max pads with -1e30f and starts from -inf
 * (lower.cc:80-86); avg divides the padded-zero sum by KH*KW. */
void kxc_oracle_pool2d_f32(const float* x, float* y,
                           int64_t N, int64_t C, int64_t H, int64_t W,
                           int KH, int KW, int SH, int SW,
                           int pad_t, int pad_l, int pad_b, int pad_r,
                           int ceil_mode, int is_avg);

/* include/te/topi/nn.h:260-287: sequential sum over rh,rw then fp32 division by H*W. */
void kxc_oracle_global_avg_pool2d_f32(const float* x, float* y,
                                      int64_t N, int64_t C, int64_t H, int64_t W);

/* include/te/topi/nn.h:48-80: out[i,j] = sum_k A[i,k] * B[j,k]. */
void kxc_oracle_dense_f32(const float* a, const float* b, float* y,
                          int64_t M, int64_t N, int64_t K);

/* include/te/topi/nn.h:84-101: out[i,j] = sum_k A[i,k] * B[k,j]. */
void kxc_oracle_matmul_f32(const float* a, const float* b, float* y,
                           int64_t M, int64_t N, int64_t K);

/* src/relay/op/nn/dense.cc:34-61 (nn_gemm, transA must be 0).  c has c_len
 * elements broadcast over the last axis (c_len == N or 1). */
void kxc_oracle_gemm_f32(const float* a, const float* b, const float* c, float* y,
                         int64_t M, int64_t N, int64_t K,
                         float alpha, float beta, int transB, int64_t c_len);

/* src/relay/op/tensor/transform.cc:140-182: row-major copy. */
void kxc_oracle_flatten_f32(const float* x, float* y, int64_t n);

/* ---- int8 family: defined by this build (the reference has no int8 operator). ---- */

/* q = clamp(rint_half_even(v / scale), -127, 127). */
void kxc_oracle_quantize_f32_i8(const float* x, int8_t* q, int64_t n, float scale);

/* acc = sum_{rc,rh,rw} x*w in int32 (padding contributes 0) + bias[o] (may be NULL);
 * v = (float)acc * mult[o]                       (one rounded fp32 multiply)
 * if residual: v = v + (float)residual * res_mult (one rounded multiply, one rounded add)
 * q = clamp(rint_half_even(v), relu ? 0 : -128, 127). */
void kxc_oracle_qconv2d_nchw_i8(const int8_t* x, const int8_t* w, const int32_t* bias,
                                const float* mult, const int8_t* residual, float res_mult,
                                int8_t* y,
                                int64_t N, int64_t C, int64_t H, int64_t W,
                                int64_t O, int64_t KH, int64_t KW,
                                int stride_h, int stride_w, int pad_h, int pad_w, int relu);

/* Same accumulation, int32 result without requantisation. */
void kxc_oracle_qconv2d_nchw_i8_acc(const int8_t* x, const int8_t* w, int32_t* acc,
                                    int64_t N, int64_t C, int64_t H, int64_t W,
                                    int64_t O, int64_t KH, int64_t KW,
                                    int stride_h, int stride_w, int pad_h, int pad_w);

/* acc[i,j] = sum_k a[i,k]*b[j,k] + bias[j]; y = (float)acc * mult[j] (fp32 logits out). */
void kxc_oracle_qdense_i8(const int8_t* a, const int8_t* b, const int32_t* bias,
                          const float* mult, float* y, int64_t M, int64_t N, int64_t K);

/* int8 max pool (pad candidate -128, exact) and int8 global average:
 * q = clamp(rint_half_even((float)sum * mult), -128, 127). */
void kxc_oracle_maxpool2d_i8(const int8_t* x, int8_t* y,
                             int64_t N, int64_t C, int64_t H, int64_t W,
                             int KH, int KW, int SH, int SW,
                             int pad_t, int pad_l, int pad_b, int pad_r);
void kxc_oracle_global_avg_pool2d_i8(const int8_t* x, int8_t* y,
                                     int64_t N, int64_t C, int64_t H, int64_t W, float mult);

/* ---- ResNet-18, the graph of the reference's test/resnet18_ir_dump.cpp:191-452 ---- */

/* consts: the 42 constant tensors in the lowered function's parameter order
 * (depth-first argument order, src/relay/backend/lower.cc:201-233), that is
 * conv1.w, conv1.b, then per BasicBlock conv1.w,b, conv2.w,b and, for the first
 * block of stages 2-4, downsample.w,b AFTER conv2 (it is the second operand of
 * the add), and fc.w, fc.b last.
 * Runs the unfused operator chain (conv, bias add, relu, add ...) exactly as
 * the lowered loop nests do.  input is [N,3,HW,HW] (HW = 224 in the reference graph).  taps (may be NULL): receives pointers to malloc'ed
 * copies of 9 named activations for layer-wise comparison; caller frees. */
int kxc_oracle_resnet18_f32(int64_t N, int64_t HW, const float* input, const float* const* consts,
                            float* logits, float** taps);

#define KXC_ORACLE_RESNET18_NUM_CONSTS 42
#define KXC_ORACLE_RESNET18_NUM_TAPS 9

#ifdef __cplusplus
}
#endif
#endif  /* KXC_ORACLE_H_ */
