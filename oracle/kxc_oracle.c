/*
 * kxc_oracle.c -- CPU restatement of the reference's lowered-operator semantics.
 *
 * TEST INFRASTRUCTURE ONLY (checker + timed CPU baseline); see kxc_oracle.h.
 * Build flags matter: -ffp-contract=off, no fast-math, so that every multiply
 * and add is rounded separately like the reference's LLVM IR (FMul, FAdd
 * without contract flags, src/codegen/codegen_llvm.cc:295-306).
 */
#include "kxc_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------ conv2d */

/* include/te/topi/nn.h:107-158.  Loop nest as lowered by
 * src/relay/backend/lower.cc:381-444: data axes n,o,h,w outermost in that
 * order; Store(init 0.0f); reduce loops rc,rh,rw (rc outermost); the update is
 * out = out + (select(in-bounds, x, 0.0f) * w), accumulated through memory.
 * A padded tap still performs the add of (0.0f * w). */
void kxc_oracle_conv2d_nchw_f32(const float* x, const float* w, float* y,
                                int64_t N, int64_t C, int64_t H, int64_t W,
                                int64_t O, int64_t KH, int64_t KW,
                                int stride_h, int stride_w, int pad_h, int pad_w,
                                int dil_h, int dil_w) {
    /* nn.h:119-123 */
    const int64_t dil_kh = (KH - 1) * dil_h + 1;
    const int64_t dil_kw = (KW - 1) * dil_w + 1;
    const int64_t OH = (H + 2 * pad_h - dil_kh) / stride_h + 1;
    const int64_t OW = (W + 2 * pad_w - dil_kw) / stride_w + 1;
    for (int64_t n = 0; n < N; ++n)
    for (int64_t o = 0; o < O; ++o)
    for (int64_t h = 0; h < OH; ++h)
    for (int64_t ww = 0; ww < OW; ++ww) {
        float acc = 0.0f;
        for (int64_t rc = 0; rc < C; ++rc)
        for (int64_t rh = 0; rh < KH; ++rh)
        for (int64_t rw = 0; rw < KW; ++rw) {
            const int64_t h_in = h * stride_h + rh * dil_h - pad_h;
            const int64_t w_in = ww * stride_w + rw * dil_w - pad_w;
            const int inb = (h_in >= 0) && (h_in < H) && (w_in >= 0) && (w_in < W);
            const float v = inb ? x[((n * C + rc) * H + h_in) * W + w_in] : 0.0f;
            const float prod = v * w[((o * C + rc) * KH + rh) * KW + rw];
            acc = acc + prod;
        }
        y[((n * O + o) * OH + h) * OW + ww] = acc;
    }
}

/* src/relay/op/nn/convolution.cc:72-74 */
void kxc_oracle_bias_add_nchw_f32(const float* x, const float* bias, float* y,
                                  int64_t N, int64_t O, int64_t HW) {
    for (int64_t n = 0; n < N; ++n)
    for (int64_t o = 0; o < O; ++o) {
        const float b = bias[o];
        const float* xs = x + (n * O + o) * HW;
        float* ys = y + (n * O + o) * HW;
        for (int64_t i = 0; i < HW; ++i) ys[i] = xs[i] + b;
    }
}

/* include/te/topi/nn.h:19-30; Max(a,b) = (a > b) ? a : b with an ordered
 * compare (src/codegen/codegen_llvm.cc:326-333): NaN -> 0, -0 -> +0. */
void kxc_oracle_relu_f32(const float* x, float* y, int64_t n) {
    for (int64_t i = 0; i < n; ++i) {
        const float v = x[i];
        y[i] = (v > 0.0f) ? v : 0.0f;
    }
}

/* ------------------------------------------------------- broadcast binary */

/* include/te/topi/broadcast.h:18-42 (index mapping), :90-113 (ops). */
void kxc_oracle_broadcast_binary_f32(int op, const float* a, const int64_t* a_shape, int a_ndim,
                                     const float* b, const int64_t* b_shape, int b_ndim,
                                     float* y, const int64_t* y_shape, int y_ndim) {
    int64_t idx[8] = {0};
    int64_t total = 1;
    for (int i = 0; i < y_ndim; ++i) total *= y_shape[i];
    const int a_off = y_ndim - a_ndim;
    const int b_off = y_ndim - b_ndim;
    for (int64_t lin = 0; lin < total; ++lin) {
        int64_t rem = lin;
        for (int i = y_ndim - 1; i >= 0; --i) {
            idx[i] = rem % y_shape[i];
            rem /= y_shape[i];
        }
        int64_t ai = 0, bi = 0;
        for (int i = 0; i < a_ndim; ++i) {
            const int64_t id = (a_shape[i] == 1) ? 0 : idx[i + a_off];
            ai = ai * a_shape[i] + id;
        }
        for (int i = 0; i < b_ndim; ++i) {
            const int64_t id = (b_shape[i] == 1) ? 0 : idx[i + b_off];
            bi = bi * b_shape[i] + id;
        }
        const float va = a[ai], vb = b[bi];
        float r;
        switch (op) {
            case 0: r = va + vb; break;
            case 1: r = va - vb; break;
            case 2: r = va * vb; break;
            default: r = va / vb; break;
        }
        y[lin] = r;
    }
}

/* ------------------------------------------------------------------ pooling */

/* include/te/topi/nn.h:161-258.  Max: init -inf (lower.cc:80-86), update
 * old > src ? old : src, out-of-bounds taps contribute (float)-1e30.
 * Avg: sum of select(inb, x, 0) from 0.0f, then a second pass sum / (KH*KW). */
void kxc_oracle_pool2d_f32(const float* x, float* y,
                           int64_t N, int64_t C, int64_t H, int64_t W,
                           int KH, int KW, int SH, int SW,
                           int pad_t, int pad_l, int pad_b, int pad_r,
                           int ceil_mode, int is_avg) {
    const int64_t h_num = H + pad_t + pad_b - KH;
    const int64_t w_num = W + pad_l + pad_r - KW;
    const int64_t OH = ceil_mode ? ((h_num + SH - 1) / SH + 1) : (h_num / SH + 1);
    const int64_t OW = ceil_mode ? ((w_num + SW - 1) / SW + 1) : (w_num / SW + 1);
    const float pad_value = (float)-1e30;
    const float denom = (float)(KH * KW);
    for (int64_t n = 0; n < N; ++n)
    for (int64_t c = 0; c < C; ++c)
    for (int64_t h = 0; h < OH; ++h)
    for (int64_t ww = 0; ww < OW; ++ww) {
        float acc = is_avg ? 0.0f : -INFINITY;
        for (int rh = 0; rh < KH; ++rh)
        for (int rw = 0; rw < KW; ++rw) {
            const int64_t h_in = h * SH + rh - pad_t;
            const int64_t w_in = ww * SW + rw - pad_l;
            const int inb = (h_in >= 0) && (h_in < H) && (w_in >= 0) && (w_in < W);
            if (is_avg) {
                const float v = inb ? x[((n * C + c) * H + h_in) * W + w_in] : 0.0f;
                acc = acc + v;
            } else {
                const float v = inb ? x[((n * C + c) * H + h_in) * W + w_in] : pad_value;
                acc = (acc > v) ? acc : v;
            }
        }
        y[((n * C + c) * OH + h) * OW + ww] = is_avg ? (acc / denom) : acc;
    }
}

/* include/te/topi/nn.h:260-287.  The divisor is the int64 constant H*W
 * converted to float (src/codegen/codegen_llvm.cc:266-273): a true division. */
void kxc_oracle_global_avg_pool2d_f32(const float* x, float* y,
                                      int64_t N, int64_t C, int64_t H, int64_t W) {
    const float denom = (float)(H * W);
    for (int64_t n = 0; n < N; ++n)
    for (int64_t c = 0; c < C; ++c) {
        const float* xs = x + (n * C + c) * H * W;
        float acc = 0.0f;
        for (int64_t rh = 0; rh < H; ++rh)
        for (int64_t rw = 0; rw < W; ++rw) acc = acc + xs[rh * W + rw];
        y[n * C + c] = acc / denom;
    }
}

/* -------------------------------------------------------------- dense/gemm */

/* include/te/topi/nn.h:48-80 */
void kxc_oracle_dense_f32(const float* a, const float* b, float* y,
                          int64_t M, int64_t N, int64_t K) {
    for (int64_t i = 0; i < M; ++i)
    for (int64_t j = 0; j < N; ++j) {
        float acc = 0.0f;
        for (int64_t k = 0; k < K; ++k) {
            const float prod = a[i * K + k] * b[j * K + k];
            acc = acc + prod;
        }
        y[i * N + j] = acc;
    }
}

/* include/te/topi/nn.h:84-101 */
void kxc_oracle_matmul_f32(const float* a, const float* b, float* y,
                           int64_t M, int64_t N, int64_t K) {
    for (int64_t i = 0; i < M; ++i)
    for (int64_t j = 0; j < N; ++j) {
        float acc = 0.0f;
        for (int64_t k = 0; k < K; ++k) {
            const float prod = a[i * K + k] * b[k * N + j];
            acc = acc + prod;
        }
        y[i * N + j] = acc;
    }
}

/* src/relay/op/nn/dense.cc:34-61: product, then "* alpha" only when alpha != 1
 * (ScaleTensor :17-24), bias "* beta" only when beta != 1, then broadcast add. */
void kxc_oracle_gemm_f32(const float* a, const float* b, const float* c, float* y,
                         int64_t M, int64_t N, int64_t K,
                         float alpha, float beta, int transB, int64_t c_len) {
    if (transB) kxc_oracle_dense_f32(a, b, y, M, N, K);
    else kxc_oracle_matmul_f32(a, b, y, M, N, K);
    for (int64_t i = 0; i < M; ++i)
    for (int64_t j = 0; j < N; ++j) {
        float v = y[i * N + j];
        if ((double)alpha != 1.0) v = v * alpha;
        float cb = c[c_len == 1 ? 0 : j];
        if ((double)beta != 1.0) cb = cb * beta;
        y[i * N + j] = v + cb;
    }
}

/* src/relay/op/tensor/transform.cc:140-182 */
void kxc_oracle_flatten_f32(const float* x, float* y, int64_t n) {
    memcpy(y, x, (size_t)n * sizeof(float));
}

/* ------------------------------------------------------------------- int8 */

static inline int32_t clamp_i32(int32_t v, int32_t lo, int32_t hi) {
    return v < lo ? lo : (v > hi ? hi : v);
}

/* Round half to even on a float, then saturate.  nearbyintf honours the
 * default rounding mode (to nearest, ties to even).  Values beyond the int32
 * range saturate; NaN maps to 0. */
static inline int32_t rint_sat(float v, int32_t lo, int32_t hi) {
    if (!(v == v)) return clamp_i32(0, lo, hi);
    const float r = nearbyintf(v);
    if (r <= (float)lo) return lo;
    if (r >= (float)hi) return hi;
    return (int32_t)r;
}

void kxc_oracle_quantize_f32_i8(const float* x, int8_t* q, int64_t n, float scale) {
    for (int64_t i = 0; i < n; ++i) q[i] = (int8_t)rint_sat(x[i] / scale, -127, 127);
}

void kxc_oracle_qconv2d_nchw_i8_acc(const int8_t* x, const int8_t* w, int32_t* acc_out,
                                    int64_t N, int64_t C, int64_t H, int64_t W,
                                    int64_t O, int64_t KH, int64_t KW,
                                    int stride_h, int stride_w, int pad_h, int pad_w) {
    const int64_t OH = (H + 2 * pad_h - KH) / stride_h + 1;
    const int64_t OW = (W + 2 * pad_w - KW) / stride_w + 1;
    for (int64_t n = 0; n < N; ++n)
    for (int64_t o = 0; o < O; ++o)
    for (int64_t h = 0; h < OH; ++h)
    for (int64_t ww = 0; ww < OW; ++ww) {
        int32_t acc = 0;
        for (int64_t rc = 0; rc < C; ++rc)
        for (int64_t rh = 0; rh < KH; ++rh) {
            const int64_t h_in = h * stride_h + rh - pad_h;
            if (h_in < 0 || h_in >= H) continue;
            for (int64_t rw = 0; rw < KW; ++rw) {
                const int64_t w_in = ww * stride_w + rw - pad_w;
                if (w_in < 0 || w_in >= W) continue;
                acc += (int32_t)x[((n * C + rc) * H + h_in) * W + w_in] *
                       (int32_t)w[((o * C + rc) * KH + rh) * KW + rw];
            }
        }
        acc_out[((n * O + o) * OH + h) * OW + ww] = acc;
    }
}

void kxc_oracle_qconv2d_nchw_i8(const int8_t* x, const int8_t* w, const int32_t* bias,
                                const float* mult, const int8_t* residual, float res_mult,
                                int8_t* y,
                                int64_t N, int64_t C, int64_t H, int64_t W,
                                int64_t O, int64_t KH, int64_t KW,
                                int stride_h, int stride_w, int pad_h, int pad_w, int relu) {
    const int64_t OH = (H + 2 * pad_h - KH) / stride_h + 1;
    const int64_t OW = (W + 2 * pad_w - KW) / stride_w + 1;
    const int64_t total = N * O * OH * OW;
    int32_t* acc = (int32_t*)malloc((size_t)total * sizeof(int32_t));
    kxc_oracle_qconv2d_nchw_i8_acc(x, w, acc, N, C, H, W, O, KH, KW,
                                   stride_h, stride_w, pad_h, pad_w);
    const int32_t lo = relu ? 0 : -128;
    for (int64_t n = 0; n < N; ++n)
    for (int64_t o = 0; o < O; ++o)
    for (int64_t p = 0; p < OH * OW; ++p) {
        const int64_t i = (n * O + o) * OH * OW + p;
        int32_t a = acc[i];
        if (bias) a += bias[o];
        float v = (float)a * mult[o];
        if (residual) {
            const float r = (float)residual[i] * res_mult;
            v = v + r;
        }
        y[i] = (int8_t)rint_sat(v, lo, 127);
    }
    free(acc);
}

void kxc_oracle_qdense_i8(const int8_t* a, const int8_t* b, const int32_t* bias,
                          const float* mult, float* y, int64_t M, int64_t N, int64_t K) {
    for (int64_t i = 0; i < M; ++i)
    for (int64_t j = 0; j < N; ++j) {
        int32_t acc = 0;
        for (int64_t k = 0; k < K; ++k) acc += (int32_t)a[i * K + k] * (int32_t)b[j * K + k];
        if (bias) acc += bias[j];
        y[i * N + j] = (float)acc * mult[j];
    }
}

void kxc_oracle_maxpool2d_i8(const int8_t* x, int8_t* y,
                             int64_t N, int64_t C, int64_t H, int64_t W,
                             int KH, int KW, int SH, int SW,
                             int pad_t, int pad_l, int pad_b, int pad_r) {
    const int64_t OH = (H + pad_t + pad_b - KH) / SH + 1;
    const int64_t OW = (W + pad_l + pad_r - KW) / SW + 1;
    for (int64_t n = 0; n < N; ++n)
    for (int64_t c = 0; c < C; ++c)
    for (int64_t h = 0; h < OH; ++h)
    for (int64_t ww = 0; ww < OW; ++ww) {
        int32_t m = -128;
        for (int rh = 0; rh < KH; ++rh)
        for (int rw = 0; rw < KW; ++rw) {
            const int64_t h_in = h * SH + rh - pad_t;
            const int64_t w_in = ww * SW + rw - pad_l;
            if (h_in < 0 || h_in >= H || w_in < 0 || w_in >= W) continue;
            const int32_t v = x[((n * C + c) * H + h_in) * W + w_in];
            if (v > m) m = v;
        }
        y[((n * C + c) * OH + h) * OW + ww] = (int8_t)m;
    }
}

void kxc_oracle_global_avg_pool2d_i8(const int8_t* x, int8_t* y,
                                     int64_t N, int64_t C, int64_t H, int64_t W, float mult) {
    for (int64_t i = 0; i < N * C; ++i) {
        int32_t s = 0;
        for (int64_t p = 0; p < H * W; ++p) s += x[i * H * W + p];
        y[i] = (int8_t)rint_sat((float)s * mult, -128, 127);
    }
}

/* -------------------------------------------------------------- ResNet-18 */

typedef struct {
    int64_t n, c, h, w;
    float* d;
} act_t;

static act_t act_alloc(int64_t n, int64_t c, int64_t h, int64_t w) {
    act_t a;
    a.n = n; a.c = c; a.h = h; a.w = w;
    a.d = (float*)malloc((size_t)(n * c * h * w) * sizeof(float));
    return a;
}

/* One nn_conv2d call with bias: two stages, T_conv2d then T_conv2d_bias_add
 * (src/relay/op/nn/convolution.cc:38-75). */
static act_t conv_bias(act_t x, const float* w, const float* b, int64_t O, int k, int s, int p) {
    const int64_t OH = (x.h + 2 * p - k) / s + 1;
    const int64_t OW = (x.w + 2 * p - k) / s + 1;
    act_t t = act_alloc(x.n, O, OH, OW);
    kxc_oracle_conv2d_nchw_f32(x.d, w, t.d, x.n, x.c, x.h, x.w, O, k, k, s, s, p, p, 1, 1);
    act_t y = act_alloc(x.n, O, OH, OW);
    kxc_oracle_bias_add_nchw_f32(t.d, b, y.d, x.n, O, OH * OW);
    free(t.d);
    return y;
}

static act_t relu_new(act_t x) {
    act_t y = act_alloc(x.n, x.c, x.h, x.w);
    kxc_oracle_relu_f32(x.d, y.d, x.n * x.c * x.h * x.w);
    return y;
}

static act_t add_new(act_t a, act_t b) {
    act_t y = act_alloc(a.n, a.c, a.h, a.w);
    const int64_t shp[4] = {a.n, a.c, a.h, a.w};
    kxc_oracle_broadcast_binary_f32(0, a.d, shp, 4, b.d, shp, 4, y.d, shp, 4);
    return y;
}

static float* tap_copy(act_t a) {
    const size_t bytes = (size_t)(a.n * a.c * a.h * a.w) * sizeof(float);
    float* p = (float*)malloc(bytes);
    memcpy(p, a.d, bytes);
    return p;
}

/* test/resnet18_ir_dump.cpp:281-452.  BasicBlock: conv1 -> relu -> conv2 ->
 * add(conv2_out, identity) -> relu, identity = block input or the 1x1/2
 * downsample conv of it. */
static act_t basic_block(act_t x, const float* const** cp, int64_t O, int stride, int downsample) {
    const float* const* c = *cp;
    act_t a = conv_bias(x, c[0], c[1], O, 3, stride, 1);
    act_t ar = relu_new(a); free(a.d);
    act_t b = conv_bias(ar, c[2], c[3], O, 3, 1, 1); free(ar.d);
    act_t id = x;
    if (downsample) {
        id = conv_bias(x, c[4], c[5], O, 1, stride, 0);
        *cp += 6;
    } else {
        *cp += 4;
    }
    act_t s = add_new(b, id); free(b.d);
    if (downsample) free(id.d);
    act_t r = relu_new(s); free(s.d);
    return r;
}

int kxc_oracle_resnet18_f32(int64_t N, int64_t HW, const float* input, const float* const* consts,
                            float* logits, float** taps) {
    const float* const* c = consts;
    int tap = 0;
    act_t x; x.n = N; x.c = 3; x.h = HW; x.w = HW; x.d = (float*)input;

    act_t c1 = conv_bias(x, c[0], c[1], 64, 7, 2, 3); c += 2;
    act_t r1 = relu_new(c1); free(c1.d);
    if (taps) taps[tap++] = tap_copy(r1);                      /* 0: conv1+relu */
    act_t mp = act_alloc(N, 64, (r1.h + 2 - 3) / 2 + 1, (r1.w + 2 - 3) / 2 + 1);
    kxc_oracle_pool2d_f32(r1.d, mp.d, N, 64, r1.h, r1.w, 3, 3, 2, 2, 1, 1, 1, 1, 0, 0);
    free(r1.d);
    if (taps) taps[tap++] = tap_copy(mp);                      /* 1: maxpool */

    act_t cur = mp;
    const int64_t chans[4] = {64, 128, 256, 512};
    for (int stage = 0; stage < 4; ++stage) {
        for (int blk = 0; blk < 2; ++blk) {
            const int first = (blk == 0 && stage > 0);
            act_t nxt = basic_block(cur, &c, chans[stage], first ? 2 : 1, first);
            free(cur.d);
            cur = nxt;
        }
        if (taps) taps[tap++] = tap_copy(cur);                 /* 2..5: stage outputs */
    }

    act_t gap = act_alloc(N, 512, 1, 1);
    kxc_oracle_global_avg_pool2d_f32(cur.d, gap.d, N, 512, cur.h, cur.w);
    free(cur.d);
    if (taps) taps[tap++] = tap_copy(gap);                     /* 6: global avg pool */
    act_t fl = act_alloc(N, 512, 1, 1);
    kxc_oracle_flatten_f32(gap.d, fl.d, N * 512);
    free(gap.d);
    if (taps) taps[tap++] = tap_copy(fl);                      /* 7: flatten */
    kxc_oracle_gemm_f32(fl.d, c[0], c[1], logits, N, 1000, 512, 1.0f, 1.0f, 1, 1000);
    free(fl.d);
    if (taps) {
        act_t lg; lg.n = N; lg.c = 1000; lg.h = 1; lg.w = 1; lg.d = logits;
        taps[tap++] = tap_copy(lg);                            /* 8: logits */
    }
    return 0;
}
