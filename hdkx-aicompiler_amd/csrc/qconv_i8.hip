// qconv_i8.hip -- int8 convolution with int32 accumulation and per-output-channel requantisation.
//
// The reference compiler has no quantised operator; the definition implemented here is
//   acc  = sum_{c,rh,rw} (int32)x * (int32)w              (padding contributes 0)   [+ bias[o]]
//   v    = (float)acc * mult[o]                            one rounded fp32 multiply
//   v    = v + (float)residual * res_mult                  optional; one multiply, one add, each rounded
//   y    = clamp(rint_half_even(v), relu ? 0 : -128, 127)
// Integer accumulation is exact and order independent, so any tiling is bit-exact; the float tail is
// three individually rounded operations, kept from being contracted with __fmul_rn / __fadd_rn.
#include <cstring>

#include "common.h"

using namespace kxc_hip;

namespace {

struct QConvArgs {
    const int8_t* x;
    const int8_t* w;
    const int32_t* bias;
    const float* mult;
    const int8_t* res;
    int8_t* y;
    int32_t N, C, H, W, O, OH, OW, KH, KW;
    int32_t sh, sw, ph, pw;
    float res_mult;
    uint32_t flags;
};

__device__ __forceinline__ int8_t requant(int32_t acc, float mult, bool has_res, int32_t res, float res_mult, bool relu) {
    float v = __fmul_rn(static_cast<float>(acc), mult);
    if (has_res) v = __fadd_rn(v, __fmul_rn(static_cast<float>(res), res_mult));
    float r = rintf(v);                      // v_rndne_f32: round half to even
    r = (v == v) ? r : 0.0f;
    r = fminf(fmaxf(r, relu ? 0.0f : -128.0f), 127.0f);
    return static_cast<int8_t>(static_cast<int32_t>(r));
}

__global__ void __launch_bounds__(256) qconv_direct_kernel(const QConvArgs a, int64_t total) {
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
        const int8_t* xn = a.x + n * a.C * a.H * a.W;
        const int8_t* wo = a.w + static_cast<int64_t>(o) * a.C * a.KH * a.KW;
        int32_t acc = 0;
        for (int32_t rc = 0; rc < a.C; ++rc)
            for (int32_t rh = 0; rh < a.KH; ++rh) {
                const int32_t ih = oh * a.sh + rh - a.ph;
                if (ih < 0 || ih >= a.H) continue;
                for (int32_t rw = 0; rw < a.KW; ++rw) {
                    const int32_t iw = ow * a.sw + rw - a.pw;
                    if (iw < 0 || iw >= a.W) continue;
                    acc += static_cast<int32_t>(xn[(static_cast<int64_t>(rc) * a.H + ih) * a.W + iw]) *
                           static_cast<int32_t>(wo[(rc * a.KH + rh) * a.KW + rw]);
                }
            }
        if (has_bias) acc += a.bias[o];
        a.y[e] = requant(acc, a.mult[o], has_res, has_res ? a.res[e] : 0, a.res_mult, do_relu);
    }
}

}  // namespace

extern "C" {

int32_t kxc_hip_qconv2d_nchw_i8(const kxc_hip_qconv2d_desc* d, const int8_t* x, const int8_t* w, const int32_t* bias,
                                const float* mult, const int8_t* residual, int8_t* y, void* stream) {
    KXC_HIP_REQUIRE(d != nullptr, "kxc_hip_qconv2d_nchw_i8: desc is NULL");
    KXC_HIP_REQUIRE(d->n >= 0 && d->c > 0 && d->h > 0 && d->w > 0 && d->o > 0 && d->kh > 0 && d->kw > 0,
                    "kxc_hip_qconv2d_nchw_i8: bad shape");
    KXC_HIP_REQUIRE(d->stride_h > 0 && d->stride_w > 0 && d->pad_h >= 0 && d->pad_w >= 0,
                    "kxc_hip_qconv2d_nchw_i8: bad stride or padding");
    const int64_t nh = static_cast<int64_t>(d->h) + 2 * d->pad_h - d->kh;
    const int64_t nw = static_cast<int64_t>(d->w) + 2 * d->pad_w - d->kw;
    KXC_HIP_REQUIRE(nh >= 0 && nw >= 0, "kxc_hip_qconv2d_nchw_i8: window is larger than input");
    KXC_HIP_REQUIRE(static_cast<int64_t>(d->c) * d->kh * d->kw <= 2147483647LL / (128 * 128),
                    "kxc_hip_qconv2d_nchw_i8: reduction too long for int32 accumulation");
    QConvArgs a;
    std::memset(&a, 0, sizeof(a));
    a.N = d->n; a.C = d->c; a.H = d->h; a.W = d->w; a.O = d->o; a.KH = d->kh; a.KW = d->kw;
    a.OH = static_cast<int32_t>(nh / d->stride_h + 1);
    a.OW = static_cast<int32_t>(nw / d->stride_w + 1);
    a.sh = d->stride_h; a.sw = d->stride_w; a.ph = d->pad_h; a.pw = d->pad_w;
    a.res_mult = d->res_mult; a.flags = d->flags;
    const int64_t total = static_cast<int64_t>(a.N) * a.O * a.OH * a.OW;
    if (total == 0) return KXC_HIP_OK;
    KXC_HIP_REQUIRE(x && w && mult && y, "kxc_hip_qconv2d_nchw_i8: NULL pointer");
    KXC_HIP_REQUIRE(!(d->flags & KXC_HIP_CONV_BIAS) || bias, "kxc_hip_qconv2d_nchw_i8: bias flag without bias");
    KXC_HIP_REQUIRE(!(d->flags & KXC_HIP_CONV_RESIDUAL) || residual,
                    "kxc_hip_qconv2d_nchw_i8: residual flag without residual");
    a.x = x; a.w = w; a.bias = bias; a.mult = mult; a.res = residual; a.y = y;
    int64_t g = CeilDiv(total, 256);
    if (g > 256 * 64) g = 256 * 64;
    qconv_direct_kernel<<<NoteGrid(static_cast<int>(g)), NoteBlock(256), NoteLds(0), ResolveStream(stream)>>>(a, total);
    return CheckLaunch("qconv_direct");
}

}  // extern "C"
