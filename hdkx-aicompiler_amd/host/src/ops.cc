// ops.cc -- built-in operator registrations: shape rule, TE compute definition (the CPU / generic
// definition, src/relay/op/nn/*.cc and src/relay/op/tensor/*.cc of the reference) and, where a
// hand-written gfx950 kernel exists, the FHIPDispatch hook that adds its launch to a plan.
#include <algorithm>
#include <cstdlib>

#include "kxc/op.h"
#include "kxc/topi.h"
#include "kxc_hip.h"

namespace kxc {
namespace relay {

namespace {

int Read2D(const std::vector<int64_t>& v, int idx, int dflt) {
    return idx >= 0 && static_cast<size_t>(idx) < v.size() ? static_cast<int>(v[idx]) : dflt;
}
std::vector<int> ReadPair(const std::vector<int64_t>& v, int dflt) {
    if (v.size() >= 2) return {static_cast<int>(v[0]), static_cast<int>(v[1])};
    return {dflt, dflt};
}
std::vector<int> ReadPad4(const std::vector<int64_t>& v) {
    if (v.size() >= 4) return {static_cast<int>(v[0]), static_cast<int>(v[1]), static_cast<int>(v[2]), static_cast<int>(v[3])};
    if (v.size() >= 2) return {static_cast<int>(v[0]), static_cast<int>(v[1]), static_cast<int>(v[0]), static_cast<int>(v[1])};
    return {0, 0, 0, 0};
}
const TensorTypeNode* TT(const Type& t) { return t.As<TensorTypeNode>(); }
kxc_hip_buf B(const HIPBuffer& b) { return kxc_hip_buf{b.kind, b.index_or_offset}; }
bool IsF32(const Type& t) { return TT(t) && TT(t)->dtype == "float32"; }
void Check(int32_t rc, const char* what) {
    if (rc != 0) throw std::runtime_error(std::string(what) + ": " + kxc_hip_last_error());
}

// ---------------------------------------------------------------- nn_conv2d (src/relay/op/nn/convolution.cc:38-75)
te::Tensor Conv2DCompute(const Attrs& attrs, const Array<te::Tensor>& in, const Type&) {
    if (in.size() < 2 || in.size() > 3) throw std::runtime_error("nn_conv2d expects 2 or 3 inputs (data, weight[, bias])");
    const auto* p = attrs.As<Conv2DAttrsNode>();
    if (!p) throw std::runtime_error("nn_conv2d expects Conv2DAttrs");
    if (p->data_layout != "NCHW" && !p->data_layout.empty()) throw std::runtime_error("nn_conv2d currently only supports NCHW");
    if (in[0]->shape.size() != 4 || in[1]->shape.size() != 4)
        throw std::runtime_error("nn_conv2d currently expects NCHW/OIHW rank-4 tensors");
    if (in.size() == 3 && in[2]->shape.size() != 1) throw std::runtime_error("nn_conv2d bias must be rank-1");
    // padding[0], padding[1] are applied on both sides (convolution.cc:53-54)
    te::Tensor conv = te::topi::conv2d_nchw(in[0], in[1], Read2D(p->strides, 0, 1), Read2D(p->strides, 1, 1),
                                            Read2D(p->padding, 0, 0), Read2D(p->padding, 1, 0), Read2D(p->dilation, 0, 1),
                                            Read2D(p->dilation, 1, 1), "T_conv2d");
    if (in.size() == 2) return conv;
    te::Tensor bias = in[2];
    return te::compute(conv->shape, [&](const Array<tir::Var>& ax) { return conv(ax) + bias(ax[1]); }, "T_conv2d_bias_add");
}

bool ConvDesc(const Attrs& attrs, const Array<Type>& input_types, kxc_hip_conv2d_desc* out) {
    const auto* p = attrs.As<Conv2DAttrsNode>();
    if (!p || input_types.size() < 2 || !IsF32(input_types[0]) || !IsF32(input_types[1])) return false;
    const auto* x = TT(input_types[0]);
    const auto* w = TT(input_types[1]);
    if (x->shape.size() != 4 || w->shape.size() != 4) return false;
    kxc_hip_conv2d_desc d{};
    d.n = static_cast<int32_t>(x->shape[0]); d.c = static_cast<int32_t>(x->shape[1]);
    d.h = static_cast<int32_t>(x->shape[2]); d.w = static_cast<int32_t>(x->shape[3]);
    d.o = static_cast<int32_t>(w->shape[0]); d.kh = static_cast<int32_t>(w->shape[2]); d.kw = static_cast<int32_t>(w->shape[3]);
    d.stride_h = Read2D(p->strides, 0, 1); d.stride_w = Read2D(p->strides, 1, 1);
    d.pad_h = Read2D(p->padding, 0, 0); d.pad_w = Read2D(p->padding, 1, 0);
    d.dil_h = Read2D(p->dilation, 0, 1); d.dil_w = Read2D(p->dilation, 1, 1);
    *out = d;
    return true;
}

// A residual block's first convolution (A) and its 1x1 downsample (B: same input, same strides, no padding, same
// number of output channels) run as one launch when the library has a kernel with a second output for A's shape
// and A would not rather run as Winograd.
bool Conv2DPairQuery(const Attrs& a_attrs, const Array<Type>& a_inputs, const std::vector<bool>& a_constant, const Attrs& b_attrs,
                     const Array<Type>& b_inputs) {
    kxc_hip_conv2d_desc a{}, b{};
    if (!ConvDesc(a_attrs, a_inputs, &a) || !ConvDesc(b_attrs, b_inputs, &b)) return false;
    if (b.kh != 1 || b.kw != 1 || b.pad_h != 0 || b.pad_w != 0 || b.o != a.o || b.c != a.c) return false;
    if (b.stride_h != a.stride_h || b.stride_w != a.stride_w) return false;
    if (a_constant.size() > 1 && a_constant[1] && kxc_hip_conv2d_winograd_preferred(&a)) return false;
    return kxc_hip_conv2d_pair_supported(&a) != 0;
}

// conv -> relu -> max pool (3x3, stride 2, padding 1): the convolution's launch takes the maximum over the three
// columns of every window while an output row is in registers and writes a map half as wide; a 3x1 / stride (2,1)
// max pool finishes the window.  Offered when the library has that epilogue for the shape and expects the two
// launches to beat convolution + 3x3 pool.
bool Conv2DPoolQuery(const Attrs& attrs, const Array<Type>& inputs, bool fused_relu, bool has_residual, const std::string& pool_op,
                     const Attrs& pool_attrs) {
    kxc_hip_conv2d_desc d{};
    const auto* p = pool_attrs.As<MaxPool2DAttrsNode>();
    if (pool_op != "nn_max_pool2d" || !p || !fused_relu || has_residual || !ConvDesc(attrs, inputs, &d)) return false;
    if (!p->layout.empty() && p->layout != "NCHW") return false;
    const auto ks = ReadPair(p->pool_size, 1), st = ReadPair(p->strides, 1), pd = ReadPad4(p->padding);
    if (ks[0] != 3 || ks[1] != 3 || st[0] != 2 || st[1] != 2 || pd[0] != 1 || pd[1] != 1 || pd[2] != 1 || pd[3] != 1 || p->ceil_mode)
        return false;
    d.flags = (inputs.size() == 3 ? KXC_HIP_CONV_BIAS : 0u) | KXC_HIP_CONV_RELU;
    return kxc_hip_conv2d_hpool_preferred(&d) != 0;
}

std::string Conv2DDispatch(const HIPDispatchContext& c, kxc_hip_plan* plan) {
    kxc_hip_conv2d_desc d{};
    if (!ConvDesc(c.attrs, c.input_types, &d) || !IsF32(c.out_type)) return "";
    const bool has_bias = c.inputs.size() == 3;
    d.flags = (has_bias ? KXC_HIP_CONV_BIAS : 0u) | (c.has_residual ? KXC_HIP_CONV_RESIDUAL : 0u) |
              (c.fused_relu ? KXC_HIP_CONV_RELU : 0u);
    const kxc_hip_buf none{KXC_HIP_BUF_NONE, 0};
    if (c.has_pool) {
        // (Conv2DPoolQuery said yes for exactly this call: 3x3 / stride 2 / padding 1 behind a ReLU)
        if (c.has_pair || c.has_residual || !c.fused_relu || !c.alloc_temp) return "";
        d.flags |= KXC_HIP_CONV_HPOOL;
        const int64_t oh = (d.h + 2 * d.pad_h - (d.dil_h * (d.kh - 1) + 1)) / d.stride_h + 1;
        const int64_t ow = (d.w + 2 * d.pad_w - (d.dil_w * (d.kw - 1) + 1)) / d.stride_w + 1;
        const HIPBuffer half = c.alloc_temp(static_cast<int64_t>(d.n) * d.o * oh * (ow / 2) * 4);
        Check(kxc_hip_plan_add_conv2d(plan, &d, B(c.inputs[0]), B(c.inputs[1]), has_bias ? B(c.inputs[2]) : none, none, B(half)),
              "nn_conv2d dispatch");
        kxc_hip_pool2d_desc q{};
        q.n = d.n; q.c = d.o; q.h = static_cast<int32_t>(oh); q.w = static_cast<int32_t>(ow / 2);
        q.kh = 3; q.kw = 1; q.stride_h = 2; q.stride_w = 1;
        q.pad_top = 1; q.pad_bottom = 1;
        Check(kxc_hip_plan_add_pool2d(plan, &q, B(half), B(c.output)), "nn_conv2d dispatch (column pool)");
        return std::string("kxc_conv2d_nchw_f32.") + kxc_hip_conv2d_variant(&d) + (has_bias ? "+bias" : "") + "+relu+maxpool3w";
    }
    if (c.has_pair) {
        const bool bias2 = c.pair_inputs.size() == 3;
        Check(kxc_hip_plan_add_conv2d_pair(plan, &d, B(c.inputs[0]), B(c.inputs[1]), has_bias ? B(c.inputs[2]) : none,
                                           c.has_residual ? B(c.residual) : none, B(c.output), B(c.pair_inputs[1]),
                                           bias2 ? B(c.pair_inputs[2]) : none, B(c.pair_output)),
              "nn_conv2d pair dispatch");
        return std::string("kxc_conv2d_nchw_f32.") + kxc_hip_conv2d_pair_variant(&d) + (has_bias ? "+bias" : "") +
               (c.has_residual ? "+add" : "") + (c.fused_relu ? "+relu" : "") + "|conv1x1" + (bias2 ? "+bias" : "");
    }
    // 3x3 stride-1 convolutions with constant weights run as Winograd F(2x2,3x3) when the library expects that to
    // be faster for the shape; the transformed weights get a workspace region of their own.
    if (c.winograd_allowed && c.alloc_persistent && c.input_constant.size() > 1 && c.input_constant[1] &&
        kxc_hip_conv2d_winograd_preferred(&d)) {
        size_t u_bytes = 0;
        Check(kxc_hip_conv2d_winograd_weight_bytes(&d, &u_bytes), "nn_conv2d dispatch");
        const HIPBuffer u = c.alloc_persistent(static_cast<int64_t>(u_bytes));
        Check(kxc_hip_plan_add_conv2d_winograd(plan, &d, B(c.inputs[0]), B(c.inputs[1]), has_bias ? B(c.inputs[2]) : none,
                                               c.has_residual ? B(c.residual) : none, B(c.output), B(u)),
              "nn_conv2d dispatch");
        return std::string("kxc_conv2d_nchw_f32.") + kxc_hip_conv2d_winograd_variant(&d) + (has_bias ? "+bias" : "") +
               (c.has_residual ? "+add" : "") + (c.fused_relu ? "+relu" : "");
    }
    Check(kxc_hip_plan_add_conv2d(plan, &d, B(c.inputs[0]), B(c.inputs[1]), has_bias ? B(c.inputs[2]) : none,
                                  c.has_residual ? B(c.residual) : none, B(c.output)),
          "nn_conv2d dispatch");
    return std::string("kxc_conv2d_nchw_f32.") + kxc_hip_conv2d_variant(&d) + (has_bias ? "+bias" : "") +
           (c.has_residual ? "+add" : "") + (c.fused_relu ? "+relu" : "");
}

// ---------------------------------------------------------------- pooling (src/relay/op/nn/pooling.cc:50-98)
te::Tensor PoolCompute(const char* op, const char* type, const char* tname, const Attrs& attrs, const Array<te::Tensor>& in) {
    if (in.size() != 1) throw std::runtime_error(std::string(op) + " expects exactly 1 input");
    const auto* p = attrs.As<MaxPool2DAttrsNode>();
    if (!p) throw std::runtime_error(std::string(op) + " expects MaxPool2DAttrs");
    if ((p->layout != "NCHW" && !p->layout.empty()) || in[0]->shape.size() != 4)
        throw std::runtime_error(std::string(op) + " expects NCHW rank-4 input");
    return te::topi::pool2d(in[0], ReadPair(p->pool_size, 1), ReadPair(p->strides, 1), ReadPad4(p->padding), type,
                            p->ceil_mode, tname);
}

std::string PoolDispatch(bool is_avg, const HIPDispatchContext& c, kxc_hip_plan* plan) {
    const auto* p = c.attrs.As<MaxPool2DAttrsNode>();
    const bool i8 = !is_avg && TT(c.input_types[0]) && TT(c.input_types[0])->dtype == "int8";
    if (!p || !(IsF32(c.input_types[0]) || i8)) return "";
    const auto* x = TT(c.input_types[0]);
    const auto ks = ReadPair(p->pool_size, 1), st = ReadPair(p->strides, 1), pd = ReadPad4(p->padding);
    kxc_hip_pool2d_desc d{};
    d.n = static_cast<int32_t>(x->shape[0]); d.c = static_cast<int32_t>(x->shape[1]);
    d.h = static_cast<int32_t>(x->shape[2]); d.w = static_cast<int32_t>(x->shape[3]);
    d.kh = ks[0]; d.kw = ks[1]; d.stride_h = st[0]; d.stride_w = st[1];
    d.pad_top = pd[0]; d.pad_left = pd[1]; d.pad_bottom = pd[2]; d.pad_right = pd[3];
    d.ceil_mode = p->ceil_mode ? 1 : 0;
    d.is_avg = is_avg ? 1 : 0;
    if (i8) {
        // int8 max pool (the padding candidate is -128, the dtype's lowest value): channel-blocked or NCHW
        const bool blocked = !c.input_layouts.empty() && c.input_layouts[0] == kHIPLayoutC16;
        if (blocked != (c.output_layout == kHIPLayoutC16)) return "";
        Check(blocked ? kxc_hip_plan_add_maxpool2d_c16_i8(plan, &d, B(c.inputs[0]), B(c.output))
                      : kxc_hip_plan_add_maxpool2d_i8(plan, &d, B(c.inputs[0]), B(c.output)),
              "int8 max pool dispatch");
        return blocked ? "kxc_max_pool2d_c16_i8" : "kxc_max_pool2d_i8";
    }
    Check(kxc_hip_plan_add_pool2d(plan, &d, B(c.inputs[0]), B(c.output)), "pool2d dispatch");
    return is_avg ? "kxc_avg_pool2d_f32" : "kxc_max_pool2d_f32";
}

std::string GapDispatch(const HIPDispatchContext& c, kxc_hip_plan* plan) {
    if (!IsF32(c.input_types[0])) return "";
    const auto* x = TT(c.input_types[0]);
    Check(kxc_hip_plan_add_global_avg_pool2d(plan, x->shape[0], x->shape[1], x->shape[2], x->shape[3], B(c.inputs[0]),
                                             B(c.output)),
          "nn_global_avg_pool2d dispatch");
    return "kxc_global_avg_pool2d_f32";
}

// ---------------------------------------------------------------- dense / gemm (src/relay/op/nn/dense.cc:17-61)
te::Tensor ScaleTensor(const te::Tensor& t, double scale, const std::string& name) {
    if (scale == 1.0) return t;
    return te::compute(t->shape, [&](const Array<tir::Var>& ax) { return t(ax) * te::topi::make_const(t->dtype, scale); }, name);
}

te::Tensor GemmCompute(const Attrs& attrs, const Array<te::Tensor>& in, const Type&) {
    if (in.size() != 3) throw std::runtime_error("nn_gemm expects exactly 3 inputs");
    const auto* p = attrs.As<GemmAttrsNode>();
    if (!p) throw std::runtime_error("nn_gemm expects GemmAttrs");
    if (p->transA != 0) throw std::runtime_error("nn_gemm currently does not support transA=1");
    te::Tensor out = p->transB == 1 ? te::topi::dense(in[0], in[1], "T_gemm_dense") : te::topi::matmul(in[0], in[1], "T_gemm_matmul");
    out = ScaleTensor(out, p->alpha, "T_gemm_alpha");
    te::Tensor bias = in[2];
    if (p->beta != 1.0) bias = ScaleTensor(in[2], p->beta, "T_gemm_beta");
    return te::topi::add(out, bias, "T_gemm_out");
}

std::string GemmDispatch(const HIPDispatchContext& c, kxc_hip_plan* plan) {
    const auto* p = c.attrs.As<GemmAttrsNode>();
    if (!p || p->transA != 0 || !IsF32(c.input_types[0])) return "";
    const auto* a = TT(c.input_types[0]);
    const auto* o = TT(c.out_type);
    const auto* bias = TT(c.input_types[2]);
    const int64_t c_len = Product(bias->shape);
    if (bias->shape.size() > 1 || (c_len != o->shape[1] && c_len != 1)) return "";   // general bias shapes: generic path
    Check(kxc_hip_plan_add_gemm(plan, o->shape[0], o->shape[1], a->shape[1], p->alpha, p->beta, p->transB, c_len,
                                B(c.inputs[0]), B(c.inputs[1]), B(c.inputs[2]), B(c.output)),
          "nn_gemm dispatch");
    return "kxc_gemm_f32";
}

std::string DenseDispatch(bool transB, const HIPDispatchContext& c, kxc_hip_plan* plan) {
    if (!IsF32(c.input_types[0])) return "";
    const auto* a = TT(c.input_types[0]);
    const auto* o = TT(c.out_type);
    const kxc_hip_buf none{KXC_HIP_BUF_NONE, 0};
    Check(kxc_hip_plan_add_gemm(plan, o->shape[0], o->shape[1], a->shape[1], 1.0f, 1.0f, transB ? 1 : 0, 0, B(c.inputs[0]),
                                B(c.inputs[1]), none, B(c.output)),
          "nn_dense dispatch");
    return "kxc_gemm_f32";
}

// ---------------------------------------------------------------- quantised operators (no counterpart in the reference)
bool IsDType(const Type& t, const char* dtype) { return TT(t) && TT(t)->dtype == dtype; }

te::Tensor QnnConv2DCompute(const Attrs& attrs, const Array<te::Tensor>& in, const Type&) {
    const auto* p = attrs.As<QnnConv2DAttrsNode>();
    if (!p) throw std::runtime_error("qnn_conv2d expects QnnConv2DAttrs");
    if (in.size() != 4 && in.size() != 5) throw std::runtime_error("qnn_conv2d expects data, weight, bias, mult[, residual]");
    const auto st = ReadPair(p->strides, 1), pd = ReadPair(p->padding, 0);
    return te::topi::qnn_conv2d_nchw(in[0], in[1], in[2], in[3], in.size() == 5 ? in[4] : te::Tensor(), static_cast<int>(st[0]),
                                     static_cast<int>(st[1]), static_cast<int>(pd[0]), static_cast<int>(pd[1]), p->relu, p->res_mult,
                                     "T_qnn_conv2d");
}

bool QnnConvDesc(const Attrs& attrs, const Array<Type>& input_types, kxc_hip_qconv2d_desc* out) {
    const auto* p = attrs.As<QnnConv2DAttrsNode>();
    if (!p || input_types.size() < 4 || !IsDType(input_types[0], "int8") || !IsDType(input_types[1], "int8")) return false;
    const auto* x = TT(input_types[0]);
    const auto* w = TT(input_types[1]);
    if (x->shape.size() != 4 || w->shape.size() != 4) return false;
    const auto st = ReadPair(p->strides, 1), pd = ReadPair(p->padding, 0);
    kxc_hip_qconv2d_desc d{};
    d.n = static_cast<int32_t>(x->shape[0]); d.c = static_cast<int32_t>(x->shape[1]);
    d.h = static_cast<int32_t>(x->shape[2]); d.w = static_cast<int32_t>(x->shape[3]);
    d.o = static_cast<int32_t>(w->shape[0]); d.kh = static_cast<int32_t>(w->shape[2]); d.kw = static_cast<int32_t>(w->shape[3]);
    d.stride_h = static_cast<int32_t>(st[0]); d.stride_w = static_cast<int32_t>(st[1]);
    d.pad_h = static_cast<int32_t>(pd[0]); d.pad_w = static_cast<int32_t>(pd[1]);
    const bool has_res = input_types.size() == 5;
    d.flags = KXC_HIP_CONV_BIAS | (has_res ? KXC_HIP_CONV_RESIDUAL : 0u) | (p->relu ? KXC_HIP_CONV_RELU : 0u);
    d.res_mult = has_res ? static_cast<float>(p->res_mult) : 0.0f;
    *out = d;
    return true;
}

bool MatrixCoresDisabled() {
    const char* e = std::getenv("KXC_HIP_QNN_MFMA");       // "0": every quantised operator keeps NCHW and its scalar kernel
    return e && e[0] == '0';
}

// The matrix-core kernels read channel-blocked activations and weights packed for them.  The weights must be
// readable before the first launch of a run (a parameter or a constant) because they are packed at its start.
HIPLayoutChoice QnnConv2DLayout(const Attrs& attrs, const Array<Type>& in, const Type&, const std::vector<int>& offered,
                                const std::vector<bool>& input_argument) {
    HIPLayoutChoice plain;
    plain.inputs.assign(in.size(), kHIPLayoutPlain);
    kxc_hip_qconv2d_desc d{};
    if (MatrixCoresDisabled() || !QnnConvDesc(attrs, in, &d) || input_argument.size() < 2 || !input_argument[1]) return plain;
    HIPLayoutChoice blocked = plain;
    blocked.output = kHIPLayoutC16;
    if (in.size() == 5) blocked.inputs[4] = kHIPLayoutC16;
    // the 4-channel input layout only ever comes from a producer that follows this call (qnn_quantize)
    if ((offered[0] == kHIPLayoutAny || offered[0] == kHIPLayoutC4) && in.size() == 4 && kxc_hip_qconv2d_c4_supported(&d)) {
        blocked.inputs[0] = kHIPLayoutC4;
        return blocked;
    }
    if (!kxc_hip_qconv2d_c16_supported(&d)) return plain;
    blocked.inputs[0] = kHIPLayoutC16;
    return blocked;
}

// A residual block's first convolution (A: ReLU, no residual) and its 1x1 downsample (B: same input and strides, no
// padding, no ReLU, no residual, same number of output channels) as one launch on the matrix cores.
bool QnnConv2DPairQuery(const Attrs& a_attrs, const Array<Type>& a_inputs, const std::vector<bool>&, const Attrs& b_attrs,
                        const Array<Type>& b_inputs) {
    kxc_hip_qconv2d_desc a{}, b{};
    if (MatrixCoresDisabled() || !QnnConvDesc(a_attrs, a_inputs, &a) || !QnnConvDesc(b_attrs, b_inputs, &b)) return false;
    if (a_inputs.size() != 4 || b_inputs.size() != 4) return false;
    if (b.kh != 1 || b.kw != 1 || b.pad_h != 0 || b.pad_w != 0 || b.o != a.o || b.c != a.c) return false;
    if (b.stride_h != a.stride_h || b.stride_w != a.stride_w || (b.flags & KXC_HIP_CONV_RELU)) return false;
    const char* e = std::getenv("KXC_HIP_QPAIR");
    if (e && e[0] == '0') return false;
    return kxc_hip_qconv2d_c16_pair_supported(&a) != 0;
}

// The first layer on its 4-channel input followed by nn_max_pool2d(3x3, stride 2, padding 1) as one kernel whose
// output is the pooled map (asked once the layouts are known: the call's first input is not plain).
bool QnnConv2DPoolQuery(const Attrs& attrs, const Array<Type>& inputs, bool, bool, const std::string& pool_op, const Attrs& pool_attrs) {
    kxc_hip_qconv2d_desc d{};
    const auto* p = pool_attrs.As<MaxPool2DAttrsNode>();
    if (MatrixCoresDisabled() || pool_op != "nn_max_pool2d" || !p || inputs.size() != 4 || !QnnConvDesc(attrs, inputs, &d)) return false;
    if (!p->layout.empty() && p->layout != "NCHW") return false;
    const auto ks = ReadPair(p->pool_size, 1), st = ReadPair(p->strides, 1), pd = ReadPad4(p->padding);
    if (ks[0] != 3 || ks[1] != 3 || st[0] != 2 || st[1] != 2 || pd[0] != 1 || pd[1] != 1 || pd[2] != 1 || pd[3] != 1 || p->ceil_mode)
        return false;
    return kxc_hip_qconv2d_c4_supported(&d) != 0 && kxc_hip_qconv2d_c4_maxpool_supported(&d) != 0;
}

std::string QnnConv2DDispatch(const HIPDispatchContext& c, kxc_hip_plan* plan) {
    kxc_hip_qconv2d_desc d{};
    if (!QnnConvDesc(c.attrs, c.input_types, &d) || !IsDType(c.out_type, "int8")) return "";
    const bool has_res = c.inputs.size() == 5;
    const kxc_hip_buf none{KXC_HIP_BUF_NONE, 0};
    const int in_layout = c.input_layouts.empty() ? kHIPLayoutPlain : c.input_layouts[0];
    if (c.has_pool && (in_layout != kHIPLayoutC4 || c.has_pair)) return "";
    if (in_layout == kHIPLayoutPlain) {
        if (c.output_layout != kHIPLayoutPlain || c.has_pair) return "";
        Check(kxc_hip_plan_add_qconv2d(plan, &d, B(c.inputs[0]), B(c.inputs[1]), B(c.inputs[2]), B(c.inputs[3]),
                                       has_res ? B(c.inputs[4]) : none, B(c.output)),
              "qnn_conv2d dispatch");
        return "kxc_qconv2d_nchw_i8";
    }
    // matrix cores: the weights are packed into a region of the module's own at the start of a run (every run when
    // they are a parameter rather than a constant)
    if (c.output_layout != kHIPLayoutC16 || !c.alloc_persistent || (has_res && c.input_layouts[4] != kHIPLayoutC16)) return "";
    if (c.has_pair && (in_layout != kHIPLayoutC16 || c.pair_inputs.size() != 4 || c.pair_output_layout != kHIPLayoutC16)) return "";
    const int every_run = c.input_constant.size() > 1 && c.input_constant[1] ? 0 : 1;
    size_t bytes = 0;
    if (in_layout == kHIPLayoutC4) {
        Check(kxc_hip_qconv2d_c4_packed_bytes(&d, &bytes), "qnn_conv2d dispatch");
        const HIPBuffer wp = c.alloc_persistent(static_cast<int64_t>(bytes));
        Check(kxc_hip_plan_add_qconv_weight_pack(plan, KXC_HIP_QPACK_C4, &d, B(c.inputs[1]), B(wp), every_run), "qnn_conv2d weight pack");
        if (c.has_pool) {
            Check(kxc_hip_plan_add_qconv2d_c4_maxpool(plan, &d, B(c.inputs[0]), B(wp), B(c.inputs[2]), B(c.inputs[3]), B(c.output)),
                  "qnn_conv2d dispatch (with the max pool)");
            return std::string("kxc_qconv2d_c4_i8:qmfma_k7x7s2_c4") + ((d.flags & KXC_HIP_CONV_RELU) ? "+relu" : "") + "+maxpool3x3s2";
        }
        Check(kxc_hip_plan_add_qconv2d_c4(plan, &d, B(c.inputs[0]), B(wp), B(c.inputs[2]), B(c.inputs[3]), B(c.output)),
              "qnn_conv2d dispatch");
        return std::string("kxc_qconv2d_c4_i8:qmfma_k7x7s2_c4") + ((d.flags & KXC_HIP_CONV_RELU) ? "+relu" : "");
    }
    Check(kxc_hip_qconv2d_c16_packed_bytes(&d, &bytes), "qnn_conv2d dispatch");
    const HIPBuffer wp = c.alloc_persistent(static_cast<int64_t>(bytes));
    Check(kxc_hip_plan_add_qconv_weight_pack(plan, KXC_HIP_QPACK_C16, &d, B(c.inputs[1]), B(wp), every_run), "qnn_conv2d weight pack");
    const std::string tail = std::string(has_res ? "+add" : "") + ((d.flags & KXC_HIP_CONV_RELU) ? "+relu" : "");
    if (c.has_pair) {
        size_t bytes2 = 0;
        Check(kxc_hip_qconv2d_c16_pair_packed_bytes(&d, &bytes2), "qnn_conv2d pair dispatch");
        const HIPBuffer wp2 = c.alloc_persistent(static_cast<int64_t>(bytes2));
        Check(kxc_hip_plan_add_qconv_weight_pack(plan, KXC_HIP_QPACK_C16_PAIR, &d, B(c.pair_inputs[1]), B(wp2), every_run),
              "qnn_conv2d pair weight pack");
        Check(kxc_hip_plan_add_qconv2d_c16_pair(plan, &d, B(c.inputs[0]), B(wp), B(c.inputs[2]), B(c.inputs[3]),
                                                has_res ? B(c.inputs[4]) : none, B(c.output), B(wp2), B(c.pair_inputs[2]),
                                                B(c.pair_inputs[3]), B(c.pair_output)),
              "qnn_conv2d pair dispatch");
        return std::string("kxc_qconv2d_c16_i8:") + kxc_hip_qconv2d_c16_variant(&d) + tail + "|qconv1x1+bias";
    }
    Check(kxc_hip_plan_add_qconv2d_c16(plan, &d, B(c.inputs[0]), B(wp), B(c.inputs[2]), B(c.inputs[3]),
                                       has_res ? B(c.inputs[4]) : none, B(c.output)),
          "qnn_conv2d dispatch");
    return std::string("kxc_qconv2d_c16_i8:") + kxc_hip_qconv2d_c16_variant(&d) + tail;
}

std::string QnnDenseDispatch(const HIPDispatchContext& c, kxc_hip_plan* plan) {
    if (c.inputs.size() != 4 || !IsDType(c.input_types[0], "int8") || !IsF32(c.out_type)) return "";
    const auto* a = TT(c.input_types[0]);
    const auto* o = TT(c.out_type);
    Check(kxc_hip_plan_add_qdense(plan, o->shape[0], o->shape[1], a->shape[1], B(c.inputs[0]), B(c.inputs[1]), B(c.inputs[2]),
                                  B(c.inputs[3]), B(c.output)),
          "qnn_dense dispatch");
    return "kxc_qdense_i8";
}

std::string QnnQuantizeDispatch(const HIPDispatchContext& c, kxc_hip_plan* plan) {
    const auto* p = c.attrs.As<QnnQuantizeAttrsNode>();
    if (!p || !IsF32(c.input_types[0])) return "";
    const auto* x = TT(c.input_types[0]);
    if (c.output_layout == kHIPLayoutPlain) {
        Check(kxc_hip_plan_add_quantize(plan, Product(x->shape), static_cast<float>(p->scale), B(c.inputs[0]), B(c.output)),
              "qnn_quantize dispatch");
        return "kxc_quantize_f32_i8";
    }
    if (x->shape.size() != 4) return "";
    const int64_t hw = x->shape[2] * x->shape[3];
    if (c.output_layout == kHIPLayoutC4) {
        Check(kxc_hip_plan_add_quantize_c4(plan, x->shape[0], x->shape[1], hw, static_cast<float>(p->scale), B(c.inputs[0]), B(c.output)),
              "qnn_quantize dispatch");
        return "kxc_quantize_f32_nchw_to_c4_i8";
    }
    Check(kxc_hip_plan_add_quantize_c16(plan, x->shape[0], x->shape[1], hw, static_cast<float>(p->scale), B(c.inputs[0]), B(c.output)),
          "qnn_quantize dispatch");
    return "kxc_quantize_f32_nchw_to_c16_i8";
}

// int8 max pool and the requantising global average pool keep whatever layout their input has.
HIPLayoutChoice Int8PoolLayout(const Attrs&, const Array<Type>& in, const Type&, const std::vector<int>& offered,
                               const std::vector<bool>&) {
    HIPLayoutChoice choice;
    choice.inputs.assign(in.size(), kHIPLayoutPlain);
    if (!MatrixCoresDisabled() && IsDType(in[0], "int8") && TT(in[0])->shape.size() == 4 && offered[0] == kHIPLayoutC16) {
        choice.inputs[0] = kHIPLayoutC16;
        choice.output = kHIPLayoutC16;
    }
    return choice;
}
HIPLayoutChoice QnnGapLayout(const Attrs&, const Array<Type>& in, const Type&, const std::vector<int>& offered,
                             const std::vector<bool>&) {
    // [N][C/16][1][1][16] is plain [N, C, 1, 1] when the channels fill their blocks
    HIPLayoutChoice choice;
    choice.inputs.assign(in.size(), kHIPLayoutPlain);
    if (!MatrixCoresDisabled() && offered[0] == kHIPLayoutC16 && TT(in[0])->shape[1] % 16 == 0) choice.inputs[0] = kHIPLayoutC16;
    return choice;
}

std::string QnnGapDispatch(const HIPDispatchContext& c, kxc_hip_plan* plan) {
    const auto* p = c.attrs.As<QnnRequantAttrsNode>();
    if (!p || !IsDType(c.input_types[0], "int8") || c.output_layout != kHIPLayoutPlain) return "";
    const auto* x = TT(c.input_types[0]);
    const bool blocked = !c.input_layouts.empty() && c.input_layouts[0] == kHIPLayoutC16;
    Check(blocked ? kxc_hip_plan_add_global_avg_pool2d_c16_i8(plan, x->shape[0], x->shape[1], x->shape[2], x->shape[3],
                                                              static_cast<float>(p->mult), B(c.inputs[0]), B(c.output))
                  : kxc_hip_plan_add_global_avg_pool2d_i8(plan, x->shape[0], x->shape[1], x->shape[2], x->shape[3],
                                                          static_cast<float>(p->mult), B(c.inputs[0]), B(c.output)),
          "qnn_global_avg_pool2d dispatch");
    return blocked ? "kxc_global_avg_pool2d_c16_i8" : "kxc_global_avg_pool2d_i8";
}

// ---------------------------------------------------------------- elementwise
std::string BinaryDispatch(int op, const HIPDispatchContext& c, kxc_hip_plan* plan) {
    if (!IsF32(c.input_types[0]) || !IsF32(c.input_types[1])) return "";
    const auto* a = TT(c.input_types[0]);
    const auto* b = TT(c.input_types[1]);
    if (a->shape.size() > 6 || b->shape.size() > 6) return "";
    Check(kxc_hip_plan_add_binary(plan, op, a->shape.data(), static_cast<int32_t>(a->shape.size()), b->shape.data(),
                                  static_cast<int32_t>(b->shape.size()), c.fused_relu ? 1 : 0, B(c.inputs[0]), B(c.inputs[1]),
                                  B(c.output)),
          "broadcast dispatch");
    static const char* names[4] = {"kxc_add_f32", "kxc_subtract_f32", "kxc_multiply_f32", "kxc_divide_f32"};
    return std::string(names[op]) + (c.fused_relu ? "+relu" : "");
}

std::string ReluDispatch(const HIPDispatchContext& c, kxc_hip_plan* plan) {
    if (!IsF32(c.input_types[0])) return "";
    Check(kxc_hip_plan_add_relu(plan, Product(TT(c.input_types[0])->shape), B(c.inputs[0]), B(c.output)), "nn_relu dispatch");
    return "kxc_relu_f32";
}

FRelayToTE BinaryCompute(int op, const char* name) {
    return [op, name](const Attrs&, const Array<te::Tensor>& in, const Type&) {
        if (in.size() != 2) throw std::runtime_error(std::string(name) + " expects exactly 2 inputs");
        static const char* tnames[4] = {"T_add", "T_subtract", "T_multiply", "T_divide"};
        return te::topi::broadcast_binary(op, in[0], in[1], tnames[op]);
    };
}

bool g_registered = false;

}  // namespace

void EnsureBuiltinOpsRegistered() {
    static bool done = [] {
        g_registered = true;
        OpRegEntry::Register("nn_conv2d")
            .describe("2D convolution, NCHW data and OIHW weights, optional rank-1 bias.")
            .set_num_inputs(-1)
            .add_argument("data", "Tensor", "The input tensor.")
            .add_argument("weight", "Tensor", "The weight tensor.")
            .set_attr<std::string>("TAttrs", "Conv2DAttrs")
            .set_attr<FInferType>("FInferType", Conv2DInferType)
            .set_attr<FRelayToTE>("FRelayToTE", Conv2DCompute)
            .set_attr<bool>("THIPFusable", true)
            .set_attr<FHIPDispatch>("FHIPDispatch", Conv2DDispatch)
            .set_attr<FHIPPairQuery>("FHIPPairQuery", Conv2DPairQuery)
            .set_attr<FHIPPoolQuery>("FHIPPoolQuery", Conv2DPoolQuery);
        OpRegEntry::Register("nn_relu")
            .describe("Rectified Linear Unit activation")
            .set_num_inputs(1)
            .add_argument("data", "Tensor", "The input tensor.")
            .set_attr<std::string>("TAttrs", "ReluAttrs")
            .set_attr<FInferType>("FInferType", UnarySameInferType)
            .set_attr<FRelayToTE>("FRelayToTE", [](const Attrs&, const Array<te::Tensor>& in, const Type&) {
                if (in.size() != 1) throw std::runtime_error("nn_relu expects exactly 1 input");
                return te::topi::relu(in[0], "T_relu");
            })
            .set_attr<FHIPDispatch>("FHIPDispatch", ReluDispatch);
        OpRegEntry::Register("nn_max_pool2d")
            .describe("2D max pooling operation.")
            .set_num_inputs(1)
            .add_argument("data", "Tensor", "The input tensor.")
            .set_attr<std::string>("TAttrs", "MaxPool2DAttrs")
            .set_attr<FInferType>("FInferType", Pool2DInferType)
            .set_attr<FRelayToTE>("FRelayToTE", [](const Attrs& a, const Array<te::Tensor>& in, const Type&) {
                return PoolCompute("nn_max_pool2d", "max", "T_max_pool2d", a, in);
            })
            .set_attr<FHIPLayoutQuery>("FHIPLayoutQuery", Int8PoolLayout)
            .set_attr<FHIPDispatch>("FHIPDispatch", [](const HIPDispatchContext& c, kxc_hip_plan* p) { return PoolDispatch(false, c, p); });
        OpRegEntry::Register("nn_avg_pool2d")
            .describe("2D average pooling operation.")
            .set_num_inputs(1)
            .add_argument("data", "Tensor", "The input tensor.")
            .set_attr<std::string>("TAttrs", "MaxPool2DAttrs")
            .set_attr<FInferType>("FInferType", Pool2DInferType)
            .set_attr<FRelayToTE>("FRelayToTE", [](const Attrs& a, const Array<te::Tensor>& in, const Type&) {
                return PoolCompute("nn_avg_pool2d", "avg", "T_avg_pool2d", a, in);
            })
            .set_attr<FHIPDispatch>("FHIPDispatch", [](const HIPDispatchContext& c, kxc_hip_plan* p) { return PoolDispatch(true, c, p); });
        OpRegEntry::Register("nn_global_avg_pool2d")
            .describe("Global average pooling: reduces H and W to 1x1 by averaging.")
            .set_num_inputs(1)
            .add_argument("data", "Tensor", "The input tensor.")
            .set_attr<std::string>("TAttrs", "GlobalAvgPool2DAttrs")
            .set_attr<FInferType>("FInferType", GlobalAvgPool2DInferType)
            .set_attr<FRelayToTE>("FRelayToTE", [](const Attrs&, const Array<te::Tensor>& in, const Type&) {
                if (in.size() != 1) throw std::runtime_error("nn_global_avg_pool2d expects exactly 1 input");
                if (in[0]->shape.size() != 4) throw std::runtime_error("nn_global_avg_pool2d expects NCHW rank-4 input");
                return te::topi::global_avg_pool2d(in[0], "T_global_avg_pool2d");
            })
            .set_attr<FHIPDispatch>("FHIPDispatch", GapDispatch);
        OpRegEntry::Register("nn_dense")
            .describe("Dense (fully connected) layer")
            .set_num_inputs(2)
            .add_argument("data", "Tensor", "The input tensor.")
            .add_argument("weight", "Tensor", "The weight tensor.")
            .set_attr<std::string>("TAttrs", "DenseAttrs")
            .set_attr<FInferType>("FInferType", DenseInferType)
            .set_attr<FRelayToTE>("FRelayToTE", [](const Attrs&, const Array<te::Tensor>& in, const Type&) {
                if (in.size() != 2) throw std::runtime_error("nn_dense expects exactly 2 inputs");
                return te::topi::dense(in[0], in[1], "T_dense");
            })
            .set_attr<FHIPDispatch>("FHIPDispatch", [](const HIPDispatchContext& c, kxc_hip_plan* p) { return DenseDispatch(true, c, p); });
        OpRegEntry::Register("qnn_conv2d")
            .describe("int8 2D convolution with int32 accumulation and per-output-channel requantisation (NCHW / OIHW).")
            .set_num_inputs(-1)
            .add_argument("data", "Tensor", "int8 input.")
            .add_argument("weight", "Tensor", "int8 weights.")
            .add_argument("bias", "Tensor", "int32 bias per output channel.")
            .add_argument("mult", "Tensor", "float32 requantisation multiplier per output channel.")
            .set_attr<std::string>("TAttrs", "QnnConv2DAttrs")
            .set_attr<FInferType>("FInferType", QnnConv2DInferType)
            .set_attr<FRelayToTE>("FRelayToTE", QnnConv2DCompute)
            .set_attr<FHIPLayoutQuery>("FHIPLayoutQuery", QnnConv2DLayout)
            .set_attr<FHIPPairQuery>("FHIPPairQuery", QnnConv2DPairQuery)
            .set_attr<FHIPPoolQuery>("FHIPPoolQuery", QnnConv2DPoolQuery)
            .set_attr<FHIPDispatch>("FHIPDispatch", QnnConv2DDispatch);
        OpRegEntry::Register("qnn_dense")
            .describe("int8 dense layer with int32 accumulation; float32 output (acc + bias) * mult.")
            .set_num_inputs(4)
            .add_argument("data", "Tensor", "int8 input [M, K].")
            .add_argument("weight", "Tensor", "int8 weights [N, K].")
            .add_argument("bias", "Tensor", "int32 bias [N].")
            .add_argument("mult", "Tensor", "float32 multiplier [N].")
            .set_attr<FInferType>("FInferType", QnnDenseInferType)
            .set_attr<FRelayToTE>("FRelayToTE", [](const Attrs&, const Array<te::Tensor>& in, const Type&) {
                if (in.size() != 4) throw std::runtime_error("qnn_dense expects data, weight, bias, mult");
                return te::topi::qnn_dense(in[0], in[1], in[2], in[3], "T_qnn_dense");
            })
            .set_attr<FHIPDispatch>("FHIPDispatch", QnnDenseDispatch);
        OpRegEntry::Register("qnn_quantize")
            .describe("float32 -> int8 with a per-tensor scale: clamp(rint(x / scale), -127, 127).")
            .set_num_inputs(1)
            .add_argument("data", "Tensor", "float32 input.")
            .set_attr<std::string>("TAttrs", "QnnQuantizeAttrs")
            .set_attr<FInferType>("FInferType", QnnQuantizeInferType)
            .set_attr<FRelayToTE>("FRelayToTE", [](const Attrs& attrs, const Array<te::Tensor>& in, const Type&) {
                const auto* p = attrs.As<QnnQuantizeAttrsNode>();
                if (!p || in.size() != 1) throw std::runtime_error("qnn_quantize expects one input and QnnQuantizeAttrs");
                return te::topi::qnn_quantize(in[0], p->scale, "T_qnn_quantize");
            })
            .set_attr<bool>("THIPLayoutFollowsConsumers", true)      // its kernels write NCHW, c16 or c4
            .set_attr<FHIPDispatch>("FHIPDispatch", QnnQuantizeDispatch);
        OpRegEntry::Register("qnn_global_avg_pool2d")
            .describe("int8 global average pool: the int32 sum over H and W, requantised with one multiplier, as int8 [N,C,1,1].")
            .set_num_inputs(1)
            .add_argument("data", "Tensor", "int8 input [N, C, H, W].")
            .set_attr<std::string>("TAttrs", "QnnRequantAttrs")
            .set_attr<FInferType>("FInferType", QnnGlobalAvgPool2DInferType)
            .set_attr<FRelayToTE>("FRelayToTE", [](const Attrs& attrs, const Array<te::Tensor>& in, const Type&) {
                const auto* p = attrs.As<QnnRequantAttrsNode>();
                if (!p || in.size() != 1) throw std::runtime_error("qnn_global_avg_pool2d expects one input and QnnRequantAttrs");
                return te::topi::qnn_global_avg_pool2d(in[0], p->mult, "T_qnn_global_avg_pool2d");
            })
            .set_attr<FHIPLayoutQuery>("FHIPLayoutQuery", QnnGapLayout)
            .set_attr<FHIPDispatch>("FHIPDispatch", QnnGapDispatch);
        OpRegEntry::Register("matmul")
            .describe("Matrix multiplication [M,K] x [K,N]")
            .set_num_inputs(2)
            .add_argument("lhs", "Tensor", "The first input tensor.")
            .add_argument("rhs", "Tensor", "The second input tensor.")
            .set_attr<FInferType>("FInferType", MatmulInferType)
            .set_attr<FRelayToTE>("FRelayToTE", [](const Attrs&, const Array<te::Tensor>& in, const Type&) {
                if (in.size() != 2) throw std::runtime_error("matmul expects exactly 2 inputs");
                return te::topi::matmul(in[0], in[1], "T_matmul");
            })
            .set_attr<FHIPDispatch>("FHIPDispatch", [](const HIPDispatchContext& c, kxc_hip_plan* p) { return DenseDispatch(false, c, p); });
        OpRegEntry::Register("nn_gemm")
            .describe("General matrix multiplication.")
            .set_num_inputs(3)
            .add_argument("A", "Tensor", "The first input tensor.")
            .add_argument("B", "Tensor", "The second input tensor.")
            .add_argument("C", "Tensor", "The third input tensor (bias).")
            .set_attr<std::string>("TAttrs", "GemmAttrs")
            .set_attr<FInferType>("FInferType", GemmInferType)
            .set_attr<FRelayToTE>("FRelayToTE", GemmCompute)
            .set_attr<FHIPDispatch>("FHIPDispatch", GemmDispatch);
        struct Bin { const char* name; int op; };
        for (Bin b : {Bin{"add", 0}, Bin{"subtract", 1}, Bin{"mul", 2}, Bin{"multiply", 2}, Bin{"divide", 3}}) {
            const int op = b.op;
            OpRegEntry::Register(b.name)
                .describe("Elementwise binary operator with numpy-style broadcasting")
                .set_num_inputs(2)
                .add_argument("lhs", "Tensor", "The first input tensor.")
                .add_argument("rhs", "Tensor", "The second input tensor.")
                .set_attr<FInferType>("FInferType", BroadcastInferType)
                .set_attr<FRelayToTE>("FRelayToTE", BinaryCompute(op, b.name))
                .set_attr<bool>("THIPFusableRelu", true)
                .set_attr<FHIPDispatch>("FHIPDispatch", [op](const HIPDispatchContext& c, kxc_hip_plan* p) { return BinaryDispatch(op, c, p); });
        }
        for (const char* fn : {"sqrt", "exp", "log"}) {
            const std::string name = fn;
            OpRegEntry::Register(name)
                .describe("Elementwise " + name)
                .set_num_inputs(1)
                .add_argument("data", "Tensor", "The input tensor.")
                .set_attr<FInferType>("FInferType", UnarySameInferType)
                .set_attr<FRelayToTE>("FRelayToTE", [name](const Attrs&, const Array<te::Tensor>& in, const Type&) {
                    if (in.size() != 1) throw std::runtime_error(name + " expects exactly 1 input");
                    return te::topi::unary_call(in[0], name, "T_" + name);
                });
        }
        OpRegEntry::Register("nn_flatten")
            .describe("Flattens all axes from `axis` on into one")
            .set_num_inputs(1)
            .add_argument("data", "Tensor", "The input tensor.")
            .set_attr<std::string>("TAttrs", "FlattenAttrs")
            .set_attr<FInferType>("FInferType", FlattenInferType)
            .set_attr<FRelayToTE>("FRelayToTE", [](const Attrs&, const Array<te::Tensor>& in, const Type& out) {
                return te::topi::reshape(in[0], out.As<TensorTypeNode>()->shape, "T_flatten");
            })
            .set_attr<bool>("THIPAlias", true);      // row-major view of the same memory: no launch
        OpRegEntry::Register("reshape")
            .describe("Row-major reshape")
            .set_num_inputs(1)
            .add_argument("data", "Tensor", "The input tensor.")
            .set_attr<std::string>("TAttrs", "ReshapeAttrs")
            .set_attr<FInferType>("FInferType", ReshapeInferType)
            .set_attr<FRelayToTE>("FRelayToTE", [](const Attrs&, const Array<te::Tensor>& in, const Type& out) {
                return te::topi::reshape(in[0], out.As<TensorTypeNode>()->shape, "T_reshape");
            })
            .set_attr<bool>("THIPAlias", true);
        OpRegEntry::Register("transpose")
            .describe("Axis permutation")
            .set_num_inputs(1)
            .add_argument("data", "Tensor", "The input tensor.")
            .set_attr<std::string>("TAttrs", "TransposeAttrs")
            .set_attr<FInferType>("FInferType", TransposeInferType)
            .set_attr<FRelayToTE>("FRelayToTE", [](const Attrs& attrs, const Array<te::Tensor>& in, const Type&) {
                const auto* a = attrs.As<TransposeAttrsNode>();
                std::vector<int> axes;
                if (a) for (auto v : a->axes) axes.push_back(static_cast<int>(v));
                if (axes.empty()) for (int i = static_cast<int>(in[0]->shape.size()) - 1; i >= 0; --i) axes.push_back(i);
                return te::topi::transpose(in[0], axes, "T_transpose");
            });
        OpRegEntry::Register("reduce_mean")
            .describe("Mean over the given axes")
            .set_num_inputs(1)
            .add_argument("data", "Tensor", "The input tensor.")
            .set_attr<std::string>("TAttrs", "ReduceMeanAttrs")
            .set_attr<FInferType>("FInferType", ReduceMeanInferType)
            .set_attr<FRelayToTE>("FRelayToTE", [](const Attrs& attrs, const Array<te::Tensor>& in, const Type&) {
                const auto* a = attrs.As<ReduceMeanAttrsNode>();
                if (!a) throw std::runtime_error("reduce_mean expects ReduceMeanAttrs");
                std::vector<int> axes;
                for (auto v : a->axes) axes.push_back(static_cast<int>(v));
                return te::topi::reduce_mean(in[0], axes, a->keepdims != 0, "T_reduce_mean");
            });
        OpRegEntry::Register("softmax")
            .describe("Computes softmax along one tensor axis.")
            .set_num_inputs(1)
            .add_argument("data", "Tensor", "The input tensor.")
            .set_attr<std::string>("TAttrs", "SoftmaxAttrs")
            .set_attr<FInferType>("FInferType", SoftmaxInferType)
            .set_attr<FRelayToTE>("FRelayToTE", [](const Attrs& attrs, const Array<te::Tensor>& in, const Type&) {
                if (in.size() != 1) throw std::runtime_error("softmax expects exactly 1 input(s)");
                if (in[0]->dtype.code != 2) throw std::runtime_error("softmax lowering requires floating-point input");
                const auto* a = attrs.As<SoftmaxAttrsNode>();
                const int nd = static_cast<int>(in[0]->shape.size());
                int64_t axis = a ? a->axis : -1;
                if (axis < 0) axis += nd;
                if (axis < 0 || axis >= nd) throw std::runtime_error("softmax axis out of range");
                return te::topi::softmax(in[0], static_cast<int>(axis), "T_softmax");
            });
        OpRegEntry::Register("cast")
            .describe("Converts the elements to another dtype.")
            .set_num_inputs(1)
            .add_argument("data", "Tensor", "The input tensor.")
            .set_attr<std::string>("TAttrs", "CastAttrs")
            .set_attr<FInferType>("FInferType", CastInferType)
            .set_attr<FRelayToTE>("FRelayToTE", [](const Attrs& attrs, const Array<te::Tensor>& in, const Type&) {
                if (in.size() != 1) throw std::runtime_error("cast expects exactly 1 input(s)");
                const auto* a = attrs.As<CastAttrsNode>();
                if (!a) throw std::runtime_error("cast expects CastAttrs");
                return te::topi::cast(in[0], tir::DTypeFromString(CastDTypeFromCode(a->to)), "T_cast");
            });
        return true;
    }();
    (void)done;
}

}  // namespace relay
}  // namespace kxc
