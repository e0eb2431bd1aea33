// relay.cc -- host NDArray, type printing, operator registry, attribute factories, shape rules and
// the InferType pass.
#include <algorithm>
#include <mutex>
#include <sstream>

#include "kxc/op.h"
#include "kxc/tir.h"

namespace kxc {

std::string TypeToString(const Type& t) {
    if (!t.defined()) return "<none>";
    if (const auto* tt = t.As<TensorTypeNode>()) {
        std::ostringstream os;
        os << "TensorType([";
        for (size_t i = 0; i < tt->shape.size(); ++i) os << (i ? ", " : "") << tt->shape[i];
        os << "], " << tt->dtype << ")";
        return os.str();
    }
    return "<Type>";
}

namespace runtime {
NDArray::NDArray(Array<int64_t> shape, std::string dtype) {
    auto n = std::make_shared<NDArrayNode>();
    n->shape = shape;
    n->dtype = dtype;
    const int64_t count = Product(n->shape);
    const tir::DataType dt = tir::DTypeFromString(dtype);
    n->bytes.assign(static_cast<size_t>(count) * dt.bytes(), 0);
    n->dl_tensor.dtype.code = static_cast<uint8_t>(dt.code);       // 0 int, 1 uint (bool: 1 bit), 2 float
    n->dl_tensor.dtype.bits = static_cast<uint8_t>(dt.bits);
    n->dl_tensor.dtype.lanes = 1;
    ptr_ = n;
}
void NDArray::CopyFromBytes(const void* src, size_t nbytes) {
    if (!ptr_ || nbytes != ptr_->bytes.size()) throw std::runtime_error("NDArray::CopyFromBytes: size mismatch");
    std::memcpy(ptr_->bytes.data(), src, nbytes);
}
void NDArray::CopyToBytes(void* dst, size_t nbytes) const {
    if (!ptr_ || nbytes != ptr_->bytes.size()) throw std::runtime_error("NDArray::CopyToBytes: size mismatch");
    std::memcpy(dst, ptr_->bytes.data(), nbytes);
}
}  // namespace runtime

namespace relay {

// ------------------------------------------------------------------ registry
namespace {
struct Registry {
    std::mutex mu;
    std::unordered_map<std::string, Op> ops;
};
Registry& Reg() {
    static Registry* r = new Registry();   // never destroyed: static registrations may outlive main's statics
    return *r;
}
std::shared_ptr<OpNode> GetOrCreate(const std::string& name) {
    Registry& r = Reg();
    std::lock_guard<std::mutex> lock(r.mu);
    auto it = r.ops.find(name);
    if (it == r.ops.end()) {
        auto n = std::make_shared<OpNode>();
        n->name = name;
        it = r.ops.emplace(name, Op(n)).first;
    }
    return std::static_pointer_cast<OpNode>(it->second.shared());
}
}  // namespace

const Op& Op::Get(const std::string& name) {
    EnsureBuiltinOpsRegistered();
    GetOrCreate(name);
    Registry& r = Reg();
    std::lock_guard<std::mutex> lock(r.mu);
    return r.ops.find(name)->second;
}

OpRegEntry OpRegEntry::Register(const std::string& name) { return OpRegEntry(GetOrCreate(name)); }

// ------------------------------------------------------------------ attribute factories
Conv2DAttrs Conv2DAttrs::Create(std::vector<int64_t> strides, std::vector<int64_t> padding, std::vector<int64_t> dilation,
                                int groups, int channels, std::vector<int64_t> kernel_size, std::string data_layout,
                                std::string kernel_layout, std::string out_layout, std::string out_dtype) {
    auto n = std::make_shared<Conv2DAttrsNode>();
    n->strides = std::move(strides); n->padding = std::move(padding); n->dilation = std::move(dilation);
    n->groups = groups; n->channels = channels; n->kernel_size = std::move(kernel_size);
    n->data_layout = std::move(data_layout); n->kernel_layout = std::move(kernel_layout);
    n->out_layout = std::move(out_layout); n->out_dtype = std::move(out_dtype);
    return Conv2DAttrs(n);
}
MaxPool2DAttrs MaxPool2DAttrs::Create(std::vector<int64_t> strides, std::vector<int64_t> padding,
                                      std::vector<int64_t> dilation, std::vector<int64_t> pool_size, std::string layout,
                                      bool ceil_mode) {
    auto n = std::make_shared<MaxPool2DAttrsNode>();
    n->strides = std::move(strides); n->padding = std::move(padding); n->dilation = std::move(dilation);
    n->pool_size = std::move(pool_size); n->layout = std::move(layout); n->ceil_mode = ceil_mode;
    return MaxPool2DAttrs(n);
}
DenseAttrs DenseAttrs::Create(int64_t units, std::string out_dtype) {
    auto n = std::make_shared<DenseAttrsNode>();
    n->units = units; n->out_dtype = std::move(out_dtype);
    return DenseAttrs(n);
}
GemmAttrs GemmAttrs::Create(float alpha, float beta, int transA, int transB) {
    auto n = std::make_shared<GemmAttrsNode>();
    n->alpha = alpha; n->beta = beta; n->transA = transA; n->transB = transB;
    return GemmAttrs(n);
}
FlattenAttrs FlattenAttrs::Create(int axis) {
    auto n = std::make_shared<FlattenAttrsNode>();
    n->axis = axis;
    return FlattenAttrs(n);
}
ReshapeAttrs ReshapeAttrs::Create(std::vector<int64_t> newshape) {
    auto n = std::make_shared<ReshapeAttrsNode>();
    n->newshape = std::move(newshape);
    return ReshapeAttrs(n);
}
TransposeAttrs TransposeAttrs::Create(std::vector<int64_t> axes) {
    auto n = std::make_shared<TransposeAttrsNode>();
    n->axes = std::move(axes);
    return TransposeAttrs(n);
}
ReduceMeanAttrs ReduceMeanAttrs::Create(std::vector<int64_t> axes, int keepdims) {
    auto n = std::make_shared<ReduceMeanAttrsNode>();
    n->axes = std::move(axes); n->keepdims = keepdims;
    return ReduceMeanAttrs(n);
}

SoftmaxAttrs SoftmaxAttrs::Create(int64_t axis) {
    auto n = std::make_shared<SoftmaxAttrsNode>();
    n->axis = axis;
    return SoftmaxAttrs(n);
}
QnnConv2DAttrs QnnConv2DAttrs::Create(std::vector<int64_t> strides, std::vector<int64_t> padding, bool relu, double res_mult) {
    auto n = std::make_shared<QnnConv2DAttrsNode>();
    n->strides = std::move(strides); n->padding = std::move(padding); n->relu = relu; n->res_mult = res_mult;
    return QnnConv2DAttrs(n);
}
QnnQuantizeAttrs QnnQuantizeAttrs::Create(double scale) {
    auto n = std::make_shared<QnnQuantizeAttrsNode>();
    n->scale = scale;
    return QnnQuantizeAttrs(n);
}
QnnRequantAttrs QnnRequantAttrs::Create(double mult) {
    auto n = std::make_shared<QnnRequantAttrsNode>();
    n->mult = mult;
    return QnnRequantAttrs(n);
}
CastAttrs CastAttrs::Create(int to) {
    auto n = std::make_shared<CastAttrsNode>();
    n->to = to;
    return CastAttrs(n);
}
std::string CastDTypeFromCode(int code) {
    static const char* const names[] = {"float32", "int32", "int64", "float64", "bool", "int8", "uint8"};
    if (code < 0 || code > 6) throw std::runtime_error("cast has unsupported dtype code: " + std::to_string(code));
    return names[code];
}

// ------------------------------------------------------------------ shape rules
namespace {
const TensorTypeNode* RequireTensor(const std::string& op, const Type& t, const char* what) {
    const auto* tt = t.As<TensorTypeNode>();
    if (!tt) throw std::runtime_error(op + " expects a tensor for " + what);
    return tt;
}
void RequireArity(const std::string& op, const Array<Type>& in, size_t n) {
    if (in.size() != n) throw std::runtime_error(op + " expects exactly " + std::to_string(n) + " input" + (n == 1 ? "" : "s"));
}
void RequireSameDType(const std::string& op, const TensorTypeNode* a, const TensorTypeNode* b) {
    if (a->dtype != b->dtype) throw std::runtime_error(op + " expects inputs of the same dtype");
}
std::vector<int64_t> ReadPair(const std::vector<int64_t>& v, int64_t d) {
    if (v.empty()) return {d, d};
    if (v.size() == 1) return {v[0], v[0]};
    return {v[0], v[1]};
}
std::vector<int64_t> ReadPadding(const std::vector<int64_t>& v) {
    if (v.empty()) return {0, 0, 0, 0};
    if (v.size() == 1) return {v[0], v[0], v[0], v[0]};
    if (v.size() == 2) return {v[0], v[1], v[0], v[1]};
    return {v[0], v[1], v[2], v[3]};
}
// src/relay/type_infer.cc:166-184
int64_t WindowOutputDim(const std::string& op, int64_t input, int64_t kernel, int64_t pad_before, int64_t pad_after,
                        int64_t stride, int64_t dilation, bool ceil_mode) {
    if (stride <= 0 || dilation <= 0) throw std::runtime_error(op + " stride and dilation must be positive");
    const int64_t eff = dilation * (kernel - 1) + 1;
    const int64_t num = input + pad_before + pad_after - eff;
    if (num < 0) throw std::runtime_error(op + " window is larger than input");
    return ceil_mode ? (num + stride - 1) / stride + 1 : num / stride + 1;
}
std::vector<int64_t> BroadcastShape(const std::string& op, const std::vector<int64_t>& a, const std::vector<int64_t>& b) {
    const size_t n = std::max(a.size(), b.size());
    std::vector<int64_t> out(n);
    for (size_t i = 0; i < n; ++i) {
        const int64_t da = i >= n - a.size() ? a[i - (n - a.size())] : 1;
        const int64_t db = i >= n - b.size() ? b[i - (n - b.size())] : 1;
        if (da != db && da != 1 && db != 1) throw std::runtime_error(op + " shapes are not broadcast-compatible");
        out[i] = da == 1 ? db : da;
    }
    return out;
}
}  // namespace

Type Conv2DInferType(const Attrs& attrs, const Array<Type>& in) {
    if (in.size() != 2 && in.size() != 3) throw std::runtime_error("nn_conv2d expects data, weight[, bias]");
    const auto* data = RequireTensor("nn_conv2d", in[0], "data");
    const auto* weight = RequireTensor("nn_conv2d", in[1], "weight");
    RequireSameDType("nn_conv2d", data, weight);
    if (data->shape.size() != 4 || weight->shape.size() != 4)
        throw std::runtime_error("nn_conv2d expects NCHW/OIHW rank-4 tensors");
    const auto* a = attrs.As<Conv2DAttrsNode>();
    if (a && !a->data_layout.empty() && a->data_layout != "NCHW")
        throw std::runtime_error("nn_conv2d only supports NCHW data layout in type inference");
    if (a && !a->kernel_layout.empty() && a->kernel_layout != "OIHW")
        throw std::runtime_error("nn_conv2d only supports OIHW kernel layout in type inference");
    const int64_t groups = a ? std::max<int64_t>(1, a->groups) : 1;
    if (data->shape[1] != weight->shape[1] * groups) throw std::runtime_error("nn_conv2d input channel mismatch");
    const auto strides = ReadPair(a ? a->strides : std::vector<int64_t>{}, 1);
    const auto dilation = ReadPair(a ? a->dilation : std::vector<int64_t>{}, 1);
    const auto padding = ReadPadding(a ? a->padding : std::vector<int64_t>{});
    if (a && !a->kernel_size.empty()) {
        const auto ks = ReadPair(a->kernel_size, 0);
        if (ks[0] != weight->shape[2] || ks[1] != weight->shape[3])
            throw std::runtime_error("nn_conv2d kernel_size does not match weight shape");
    }
    const int64_t channels = a && a->channels > 0 ? a->channels : weight->shape[0];
    if (in.size() == 3) {
        const auto* bias = RequireTensor("nn_conv2d", in[2], "bias");
        RequireSameDType("nn_conv2d", data, bias);
        if (bias->shape.size() != 1 || bias->shape[0] != channels)
            throw std::runtime_error("nn_conv2d bias must be rank-1 with output channels");
    }
    const int64_t oh = WindowOutputDim("nn_conv2d", data->shape[2], weight->shape[2], padding[0], padding[2], strides[0], dilation[0], false);
    const int64_t ow = WindowOutputDim("nn_conv2d", data->shape[3], weight->shape[3], padding[1], padding[3], strides[1], dilation[1], false);
    const std::string dtype = a && !a->out_dtype.empty() ? a->out_dtype : data->dtype;
    return TensorType({data->shape[0], channels, oh, ow}, dtype);
}

namespace {
void RequireDType(const char* op, const TensorTypeNode* t, const char* what, const char* dtype) {
    if (t->dtype != dtype) throw std::runtime_error(std::string(op) + " expects " + what + " of dtype " + dtype + ", got " + t->dtype);
}
void RequireChannelVector(const char* op, const TensorTypeNode* t, const char* what, int64_t channels) {
    if (t->shape.size() != 1 || t->shape[0] != channels)
        throw std::runtime_error(std::string(op) + " " + what + " must be rank-1 with one entry per output channel");
}
}  // namespace

Type QnnConv2DInferType(const Attrs& attrs, const Array<Type>& in) {
    if (in.size() != 4 && in.size() != 5) throw std::runtime_error("qnn_conv2d expects data, weight, bias, mult[, residual]");
    const auto* a = attrs.As<QnnConv2DAttrsNode>();
    if (!a) throw std::runtime_error("qnn_conv2d expects QnnConv2DAttrs");
    const auto* data = RequireTensor("qnn_conv2d", in[0], "data");
    const auto* weight = RequireTensor("qnn_conv2d", in[1], "weight");
    const auto* bias = RequireTensor("qnn_conv2d", in[2], "bias");
    const auto* mult = RequireTensor("qnn_conv2d", in[3], "mult");
    RequireDType("qnn_conv2d", data, "data", "int8"); RequireDType("qnn_conv2d", weight, "weight", "int8");
    RequireDType("qnn_conv2d", bias, "bias", "int32"); RequireDType("qnn_conv2d", mult, "mult", "float32");
    if (data->shape.size() != 4 || weight->shape.size() != 4) throw std::runtime_error("qnn_conv2d expects NCHW/OIHW rank-4 tensors");
    if (data->shape[1] != weight->shape[1]) throw std::runtime_error("qnn_conv2d input channel mismatch");
    RequireChannelVector("qnn_conv2d", bias, "bias", weight->shape[0]);
    RequireChannelVector("qnn_conv2d", mult, "mult", weight->shape[0]);
    const auto strides = ReadPair(a->strides, 1);
    const auto pads = ReadPair(a->padding, 0);
    const int64_t oh = WindowOutputDim("qnn_conv2d", data->shape[2], weight->shape[2], pads[0], pads[0], strides[0], 1, false);
    const int64_t ow = WindowOutputDim("qnn_conv2d", data->shape[3], weight->shape[3], pads[1], pads[1], strides[1], 1, false);
    const std::vector<int64_t> oshape = {data->shape[0], weight->shape[0], oh, ow};
    if (in.size() == 5) {
        const auto* res = RequireTensor("qnn_conv2d", in[4], "residual");
        RequireDType("qnn_conv2d", res, "residual", "int8");
        if (res->shape != oshape) throw std::runtime_error("qnn_conv2d residual must have the output's shape");
    }
    return TensorType(oshape, "int8");
}

Type QnnDenseInferType(const Attrs&, const Array<Type>& in) {
    RequireArity("qnn_dense", in, 4);
    const auto* data = RequireTensor("qnn_dense", in[0], "data");
    const auto* weight = RequireTensor("qnn_dense", in[1], "weight");
    const auto* bias = RequireTensor("qnn_dense", in[2], "bias");
    const auto* mult = RequireTensor("qnn_dense", in[3], "mult");
    RequireDType("qnn_dense", data, "data", "int8"); RequireDType("qnn_dense", weight, "weight", "int8");
    RequireDType("qnn_dense", bias, "bias", "int32"); RequireDType("qnn_dense", mult, "mult", "float32");
    if (data->shape.size() != 2 || weight->shape.size() != 2) throw std::runtime_error("qnn_dense expects rank-2 data and weight");
    if (data->shape[1] != weight->shape[1]) throw std::runtime_error("qnn_dense input dimension mismatch");
    RequireChannelVector("qnn_dense", bias, "bias", weight->shape[0]);
    RequireChannelVector("qnn_dense", mult, "mult", weight->shape[0]);
    return TensorType({data->shape[0], weight->shape[0]}, "float32");
}

Type QnnGlobalAvgPool2DInferType(const Attrs& attrs, const Array<Type>& in) {
    RequireArity("qnn_global_avg_pool2d", in, 1);
    const auto* a = attrs.As<QnnRequantAttrsNode>();
    if (!a || !(a->mult > 0.0)) throw std::runtime_error("qnn_global_avg_pool2d expects QnnRequantAttrs with a positive multiplier");
    const auto* x = RequireTensor("qnn_global_avg_pool2d", in[0], "data");
    RequireDType("qnn_global_avg_pool2d", x, "data", "int8");
    if (x->shape.size() != 4) throw std::runtime_error("qnn_global_avg_pool2d expects an NCHW rank-4 input");
    return TensorType({x->shape[0], x->shape[1], 1, 1}, "int8");
}

int64_t HIPLayoutBytes(const Type& t, int layout) {
    const auto* tt = t.As<TensorTypeNode>();
    if (!tt) throw std::runtime_error("HIPLayoutBytes: not a tensor type");
    const int64_t elem = tir::DTypeFromString(tt->dtype).bytes();
    if (layout == kHIPLayoutPlain || layout == kHIPLayoutAny) return Product(tt->shape) * elem;
    if (tt->shape.size() != 4 || elem != 1) throw std::runtime_error("a channel-blocked layout needs a rank-4 int8 tensor");
    const int64_t cbytes = layout == kHIPLayoutC16 ? (tt->shape[1] + 15) / 16 * 16 : 4;
    if (layout == kHIPLayoutC4 && tt->shape[1] > 4) throw std::runtime_error("the 4-channel layout holds at most four channels");
    return tt->shape[0] * cbytes * tt->shape[2] * tt->shape[3];
}

Type QnnQuantizeInferType(const Attrs& attrs, const Array<Type>& in) {
    RequireArity("qnn_quantize", in, 1);
    const auto* a = attrs.As<QnnQuantizeAttrsNode>();
    if (!a || !(a->scale > 0.0)) throw std::runtime_error("qnn_quantize expects QnnQuantizeAttrs with a positive scale");
    const auto* x = RequireTensor("qnn_quantize", in[0], "data");
    RequireDType("qnn_quantize", x, "data", "float32");
    return TensorType(x->shape, "int8");
}

Type Pool2DInferType(const Attrs& attrs, const Array<Type>& in) {
    RequireArity("pool2d", in, 1);
    const auto* data = RequireTensor("pool2d", in[0], "data");
    if (data->shape.size() != 4) throw std::runtime_error("pool2d expects NCHW rank-4 input");
    const auto* a = attrs.As<MaxPool2DAttrsNode>();
    if (a && !a->layout.empty() && a->layout != "NCHW") throw std::runtime_error("pool2d only supports NCHW layout in type inference");
    const auto ps = ReadPair(a ? a->pool_size : std::vector<int64_t>{}, 1);
    const auto st = ReadPair(a ? a->strides : std::vector<int64_t>{}, 1);
    const auto dl = ReadPair(a ? a->dilation : std::vector<int64_t>{}, 1);
    const auto pd = ReadPadding(a ? a->padding : std::vector<int64_t>{});
    const bool ceil_mode = a && a->ceil_mode;
    const int64_t oh = WindowOutputDim("pool2d", data->shape[2], ps[0], pd[0], pd[2], st[0], dl[0], ceil_mode);
    const int64_t ow = WindowOutputDim("pool2d", data->shape[3], ps[1], pd[1], pd[3], st[1], dl[1], ceil_mode);
    return TensorType({data->shape[0], data->shape[1], oh, ow}, data->dtype);
}

Type GlobalAvgPool2DInferType(const Attrs&, const Array<Type>& in) {
    RequireArity("nn_global_avg_pool2d", in, 1);
    const auto* data = RequireTensor("nn_global_avg_pool2d", in[0], "data");
    if (data->shape.size() != 4) throw std::runtime_error("nn_global_avg_pool2d expects NCHW rank-4 input");
    return TensorType({data->shape[0], data->shape[1], 1, 1}, data->dtype);
}

Type DenseInferType(const Attrs& attrs, const Array<Type>& in) {
    RequireArity("nn_dense", in, 2);
    const auto* data = RequireTensor("nn_dense", in[0], "data");
    const auto* weight = RequireTensor("nn_dense", in[1], "weight");
    RequireSameDType("nn_dense", data, weight);
    if (data->shape.size() != 2 || weight->shape.size() != 2) throw std::runtime_error("nn_dense expects rank-2 data and weight");
    if (data->shape[1] != weight->shape[1]) throw std::runtime_error("nn_dense input dimension mismatch");
    const auto* a = attrs.As<DenseAttrsNode>();
    const int64_t units = a && a->units > 0 ? a->units : weight->shape[0];
    return TensorType({data->shape[0], units}, a && !a->out_dtype.empty() ? a->out_dtype : data->dtype);
}

Type GemmInferType(const Attrs& attrs, const Array<Type>& in) {
    RequireArity("nn_gemm", in, 3);
    const auto* A = RequireTensor("nn_gemm", in[0], "A");
    const auto* B = RequireTensor("nn_gemm", in[1], "B");
    const auto* C = RequireTensor("nn_gemm", in[2], "C");
    RequireSameDType("nn_gemm", A, B);
    RequireSameDType("nn_gemm", A, C);
    if (A->shape.size() != 2 || B->shape.size() != 2) throw std::runtime_error("nn_gemm expects rank-2 A and B");
    const auto* a = attrs.As<GemmAttrsNode>();
    const bool ta = a && a->transA != 0, tb = a && a->transB != 0;
    const int64_t m = ta ? A->shape[1] : A->shape[0], ka = ta ? A->shape[0] : A->shape[1];
    const int64_t kb = tb ? B->shape[1] : B->shape[0], n = tb ? B->shape[0] : B->shape[1];
    if (ka != kb) throw std::runtime_error("nn_gemm reduction dimension mismatch");
    BroadcastShape("nn_gemm bias", C->shape, {m, n});
    return TensorType({m, n}, A->dtype);
}

Type MatmulInferType(const Attrs&, const Array<Type>& in) {
    RequireArity("matmul", in, 2);
    const auto* A = RequireTensor("matmul", in[0], "lhs");
    const auto* B = RequireTensor("matmul", in[1], "rhs");
    RequireSameDType("matmul", A, B);
    if (A->shape.size() != 2 || B->shape.size() != 2) throw std::runtime_error("matmul expects rank-2 inputs");
    if (A->shape[1] != B->shape[0]) throw std::runtime_error("matmul reduction dimension mismatch");
    return TensorType({A->shape[0], B->shape[1]}, A->dtype);
}

Type UnarySameInferType(const Attrs&, const Array<Type>& in) {
    RequireArity("unary op", in, 1);
    const auto* x = RequireTensor("unary op", in[0], "data");
    return TensorType(x->shape, x->dtype);
}

Type BroadcastInferType(const Attrs&, const Array<Type>& in) {
    RequireArity("broadcast op", in, 2);
    const auto* a = RequireTensor("broadcast op", in[0], "lhs");
    const auto* b = RequireTensor("broadcast op", in[1], "rhs");
    RequireSameDType("broadcast op", a, b);
    return TensorType(BroadcastShape("broadcast op", a->shape, b->shape), a->dtype);
}

Type FlattenInferType(const Attrs& attrs, const Array<Type>& in) {
    RequireArity("nn_flatten", in, 1);
    const auto* x = RequireTensor("nn_flatten", in[0], "data");
    const auto* a = attrs.As<FlattenAttrsNode>();
    int axis = a ? a->axis : 1;
    if (axis < 0) axis += static_cast<int>(x->shape.size());
    if (axis < 0 || axis > static_cast<int>(x->shape.size())) throw std::runtime_error("nn_flatten axis out of range");
    int64_t outer = 1, inner = 1;
    for (int i = 0; i < static_cast<int>(x->shape.size()); ++i) (i < axis ? outer : inner) *= x->shape[i];
    return TensorType({outer, inner}, x->dtype);
}

Type ReshapeInferType(const Attrs& attrs, const Array<Type>& in) {
    RequireArity("reshape", in, 1);
    const auto* x = RequireTensor("reshape", in[0], "data");
    const auto* a = attrs.As<ReshapeAttrsNode>();
    if (!a) throw std::runtime_error("reshape expects ReshapeAttrs");
    std::vector<int64_t> shape = a->newshape;
    const int64_t total = Product(x->shape);
    int64_t known = 1;
    int infer = -1;
    for (size_t i = 0; i < shape.size(); ++i) {
        if (shape[i] == -1) { if (infer >= 0) throw std::runtime_error("reshape allows a single -1"); infer = static_cast<int>(i); }
        else known *= shape[i];
    }
    if (infer >= 0) shape[infer] = known ? total / known : 0;
    if (Product(shape) != total) throw std::runtime_error("reshape element count mismatch");
    return TensorType(shape, x->dtype);
}

Type TransposeInferType(const Attrs& attrs, const Array<Type>& in) {
    RequireArity("transpose", in, 1);
    const auto* x = RequireTensor("transpose", in[0], "data");
    const auto* a = attrs.As<TransposeAttrsNode>();
    std::vector<int64_t> axes = a ? a->axes : std::vector<int64_t>{};
    if (axes.empty()) for (int i = static_cast<int>(x->shape.size()) - 1; i >= 0; --i) axes.push_back(i);
    if (axes.size() != x->shape.size()) throw std::runtime_error("transpose axes rank mismatch");
    std::vector<int64_t> shape;
    for (auto ax : axes) {
        if (ax < 0 || ax >= static_cast<int64_t>(x->shape.size())) throw std::runtime_error("transpose axis out of range");
        shape.push_back(x->shape[ax]);
    }
    return TensorType(shape, x->dtype);
}

Type ReduceMeanInferType(const Attrs& attrs, const Array<Type>& in) {
    RequireArity("reduce_mean", in, 1);
    const auto* x = RequireTensor("reduce_mean", in[0], "data");
    const auto* a = attrs.As<ReduceMeanAttrsNode>();
    if (!a) throw std::runtime_error("reduce_mean expects ReduceMeanAttrs");
    const int nd = static_cast<int>(x->shape.size());
    std::vector<bool> red(nd, false);
    for (auto ax : a->axes) {
        int v = static_cast<int>(ax < 0 ? ax + nd : ax);
        if (v < 0 || v >= nd) throw std::runtime_error("reduce_mean axis out of range");
        red[v] = true;
    }
    std::vector<int64_t> shape;
    for (int i = 0; i < nd; ++i) {
        if (!red[i]) shape.push_back(x->shape[i]);
        else if (a->keepdims) shape.push_back(1);
    }
    return TensorType(shape, x->dtype);
}

Type SoftmaxInferType(const Attrs& attrs, const Array<Type>& in) {
    RequireArity("softmax", in, 1);
    const auto* x = RequireTensor("softmax", in[0], "data");
    const auto* a = attrs.As<SoftmaxAttrsNode>();
    const int nd = static_cast<int>(x->shape.size());
    int64_t axis = a ? a->axis : -1;
    if (axis < 0) axis += nd;
    if (axis < 0 || axis >= nd) throw std::runtime_error("softmax axis out of range");
    return TensorType(x->shape, x->dtype);
}

Type CastInferType(const Attrs& attrs, const Array<Type>& in) {
    RequireArity("cast", in, 1);
    const auto* x = RequireTensor("cast", in[0], "data");
    const auto* a = attrs.As<CastAttrsNode>();
    return TensorType(x->shape, a ? CastDTypeFromCode(a->to) : x->dtype);
}

// ------------------------------------------------------------------ InferType
namespace {
void InferExpr(const Expr& e, std::unordered_map<const RelayExprNode*, bool>* done) {
    if (!e.defined() || done->count(e.get())) return;
    (*done)[e.get()] = true;
    if (const auto* v = e.As<VarNode>()) {
        if (!v->type_annotation.defined()) throw std::runtime_error("InferType: variable '" + v->vid->name_hint + "' has no type annotation");
        v->checked_type_ = v->type_annotation;
    } else if (const auto* c = e.As<ConstantNode>()) {
        c->checked_type_ = TensorType(c->data->shape, c->data->dtype);
    } else if (const auto* call = e.As<CallNode>()) {
        Array<Type> in;
        for (const auto& arg : call->args) {
            InferExpr(arg, done);
            in.push_back(arg.checked_type());
        }
        const auto* op = call->op.As<OpNode>();
        if (!op) throw std::runtime_error("InferType: Call.op is not an operator");
        if (op->num_inputs >= 0 && static_cast<int>(call->args.size()) != op->num_inputs)
            throw std::runtime_error(op->name + " expects " + std::to_string(op->num_inputs) + " inputs, got " +
                                     std::to_string(call->args.size()));
        auto it = op->attrs.find("FInferType");
        if (it == op->attrs.end()) throw std::runtime_error("No FInferType registered for op: " + op->name);
        const auto* fn = std::any_cast<FInferType>(&it->second);
        if (!fn) throw std::runtime_error("Bad FInferType type for op: " + op->name);
        call->checked_type_ = (*fn)(call->attrs, in);
    } else if (e.As<OpNode>()) {
        // operators carry no type
    } else {
        throw std::runtime_error("InferType: unsupported Relay node");
    }
}
}  // namespace

Function InferTypePass(const Function& f) {
    if (!f.defined()) throw std::runtime_error("InferType: undefined function");
    std::unordered_map<const RelayExprNode*, bool> done;
    for (const auto& p : f->params) InferExpr(p, &done);
    InferExpr(f->body, &done);
    f->checked_type_ = f->body.checked_type();
    return f;
}

// ---------------------------------------------------------------- SplitBatch
namespace {
struct SplitState {
    int64_t batch = 0;
    std::unordered_map<const RelayExprNode*, bool> batched;     // value carries the batch on axis 0
    std::unordered_map<const RelayExprNode*, Expr> clone;
};

const TensorTypeNode* TTy(const Expr& e) { return e.checked_type().As<TensorTypeNode>(); }

// an operand without the batch beside a batched one of rank `rank`: it must broadcast along axis 0
bool BroadcastsOverBatch(const Expr& shared, size_t rank) {
    const auto* t = TTy(shared);
    return t && (t->shape.size() < rank || (t->shape.size() == rank && t->shape[0] == 1));
}

// Clones `e` for one share of the batch; false when the graph is not separable.
bool SplitExpr(const Expr& e, SplitState* st, Expr* out) {
    auto it = st->clone.find(e.get());
    if (it != st->clone.end()) { *out = it->second; return true; }
    if (e.As<ConstantNode>()) {
        st->batched[e.get()] = false;
        st->clone[e.get()] = e;          // shared between the shares
        *out = e;
        return true;
    }
    const auto* call = e.As<CallNode>();
    const auto* op = call ? call->op.As<OpNode>() : nullptr;
    if (!op || !TTy(e)) return false;
    Array<Expr> args;
    std::vector<bool> b;
    for (const auto& a : call->args) {
        Expr c;
        if (!SplitExpr(a, st, &c)) return false;
        args.push_back(c);
        b.push_back(st->batched.at(a.get()));
    }
    const std::string& name = op->name;
    const size_t n = b.size();
    bool any = false;
    for (bool x : b) any = any || x;
    bool result_batched = false;
    if (!any) {
        result_batched = false;        // no operand depends on the batch: every share computes the same value
    } else {
        const auto* t0 = TTy(call->args[0]);
        if (!t0 || t0->shape.empty()) return false;
        const size_t rank0 = t0->shape.size();
        auto only_first = [&]() -> bool { for (size_t i = 1; i < n; ++i) if (b[i]) return false; return b[0]; };
        if (name == "nn_conv2d" || name == "nn_dense" || name == "matmul" || name == "qnn_dense") {
            if (!only_first()) return false;
        } else if (name == "qnn_conv2d") {
            // data [, weight, bias, mult] [, residual of the output's shape]
            for (size_t i = 1; i < n; ++i) if (b[i] && i != 4) return false;
            if (!b[0] || (n == 5 && !b[4])) return false;
        } else if (name == "nn_gemm") {
            const auto* g = call->attrs.As<GemmAttrsNode>();
            if (!only_first() || (g && g->transA != 0)) return false;
            if (n == 3 && !BroadcastsOverBatch(call->args[2], 2)) return false;
        } else if (name == "nn_relu" || name == "sqrt" || name == "exp" || name == "log" || name == "cast" ||
                   name == "qnn_quantize" || name == "nn_max_pool2d" || name == "nn_avg_pool2d" ||
                   name == "nn_global_avg_pool2d" || name == "qnn_global_avg_pool2d") {
            if (n != 1) return false;
        } else if (name == "add" || name == "subtract" || name == "mul" || name == "multiply" || name == "divide") {
            if (n != 2) return false;
            const auto* t1 = TTy(call->args[1]);
            if (!t1) return false;
            if (b[0] && b[1]) {
                if (rank0 != t1->shape.size() || t0->shape[0] != st->batch || t1->shape[0] != st->batch) return false;
            } else {
                const Expr& shared = b[0] ? call->args[1] : call->args[0];
                const size_t rank = b[0] ? rank0 : t1->shape.size();
                if (!BroadcastsOverBatch(shared, rank)) return false;
            }
        } else if (name == "nn_flatten") {
            const auto* a = call->attrs.As<FlattenAttrsNode>();
            if (!a || a->axis < 1) return false;
        } else if (name == "softmax") {
            const auto* a = call->attrs.As<SoftmaxAttrsNode>();
            const int64_t axis = a ? (a->axis < 0 ? a->axis + static_cast<int64_t>(rank0) : a->axis) : static_cast<int64_t>(rank0) - 1;
            if (axis == 0) return false;
        } else if (name == "reduce_mean") {
            const auto* a = call->attrs.As<ReduceMeanAttrsNode>();
            if (!a || a->axes.empty()) return false;
            for (int64_t ax : a->axes) if (ax == 0 || ax + static_cast<int64_t>(rank0) == 0) return false;
        } else if (name == "transpose") {
            const auto* a = call->attrs.As<TransposeAttrsNode>();
            if (!a || a->axes.empty() || a->axes[0] != 0) return false;
        } else {
            return false;      // (reshape and operators this list does not know keep the batch whole)
        }
        const auto* to = TTy(e);
        if (to->shape.empty() || to->shape[0] != st->batch) return false;
        result_batched = true;
    }
    Call c(call->op, args, call->attrs);
    st->batched[e.get()] = result_batched;
    st->clone[e.get()] = c;
    *out = c;
    return true;
}
}  // namespace

Function SplitBatch(const Function& f, int lanes) {
    if (!f.defined() || lanes < 2 || f->params.empty()) return Function();
    const auto* t0 = f->params[0].checked_type().As<TensorTypeNode>();
    if (!t0 || t0->shape.empty() || t0->shape[0] < lanes || t0->shape[0] % lanes != 0) return Function();
    SplitState st;
    st.batch = t0->shape[0];
    Array<Var> params;
    for (size_t i = 0; i < f->params.size(); ++i) {
        const Var& p = f->params[i];
        const auto* t = p.checked_type().As<TensorTypeNode>();
        if (!t) return Function();
        std::vector<int64_t> shape = t->shape;
        if (i == 0) shape[0] /= lanes;
        Var v(p->vid->name_hint, TensorType(shape, t->dtype));
        params.push_back(v);
        st.batched[p.get()] = i == 0;
        st.clone[p.get()] = v;
    }
    Expr body;
    if (!SplitExpr(f->body, &st, &body) || !st.batched.at(f->body.get())) return Function();
    Function share(params, body);
    try {
        share = InferTypePass(share);
    } catch (const std::exception&) {
        return Function();
    }
    const auto* full = f->body.checked_type().As<TensorTypeNode>();
    const auto* part = share->body.checked_type().As<TensorTypeNode>();
    if (!full || !part || full->shape.size() != part->shape.size() || part->shape[0] * lanes != full->shape[0]) return Function();
    for (size_t i = 1; i < full->shape.size(); ++i)
        if (full->shape[i] != part->shape[i]) return Function();
    return share;
}

}  // namespace relay
}  // namespace kxc
