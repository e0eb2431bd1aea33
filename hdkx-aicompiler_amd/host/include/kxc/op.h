// op.h -- operator registry, attribute types and the per-operator hooks.
//
// Same registration DSL and hook types as the reference (include/relay/op_macros.h:16-40,
// include/relay/op_attr_types.h:17-23, include/relay/op.h:29-54,104-382):
//   KXC_REGISTER_OP(nn_conv2d).describe(..).set_num_inputs(-1).add_argument(..)
//       .set_attr<FInferType>("FInferType", ..).set_attr<FRelayToTE>("FRelayToTE", ..)
// plus one hook of this backend registered alongside them: "FHIPDispatch", which maps a call (and
// what was fused into it) to a hand-written gfx950 kernel of the C-ABI library.  Operators without
// it go through FRelayToTE -> TIR -> the HIP code generator.
#pragma once

#include <any>
#include <functional>
#include <unordered_map>

#include "kxc/relay.h"
#include "kxc/te.h"

struct kxc_hip_plan;   // C ABI (kxc_hip.h)

namespace kxc {
namespace relay {

struct ArgumentInfo {
    std::string name, type, description;
};

struct OpNode : RelayExprNode {
    std::string name;
    std::string description;
    Array<ArgumentInfo> arguments;
    int num_inputs = -1;
    std::unordered_map<std::string, std::any> attrs;
};

class Op : public Expr {
public:
    Op() = default;
    explicit Op(std::shared_ptr<OpNode> n) { ptr_ = n; }
    const OpNode* operator->() const { return static_cast<const OpNode*>(ptr_.get()); }
    // Looks the operator up in the global table, creating an empty entry if absent (src/base/op.cc:19-39).
    static const Op& Get(const std::string& name);
};

using FInferType = std::function<Type(const Attrs&, const Array<Type>&)>;
using FRelayToTE = std::function<te::Tensor(const Attrs&, const Array<te::Tensor>&, const Type&)>;

// ---- this backend's hook -------------------------------------------------------------------
// A device buffer operand of a launch: a packed argument or a workspace slot.
struct HIPBuffer {
    int kind = 2;            // KXC_HIP_BUF_ARG / _WORKSPACE / _NONE
    int64_t index_or_offset = 0;
};
// How a rank-4 int8 activation lies in memory between two launches.  kHIPLayoutPlain is the tensor type's own
// row-major (NCHW) layout, the only one function parameters, constants and the result ever have; kHIPLayoutC16
// stores [N][ceil(C/16)][H][W][16] (one pixel's 16 channels contiguous: the operand slice of the int8 matrix
// instruction), kHIPLayoutC4 [N][H][W][4] (inputs of at most four channels).  An operator's "FHIPLayoutQuery" says
// which layouts its hand-written kernel takes and writes for a call; the graph pass places a converter on every
// edge whose two ends disagree.  kHIPLayoutAny (in `offered` only) marks an input whose producer writes whatever
// its consumers ask for.
enum HIPLayout : int { kHIPLayoutAny = -1, kHIPLayoutPlain = 0, kHIPLayoutC16 = 1, kHIPLayoutC4 = 2 };
struct HIPLayoutChoice {
    std::vector<int> inputs;             // one per input; empty = all plain
    int output = kHIPLayoutPlain;
};
// offered[i]: the layout input i exists in (kHIPLayoutAny: the producer follows this call).  input_argument[i]: the
// input is a packed argument (a parameter or a constant), i.e. readable before the first launch of a run.
using FHIPLayoutQuery = std::function<HIPLayoutChoice(const Attrs& attrs, const Array<Type>& input_types, const Type& out_type,
                                                      const std::vector<int>& offered, const std::vector<bool>& input_argument)>;
// Bytes of a tensor of type `t` in layout `layout`.
int64_t HIPLayoutBytes(const Type& t, int layout);

struct HIPDispatchContext {
    Attrs attrs;
    Array<Type> input_types;
    Type out_type;
    Array<HIPBuffer> inputs;
    HIPBuffer output;
    // the layouts the inputs arrive in and the output is expected in: what the operator's FHIPLayoutQuery chose
    // (all plain for operators without one)
    std::vector<int> input_layouts;
    int output_layout = kHIPLayoutPlain;
    int pair_output_layout = kHIPLayoutPlain;
    // input_argument[i]: input i is a packed argument of the run; input_constant[i]: it is a module constant
    std::vector<bool> input_argument;
    bool winograd_allowed = false;
    // what the graph pass fused behind this call (only offered to operators that declare "THIPFusable")
    bool fused_relu = false;
    bool has_residual = false;
    HIPBuffer residual;
    // input_constant[i]: input i is a module constant (same tensor on every run).  alloc_persistent(bytes) hands
    // out a workspace region that lives as long as the module, for a re-laid-out copy of such a constant.
    std::vector<bool> input_constant;
    std::function<HIPBuffer(int64_t)> alloc_persistent;
    // A second call of the same operator on the same first input whose value this launch produces as well (offered
    // only after the operator's "FHIPPairQuery" said yes for the two calls): its attributes, input types, inputs
    // (the first one equals inputs[0]) and output.
    bool has_pair = false;
    Attrs pair_attrs;
    Array<Type> pair_input_types;
    Array<HIPBuffer> pair_inputs;
    HIPBuffer pair_output;
    // A pooling call that is the sole reader of this launch's value and that the operator's "FHIPPoolQuery" agreed
    // to produce as well: `output` and `out_type` are then the pooling call's, and alloc_temp(bytes) hands out
    // workspace that lives until the call's launches have been appended (for what passes between them).
    bool has_pool = false;
    std::string pool_op;
    Attrs pool_attrs;
    std::function<HIPBuffer(int64_t)> alloc_temp;
};
// Whether the launch(es) of a call (attributes, input types, what is fused behind it) can also produce the pooling
// call `pool_op` (nn_max_pool2d / nn_avg_pool2d, MaxPool2DAttrs) that reads its value.
using FHIPPoolQuery = std::function<bool(const Attrs& attrs, const Array<Type>& inputs, bool fused_relu, bool has_residual,
                                         const std::string& pool_op, const Attrs& pool_attrs)>;
// Whether one launch of call A (attrs, input types, and whether a ReLU / residual is fused behind it is irrelevant)
// can also produce call B, an unfused call of the same operator on the same first input.
using FHIPPairQuery = std::function<bool(const Attrs& a_attrs, const Array<Type>& a_inputs, const std::vector<bool>& a_constant,
                                         const Attrs& b_attrs, const Array<Type>& b_inputs)>;
// Appends the launch(es) for one call to the plan; returns the kernel_symbol, or "" to decline (the
// call is then compiled through the code generator).
using FHIPDispatch = std::function<std::string(const HIPDispatchContext&, kxc_hip_plan*)>;

class OpRegEntry {
public:
    explicit OpRegEntry(std::shared_ptr<OpNode> op) : op_(std::move(op)) {}
    OpRegEntry& describe(const std::string& text) { op_->description = text; return *this; }
    OpRegEntry& set_num_inputs(int n) { op_->num_inputs = n; return *this; }
    OpRegEntry& add_argument(const std::string& name, const std::string& type, const std::string& desc) {
        op_->arguments.push_back({name, type, desc});
        return *this;
    }
    template <typename T>
    OpRegEntry& set_attr(const std::string& key, const T& value) {
        op_->attrs[key] = value;
        return *this;
    }
    static OpRegEntry Register(const std::string& name);

private:
    std::shared_ptr<OpNode> op_;
};

#define KXC_OP_CONCAT_(a, b) a##b
#define KXC_OP_CONCAT(a, b) KXC_OP_CONCAT_(a, b)
#define KXC_REGISTER_OP(OpName) \
    static ::kxc::relay::OpRegEntry KXC_OP_CONCAT(kxc_op_reg_, __COUNTER__) = ::kxc::relay::OpRegEntry::Register(#OpName)

// Force the built-in operator registrations to be linked (static initialisers in ops.cc).
void EnsureBuiltinOpsRegistered();

// ------------------------------------------------------------------ attribute types
#define KXC_ATTRS_REF(TypeName)                                                                      \
    class TypeName : public Attrs {                                                                  \
    public:                                                                                          \
        TypeName() = default;                                                                        \
        explicit TypeName(std::shared_ptr<TypeName##Node> n) : Attrs(n) {}                           \
        const TypeName##Node* operator->() const { return static_cast<const TypeName##Node*>(ptr_.get()); }

struct Conv2DAttrsNode : AttrsNode {
    std::vector<int64_t> strides, padding, dilation, kernel_size;
    int groups = 1, channels = 0;
    std::string data_layout, kernel_layout, out_layout, out_dtype;
};
KXC_ATTRS_REF(Conv2DAttrs)
    static Conv2DAttrs Create(std::vector<int64_t> strides, std::vector<int64_t> padding, std::vector<int64_t> dilation,
                              int groups, int channels, std::vector<int64_t> kernel_size, std::string data_layout,
                              std::string kernel_layout, std::string out_layout, std::string out_dtype);
};

struct MaxPool2DAttrsNode : AttrsNode {
    std::vector<int64_t> strides, padding, dilation, pool_size;
    std::string layout;
    bool ceil_mode = false;
};
KXC_ATTRS_REF(MaxPool2DAttrs)
    // strides first, pool_size fourth (include/relay/op.h:172-174)
    static MaxPool2DAttrs Create(std::vector<int64_t> strides, std::vector<int64_t> padding, std::vector<int64_t> dilation,
                                 std::vector<int64_t> pool_size, std::string layout, bool ceil_mode);
};

struct DenseAttrsNode : AttrsNode { int64_t units = 0; std::string out_dtype; };
KXC_ATTRS_REF(DenseAttrs)
    static DenseAttrs Create(int64_t units, std::string out_dtype);
};

struct GemmAttrsNode : AttrsNode { float alpha = 1.0f, beta = 1.0f; int transA = 0, transB = 0; };
KXC_ATTRS_REF(GemmAttrs)
    static GemmAttrs Create(float alpha = 1.0f, float beta = 1.0f, int transA = 0, int transB = 0);
};

struct FlattenAttrsNode : AttrsNode { int axis = 1; };
KXC_ATTRS_REF(FlattenAttrs)
    static FlattenAttrs Create(int axis = 1);
};

struct ReshapeAttrsNode : AttrsNode { std::vector<int64_t> newshape; };
KXC_ATTRS_REF(ReshapeAttrs)
    static ReshapeAttrs Create(std::vector<int64_t> newshape);
};

struct TransposeAttrsNode : AttrsNode { std::vector<int64_t> axes; };
KXC_ATTRS_REF(TransposeAttrs)
    static TransposeAttrs Create(std::vector<int64_t> axes);
};

struct ReduceMeanAttrsNode : AttrsNode { std::vector<int64_t> axes; int keepdims = 0; };
KXC_ATTRS_REF(ReduceMeanAttrs)
    static ReduceMeanAttrs Create(std::vector<int64_t> axes, int keepdims);
};

// softmax (src/relay/op/nn/softmax.cc): axis may be negative
struct SoftmaxAttrsNode : AttrsNode { int64_t axis = -1; };
KXC_ATTRS_REF(SoftmaxAttrs)
    static SoftmaxAttrs Create(int64_t axis = -1);
};

// cast (src/relay/op/tensor/transform.cc:84-104): `to` is a dtype code -- 0 float32, 1 int32, 2 int64, 3 float64,
// 4 bool, 5 int8, 6 uint8
// Quantised operators.  The reference has no int8 operator (grep for int8 / quant finds dtype plumbing only); these
// follow its rules for adding one (docs/relay-op-integration/04-lowering-backend.md:142-152: attributes, type rule,
// TOPI compute with a tir::Call for the new intrinsic `rint`, code-generator mapping, numeric test):
//   qnn_quantize(x f32)                                   -> int8  clamp(rint(x / scale), -127, 127), NaN -> 0
//   qnn_conv2d(x i8, w i8, bias i32, mult f32[, res i8])  -> int8  acc = sum x*w in int32 + bias[o];
//        v = (float)acc * mult[o] [+ (float)res * res_mult];  clamp(rint(v), relu ? 0 : -128, 127), NaN -> 0
//   qnn_dense(x i8 [M,K], w i8 [N,K], bias i32, mult f32) -> float32  (float)(acc + bias[j]) * mult[j]
// rint rounds to nearest, ties to even; every float operation is rounded separately.
struct QnnConv2DAttrsNode : AttrsNode {
    std::vector<int64_t> strides, padding;      // {h, w}; padding symmetric {h, w}
    bool relu = true;
    double res_mult = 0.0;
};
KXC_ATTRS_REF(QnnConv2DAttrs)
    static QnnConv2DAttrs Create(std::vector<int64_t> strides, std::vector<int64_t> padding, bool relu, double res_mult = 0.0);
};
struct QnnQuantizeAttrsNode : AttrsNode { double scale = 1.0; };
KXC_ATTRS_REF(QnnQuantizeAttrs)
    static QnnQuantizeAttrs Create(double scale);
};
//   qnn_global_avg_pool2d(x i8 [N,C,H,W]) -> int8 [N,C,1,1]  clamp(rint((float)(sum over H, W in int32) * mult), -128, 127)
//        (mult = s_in / (H * W * s_out), computed by whoever quantised the model)
struct QnnRequantAttrsNode : AttrsNode { double mult = 1.0; };
KXC_ATTRS_REF(QnnRequantAttrs)
    static QnnRequantAttrs Create(double mult);
};

struct CastAttrsNode : AttrsNode { int to = 0; };
KXC_ATTRS_REF(CastAttrs)
    static CastAttrs Create(int to);
};

#define KXC_SIMPLE_ATTRS(TypeName)                \
    struct TypeName##Node : AttrsNode {};         \
    KXC_ATTRS_REF(TypeName)                       \
        static TypeName Create() { return TypeName(std::make_shared<TypeName##Node>()); } \
    };
KXC_SIMPLE_ATTRS(ReluAttrs)
KXC_SIMPLE_ATTRS(AddAttrs)
KXC_SIMPLE_ATTRS(GlobalAvgPool2DAttrs)

// ------------------------------------------------------------------ shape rules (src/relay/type_infer.cc)
Type Conv2DInferType(const Attrs& attrs, const Array<Type>& inputs);
Type Pool2DInferType(const Attrs& attrs, const Array<Type>& inputs);
Type GlobalAvgPool2DInferType(const Attrs& attrs, const Array<Type>& inputs);
Type DenseInferType(const Attrs& attrs, const Array<Type>& inputs);
Type QnnConv2DInferType(const Attrs& attrs, const Array<Type>& inputs);
Type QnnDenseInferType(const Attrs& attrs, const Array<Type>& inputs);
Type QnnQuantizeInferType(const Attrs& attrs, const Array<Type>& inputs);
Type QnnGlobalAvgPool2DInferType(const Attrs& attrs, const Array<Type>& inputs);
Type GemmInferType(const Attrs& attrs, const Array<Type>& inputs);
Type MatmulInferType(const Attrs& attrs, const Array<Type>& inputs);
Type UnarySameInferType(const Attrs& attrs, const Array<Type>& inputs);
Type BroadcastInferType(const Attrs& attrs, const Array<Type>& inputs);
Type FlattenInferType(const Attrs& attrs, const Array<Type>& inputs);
Type ReshapeInferType(const Attrs& attrs, const Array<Type>& inputs);
Type TransposeInferType(const Attrs& attrs, const Array<Type>& inputs);
Type ReduceMeanInferType(const Attrs& attrs, const Array<Type>& inputs);
Type SoftmaxInferType(const Attrs& attrs, const Array<Type>& inputs);
Type CastInferType(const Attrs& attrs, const Array<Type>& inputs);
// dtype string of a cast code; throws "cast has unsupported dtype code: N"
std::string CastDTypeFromCode(int code);

// InferTypePass (src/relay/transforms/infer_type.cc:41-222): fills checked_type_ of every node.
Function InferTypePass(const Function& f);
// The same function on 1/lanes of the batch: parameter 0 (the only parameter that may carry the batch) gets a
// leading extent divided by `lanes`, constants are shared, every call keeps its operator and attributes.  Returns an
// undefined Function when the graph cannot be proven separable along the batch: every operator between parameter 0
// and the result must treat the leading axis of a batched operand as independent samples (convolutions, pools,
// dense / gemm / matmul on the left operand, element-wise operators with broadcast operands that have no batch
// axis, flatten, softmax / reduce_mean / transpose that leave axis 0 alone, cast, the quantised operators), the
// result must carry the batch, and the batch must divide.  `f` must be typed; the result is typed.  (No counterpart
// in the reference; used by the hip back end to run the shares of a batch side by side.)
Function SplitBatch(const Function& f, int lanes);

}  // namespace relay
}  // namespace kxc
