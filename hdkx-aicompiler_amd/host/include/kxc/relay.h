// relay.h -- graph-level IR: types, Var / Constant / Call / Function, and the host NDArray.
// Surface of the reference's include/relay/relay.h:49-169 and include/base/ndarray.h:72-82 as far as
// graph construction needs it.
#pragma once

#include <cstring>

#include "kxc/base.h"

namespace kxc {

// ------------------------------------------------------------------ types
struct TypeNode : Object {};
struct TensorTypeNode : TypeNode {
    std::vector<int64_t> shape;
    std::string dtype;
};
class Type : public Ref<TypeNode> {
public:
    Type() = default;
    explicit Type(std::shared_ptr<TypeNode> n) : Ref<TypeNode>(std::move(n)) {}
};
class TensorType : public Type {
public:
    TensorType() = default;
    TensorType(Array<int64_t> shape, std::string dtype) {
        auto n = std::make_shared<TensorTypeNode>();
        n->shape = shape;
        n->dtype = std::move(dtype);
        ptr_ = n;
    }
    const TensorTypeNode* operator->() const { return static_cast<const TensorTypeNode*>(ptr_.get()); }
};
std::string TypeToString(const Type& t);

// ------------------------------------------------------------------ host tensor
}  // namespace kxc
// Element type of a host tensor as the reference's NDArray exposes it (include/base/ndarray.h:19-31).
extern "C" {
typedef enum { kDLInt = 0U, kDLUint = 1U, kDLFloat = 2U, kDLBfloat = 4U, kDLComplex = 5U } DLDataTypeCode;
typedef struct {
    uint8_t code;
    uint8_t bits;
    uint16_t lanes;
} DLDataType;
}
namespace kxc {
namespace runtime {
struct NDArrayNode : Object {
    std::vector<int64_t> shape;
    std::string dtype;
    struct {
        DLDataType dtype;
    } dl_tensor;                   // dtype as {code, bits, lanes}, filled on construction
    std::vector<char> bytes;       // zero-filled on construction (src/base/ndarray.cc:35-62)
    void* data() { return bytes.data(); }
    const void* data() const { return bytes.data(); }
};
class NDArray : public Ref<NDArrayNode> {
public:
    NDArray() = default;
    NDArray(Array<int64_t> shape, std::string dtype);
    void CopyFromBytes(const void* src, size_t nbytes);
    void CopyToBytes(void* dst, size_t nbytes) const;
    size_t nbytes() const { return ptr_ ? ptr_->bytes.size() : 0; }
};
}  // namespace runtime

// ------------------------------------------------------------------ expressions
struct RelayExprNode : Object {
    mutable Type checked_type_;     // filled by InferType
};
class Expr : public Ref<RelayExprNode> {
public:
    Expr() = default;
    explicit Expr(std::shared_ptr<RelayExprNode> n) : Ref<RelayExprNode>(std::move(n)) {}
    const Type& checked_type() const { return ptr_->checked_type_; }
};

struct IdNode { std::string name_hint; };
struct VarNode : RelayExprNode {
    std::shared_ptr<IdNode> vid;
    Type type_annotation;
};
class Var : public Expr {
public:
    Var() = default;
    Var(std::string name, Type annotation) {
        auto n = std::make_shared<VarNode>();
        n->vid = std::make_shared<IdNode>();
        n->vid->name_hint = std::move(name);
        n->type_annotation = annotation;
        ptr_ = n;
    }
    const VarNode* operator->() const { return static_cast<const VarNode*>(ptr_.get()); }
};

struct ConstantNode : RelayExprNode {
    runtime::NDArray data;
};
class Constant : public Expr {
public:
    Constant() = default;
    explicit Constant(runtime::NDArray data) {
        auto n = std::make_shared<ConstantNode>();
        n->data = data;
        ptr_ = n;
    }
    const ConstantNode* operator->() const { return static_cast<const ConstantNode*>(ptr_.get()); }
};

struct AttrsNode : Object {};
class Attrs : public Ref<AttrsNode> {
public:
    Attrs() = default;
    explicit Attrs(std::shared_ptr<AttrsNode> n) : Ref<AttrsNode>(std::move(n)) {}
};

struct CallNode : RelayExprNode {
    Expr op;
    Array<Expr> args;
    Attrs attrs;
};
class Call : public Expr {
public:
    Call() = default;
    Call(Expr op, Array<Expr> args, Attrs attrs = Attrs()) {
        auto n = std::make_shared<CallNode>();
        n->op = op;
        n->args = args;
        n->attrs = attrs;
        ptr_ = n;
    }
    const CallNode* operator->() const { return static_cast<const CallNode*>(ptr_.get()); }
};

struct FunctionNode : RelayExprNode {
    Array<Var> params;
    Expr body;
};
class Function : public Expr {
public:
    Function() = default;
    Function(Array<Var> params, Expr body) {
        auto n = std::make_shared<FunctionNode>();
        n->params = params;
        n->body = body;
        ptr_ = n;
    }
    const FunctionNode* operator->() const { return static_cast<const FunctionNode*>(ptr_.get()); }
};

}  // namespace kxc
