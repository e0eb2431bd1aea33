// te.h -- tensor expressions: placeholders and compute definitions that the lowering turns into loops.
// Counterpart of the reference's TE layer (include/te/te.h:177-319, src/te/te.cc:92-155): a compute
// tensor has data axes named ax0.., a single body expression, and at most one reduction at the top
// of the body.
#pragma once

#include <functional>

#include "kxc/tir.h"

namespace kxc {
namespace tir {
struct TensorNode {
    std::vector<PrimExpr> shape;
    DataType dtype;
    std::string name;
    std::string tag;
    bool is_placeholder = true;
    std::vector<Var> axis;      // data axes (compute only)
    PrimExpr body;              // compute only; may be a kReduce node
};
}  // namespace tir

namespace te {

using tir::PrimExpr;

struct IterVar {
    tir::Var var;
    PrimExpr dom_min, dom_extent;
};

class Tensor : public Ref<tir::TensorNode> {
public:
    Tensor() = default;
    explicit Tensor(std::shared_ptr<tir::TensorNode> n) : Ref<tir::TensorNode>(std::move(n)) {}
    // element access inside a compute body
    PrimExpr operator()(const std::vector<PrimExpr>& indices) const;
    PrimExpr operator()(const Array<tir::Var>& indices) const;
    template <typename... Args>
    PrimExpr operator()(PrimExpr first, Args... rest) const {
        return (*this)(std::vector<PrimExpr>{first, PrimExpr(rest)...});
    }
    std::vector<int64_t> const_shape() const;
};

enum ReduceType { kSum = 0, kMax = 1, kMin = 2 };

Tensor placeholder(std::vector<PrimExpr> shape, tir::DataType dtype, std::string name);
Tensor compute(std::vector<PrimExpr> shape, std::function<PrimExpr(const Array<tir::Var>&)> fcompute,
               std::string name = "compute", std::string tag = "");
IterVar reduce_axis(PrimExpr min, PrimExpr extent, std::string name);
PrimExpr sum(PrimExpr source, std::vector<IterVar> axes);
PrimExpr max(PrimExpr source, std::vector<IterVar> axes);
PrimExpr min(PrimExpr source, std::vector<IterVar> axes);

}  // namespace te
}  // namespace kxc
