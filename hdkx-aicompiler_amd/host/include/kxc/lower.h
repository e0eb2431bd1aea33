// lower.h -- Relay function -> TE -> one TIR PrimFunc of naive loop nests.
// Reproduces the reference's LowerToTIR contract (src/relay/backend/lower.cc:470-663):
//   * parameters: function inputs, then constants named const_<k> in depth-first argument order
//     (:201-233), then outputs named <tensor>_out (:451-468);
//   * intermediates: nested Allocate nodes around the body (:603-609);
//   * every compute stage: data loops outermost in axis order, and for a reduction
//     Store(init) followed by the reduce loops (first axis outermost) around
//     Store(Load(out) + source) (:389-449); flat row-major indices (:59-71);
//   * attrs global_symbol, tir.noalias, kxc.input_count / constant_count / output_count /
//     output_param_start (:619-629).
#pragma once

#include "kxc/op.h"
#include "kxc/tir.h"

namespace kxc {
namespace relay {

struct LoweredFunc {
    tir::PrimFunc func;
    // constants in parameter order (their host data), so a caller can pass them again at Run
    Array<runtime::NDArray> constants;
    // names of the intermediate buffers in allocation order, with element counts and dtypes
    struct Intermediate { std::string name; tir::DataType dtype; int64_t elements; const tir::ExprNode* var; };
    std::vector<Intermediate> intermediates;
};

tir::PrimFunc LowerToTIR(const Function& f);
LoweredFunc LowerToTIRDetailed(const Function& f);

}  // namespace relay
}  // namespace kxc
