// lower.cc -- see lower.h.
#include "kxc/lower.h"

#include <limits>
#include <unordered_map>
#include <unordered_set>

namespace kxc {
namespace relay {

using te::Tensor;
using tir::DataType;
using tir::ExprKind;
using tir::PrimExpr;
using tir::Stmt;

namespace {

PrimExpr I64(int64_t v) { return tir::IntImm(v, DataType::Int(64)); }

std::vector<PrimExpr> ShapeExprs(const std::vector<int64_t>& shape) {
    std::vector<PrimExpr> out;
    for (auto d : shape) out.push_back(I64(d));
    return out;
}

// row-major flattening: ((i0 * s1 + i1) * s2 + i2) ...
PrimExpr FlattenIndex(const std::vector<PrimExpr>& indices, const std::vector<PrimExpr>& shape) {
    if (shape.empty()) return tir::IntImm(0);
    if (indices.size() != shape.size()) throw std::runtime_error("Index rank mismatch during flattening");
    PrimExpr lin = indices[0];
    for (size_t i = 1; i < indices.size(); ++i) lin = lin * shape[i] + indices[i];
    return lin;
}

PrimExpr ReduceIdentity(int rtype, DataType t) {
    if (rtype == te::kSum) return t.is_float() ? tir::FloatImm(0.0, t) : tir::IntImm(0, t);
    const bool is_max = rtype == te::kMax;
    if (t.is_float()) {
        const double inf = std::numeric_limits<double>::infinity();
        return tir::FloatImm(is_max ? -inf : inf, t);
    }
    // (the reference hands every integer type the 64-bit extremes, src/relay/backend/lower.cc:80-95; a narrower type
    // takes its own, since the 64-bit ones truncate to 0 and -1 there)
    if (t.is_uint()) return tir::IntImm(is_max ? 0 : (t.bits >= 63 ? std::numeric_limits<int64_t>::max() : (int64_t{1} << t.bits) - 1), t);
    if (t.bits < 64) return tir::IntImm(is_max ? -(int64_t{1} << (t.bits - 1)) : (int64_t{1} << (t.bits - 1)) - 1, t);
    return tir::IntImm(is_max ? std::numeric_limits<int64_t>::min() : std::numeric_limits<int64_t>::max(), t);
}

class Converter {
public:
    explicit Converter(const Function& f) {
        for (const auto& p : f->params) {
            const auto* tt = p->type_annotation.As<TensorTypeNode>();
            if (!tt) throw std::runtime_error("LowerToTIR requires TensorType on function parameters: " + p->vid->name_hint);
            Tensor t = te::placeholder(ShapeExprs(tt->shape), tir::DTypeFromString(tt->dtype), p->vid->name_hint);
            memo_[p.get()] = t;
            inputs.push_back(t);
        }
    }

    Tensor Visit(const Expr& e) {
        auto it = memo_.find(e.get());
        if (it != memo_.end()) return it->second;
        Tensor out;
        if (const auto* v = e.As<VarNode>()) {
            throw std::runtime_error("Unexpected free var in LowerToTIR: " + v->vid->name_hint);
        } else if (const auto* c = e.As<ConstantNode>()) {
            out = te::placeholder(ShapeExprs(c->data->shape), tir::DTypeFromString(c->data->dtype),
                                  "const_" + std::to_string(constants.size()));
            constants.push_back(out);
            constant_data.push_back(c->data);
        } else if (const auto* call = e.As<CallNode>()) {
            Array<Tensor> in;
            for (const auto& arg : call->args) in.push_back(Visit(arg));
            const auto* op = call->op.As<OpNode>();
            if (!op) throw std::runtime_error("Call.op is not OpNode in LowerToTIR");
            if (op->name.rfind("device.", 0) == 0)
                throw std::runtime_error("LowerToTIR does not lower device communication ops. "
                                         "Run LowerRelayToExecPlanPass before LowerToTIR.");
            if (!e.checked_type().defined())
                throw std::runtime_error("LowerToTIR requires checked_type for op: " + op->name);
            auto it2 = op->attrs.find("FRelayToTE");
            if (it2 == op->attrs.end()) throw std::runtime_error("No FRelayToTE registered for op: " + op->name);
            const auto* fn = std::any_cast<FRelayToTE>(&it2->second);
            if (!fn) throw std::runtime_error("Bad FRelayToTE type for op: " + op->name);
            out = (*fn)(call->attrs, in, e.checked_type());
        } else {
            throw std::runtime_error("Unsupported Relay node in LowerToTIR");
        }
        memo_[e.get()] = out;
        return out;
    }

    Array<Tensor> inputs, constants;
    Array<runtime::NDArray> constant_data;

private:
    std::unordered_map<const RelayExprNode*, Tensor> memo_;
};

void FindProducers(const PrimExpr& e, std::vector<Tensor>* deps) {
    if (!e.defined()) return;
    if (e->kind == ExprKind::kProducerLoad) deps->push_back(Tensor(e->tensor));
    for (const auto& a : e->args) FindProducers(a, deps);
}

void CollectDFS(const Tensor& t, std::unordered_set<const tir::TensorNode*>* seen, std::vector<Tensor>* topo) {
    if (!t.defined() || seen->count(t.get())) return;
    if (!t->is_placeholder) {
        std::vector<Tensor> deps;
        FindProducers(t->body, &deps);
        for (const auto& d : deps) CollectDFS(d, seen, topo);
    }
    seen->insert(t.get());
    topo->push_back(t);
}

class ExprLowerer {
public:
    explicit ExprLowerer(const std::unordered_map<const tir::TensorNode*, tir::Var>& vars) : vars_(vars) {}
    PrimExpr Lower(const PrimExpr& e) const {
        if (!e.defined()) return e;
        switch (e->kind) {
            case ExprKind::kIntImm: case ExprKind::kFloatImm: case ExprKind::kVar: return e;
            case ExprKind::kReduce: throw std::runtime_error("nested reduce is not supported");
            default: break;
        }
        std::vector<PrimExpr> args;
        for (const auto& a : e->args) args.push_back(Lower(a));
        if (e->kind == ExprKind::kProducerLoad) {
            auto it = vars_.find(e->tensor.get());
            if (it == vars_.end()) throw std::runtime_error("Missing buffer var for tensor '" + e->tensor->name + "'");
            return tir::Load(it->second, FlattenIndex(args, e->tensor->shape), e->dtype);
        }
        auto n = std::make_shared<tir::ExprNode>(*e.get());
        n->args = args;
        return PrimExpr(n);
    }

private:
    const std::unordered_map<const tir::TensorNode*, tir::Var>& vars_;
};

Stmt LowerCompute(const Tensor& t, const std::unordered_map<const tir::TensorNode*, tir::Var>& vars,
                  const ExprLowerer& lowerer) {
    const tir::Var out = vars.at(t.get());
    std::vector<PrimExpr> axes(t->axis.begin(), t->axis.end());
    const PrimExpr out_index = FlattenIndex(axes, t->shape);
    Stmt body;
    if (t->body->kind == ExprKind::kReduce) {
        const PrimExpr& red = t->body;
        Stmt init = tir::Store(out, ReduceIdentity(red->reduce_type, t->dtype), out_index);
        PrimExpr src = lowerer.Lower(red->args[0]);
        PrimExpr old = tir::Load(out, out_index, t->dtype);
        PrimExpr upd = red->reduce_type == te::kSum ? old + src
                       : red->reduce_type == te::kMax ? tir::Max(old, src) : tir::Min(old, src);
        Stmt update = tir::Store(out, upd, out_index);
        for (int i = static_cast<int>(red->reduce_vars.size()) - 1; i >= 0; --i)
            update = tir::For(tir::Var(red->reduce_vars[i].shared()), red->reduce_min[i], red->reduce_extent[i],
                              tir::ForType::Serial, update);
        body = tir::SeqStmt({init, update});
    } else {
        body = tir::Store(out, lowerer.Lower(t->body), out_index);
    }
    for (int i = static_cast<int>(t->axis.size()) - 1; i >= 0; --i)
        body = tir::For(t->axis[i], tir::IntImm(0), t->shape[i], tir::ForType::Serial, body);
    return body;
}

}  // namespace

LoweredFunc LowerToTIRDetailed(const Function& untyped) {
    if (!untyped.defined()) throw std::runtime_error("LowerToTIR expects a defined function");
    // types are inferred here as well (src/relay/backend/lower.cc:470-477), so an untyped graph can be lowered
    const Function f = InferTypePass(untyped);
    if (!f->body.defined()) throw std::runtime_error("LowerToTIR expects function body to be defined");
    Converter conv(f);
    Tensor out_tensor = conv.Visit(f->body);

    std::unordered_set<const tir::TensorNode*> seen;
    std::vector<Tensor> topo;
    CollectDFS(out_tensor, &seen, &topo);

    auto fn = std::make_shared<tir::PrimFuncNode>();
    std::unordered_map<const tir::TensorNode*, tir::Var> vars;
    auto add_param = [&](const Tensor& t, const std::string& name) {
        tir::Var v(name, t->dtype);
        fn->params.push_back(v);
        fn->buffer_map[v.get()] = tir::BufferInfo{t->dtype, t.const_shape(), name};
        vars[t.get()] = v;
    };
    for (const auto& t : conv.inputs) add_param(t, t->name);
    for (const auto& t : conv.constants) add_param(t, t->name);
    const int64_t input_count = static_cast<int64_t>(conv.inputs.size());
    const int64_t constant_count = static_cast<int64_t>(conv.constants.size());

    LoweredFunc result;
    if (out_tensor->is_placeholder) {
        // the function returns one of its inputs: materialise a copy stage
        Tensor src = out_tensor;
        out_tensor = te::compute(src->shape, [&](const Array<tir::Var>& i) { return src(i); }, src->name + "_copy");
        topo.push_back(out_tensor);
    }
    add_param(out_tensor, (out_tensor->name.empty() ? std::string("output") : out_tensor->name) + "_out");

    std::vector<Tensor> intermediates;
    for (const auto& t : topo) {
        if (t->is_placeholder || t.get() == out_tensor.get()) continue;
        tir::Var v(t->name, t->dtype);
        vars[t.get()] = v;
        intermediates.push_back(t);
        result.intermediates.push_back({t->name, t->dtype, Product(t.const_shape()), v.get()});
    }

    ExprLowerer lowerer(vars);
    std::vector<Stmt> seq;
    for (const auto& t : topo) {
        if (t->is_placeholder) continue;
        try {
            seq.push_back(LowerCompute(t, vars, lowerer));
        } catch (const std::exception& e) {
            throw std::runtime_error("LowerComputeStmt failed for tensor '" + t->name + "': " + e.what());
        }
    }
    Stmt body = seq.size() == 1 ? seq[0] : tir::SeqStmt(seq);
    for (int i = static_cast<int>(intermediates.size()) - 1; i >= 0; --i) {
        const Tensor& t = intermediates[i];
        body = tir::Allocate(vars[t.get()], t->dtype, t->shape, tir::IntImm(1, DataType::Bool()), body);
    }
    fn->body = body;
    fn->str_attrs["global_symbol"] = "main";
    fn->int_attrs["tir.noalias"] = 1;
    fn->int_attrs["kxc.input_count"] = input_count;
    fn->int_attrs["kxc.constant_count"] = constant_count;
    fn->int_attrs["kxc.output_count"] = 1;
    fn->int_attrs["kxc.output_param_start"] = input_count + constant_count;
    result.func = tir::PrimFunc(fn);
    result.constants = conv.constant_data;
    return result;
}

tir::PrimFunc LowerToTIR(const Function& f) { return LowerToTIRDetailed(f).func; }

}  // namespace relay
}  // namespace kxc
