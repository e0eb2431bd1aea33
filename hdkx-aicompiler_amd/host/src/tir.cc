// tir.cc -- constructors, printer and the two scalar passes of the loop-level IR.
#include "kxc/tir.h"

#include <cmath>
#include <sstream>

namespace kxc {
namespace tir {

DataType DTypeFromString(const std::string& s) {
    if (s == "float32") return DataType::Float(32);
    if (s == "float64") return DataType::Float(64);
    if (s == "int32") return DataType::Int(32);
    if (s == "int64") return DataType::Int(64);
    if (s == "int8") return DataType::Int(8);
    if (s == "uint8") return DataType::UInt(8);
    if (s == "bool") return DataType::Bool();
    throw std::runtime_error("Unsupported dtype string: " + s);
}

std::string DTypeToString(DataType t) {
    if (t.is_bool()) return "bool";
    const char* base = t.code == 0 ? "int" : t.code == 1 ? "uint" : t.code == 2 ? "float" : "handle";
    return std::string(base) + std::to_string(t.bits);
}

static PrimExpr MakeNode(ExprKind k, DataType t, std::vector<PrimExpr> args = {}) {
    auto n = std::make_shared<ExprNode>();
    n->kind = k;
    n->dtype = t;
    n->args = std::move(args);
    return PrimExpr(n);
}

PrimExpr IntImm(int64_t v, DataType t) {
    PrimExpr e = MakeNode(ExprKind::kIntImm, t);
    e.get()->ivalue = v;
    return e;
}
PrimExpr FloatImm(double v, DataType t) {
    PrimExpr e = MakeNode(ExprKind::kFloatImm, t);
    e.get()->fvalue = v;
    return e;
}
PrimExpr::PrimExpr(int v) : PrimExpr(IntImm(v, DataType::Int(32))) {}
PrimExpr::PrimExpr(int64_t v) : PrimExpr(IntImm(v, DataType::Int(64))) {}
PrimExpr::PrimExpr(float v) : PrimExpr(FloatImm(v, DataType::Float(32))) {}
PrimExpr::PrimExpr(double v) : PrimExpr(FloatImm(v, DataType::Float(64))) {}

Var::Var(std::string name, DataType dtype) {
    auto n = std::make_shared<ExprNode>();
    n->kind = ExprKind::kVar;
    n->dtype = dtype;
    n->name = std::move(name);
    ptr_ = n;
}

static void RequireDefined(const PrimExpr& a, const PrimExpr& b, const char* what) {
    if (!a.defined() || !b.defined()) throw std::runtime_error(std::string(what) + ": undefined operand");
}

// result dtype = dtype of the left operand (src/tir/expr.cc:37-44)
#define KXC_BINARY(Name, Kind)                                  \
    PrimExpr Name(PrimExpr a, PrimExpr b) {                     \
        RequireDefined(a, b, #Name);                            \
        return MakeNode(ExprKind::Kind, a.dtype(), {a, b});     \
    }
KXC_BINARY(Add, kAdd)
KXC_BINARY(Sub, kSub)
KXC_BINARY(Mul, kMul)
KXC_BINARY(Div, kDiv)
KXC_BINARY(Mod, kMod)
KXC_BINARY(Min, kMin)
KXC_BINARY(Max, kMax)
#undef KXC_BINARY
#define KXC_COMPARE(Name, Kind)                                 \
    PrimExpr Name(PrimExpr a, PrimExpr b) {                     \
        RequireDefined(a, b, #Name);                            \
        return MakeNode(ExprKind::Kind, DataType::Bool(), {a, b}); \
    }
KXC_COMPARE(EQ, kEQ)
KXC_COMPARE(LT, kLT)
KXC_COMPARE(And, kAnd)
KXC_COMPARE(Or, kOr)
#undef KXC_COMPARE
PrimExpr Not(PrimExpr a) {
    if (!a.defined()) throw std::runtime_error("Not: undefined operand");
    return MakeNode(ExprKind::kNot, DataType::Bool(), {a});
}
PrimExpr Load(Var buffer, PrimExpr index, DataType dtype) { return MakeNode(ExprKind::kLoad, dtype, {buffer, index}); }
PrimExpr Call(DataType dtype, std::string name, std::vector<PrimExpr> args) {
    PrimExpr e = MakeNode(ExprKind::kCall, dtype, std::move(args));
    e.get()->name = std::move(name);
    return e;
}
PrimExpr Select(PrimExpr cond, PrimExpr t, PrimExpr f) { return MakeNode(ExprKind::kSelect, t.dtype(), {cond, t, f}); }

bool GetConstInt(const PrimExpr& e, int64_t* out) {
    if (!e.defined() || e->kind != ExprKind::kIntImm) return false;
    *out = e->ivalue;
    return true;
}

static Stmt MakeStmt(StmtKind k) {
    auto n = std::make_shared<StmtNode>();
    n->kind = k;
    return Stmt(n);
}
Stmt LetStmt(Var var, PrimExpr value, Stmt body) {
    Stmt s = MakeStmt(StmtKind::kLetStmt);
    s.get()->var = var; s.get()->a = value; s.get()->body = {body};
    return s;
}
Stmt Store(Var buffer, PrimExpr value, PrimExpr index) {
    Stmt s = MakeStmt(StmtKind::kStore);
    s.get()->var = buffer; s.get()->a = value; s.get()->b = index;
    return s;
}
Stmt For(Var loop_var, PrimExpr min, PrimExpr extent, ForType type, Stmt body) {
    Stmt s = MakeStmt(StmtKind::kFor);
    s.get()->var = loop_var; s.get()->a = min; s.get()->b = extent; s.get()->for_type = type; s.get()->body = {body};
    return s;
}
Stmt IfThenElse(PrimExpr cond, Stmt then_case, Stmt else_case) {
    Stmt s = MakeStmt(StmtKind::kIfThenElse);
    s.get()->a = cond;
    s.get()->body = {then_case};
    if (else_case.defined()) s.get()->body.push_back(else_case);
    return s;
}
Stmt Allocate(Var buffer, DataType dtype, std::vector<PrimExpr> extents, PrimExpr condition, Stmt body) {
    Stmt s = MakeStmt(StmtKind::kAllocate);
    s.get()->var = buffer; s.get()->dtype = dtype; s.get()->extents = std::move(extents); s.get()->a = condition;
    s.get()->body = {body};
    return s;
}
Stmt SeqStmt(std::vector<Stmt> seq) {
    Stmt s = MakeStmt(StmtKind::kSeqStmt);
    s.get()->body = std::move(seq);
    return s;
}
Stmt Evaluate(PrimExpr value) {
    Stmt s = MakeStmt(StmtKind::kEvaluate);
    s.get()->a = value;
    return s;
}

namespace pass {
void IRPrinterPass::Run(const PrimFunc& func, std::ostream& os) const {
    os << "================ TIR PrimFunc ================\n";
    if (!func.defined()) { os << "<undefined>\n"; return; }
    const std::string pad(static_cast<size_t>(indent_spaces_ < 0 ? 0 : indent_spaces_), ' ');
    os << "params(" << func->params.size() << "):\n";
    for (size_t i = 0; i < func->params.size(); ++i) {
        os << pad << "[" << i << "] " << func->params[i].name_hint();
        auto it = func->buffer_map.find(func->params[i].get());
        if (it != func->buffer_map.end()) {
            os << " : buffer " << it->second.name << " " << DTypeToString(it->second.dtype) << "[";
            for (size_t d = 0; d < it->second.shape.size(); ++d) os << (d ? ", " : "") << it->second.shape[d];
            os << "]";
        }
        os << "\n";
    }
    os << "attrs:\n";
    for (const auto& kv : func->int_attrs) os << pad << kv.first << " = " << kv.second << "\n";
    for (const auto& kv : func->str_attrs) os << pad << kv.first << " = \"" << kv.second << "\"\n";
    os << "body:\n" << ToString(func->body, indent_spaces_ < 0 ? 0 : indent_spaces_);
}
void DumpPrimFunc(const PrimFunc& func, std::ostream& os, int indent_spaces) { IRPrinterPass(indent_spaces).Run(func, os); }
}  // namespace pass

DataType PromoteTypes(DataType a, DataType b) {
    if (a == b) return a;
    if (a.is_float() || b.is_float()) {
        int bits = 32;
        if (a.is_float()) bits = std::max(bits, a.bits);
        if (b.is_float()) bits = std::max(bits, b.bits);
        return DataType::Float(bits);
    }
    const int bits = std::max(a.bits == 1 ? 8 : a.bits, b.bits == 1 ? 8 : b.bits);
    return (a.is_int() || b.is_int()) ? DataType::Int(bits) : DataType::UInt(bits);
}

// ------------------------------------------------------------------ printer
static const char* OpText(ExprKind k) {
    switch (k) {
        case ExprKind::kAdd: return "+"; case ExprKind::kSub: return "-"; case ExprKind::kMul: return "*";
        case ExprKind::kDiv: return "/"; case ExprKind::kMod: return "%"; case ExprKind::kEQ: return "==";
        case ExprKind::kLT: return "<"; case ExprKind::kAnd: return "&&"; case ExprKind::kOr: return "||";
        default: return "?";
    }
}

std::string ToString(const PrimExpr& e) {
    if (!e.defined()) return "<undef>";
    std::ostringstream os;
    switch (e->kind) {
        case ExprKind::kIntImm: os << e->ivalue; break;
        case ExprKind::kFloatImm: os << e->fvalue << "f"; break;
        case ExprKind::kVar: os << e->name; break;
        case ExprKind::kMin: os << "min(" << ToString(e->args[0]) << ", " << ToString(e->args[1]) << ")"; break;
        case ExprKind::kMax: os << "max(" << ToString(e->args[0]) << ", " << ToString(e->args[1]) << ")"; break;
        case ExprKind::kNot: os << "!" << ToString(e->args[0]); break;
        case ExprKind::kLoad: os << ToString(e->args[0]) << "[" << ToString(e->args[1]) << "]"; break;
        case ExprKind::kSelect:
            os << "select(" << ToString(e->args[0]) << ", " << ToString(e->args[1]) << ", " << ToString(e->args[2]) << ")";
            break;
        case ExprKind::kCall: {
            os << e->name << "(";
            for (size_t i = 0; i < e->args.size(); ++i) os << (i ? ", " : "") << ToString(e->args[i]);
            os << ")";
            break;
        }
        case ExprKind::kProducerLoad: {
            os << "<tensor>(";
            for (size_t i = 0; i < e->args.size(); ++i) os << (i ? ", " : "") << ToString(e->args[i]);
            os << ")";
            break;
        }
        case ExprKind::kReduce: os << "reduce(" << ToString(e->args[0]) << ")"; break;
        default: os << "(" << ToString(e->args[0]) << " " << OpText(e->kind) << " " << ToString(e->args[1]) << ")";
    }
    return os.str();
}

std::string ToString(const Stmt& s, int indent) {
    if (!s.defined()) return "";
    const std::string pad(indent, ' ');
    std::ostringstream os;
    switch (s->kind) {
        case StmtKind::kFor:
            os << pad << "for (" << s->var.name_hint() << ", " << ToString(s->a) << ", " << ToString(s->b) << ") {\n"
               << ToString(s->body[0], indent + 2) << pad << "}\n";
            break;
        case StmtKind::kStore:
            os << pad << s->var.name_hint() << "[" << ToString(s->b) << "] = " << ToString(s->a) << "\n";
            break;
        case StmtKind::kLetStmt:
            os << pad << "let " << s->var.name_hint() << " = " << ToString(s->a) << "\n" << ToString(s->body[0], indent);
            break;
        case StmtKind::kAllocate: {
            os << pad << "allocate " << s->var.name_hint() << "[" << DTypeToString(s->dtype);
            for (auto& e : s->extents) os << " * " << ToString(e);
            os << "]\n" << ToString(s->body[0], indent);
            break;
        }
        case StmtKind::kIfThenElse:
            os << pad << "if (" << ToString(s->a) << ") {\n" << ToString(s->body[0], indent + 2) << pad << "}";
            if (s->body.size() > 1) os << " else {\n" << ToString(s->body[1], indent + 2) << pad << "}";
            os << "\n";
            break;
        case StmtKind::kSeqStmt:
            for (auto& b : s->body) os << ToString(b, indent);
            break;
        case StmtKind::kEvaluate: os << pad << ToString(s->a) << "\n"; break;
    }
    return os.str();
}

std::string ToString(const PrimFunc& f) {
    std::ostringstream os;
    os << "primfn(";
    for (size_t i = 0; i < f->params.size(); ++i) os << (i ? ", " : "") << f->params[i].name_hint();
    os << ") {\n" << ToString(f->body, 2) << "}\n";
    return os.str();
}

// ------------------------------------------------------------------ fold_constant + simplify_expr
static bool IsConstInt(const PrimExpr& e, int64_t v) {
    int64_t c;
    return GetConstInt(e, &c) && c == v;
}
static bool IsConstFloat(const PrimExpr& e, double v) {
    return e.defined() && e->kind == ExprKind::kFloatImm && e->fvalue == v;
}

PrimExpr FoldAndSimplify(const PrimExpr& e) {
    if (!e.defined()) return e;
    switch (e->kind) {
        case ExprKind::kIntImm: case ExprKind::kFloatImm: case ExprKind::kVar: return e;
        default: break;
    }
    std::vector<PrimExpr> args;
    bool changed = false;
    for (auto& a : e->args) {
        PrimExpr n = FoldAndSimplify(a);
        changed |= !n.same_as(a);
        args.push_back(n);
    }
    auto rebuild = [&]() -> PrimExpr {
        if (!changed) return e;
        auto n = std::make_shared<ExprNode>(*e.get());
        n->args = args;
        return PrimExpr(n);
    };
    const bool binary = args.size() == 2 && e->kind >= ExprKind::kAdd && e->kind <= ExprKind::kMax;
    if (binary) {
        int64_t x, y;
        // integer scalar folding (src/tir/transforms/fold_constant.cc:343-389); int results keep the lhs dtype
        if (GetConstInt(args[0], &x) && GetConstInt(args[1], &y) && !args[0].dtype().is_float()) {
            switch (e->kind) {
                case ExprKind::kAdd: return IntImm(x + y, e->dtype);
                case ExprKind::kSub: return IntImm(x - y, e->dtype);
                case ExprKind::kMul: return IntImm(x * y, e->dtype);
                case ExprKind::kDiv: if (y != 0) return IntImm(x / y, e->dtype); break;
                case ExprKind::kMod: if (y != 0) return IntImm(x % y, e->dtype); break;
                case ExprKind::kMin: return IntImm(x < y ? x : y, e->dtype);
                case ExprKind::kMax: return IntImm(x > y ? x : y, e->dtype);
                default: break;
            }
        }
        // x + 0, 0 + x, x - 0, x * 1, 1 * x, x / 1 (src/tir/transforms/simplify_expr.cc:17-69), integers only:
        // a float x + 0.0 is kept because it turns -0.0 into +0.0
        if (!e->dtype.is_float()) {
            if (e->kind == ExprKind::kAdd && IsConstInt(args[1], 0)) return args[0];
            if (e->kind == ExprKind::kAdd && IsConstInt(args[0], 0) && args[1].dtype() == e->dtype) return args[1];
            if (e->kind == ExprKind::kSub && IsConstInt(args[1], 0)) return args[0];
            if (e->kind == ExprKind::kMul && IsConstInt(args[1], 1)) return args[0];
            if (e->kind == ExprKind::kMul && IsConstInt(args[0], 1) && args[1].dtype() == e->dtype) return args[1];
            if (e->kind == ExprKind::kDiv && IsConstInt(args[1], 1)) return args[0];
        } else {
            if (e->kind == ExprKind::kMul && IsConstFloat(args[1], 1.0)) return args[0];
            if (e->kind == ExprKind::kDiv && IsConstFloat(args[1], 1.0)) return args[0];
        }
    }
    return rebuild();
}

Stmt FoldAndSimplify(const Stmt& s) {
    if (!s.defined()) return s;
    auto n = std::make_shared<StmtNode>(*s.get());
    if (n->a.defined()) n->a = FoldAndSimplify(n->a);
    if (n->b.defined()) n->b = FoldAndSimplify(n->b);
    for (auto& e : n->extents) e = FoldAndSimplify(e);
    for (auto& b : n->body) b = FoldAndSimplify(b);
    return Stmt(n);
}

PrimFunc RunTIRPassPipeline(const PrimFunc& f, const std::vector<std::string>& passes) {
    bool any = false;
    for (const auto& p : passes) {
        if (p == "fold_constant" || p == "simplify_expr" || p == "optimize_default") any = true;
        else throw std::runtime_error("Unknown TIR pass: " + p);
    }
    if (!any) return f;
    auto n = std::make_shared<PrimFuncNode>(*f.get());
    n->body = FoldAndSimplify(f->body);
    return PrimFunc(n);
}

}  // namespace tir
}  // namespace kxc
