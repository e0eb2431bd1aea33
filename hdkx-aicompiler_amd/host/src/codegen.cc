// codegen.cc -- see codegen.h.
#include "kxc/codegen.h"

#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <cstdio>
#include <functional>
#include <map>
#include <set>
#include <sstream>
#include <unordered_map>

namespace kxc {
namespace codegen {

using tir::DataType;
using tir::ExprKind;
using tir::ExprNode;
using tir::PrimExpr;
using tir::Stmt;
using tir::StmtKind;

namespace {

// builtin = true: spell integer types with language keywords (run-time compiled device code has no <stdint.h>)
std::string CType(DataType t, bool builtin = false) {
    if (t.is_float()) return t.bits == 64 ? "double" : "float";
    if (t.is_bool()) return "bool";
    if (builtin) {
        const int bits = t.bits == 1 ? 8 : t.bits;
        const char* base = bits == 8 ? "char" : bits == 16 ? "short" : bits == 32 ? "int" : "long long";
        return std::string(t.is_uint() ? "unsigned " : (bits == 8 ? "signed " : "")) + base;
    }
    const std::string base = "int" + std::to_string(t.bits == 1 ? 8 : t.bits) + "_t";
    return t.is_uint() ? "u" + base : base;
}

// Assigns every variable node a C identifier that is unique within one generated function/module.
class Names {
public:
    std::string Get(const ExprNode* v) {
        auto it = names_.find(v);
        if (it != names_.end()) return it->second;
        std::string base;
        for (char c : v->name) base += (std::isalnum(static_cast<unsigned char>(c)) || c == '_') ? c : '_';
        if (base.empty() || std::isdigit(static_cast<unsigned char>(base[0]))) base = "v_" + base;
        std::string name = base;
        for (int k = 1; used_.count(name); ++k) name = base + "_" + std::to_string(k);
        used_.insert(name);
        names_[v] = name;
        return name;
    }
    void Reserve(const std::string& s) { used_.insert(s); }
    bool builtin_types = false;

private:
    std::unordered_map<const ExprNode*, std::string> names_;
    std::set<std::string> used_;
};

// Expression text shared by both generators.  C's usual arithmetic conversions promote mixed operands
// to the wider / floating type, which is the reference's promotion rule
// (src/codegen/codegen_llvm.cc:189-217,266-273); Min/Max are compare + select with an ordered compare
// (:317-334), Select is a conditional (:391-442).
// overrides: text to emit in place of given nodes (the LDS-staged loads of a scheduled reduction)
using ExprOverrides = std::map<const ExprNode*, std::string>;
std::string EmitExpr(const PrimExpr& e, Names* names, const ExprOverrides* overrides = nullptr) {
    if (!e.defined()) return "0";
    if (overrides) {
        auto it = overrides->find(e.get());
        if (it != overrides->end()) return it->second;
    }
    auto A = [&](int i) { return EmitExpr(e->args[i], names, overrides); };
    char buf[64];
    switch (e->kind) {
        case ExprKind::kIntImm:
            if (e->dtype.is_bool()) return e->ivalue ? "true" : "false";
            if (e->dtype.bits == 64) return "((" + CType(e->dtype, names->builtin_types) + ")" + std::to_string(e->ivalue) + "LL)";
            return std::to_string(e->ivalue);
        case ExprKind::kFloatImm:
            if (std::isinf(e->fvalue)) return e->fvalue > 0 ? "INFINITY" : "(-INFINITY)";
            if (std::isnan(e->fvalue)) return "NAN";
            std::snprintf(buf, sizeof(buf), e->dtype.bits == 32 ? "%.9ef" : "%.17e", e->fvalue);
            return buf;
        case ExprKind::kVar: return names->Get(e.get());
        case ExprKind::kAdd: return "(" + A(0) + " + " + A(1) + ")";
        case ExprKind::kSub: return "(" + A(0) + " - " + A(1) + ")";
        case ExprKind::kMul: return "(" + A(0) + " * " + A(1) + ")";
        case ExprKind::kDiv: return "(" + A(0) + " / " + A(1) + ")";
        case ExprKind::kMod:
            if (PromoteTypes(e->args[0].dtype(), e->args[1].dtype()).is_float()) return "fmod(" + A(0) + ", " + A(1) + ")";
            return "(" + A(0) + " % " + A(1) + ")";
        case ExprKind::kMin: { std::string a = A(0), b = A(1); return "((" + a + ") < (" + b + ") ? (" + a + ") : (" + b + "))"; }
        case ExprKind::kMax: { std::string a = A(0), b = A(1); return "((" + a + ") > (" + b + ") ? (" + a + ") : (" + b + "))"; }
        case ExprKind::kEQ: return "(" + A(0) + " == " + A(1) + ")";
        case ExprKind::kLT: return "(" + A(0) + " < " + A(1) + ")";
        case ExprKind::kAnd: return "(" + A(0) + " && " + A(1) + ")";
        case ExprKind::kOr: return "(" + A(0) + " || " + A(1) + ")";
        case ExprKind::kNot: return "(!" + A(0) + ")";
        case ExprKind::kLoad: return A(0) + "[" + A(1) + "]";
        case ExprKind::kSelect: return "(" + A(0) + " ? " + A(1) + " : " + A(2) + ")";
        case ExprKind::kCall: {
            if (e->name == "cast") return "((" + CType(e->dtype, names->builtin_types) + ")(" + A(0) + "))";
            static const std::map<std::string, std::string> f32 = {{"exp", "expf"}, {"log", "logf"}, {"sqrt", "sqrtf"},
                {"floor", "floorf"}, {"ceil", "ceilf"}, {"fabs", "fabsf"}, {"tanh", "tanhf"},
                // round to nearest, ties to even (the default rounding mode): the quantised operators' rounding
                {"rint", "rintf"}};
            std::string name = e->name;
            if (name.rfind("tir.", 0) == 0) name = name.substr(4);
            auto it = f32.find(name);
            if (it == f32.end()) throw std::runtime_error("code generator: unsupported intrinsic " + e->name);
            std::string fn = e->dtype.bits == 64 ? name : it->second;
            std::string out = fn + "(";
            for (size_t i = 0; i < e->args.size(); ++i) out += (i ? ", " : "") + A(static_cast<int>(i));
            return out + ")";
        }
        default: throw std::runtime_error("code generator: TE-only expression reached the back end");
    }
}

void EmitStmt(const Stmt& s, Names* names, std::ostringstream& os, int indent) {
    if (!s.defined()) return;
    const std::string pad(indent, ' ');
    switch (s->kind) {
        case StmtKind::kFor: {
            const std::string v = names->Get(s->var.get());
            const std::string lo = EmitExpr(s->a, names), ext = EmitExpr(s->b, names);
            os << pad << "for (int " << v << " = " << lo << "; " << v << " < (" << lo << " + " << ext << "); ++" << v
               << ") {\n";
            EmitStmt(s->body[0], names, os, indent + 2);
            os << pad << "}\n";
            break;
        }
        case StmtKind::kStore:
            os << pad << names->Get(s->var.get()) << "[" << EmitExpr(s->b, names) << "] = " << EmitExpr(s->a, names) << ";\n";
            break;
        case StmtKind::kLetStmt:
            os << pad << "{\n" << pad << "  const " << CType(s->var.dtype(), names->builtin_types) << " " << names->Get(s->var.get()) << " = "
               << EmitExpr(s->a, names) << ";\n";
            EmitStmt(s->body[0], names, os, indent + 2);
            os << pad << "}\n";
            break;
        case StmtKind::kIfThenElse:
            os << pad << "if (" << EmitExpr(s->a, names) << ") {\n";
            EmitStmt(s->body[0], names, os, indent + 2);
            if (s->body.size() > 1) {
                os << pad << "} else {\n";
                EmitStmt(s->body[1], names, os, indent + 2);
            }
            os << pad << "}\n";
            break;
        case StmtKind::kSeqStmt:
            for (const auto& b : s->body) EmitStmt(b, names, os, indent);
            break;
        case StmtKind::kEvaluate: os << pad << EmitExpr(s->a, names) << ";\n"; break;
        case StmtKind::kAllocate: throw std::runtime_error("code generator: Allocate inside a compute stage");
    }
}

// Peels the Allocate nest off a PrimFunc body and returns the top-level stages.
void SplitStages(const Stmt& body, std::vector<Stmt>* allocs, std::vector<Stmt>* stages) {
    Stmt cur = body;
    while (cur.defined() && cur->kind == StmtKind::kAllocate) {
        allocs->push_back(cur);
        cur = cur->body[0];
    }
    if (!cur.defined()) return;
    if (cur->kind == StmtKind::kSeqStmt) {
        for (const auto& s : cur->body) {
            if (s.defined() && s->kind == StmtKind::kAllocate) throw std::runtime_error("code generator: nested Allocate in a sequence");
            stages->push_back(s);
        }
    } else {
        stages->push_back(cur);
    }
}

void CollectBuffers(const PrimExpr& e, std::vector<const ExprNode*>* out) {
    if (!e.defined()) return;
    if (e->kind == ExprKind::kLoad) {
        const ExprNode* b = e->args[0].get();
        if (std::find(out->begin(), out->end(), b) == out->end()) out->push_back(b);
        CollectBuffers(e->args[1], out);
        return;
    }
    for (const auto& a : e->args) CollectBuffers(a, out);
}
void CollectBuffers(const Stmt& s, std::vector<const ExprNode*>* out, std::vector<const ExprNode*>* written) {
    if (!s.defined()) return;
    if (s->kind == StmtKind::kStore) {
        const ExprNode* b = s->var.get();
        if (std::find(out->begin(), out->end(), b) == out->end()) out->push_back(b);
        if (std::find(written->begin(), written->end(), b) == written->end()) written->push_back(b);
    }
    CollectBuffers(s->a, out);
    CollectBuffers(s->b, out);
    for (const auto& b : s->body) CollectBuffers(b, out, written);
}

}  // namespace

// =================================================================== host C
std::string CodeGenC::Generate(const tir::PrimFunc& func, const std::string& name) {
    Names names;
    names.Reserve("packed_args");
    std::ostringstream os;
    os << "#include <stdint.h>\n#include <stdbool.h>\n#include <stdlib.h>\n#include <math.h>\n\n";
    os << "int32_t " << name << "(void** packed_args) {\n";
    for (size_t i = 0; i < func->params.size(); ++i) {
        const auto& p = func->params[i];
        os << "  " << CType(p.dtype()) << "* restrict " << names.Get(p.get()) << " = (" << CType(p.dtype())
           << "*)packed_args[" << i << "];\n";
    }
    std::vector<Stmt> allocs, stages;
    SplitStages(func->body, &allocs, &stages);
    std::vector<std::string> to_free;
    for (const auto& a : allocs) {
        int64_t count = 1;
        for (const auto& e : a->extents) {
            int64_t v;
            if (!tir::GetConstInt(e, &v)) throw std::runtime_error("CodeGenC: non-constant allocation extent");
            count *= v;
        }
        const std::string v = names.Get(a->var.get());
        os << "  " << CType(a->dtype) << "* restrict " << v << " = (" << CType(a->dtype) << "*)malloc((size_t)"
           << count << " * sizeof(" << CType(a->dtype) << "));\n";
        os << "  if (!" << v << ") return 1;\n";
        to_free.push_back(v);
    }
    for (const auto& st : stages) EmitStmt(st, &names, os, 2);
    for (auto it = to_free.rbegin(); it != to_free.rend(); ++it) os << "  free(" << *it << ");\n";
    os << "  return 0;\n}\n";
    return os.str();
}

// =================================================================== gfx950 HIP
namespace {

struct Affine {
    bool ok = true;
    int64_t constant = 0;
    std::map<const ExprNode*, int64_t> coef;
};

Affine AnalyzeAffine(const PrimExpr& e) {
    Affine r;
    if (!e.defined()) { r.ok = false; return r; }
    switch (e->kind) {
        case ExprKind::kIntImm: r.constant = e->ivalue; return r;
        case ExprKind::kVar: r.coef[e.get()] = 1; return r;
        case ExprKind::kAdd: case ExprKind::kSub: {
            Affine a = AnalyzeAffine(e->args[0]), b = AnalyzeAffine(e->args[1]);
            if (!a.ok || !b.ok) { r.ok = false; return r; }
            const int64_t sign = e->kind == ExprKind::kAdd ? 1 : -1;
            r = a;
            r.constant += sign * b.constant;
            for (auto& kv : b.coef) r.coef[kv.first] += sign * kv.second;
            return r;
        }
        case ExprKind::kMul: {
            Affine a = AnalyzeAffine(e->args[0]), b = AnalyzeAffine(e->args[1]);
            if (!a.ok || !b.ok) { r.ok = false; return r; }
            if (!a.coef.empty() && !b.coef.empty()) { r.ok = false; return r; }
            const Affine& lin = a.coef.empty() ? b : a;
            const int64_t k = a.coef.empty() ? a.constant : b.constant;
            r.constant = lin.constant * k;
            for (auto& kv : lin.coef) r.coef[kv.first] = kv.second * k;
            return r;
        }
        default: r.ok = false; return r;
    }
}

struct LoopNest {
    std::vector<tir::Var> vars;
    std::vector<int64_t> extents;
    Stmt body;
};

// Strips the outer data-parallel loops (constant extent, zero minimum).
LoopNest PeelLoops(Stmt s, bool stop_at_seq) {
    LoopNest n;
    while (s.defined() && s->kind == StmtKind::kFor) {
        int64_t lo, ext;
        if (!tir::GetConstInt(s->a, &lo) || !tir::GetConstInt(s->b, &ext) || lo != 0) break;
        n.vars.push_back(s->var);
        n.extents.push_back(ext);
        s = s->body[0];
        if (stop_at_seq && s.defined() && s->kind == StmtKind::kSeqStmt) break;
    }
    n.body = s;
    return n;
}

// Recognises  for data axes { out[o] = init; for reduce axes { out[o] = out[o] (+) src[o*R + r] } }  with
// contiguous rows: every data-axis coefficient of the source index is R times its coefficient in the
// output index and the reduce axes enumerate 0..R-1 in row-major order.
bool MatchRowReduce(const LoopNest& data, Stmt* init_out, PrimExpr* src_load, int64_t* R, int* reduce_kind,
                    const ExprNode** out_buf) {
    const Stmt& b = data.body;
    if (!b.defined() || b->kind != StmtKind::kSeqStmt || b->body.size() != 2) return false;
    const Stmt& init = b->body[0];
    if (init->kind != StmtKind::kStore) return false;
    LoopNest red = PeelLoops(b->body[1], false);
    if (red.vars.empty() || !red.body.defined() || red.body->kind != StmtKind::kStore) return false;
    const Stmt& upd = red.body;
    if (upd->var.get() != init->var.get()) return false;
    const PrimExpr& v = upd->a;
    if (v->kind != ExprKind::kAdd) return false;            // sums only: the staged loop keeps the order
    const PrimExpr& old = v->args[0];
    const PrimExpr& src = v->args[1];
    if (old->kind != ExprKind::kLoad || old->args[0].get() != init->var.get()) return false;
    if (src->kind != ExprKind::kLoad || src->args[0].get() == init->var.get()) return false;
    int64_t rows = 1;
    for (auto e : red.extents) rows *= e;
    if (rows < 2 || rows > 63) return false;                 // 256 rows of (R|1) floats must fit 64 KiB of LDS
    if (!src.dtype().is_float() || src.dtype().bits != 32) return false;
    Affine oi = AnalyzeAffine(init->b), ui = AnalyzeAffine(upd->b), si = AnalyzeAffine(src->args[1]);
    if (!oi.ok || !ui.ok || !si.ok || oi.constant != 0 || si.constant != 0) return false;
    if (oi.coef != ui.coef || oi.constant != ui.constant) return false;
    // output index must be the flattened data index
    int64_t stride = 1;
    for (int i = static_cast<int>(data.vars.size()) - 1; i >= 0; --i) {
        const int64_t c = oi.coef.count(data.vars[i].get()) ? oi.coef.at(data.vars[i].get()) : 0;
        if (data.extents[i] != 1 && c != stride) return false;
        const int64_t sc = si.coef.count(data.vars[i].get()) ? si.coef.at(data.vars[i].get()) : 0;
        if (data.extents[i] != 1 && sc != stride * rows) return false;
        stride *= data.extents[i];
    }
    int64_t rs = 1;
    for (int i = static_cast<int>(red.vars.size()) - 1; i >= 0; --i) {
        const int64_t c = si.coef.count(red.vars[i].get()) ? si.coef.at(red.vars[i].get()) : 0;
        if (red.extents[i] != 1 && c != rs) return false;
        if (oi.coef.count(red.vars[i].get()) && oi.coef.at(red.vars[i].get()) != 0) return false;
        rs *= red.extents[i];
    }
    *init_out = init;
    *src_load = src;
    *R = rows;
    *reduce_kind = 0;
    *out_buf = init->var.get();
    return true;
}

// Recognises  for data axes { out[o] = init; for reduce axes { out[o] = out[o] + EXPR } }  where the innermost
// reduce axis k has a constant extent of at least 16 and EXPR holds fp32 loads that walk memory contiguously along k
// (dense / matmul with a transposed operand, long row sums): every thread reads a run of consecutive floats, so the
// lanes of a wave read addresses a whole row apart.  Such loads are staged through LDS a chunk of k at a time.
struct KStage {
    Stmt init, upd;
    LoopNest red;
    PrimExpr expr;                       // EXPR
    std::vector<PrimExpr> staged;        // the load nodes that go through LDS
    int64_t extent = 0;                  // of the innermost reduce axis
    int chunk = 0;                       // floats of a row staged at a time
};

// Every load of `e` with whether it is evaluated unconditionally.  A load in a branch of a select, or in the right
// operand of a short-circuit `and` / `or`, runs only when its guard lets it (a padded window reads the input only
// inside the image); staging such a load for a whole tile of rows would read addresses the guard excludes, before
// the buffer or past its end.
void CollectLoads(const PrimExpr& e, bool guarded, std::vector<std::pair<PrimExpr, bool>>* out) {
    if (!e.defined()) return;
    if (e->kind == ExprKind::kLoad) out->emplace_back(e, guarded);
    for (size_t i = 0; i < e->args.size(); ++i) {
        const bool lazy = (e->kind == ExprKind::kSelect && i >= 1) || ((e->kind == ExprKind::kAnd || e->kind == ExprKind::kOr) && i >= 1);
        CollectLoads(e->args[i], guarded || lazy, out);
    }
}

bool MatchKStage(const LoopNest& data, KStage* m) {
    const Stmt& b = data.body;
    if (!b.defined() || b->kind != StmtKind::kSeqStmt || b->body.size() != 2 || data.vars.empty()) return false;
    const Stmt& init = b->body[0];
    if (init->kind != StmtKind::kStore) return false;
    LoopNest red = PeelLoops(b->body[1], false);
    if (red.vars.empty() || !red.body.defined() || red.body->kind != StmtKind::kStore) return false;
    const Stmt& upd = red.body;
    if (upd->var.get() != init->var.get()) return false;
    if (!upd->a.defined() || upd->a->kind != ExprKind::kAdd) return false;       // sums only: the order is kept
    const PrimExpr& old = upd->a->args[0];
    if (old->kind != ExprKind::kLoad || old->args[0].get() != init->var.get()) return false;
    Affine oi = AnalyzeAffine(init->b), ui = AnalyzeAffine(upd->b), li = AnalyzeAffine(old->args[1]);
    if (!oi.ok || !ui.ok || !li.ok || oi.coef != ui.coef || oi.constant != ui.constant || oi.coef != li.coef ||
        oi.constant != li.constant)
        return false;
    for (const auto& v : red.vars)
        if (oi.coef.count(v.get()) && oi.coef.at(v.get()) != 0) return false;     // the output does not move with the reduction
    if (!init->a.defined() || !init->a.dtype().is_float() || init->a.dtype().bits != 32) return false;
    const tir::Var& rk = red.vars.back();
    const int64_t extent = red.extents.back();
    if (extent < 16) return false;
    std::vector<std::pair<PrimExpr, bool>> loads;
    CollectLoads(upd->a->args[1], false, &loads);
    const tir::Var& lane_var = data.vars.back();
    const int64_t lane_extent = data.extents.back();
    for (const auto& entry : loads) {
        const PrimExpr& l = entry.first;
        if (l->args[0].get() == init->var.get()) return false;                  // EXPR reads the output: not a plain sum
        if (entry.second) continue;                                             // guarded: stays a lazy global load
        if (!l.dtype().is_float() || l.dtype().bits != 32) continue;
        Affine ai = AnalyzeAffine(l->args[1]);
        if (!ai.ok || !ai.coef.count(rk.get()) || ai.coef.at(rk.get()) != 1) continue;
        bool thread_dependent = false;
        for (const auto& v : data.vars)
            if (ai.coef.count(v.get()) && ai.coef.at(v.get()) != 0) thread_dependent = true;
        if (!thread_dependent) continue;
        // the same row for (nearly) every lane of a wave is a broadcast load already
        const int64_t lane_coef = ai.coef.count(lane_var.get()) ? ai.coef.at(lane_var.get()) : 0;
        if (lane_coef == 0 && lane_extent >= 64) continue;
        m->staged.push_back(l);
    }
    if (m->staged.empty() || m->staged.size() > 2) return false;
    m->init = init; m->upd = upd; m->red = red; m->expr = upd->a->args[1];
    m->extent = extent;
    m->chunk = m->staged.size() == 1 ? 32 : 16;      // 256 rows x (chunk + 1) floats per staged load: 33 / 2 x 17 KiB
    return true;
}

// Recognises  for data axes { out[o] = init; for reduce axes { out[o] = out[o] + EXPR } }  (fp32) where EXPR's loads
// split over the data axes: some loads do not move with an axis others move with (a convolution's input window does
// not depend on the output channel, its weights on nothing else).  A thread then owns a small block of outputs along up
// to two such axes and every loaded value feeds several accumulators; each output is still summed by one thread
// in the CPU order.  `tile[i]` is the block extent along `axis[i]` (an index into the data axes; -1 = unused).
struct RegTile {
    Stmt init, upd;
    LoopNest red;
    PrimExpr expr;
    int axis[2] = {-1, -1};
    int tile[2] = {1, 1};
    int64_t units = 0;                  // threads' worth of work: blocks of outputs
};

bool MatchRegTile(const LoopNest& data, int64_t min_units, RegTile* m) {
    const Stmt& b = data.body;
    if (!b.defined() || b->kind != StmtKind::kSeqStmt || b->body.size() != 2 || data.vars.size() < 2) return false;
    const Stmt& init = b->body[0];
    if (init->kind != StmtKind::kStore) return false;
    LoopNest red = PeelLoops(b->body[1], false);
    if (red.vars.empty() || !red.body.defined() || red.body->kind != StmtKind::kStore) return false;
    const Stmt& upd = red.body;
    if (upd->var.get() != init->var.get()) return false;
    if (!upd->a.defined() || upd->a->kind != ExprKind::kAdd) return false;
    const PrimExpr& old = upd->a->args[0];
    if (old->kind != ExprKind::kLoad || old->args[0].get() != init->var.get()) return false;
    Affine oi = AnalyzeAffine(init->b), ui = AnalyzeAffine(upd->b), li = AnalyzeAffine(old->args[1]);
    if (!oi.ok || !ui.ok || !li.ok || oi.coef != ui.coef || oi.constant != ui.constant || oi.coef != li.coef ||
        oi.constant != li.constant)
        return false;
    for (const auto& v : red.vars)
        if (oi.coef.count(v.get()) && oi.coef.at(v.get()) != 0) return false;
    if (!init->a.defined() || !init->a.dtype().is_float() || init->a.dtype().bits != 32) return false;
    int64_t reduce_extent = 1;
    for (auto e : red.extents) reduce_extent *= e;
    if (reduce_extent < 4) return false;
    std::vector<std::pair<PrimExpr, bool>> loads;
    CollectLoads(upd->a->args[1], false, &loads);
    CollectLoads(init->a, false, &loads);
    if (loads.size() < 2) return false;
    const int nd = static_cast<int>(data.vars.size());
    // moves[l][a]: load l's address changes with data axis a (an index that is not affine counts as moving with all)
    std::vector<std::vector<bool>> moves;
    for (const auto& entry : loads) {
        if (entry.first->args[0].get() == init->var.get()) return false;        // EXPR reads the output
        Affine ai = AnalyzeAffine(entry.first->args[1]);
        std::vector<bool> row(static_cast<size_t>(nd), true);
        if (ai.ok)
            for (int a = 0; a < nd; ++a) row[static_cast<size_t>(a)] = ai.coef.count(data.vars[a].get()) && ai.coef.at(data.vars[a].get()) != 0;
        moves.push_back(row);
    }
    const int lane = nd - 1;                                                   // consecutive lanes walk the innermost axis
    auto shares = [&](int a, bool lane_varying_only) {
        bool still = false, moving = false;
        for (const auto& row : moves) {
            if (row[static_cast<size_t>(a)]) moving = true;
            else if (!lane_varying_only || row[static_cast<size_t>(lane)]) still = true;
        }
        return still && moving;
    };
    // first axis: one along which a per-lane load (the expensive kind) is shared; else any axis that shares a load
    int a1 = -1;
    for (int pass = 0; pass < 2 && a1 < 0; ++pass)
        for (int a = 0; a < lane && a1 < 0; ++a)
            if (data.extents[a] >= 2 && shares(a, pass == 0)) a1 = a;
    if (a1 < 0) return false;
    // second axis (innermost candidate first): it must share a load that moves with the first
    int a2 = -1;
    for (int a = lane - 1; a >= 0 && a2 < 0; --a) {
        if (a == a1 || data.extents[a] < 2) continue;
        for (const auto& row : moves)
            if (row[static_cast<size_t>(a1)] && !row[static_cast<size_t>(a)]) a2 = a;
    }
    int64_t total = 1;
    for (auto e : data.extents) total *= e;
    auto units_for = [&](int t1, int t2) {
        int64_t u = total / data.extents[a1] * ((data.extents[a1] + t1 - 1) / t1);
        if (a2 >= 0) u = u / data.extents[a2] * ((data.extents[a2] + t2 - 1) / t2);
        return u;
    };
    int t1 = static_cast<int>(std::min<int64_t>(4, data.extents[a1]));
    int t2 = a2 >= 0 ? static_cast<int>(std::min<int64_t>(4, data.extents[a2])) : 1;
    // keep the machine full: fewer, fatter threads only while there is at least `min_units` of them
    while (t2 > 1 && units_for(t1, t2) < min_units) t2 = (t2 + 1) / 2;
    while (t1 > 1 && units_for(t1, t2) < min_units) t1 = (t1 + 1) / 2;
    if (t1 * t2 < 2) return false;
    if (t1 == 1) { a1 = a2; t1 = t2; a2 = -1; t2 = 1; }
    if (t2 == 1) a2 = -1;
    m->init = init; m->upd = upd; m->red = red; m->expr = upd->a->args[1];
    m->axis[0] = a1; m->axis[1] = a2; m->tile[0] = t1; m->tile[1] = t2;
    m->units = units_for(t1, t2);
    return true;
}

// Which of the two tiled axes an expression reads (bit 0: `a`, bit 1: `b`), and whether it loads from memory.
int TileDeps(const PrimExpr& e, const ExprNode* a, const ExprNode* b) {
    if (!e.defined()) return 0;
    if (e->kind == ExprKind::kVar) return (e.get() == a ? 1 : 0) | (b && e.get() == b ? 2 : 0);
    int d = 0;
    for (const auto& x : e->args) d |= TileDeps(x, a, b);
    return d;
}
bool HasLoad(const PrimExpr& e) {
    if (!e.defined()) return false;
    if (e->kind == ExprKind::kLoad) return true;
    for (const auto& x : e->args)
        if (HasLoad(x)) return true;
    return false;
}
// The largest sub-expressions with a load that read only some of the tiled axes: a block of outputs evaluates each once
// per index of the axes it does read, not once per output.  Nothing is taken out of a branch that is evaluated lazily
// (a padded window's input load stays behind its bounds test; the whole select moves).
struct SharedTerm { PrimExpr e; int deps; };
void CollectSharedTerms(const PrimExpr& e, const ExprNode* a, const ExprNode* b, std::vector<SharedTerm>* out) {
    if (!e.defined() || out->size() >= 8) return;
    const int full = 1 | (b ? 2 : 0);
    const int d = TileDeps(e, a, b);
    if (d != full) {
        if (HasLoad(e)) out->push_back({e, d});
        return;
    }
    const bool lazy = e->kind == ExprKind::kSelect || e->kind == ExprKind::kAnd || e->kind == ExprKind::kOr;
    for (size_t i = 0; i < e->args.size(); ++i)
        if (!lazy || i == 0) CollectSharedTerms(e->args[i], a, b, out);
}

}  // namespace

HIPModuleSource CodeGenHIP::Generate(const tir::PrimFunc& func, const std::string& prefix) {
    HIPModuleSource out;
    Names names;
    names.builtin_types = true;
    // identifiers the schedules below declare themselves: no buffer or loop variable may take them
    for (const char* id : {"tile", "tile0", "tile1", "rowbase0", "rowbase1", "total", "base", "rows", "row", "e", "k", "kk",
                           "k0", "kend", "acc", "gid", "rem", "valid", "r"})
        names.Reserve(id);
    for (const char* id : {"ta_base", "tb_base"}) names.Reserve(id);
    for (int i = 0; i < 4; ++i) {
        names.Reserve("ta" + std::to_string(i));
        names.Reserve("tb" + std::to_string(i));
        for (int j = 0; j < 4; ++j) names.Reserve("acc" + std::to_string(i) + std::to_string(j));
    }
    for (int k = 0; k < 8; ++k) {
        names.Reserve("u" + std::to_string(k));
        for (int i = 0; i < 4; ++i) names.Reserve("u" + std::to_string(k) + "_" + std::to_string(i));
    }
    // threads a register-tiled stage must keep (one workgroup of 256 on each of the 256 compute units)
    int64_t tile_min_units = 65536;
    if (const char* v = std::getenv("KXC_HIPGEN_TILE_MIN_UNITS")) tile_min_units = std::max<int64_t>(1, std::atoll(v));
    std::ostringstream os;
    os << "// generated by kxc CodeGenHIP for gfx950 (wave64)\n";
    os << "#ifndef INFINITY\n#define INFINITY __builtin_inff()\n#endif\n#ifndef NAN\n#define NAN __builtin_nanf(\"\")\n#endif\n\n";

    std::vector<Stmt> allocs, stages;
    SplitStages(func->body, &allocs, &stages);
    std::map<const ExprNode*, DataType> buffer_types;
    for (const auto& p : func->params) buffer_types[p.get()] = p.dtype();
    for (const auto& a : allocs) buffer_types[a->var.get()] = a->dtype;

    int index = 0;
    for (const auto& stage : stages) {
        HIPKernelSpec spec;
        std::vector<const ExprNode*> written;
        CollectBuffers(stage, &spec.buffers, &written);
        for (const ExprNode* b : spec.buffers)
            if (!buffer_types.count(b)) throw std::runtime_error("CodeGenHIP: stage uses an undeclared buffer '" + b->name + "'");
        const std::string target = written.empty() ? "stage" : names.Get(written[0]);
        spec.symbol = prefix + "_s" + std::to_string(index++) + "_" + target;
        names.Reserve(spec.symbol);

        LoopNest data = PeelLoops(stage, true);
        int64_t total = 1;
        for (auto e : data.extents) total *= e;
        if (total <= 0) total = 1;

        os << "extern \"C\" __global__ void __launch_bounds__(256) " << spec.symbol << "(";
        for (size_t i = 0; i < spec.buffers.size(); ++i) {
            const ExprNode* b = spec.buffers[i];
            const bool is_written = std::find(written.begin(), written.end(), b) != written.end();
            os << (i ? ", " : "") << (is_written ? "" : "const ") << CType(buffer_types[b], true) << "* __restrict__ " << names.Get(b);
        }
        os << ") {\n";

        Stmt init;
        PrimExpr src;
        int64_t R = 0;
        int rkind = 0;
        const ExprNode* obuf = nullptr;
        if (MatchRowReduce(data, &init, &src, &R, &rkind, &obuf)) {
            // ---- LDS-staged contiguous row reduction
            const int64_t rp = R | 1;
            spec.schedule = "lds_row_reduce";
            spec.shared_bytes = 0;   // static LDS
            const std::string o = names.Get(obuf), s = names.Get(src->args[0].get());
            os << "  __shared__ float tile[" << 256 * rp << "];\n";
            os << "  const long long total = " << total << "LL;\n";
            os << "  for (long long base = (long long)blockIdx.x * 256; base < total; base += (long long)gridDim.x * 256) {\n";
            os << "    const int rows = (int)((total - base) < 256 ? (total - base) : 256);\n";
            os << "    for (int e = threadIdx.x; e < rows * " << R << "; e += 256) {\n";
            os << "      const int row = e / " << R << ";\n";
            os << "      tile[row * " << rp << " + (e - row * " << R << ")] = " << s << "[base * " << R << " + e];\n";
            os << "    }\n    __syncthreads();\n";
            os << "    if ((int)threadIdx.x < rows) {\n";
            os << "      " << CType(buffer_types[obuf], true) << " acc = " << EmitExpr(init->a, &names) << ";\n";
            os << "      for (int r = 0; r < " << R << "; ++r) acc = acc + tile[threadIdx.x * " << rp << " + r];\n";
            os << "      " << o << "[base + threadIdx.x] = acc;\n";
            os << "    }\n    __syncthreads();\n  }\n";
        } else if (KStage ks; MatchKStage(data, &ks)) {
            // ---- reduction whose k-contiguous operands are staged through LDS, a chunk of k at a time; every
            // thread still adds its products in the CPU order (acc = acc + EXPR for k = 0, 1, ...)
            spec.schedule = "lds_k_stage";
            const int KC = ks.chunk, KP = KC + 1;
            const std::string o = names.Get(ks.init->var.get());
            const std::string rk = names.Get(ks.red.vars.back().get());
            for (size_t j = 0; j < ks.staged.size(); ++j) {
                os << "  __shared__ float tile" << j << "[" << 256 * KP << "];\n";
                os << "  __shared__ long long rowbase" << j << "[256];\n";
            }
            os << "  const long long total = " << total << "LL;\n";
            os << "  for (long long base = (long long)blockIdx.x * 256; base < total; base += (long long)gridDim.x * 256) {\n";
            os << "    const long long gid = base + threadIdx.x;\n";
            os << "    const bool valid = gid < total;\n";
            os << "    long long rem = valid ? gid : total - 1;      // threads past the end help with the loads only\n";
            for (int i = static_cast<int>(data.vars.size()) - 1; i >= 0; --i) {
                const std::string v = names.Get(data.vars[i].get());
                if (i == 0) os << "    const int " << v << " = (int)rem;\n";
                else {
                    os << "    const int " << v << " = (int)(rem % " << data.extents[i] << "LL);\n";
                    os << "    rem /= " << data.extents[i] << "LL;\n";
                }
            }
            os << "    float acc = " << EmitExpr(ks.init->a, &names) << ";\n";
            std::string pad = "    ";
            for (size_t i = 0; i + 1 < ks.red.vars.size(); ++i) {
                const std::string v = names.Get(ks.red.vars[i].get());
                os << pad << "for (int " << v << " = 0; " << v << " < " << ks.red.extents[i] << "; ++" << v << ") {\n";
                pad += "  ";
            }
            os << pad << "{ const int " << rk << " = 0;\n";
            for (size_t j = 0; j < ks.staged.size(); ++j)
                os << pad << "  rowbase" << j << "[threadIdx.x] = (long long)(" << EmitExpr(ks.staged[j]->args[1], &names) << ");\n";
            os << pad << "}\n";
            os << pad << "for (int k0 = 0; k0 < " << ks.extent << "; k0 += " << KC << ") {\n";
            os << pad << "  __syncthreads();\n";
            os << pad << "  for (int e = threadIdx.x; e < " << 256 * KC << "; e += 256) {\n";
            os << pad << "    const int row = e / " << KC << ", k = e - row * " << KC << ";\n";
            os << pad << "    if (k0 + k < " << ks.extent << ") {\n";
            ExprOverrides overrides;
            for (size_t j = 0; j < ks.staged.size(); ++j) {
                os << pad << "      tile" << j << "[row * " << KP << " + k] = " << names.Get(ks.staged[j]->args[0].get())
                   << "[rowbase" << j << "[row] + k0 + k];\n";
                overrides[ks.staged[j].get()] = "tile" + std::to_string(j) + "[threadIdx.x * " + std::to_string(KP) + " + kk]";
            }
            os << pad << "    }\n";
            os << pad << "  }\n";
            os << pad << "  __syncthreads();\n";
            os << pad << "  const int kend = (" << ks.extent << " - k0) < " << KC << " ? (" << ks.extent << " - k0) : " << KC << ";\n";
            os << pad << "  for (int kk = 0; kk < kend; ++kk) {\n";
            os << pad << "    const int " << rk << " = k0 + kk;\n";
            os << pad << "    (void)" << rk << ";\n";
            os << pad << "    acc = acc + " << EmitExpr(ks.expr, &names, &overrides) << ";\n";
            os << pad << "  }\n";
            os << pad << "}\n";
            for (size_t i = 0; i + 1 < ks.red.vars.size(); ++i) {
                pad.resize(pad.size() - 2);
                os << pad << "}\n";
            }
            os << "    if (valid) " << o << "[" << EmitExpr(ks.init->b, &names) << "] = acc;\n";
            os << "  }\n";
        } else if (RegTile rt; MatchRegTile(data, tile_min_units, &rt)) {
            // ---- register-tiled reduction: a thread owns tile[0] x tile[1] outputs along two data axes; the loads
            // that do not move with an axis are shared by the accumulators along it (the compiler merges the equal
            // loads of the repeated expression); every output is summed by its one thread in the CPU order
            spec.schedule = "reg_tile";
            const std::string o = names.Get(rt.init->var.get());
            const char* base_name[2] = {"ta_base", "tb_base"};
            const char* value_name[2] = {"ta", "tb"};
            total = rt.units;
            os << "  for (long long gid = (long long)blockIdx.x * 256 + threadIdx.x; gid < " << total
               << "LL; gid += (long long)gridDim.x * 256) {\n";
            os << "    long long rem = gid;\n";
            for (int i = static_cast<int>(data.vars.size()) - 1; i >= 0; --i) {
                const int which = i == rt.axis[0] ? 0 : (i == rt.axis[1] ? 1 : -1);
                const int64_t steps = which < 0 ? data.extents[i] : (data.extents[i] + rt.tile[which] - 1) / rt.tile[which];
                const std::string v = which < 0 ? names.Get(data.vars[i].get()) : std::string(base_name[which]);
                const std::string scale = which < 0 ? "" : " * " + std::to_string(rt.tile[which]);
                if (i == 0) os << "    const int " << v << " = (int)rem" << scale << ";\n";
                else {
                    os << "    const int " << v << " = (int)(rem % " << steps << "LL)" << scale << ";\n";
                    os << "    rem /= " << steps << "LL;\n";
                }
                // a block that hangs over the end of its axis repeats the last index; its stores are skipped below
                for (int j = 0; which >= 0 && j < rt.tile[which]; ++j)
                    os << "    const int " << value_name[which] << j << " = " << v << " + " << j << " < " << data.extents[i] << " ? " << v
                       << " + " << j << " : " << data.extents[i] - 1 << ";\n";
            }
            auto at = [&](int i, int j) {
                ExprOverrides ov;
                ov[data.vars[static_cast<size_t>(rt.axis[0])].get()] = "ta" + std::to_string(i);
                if (rt.axis[1] >= 0) ov[data.vars[static_cast<size_t>(rt.axis[1])].get()] = "tb" + std::to_string(j);
                return ov;
            };
            for (int i = 0; i < rt.tile[0]; ++i)
                for (int j = 0; j < rt.tile[1]; ++j) {
                    const ExprOverrides ov = at(i, j);
                    os << "    float acc" << i << j << " = " << EmitExpr(rt.init->a, &names, &ov) << ";\n";
                }
            std::string pad = "    ";
            for (size_t i = 0; i < rt.red.vars.size(); ++i) {
                const std::string v = names.Get(rt.red.vars[i].get());
                os << pad << "for (int " << v << " = 0; " << v << " < " << rt.red.extents[i] << "; ++" << v << ") {\n";
                pad += "  ";
            }
            const ExprNode* va = data.vars[static_cast<size_t>(rt.axis[0])].get();
            const ExprNode* vb = rt.axis[1] >= 0 ? data.vars[static_cast<size_t>(rt.axis[1])].get() : nullptr;
            std::vector<SharedTerm> shared;
            CollectSharedTerms(rt.expr, va, vb, &shared);
            for (size_t k = 0; k < shared.size(); ++k) {
                const std::string u = "u" + std::to_string(k);
                if (shared[k].deps == 0) os << pad << "const auto " << u << " = " << EmitExpr(shared[k].e, &names) << ";\n";
                for (int i = 0; shared[k].deps == 1 && i < rt.tile[0]; ++i) {
                    const ExprOverrides ov = at(i, 0);
                    os << pad << "const auto " << u << "_" << i << " = " << EmitExpr(shared[k].e, &names, &ov) << ";\n";
                }
                for (int j = 0; shared[k].deps == 2 && j < rt.tile[1]; ++j) {
                    const ExprOverrides ov = at(0, j);
                    os << pad << "const auto " << u << "_" << j << " = " << EmitExpr(shared[k].e, &names, &ov) << ";\n";
                }
            }
            for (int i = 0; i < rt.tile[0]; ++i)
                for (int j = 0; j < rt.tile[1]; ++j) {
                    ExprOverrides ov = at(i, j);
                    for (size_t k = 0; k < shared.size(); ++k) {
                        const std::string u = "u" + std::to_string(k);
                        ov[shared[k].e.get()] = shared[k].deps == 0 ? u : u + "_" + std::to_string(shared[k].deps == 1 ? i : j);
                    }
                    os << pad << "acc" << i << j << " = acc" << i << j << " + " << EmitExpr(rt.expr, &names, &ov) << ";\n";
                }
            for (size_t i = 0; i < rt.red.vars.size(); ++i) {
                pad.resize(pad.size() - 2);
                os << pad << "}\n";
            }
            for (int i = 0; i < rt.tile[0]; ++i)
                for (int j = 0; j < rt.tile[1]; ++j) {
                    const ExprOverrides ov = at(i, j);
                    os << "    if (ta_base + " << i << " < " << data.extents[static_cast<size_t>(rt.axis[0])];
                    if (rt.axis[1] >= 0) os << " && tb_base + " << j << " < " << data.extents[static_cast<size_t>(rt.axis[1])];
                    os << ") " << o << "[" << EmitExpr(rt.init->b, &names, &ov) << "] = acc" << i << j << ";\n";
                }
            os << "  }\n";
        } else {
            // ---- flat schedule: one output element per thread per grid-stride step
            spec.schedule = "flat";
            os << "  for (long long gid = (long long)blockIdx.x * 256 + threadIdx.x; gid < " << total
               << "LL; gid += (long long)gridDim.x * 256) {\n";
            // innermost data axis is lane-fastest
            os << "    long long rem = gid;\n";
            for (int i = static_cast<int>(data.vars.size()) - 1; i >= 0; --i) {
                const std::string v = names.Get(data.vars[i].get());
                if (i == 0) os << "    const int " << v << " = (int)rem;\n";
                else {
                    os << "    const int " << v << " = (int)(rem % " << data.extents[i] << "LL);\n";
                    os << "    rem /= " << data.extents[i] << "LL;\n";
                }
            }
            EmitStmt(data.body, &names, os, 4);
            os << "  }\n";
        }
        os << "}\n\n";
        int64_t blocks = (total + 255) / 256;
        if (blocks > 256 * 32) blocks = 256 * 32;       // grid-stride beyond 32 workgroups per CU
        if (blocks < 1) blocks = 1;
        spec.grid[0] = static_cast<uint32_t>(blocks);
        out.kernels.push_back(spec);
    }
    out.source = os.str();
    return out;
}

}  // namespace codegen
}  // namespace kxc
