// tir.h -- the loop-level IR the code generators consume.
//
// Node set and meaning follow the reference's TIR (include/tir/expr.h:20-220, include/tir/stmt.h:33-321):
// expressions IntImm FloatImm Var Add Sub Mul Div Mod Min Max EQ LT And Or Not Load Call Select,
// statements LetStmt Store For IfThenElse Allocate SeqStmt Evaluate, PrimFunc{params, body, buffer_map,
// attrs}.  A binary expression takes the dtype of its left operand (src/tir/expr.cc:37-44); code
// generators promote mixed operands to the wider / floating type (src/codegen/codegen_llvm.cc:189-217).
// The representation is one tagged node type per family rather than a class per node.
#pragma once

#include <ostream>

#include <functional>
#include <limits>

#include "kxc/base.h"

namespace kxc {
namespace tir {

struct DataType {
    int code = 2;   // 0 int, 1 uint, 2 float, 3 handle, 4 void
    int bits = 32;
    int lanes = 1;
    static DataType Int(int bits = 32, int lanes = 1) { return {0, bits, lanes}; }
    static DataType UInt(int bits = 32, int lanes = 1) { return {1, bits, lanes}; }
    static DataType Float(int bits = 32, int lanes = 1) { return {2, bits, lanes}; }
    static DataType Bool() { return {1, 1, 1}; }
    static DataType Handle() { return {3, 64, 1}; }
    bool is_float() const { return code == 2; }
    bool is_int() const { return code == 0; }
    bool is_uint() const { return code == 1; }
    bool is_bool() const { return code == 1 && bits == 1; }
    bool operator==(const DataType& o) const { return code == o.code && bits == o.bits && lanes == o.lanes; }
    bool operator!=(const DataType& o) const { return !(*this == o); }
    int bytes() const { return bits == 1 ? 1 : bits / 8; }
};

// dtype strings of tensor types (src/relay/backend/lower.cc:33-42)
DataType DTypeFromString(const std::string& s);
std::string DTypeToString(DataType t);

enum class ExprKind {
    kIntImm, kFloatImm, kVar, kAdd, kSub, kMul, kDiv, kMod, kMin, kMax, kEQ, kLT, kAnd, kOr, kNot,
    kLoad, kCall, kSelect,
    kProducerLoad,   // TE only: tensor(indices)
    kReduce          // TE only: reduction over axes
};

class PrimExpr;
struct ExprNode;
struct TensorNode;   // te.h

struct ExprNode {
    ExprKind kind;
    DataType dtype;
    int64_t ivalue = 0;                    // IntImm
    double fvalue = 0.0;                   // FloatImm
    std::string name;                      // Var name hint / Call name
    std::vector<PrimExpr> args;            // operands; Load: {buffer var, index}; Select: {cond, t, f}
    // TE extensions
    std::shared_ptr<TensorNode> tensor;    // ProducerLoad
    int reduce_type = 0;                   // Reduce: 0 sum, 1 max, 2 min
    std::vector<PrimExpr> reduce_vars;     // Reduce: axis vars
    std::vector<PrimExpr> reduce_min, reduce_extent;
    virtual ~ExprNode() = default;
};

class PrimExpr : public Ref<ExprNode> {
public:
    PrimExpr() = default;
    explicit PrimExpr(std::shared_ptr<ExprNode> n) : Ref<ExprNode>(std::move(n)) {}
    PrimExpr(int v);                        // IntImm int32
    PrimExpr(int64_t v);                    // IntImm int64
    PrimExpr(float v);                      // FloatImm float32
    PrimExpr(double v);                     // FloatImm float64
    DataType dtype() const { return ptr_ ? ptr_->dtype : DataType(); }
};

// A Var is a PrimExpr of kind kVar; identity is the node address.
class Var : public PrimExpr {
public:
    Var() = default;
    explicit Var(std::string name, DataType dtype = DataType::Int(32));
    explicit Var(std::shared_ptr<ExprNode> n) : PrimExpr(std::move(n)) {}
    const std::string& name_hint() const { return ptr_->name; }
};

PrimExpr IntImm(int64_t v, DataType t = DataType::Int(32));
PrimExpr FloatImm(double v, DataType t = DataType::Float(32));
PrimExpr Add(PrimExpr a, PrimExpr b);
PrimExpr Sub(PrimExpr a, PrimExpr b);
PrimExpr Mul(PrimExpr a, PrimExpr b);
PrimExpr Div(PrimExpr a, PrimExpr b);
PrimExpr Mod(PrimExpr a, PrimExpr b);
PrimExpr Min(PrimExpr a, PrimExpr b);
PrimExpr Max(PrimExpr a, PrimExpr b);
PrimExpr EQ(PrimExpr a, PrimExpr b);
PrimExpr LT(PrimExpr a, PrimExpr b);
PrimExpr And(PrimExpr a, PrimExpr b);
PrimExpr Or(PrimExpr a, PrimExpr b);
PrimExpr Not(PrimExpr a);
PrimExpr Load(Var buffer, PrimExpr index, DataType dtype);
PrimExpr Call(DataType dtype, std::string name, std::vector<PrimExpr> args);
PrimExpr Select(PrimExpr cond, PrimExpr t, PrimExpr f);

inline PrimExpr operator+(PrimExpr a, PrimExpr b) { return Add(a, b); }
inline PrimExpr operator-(PrimExpr a, PrimExpr b) { return Sub(a, b); }
inline PrimExpr operator*(PrimExpr a, PrimExpr b) { return Mul(a, b); }
inline PrimExpr operator/(PrimExpr a, PrimExpr b) { return Div(a, b); }
inline PrimExpr operator%(PrimExpr a, PrimExpr b) { return Mod(a, b); }
inline PrimExpr operator<(PrimExpr a, PrimExpr b) { return LT(a, b); }
// built from LT and Not, as the reference's TOPI helpers do (include/te/topi/utils.h:62-66)
inline PrimExpr operator>(PrimExpr a, PrimExpr b) { return LT(b, a); }
inline PrimExpr operator>=(PrimExpr a, PrimExpr b) { return Not(LT(a, b)); }
inline PrimExpr operator<=(PrimExpr a, PrimExpr b) { return Not(LT(b, a)); }
inline PrimExpr operator&&(PrimExpr a, PrimExpr b) { return And(a, b); }
inline PrimExpr operator||(PrimExpr a, PrimExpr b) { return Or(a, b); }
inline PrimExpr operator!(PrimExpr a) { return Not(a); }

bool GetConstInt(const PrimExpr& e, int64_t* out);

// ------------------------------------------------------------------ statements
enum class ForType { Serial, Parallel, Vectorized, Unrolled };
enum class StmtKind { kLetStmt, kStore, kFor, kIfThenElse, kAllocate, kSeqStmt, kEvaluate };

class Stmt;
struct StmtNode {
    StmtKind kind;
    Var var;                         // For loop var / Let var / Store & Allocate buffer var
    PrimExpr a, b;                   // For: min, extent; Store: value, index; Let: value; If: condition; Evaluate: value
    ForType for_type = ForType::Serial;
    DataType dtype;                  // Allocate element type
    std::vector<PrimExpr> extents;   // Allocate
    std::vector<Stmt> body;          // For/Let/Allocate: {body}; If: {then[, else]}; Seq: all
    virtual ~StmtNode() = default;
};

class Stmt : public Ref<StmtNode> {
public:
    Stmt() = default;
    explicit Stmt(std::shared_ptr<StmtNode> n) : Ref<StmtNode>(std::move(n)) {}
};

Stmt LetStmt(Var var, PrimExpr value, Stmt body);
Stmt Store(Var buffer, PrimExpr value, PrimExpr index);
Stmt For(Var loop_var, PrimExpr min, PrimExpr extent, ForType type, Stmt body);
Stmt IfThenElse(PrimExpr cond, Stmt then_case, Stmt else_case = Stmt());
Stmt Allocate(Var buffer, DataType dtype, std::vector<PrimExpr> extents, PrimExpr condition, Stmt body);
Stmt SeqStmt(std::vector<Stmt> seq);
Stmt Evaluate(PrimExpr value);

struct BufferInfo {
    DataType dtype;
    std::vector<int64_t> shape;
    std::string name;
};

struct PrimFuncNode {
    std::vector<Var> params;
    Stmt body;
    std::map<const ExprNode*, BufferInfo> buffer_map;   // param var -> buffer
    std::map<std::string, int64_t> int_attrs;           // kxc.input_count, kxc.constant_count, ...
    std::map<std::string, std::string> str_attrs;       // global_symbol
};

class PrimFunc : public Ref<PrimFuncNode> {
public:
    PrimFunc() = default;
    explicit PrimFunc(std::shared_ptr<PrimFuncNode> n) : Ref<PrimFuncNode>(std::move(n)) {}
};

// Text dump (for diagnostics and tests).
std::string ToString(const PrimExpr& e);
std::string ToString(const Stmt& s, int indent = 0);
std::string ToString(const PrimFunc& f);

// The two passes of the JIT pipeline (src/tir/transforms/pipeline.cc:103-121): integer/float scalar
// folding and x+0, x*1, x/1 simplification.  Neither changes floating-point evaluation order.
PrimExpr FoldAndSimplify(const PrimExpr& e);
Stmt FoldAndSimplify(const Stmt& s);
PrimFunc RunTIRPassPipeline(const PrimFunc& f, const std::vector<std::string>& passes);

// Structured text dump of a PrimFunc under the reference's names (include/tir/pass/print_ir.h:14-27).
namespace pass {
class IRPrinterPass {
public:
    explicit IRPrinterPass(int indent_spaces = 2) : indent_spaces_(indent_spaces) {}
    void Run(const PrimFunc& func, std::ostream& os) const;

private:
    int indent_spaces_;
};
void DumpPrimFunc(const PrimFunc& func, std::ostream& os, int indent_spaces = 2);
}  // namespace pass

// The type two operands are promoted to before a binary operation.
DataType PromoteTypes(DataType a, DataType b);

}  // namespace tir
}  // namespace kxc
