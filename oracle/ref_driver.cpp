// ref_driver.cpp -- TEST INFRASTRUCTURE.  Builds only where the reference
// checkout is present (this file includes the reference's public headers and
// links its object files; see the Makefile's `ref` target).  It drives the
// reference's OWN pipeline
//     InferType -> Relay passes {fold_constant, simplify_expr} -> InferType
//     -> LowerToTIR -> TIR passes {fold_constant, simplify_expr} -> CodeGenC
// (the JIT-mode pass list of src/api/compiler.cc:83-100) for a list of operator
// cases and writes the C text the reference's CodeGenC produces for each case.
// The Makefile compiles that text with the host C compiler into
// oracle/_ref/libkxc_ref_cases.so.  That library is the reference's loop nests
// verbatim: the strongest available statement of what the CPU backend computes
// (the LLVM backend emits the same TIR with the same scalar order; it needs
// LLVM >= 20 development libraries and cannot be built offline).
//
// Usage: ref_driver <out.c>
//
// Every emitted function has the reference ABI `int32_t f(void** packed_args)`
// with arguments in the order inputs, constants (lowering order), outputs.

#include <cstdint>
#include <fstream>
#include <iostream>
#include <sstream>
#include <stdexcept>
#include <string>
#include <vector>

#include "codegen/codegen_c.h"
#include "relay/op.h"
#include "relay/relay.h"
#include "relay/transforms/infer_type.h"
#include "relay/transforms/lower.h"
#include "relay/transforms/pipeline.h"
#include "tir/transforms/pipeline.h"

using namespace kxc;
using namespace kxc::relay;

namespace {

std::string EmitC(Function f, const std::string& symbol) {
    Array<String> passes = {String("fold_constant"), String("simplify_expr")};
    Function typed = relay::InferTypePass(f);
    Function opt = relay::RunRelayPassPipeline(typed, passes);
    opt = relay::InferTypePass(opt);
    tir::PrimFunc pf = relay::LowerToTIR(opt);
    pf = tir::RunTIRPassPipeline(pf, passes);
    codegen::CodeGenC cg;
    return cg.Generate(pf, symbol);
}

Var F32(const std::string& name, std::vector<int64_t> shape) {
    Array<int64_t> s;
    for (auto d : shape) s.push_back(d);
    return Var(name, TensorType(s, "float32"));
}

Conv2DAttrs ConvAttrs(int s, int p, int o, int k) {
    return Conv2DAttrs::Create({s, s}, {p, p, p, p}, {1, 1}, 1, o, {k, k}, "NCHW", "OIHW", "", "");
}

// conv (+bias) (+relu) with every tensor a function parameter.
Function ConvCase(int64_t n, int64_t c, int64_t h, int64_t w, int64_t o, int k, int s, int p,
                  bool bias, bool relu) {
    Var x = F32("data", {n, c, h, w});
    Var wt = F32("weight", {o, c, k, k});
    Array<Var> params = {x, wt};
    Array<Expr> args = {x, wt};
    if (bias) {
        Var b = F32("bias", {o});
        params.push_back(b);
        args.push_back(b);
    }
    Expr out = Call(Op::Get("nn_conv2d"), args, ConvAttrs(s, p, static_cast<int>(o), k));
    if (relu) out = Call(Op::Get("nn_relu"), {out}, ReluAttrs::Create());
    return Function(params, out);
}

// conv+bias -> add(conv_out, skip) -> relu: the residual tail of a BasicBlock.
Function ConvAddReluCase(int64_t n, int64_t c, int64_t h, int64_t w, int64_t o, int k, int s,
                         int p) {
    Var x = F32("data", {n, c, h, w});
    Var wt = F32("weight", {o, c, k, k});
    Var b = F32("bias", {o});
    const int64_t oh = (h + 2 * p - k) / s + 1, ow = (w + 2 * p - k) / s + 1;
    Var skip = F32("skip", {n, o, oh, ow});
    Expr conv = Call(Op::Get("nn_conv2d"), {x, wt, b}, ConvAttrs(s, p, static_cast<int>(o), k));
    Expr add = Call(Op::Get("add"), {conv, skip}, AddAttrs::Create());
    Expr out = Call(Op::Get("nn_relu"), {add}, ReluAttrs::Create());
    return Function({x, wt, b, skip}, out);
}

Function PoolCase(const std::string& op, int64_t n, int64_t c, int64_t h, int64_t w, int k, int s,
                  int p, bool ceil_mode) {
    Var x = F32("data", {n, c, h, w});
    auto attrs = MaxPool2DAttrs::Create({s, s}, {p, p, p, p}, {1, 1}, {k, k}, "NCHW", ceil_mode);
    return Function({x}, Call(Op::Get(op), {x}, attrs));
}

Function GapCase(int64_t n, int64_t c, int64_t h, int64_t w) {
    Var x = F32("data", {n, c, h, w});
    return Function({x},
                    Call(Op::Get("nn_global_avg_pool2d"), {x}, GlobalAvgPool2DAttrs::Create()));
}

Function AddReluCase(std::vector<int64_t> a_shape, std::vector<int64_t> b_shape, bool relu) {
    Var a = F32("a", a_shape);
    Var b = F32("b", b_shape);
    Expr out = Call(Op::Get("add"), {a, b}, AddAttrs::Create());
    if (relu) out = Call(Op::Get("nn_relu"), {out}, ReluAttrs::Create());
    return Function({a, b}, out);
}

Function DenseCase(int64_t m, int64_t n, int64_t k) {
    Var a = F32("data", {m, k});
    Var b = F32("weight", {n, k});
    return Function({a, b}, Call(Op::Get("nn_dense"), {a, b}, DenseAttrs::Create(n, "")));
}

Function GemmCase(int64_t m, int64_t n, int64_t k, float alpha, float beta, int transB) {
    Var a = F32("a", {m, k});
    Var b = transB ? F32("b", {n, k}) : F32("b", {k, n});
    Var c = F32("c", {n});
    return Function({a, b, c},
                    Call(Op::Get("nn_gemm"), {a, b, c}, GemmAttrs::Create(alpha, beta, 0, transB)));
}

// gap -> flatten -> gemm: the classifier head.
Function HeadCase(int64_t n, int64_t c, int64_t h, int64_t w, int64_t classes) {
    Var x = F32("data", {n, c, h, w});
    Var wt = F32("fc_w", {classes, c});
    Var b = F32("fc_b", {classes});
    Expr gap = Call(Op::Get("nn_global_avg_pool2d"), {x}, GlobalAvgPool2DAttrs::Create());
    Expr fl = Call(Op::Get("nn_flatten"), {gap}, FlattenAttrs::Create(1));
    Expr out = Call(Op::Get("nn_gemm"), {fl, wt, b}, GemmAttrs::Create(1.0f, 1.0f, 0, 1));
    return Function({x, wt, b}, out);
}

}  // namespace

int main(int argc, char** argv) {
    if (argc < 2) {
        std::cerr << "usage: ref_driver <out.c>\n";
        return 2;
    }
    try {
        std::ostringstream all;
        all << "#include <stdint.h>\n#include <math.h>\n";
        struct Case { std::string name; Function f; };
        std::vector<Case> cases;
        // benchmark configuration 1
        cases.push_back({"kxc_ref_conv_cfg1", ConvCase(1, 64, 56, 56, 64, 3, 1, 1, true, true)});
        // the reference test's own tiny shapes (test/op_numeric_llvm_test.cpp)
        cases.push_back({"kxc_ref_conv_kat", ConvCase(1, 1, 3, 3, 1, 2, 1, 0, false, false)});
        cases.push_back({"kxc_ref_maxpool_kat", PoolCase("nn_max_pool2d", 1, 1, 4, 4, 2, 2, 0, false)});
        cases.push_back({"kxc_ref_avgpool_kat", PoolCase("nn_avg_pool2d", 1, 1, 4, 4, 2, 2, 0, false)});
        cases.push_back({"kxc_ref_gap_kat", GapCase(1, 2, 2, 2)});
        cases.push_back({"kxc_ref_dense_kat", DenseCase(2, 2, 3)});
        cases.push_back({"kxc_ref_gemm_kat", GemmCase(2, 4, 3, 1.0f, 1.0f, 1)});
        // shape zoo at reduced batch/spatial size: every conv geometry of ResNet-18
        cases.push_back({"kxc_ref_conv7x7s2", ConvCase(2, 3, 32, 32, 16, 7, 2, 3, true, true)});
        cases.push_back({"kxc_ref_conv3x3s1", ConvCase(2, 8, 14, 14, 16, 3, 1, 1, true, true)});
        cases.push_back({"kxc_ref_conv3x3s2", ConvCase(2, 8, 14, 14, 16, 3, 2, 1, true, true)});
        cases.push_back({"kxc_ref_conv1x1s2", ConvCase(2, 8, 14, 14, 16, 1, 2, 0, true, false)});
        cases.push_back({"kxc_ref_conv_nobias", ConvCase(1, 4, 9, 11, 5, 3, 1, 1, false, false)});
        cases.push_back({"kxc_ref_conv_add_relu", ConvAddReluCase(2, 8, 14, 14, 8, 3, 1, 1)});
        cases.push_back({"kxc_ref_maxpool3x3s2", PoolCase("nn_max_pool2d", 2, 4, 16, 16, 3, 2, 1, false)});
        cases.push_back({"kxc_ref_maxpool_ceil", PoolCase("nn_max_pool2d", 1, 2, 7, 9, 3, 2, 1, true)});
        cases.push_back({"kxc_ref_avgpool3x3s2", PoolCase("nn_avg_pool2d", 2, 4, 16, 16, 3, 2, 1, false)});
        cases.push_back({"kxc_ref_gap7x7", GapCase(4, 32, 7, 7)});
        cases.push_back({"kxc_ref_add_relu", AddReluCase({4, 16, 7, 7}, {4, 16, 7, 7}, true)});
        cases.push_back({"kxc_ref_add_bcast", AddReluCase({2, 3, 4}, {3, 1}, false)});
        cases.push_back({"kxc_ref_dense", DenseCase(8, 40, 64)});
        cases.push_back({"kxc_ref_gemm_fc", GemmCase(8, 40, 64, 1.0f, 1.0f, 1)});
        cases.push_back({"kxc_ref_gemm_ab", GemmCase(4, 6, 10, 0.5f, 2.0f, 0)});
        cases.push_back({"kxc_ref_head", HeadCase(4, 32, 7, 7, 10)});
        // No whole-network case: for a graph that calls one operator twice the reference's C
        // code generator declares two stack arrays of the same name (T_conv2d, T_relu ...) in one
        // scope and its output does not compile.  Single-operator and single-block cases do.
        for (auto& c : cases) {
            all << "\n/* ---- " << c.name << " ---- */\n" << EmitC(c.f, c.name) << "\n";
        }
        std::ofstream out(argv[1]);
        out << all.str();
        std::cout << "wrote " << cases.size() << " reference-generated functions to " << argv[1]
                  << "\n";
        return 0;
    } catch (const std::exception& e) {
        std::cerr << "ref_driver: " << e.what() << "\n";
        return 1;
    }
}
