// host_tests.cpp -- test program of the C++ host layer.
//
//   host_tests op_numeric <cpu|hip|hipgen>   the known-answer operator tests of the reference's
//                                            test/op_numeric_llvm_test.cpp, graph code unchanged, with
//                                            only the target switched (hipgen: every operator through
//                                            the TIR -> HIP generator instead of hand-written kernels)
//   host_tests device_info                   the DeviceAPI / Target contract of test/device_info_test.cpp
//   host_tests codegen                       lowering and code generator checks (no GPU needed)
//   host_tests resnet18 <cpu|hip|hipgen> <dir> <batch> <hw>
//                                            builds the ResNet-18 graph, reads input.bin and const_<k>.bin
//                                            from <dir>, runs, writes logits.bin and plan.json
#include <dlfcn.h>
#include <array>
#include <cmath>
#include <set>
#include <sstream>
#include <cstdio>
#include <cstring>
#include <fstream>
#include <functional>
#include <iostream>
#include <condition_variable>
#include <mutex>
#include <thread>
#include <atomic>

#include "kxc/compiler.h"
#include "kxc/packed_func.h"
#include "kxc/models.h"
#include "kxc/onnx_importer.h"
#include "kxc/profiling.h"
#include "kxc/runtime_session.h"
#include "kxc/topi.h"
#include "kxc_hip.h"

namespace {

std::string g_mode = "cpu";

void Check(bool cond, const std::string& msg) {
    if (!cond) throw std::runtime_error(msg);
}

void ExpectNear(const std::vector<float>& actual, const std::vector<float>& expected, float tol = 1e-4f) {
    Check(actual.size() == expected.size(), "result size mismatch");
    for (size_t i = 0; i < actual.size(); ++i) {
        if (!(std::fabs(actual[i] - expected[i]) <= tol))
            throw std::runtime_error("value mismatch at " + std::to_string(i) + ": actual=" + std::to_string(actual[i]) +
                                     ", expected=" + std::to_string(expected[i]));
    }
}

kxc::api::CompileConfig MakeConfig() {
    const bool gpu = g_mode != "cpu";
    auto config = kxc::api::CompileConfig::JIT(kxc::BuildTarget(gpu ? kxc::kGPU : kxc::kCPU));
    config->opt_level = 0;
    if (g_mode == "hipgen") { config->hip_use_handwritten = false; config->hip_fuse = false; }
    return config;
}

// Buffers: (pointer, bytes, is_output).  On the GPU every buffer is staged through DeviceAPI allocations,
// the way the reference's device test drives a kernel (test/cupti_smoke_test.cpp:108-114,207-214).
struct Buf { void* host; size_t bytes; bool out; };

void CompileAndRun(const std::string& name, kxc::Function func, std::vector<Buf> bufs) {
    auto config = MakeConfig();
    auto module = kxc::api::Compiler::Compile(func, config);
    Check(module.IsReady(), name + " module should be ready: " + module.GetStatus());
    std::vector<void*> args;
    if (g_mode == "cpu") {
        for (auto& b : bufs) args.push_back(b.host);
        module.Run(args);
        return;
    }
    kxc::DeviceAPI* api = kxc::GetDeviceAPI(kxc::kGPU);
    kxc::Device dev(kxc::kGPU, 0), cpu(kxc::kCPU, 0);
    for (auto& b : bufs) {
        void* d = api->AllocDataSpace(dev, b.bytes, 256);
        if (!b.out) api->CopyDataFromTo(cpu, b.host, dev, d, b.bytes);
        args.push_back(d);
    }
    module.Run(args);
    for (size_t i = 0; i < bufs.size(); ++i) {
        if (bufs[i].out) api->CopyDataFromTo(dev, args[i], cpu, bufs[i].host, bufs[i].bytes);
        api->FreeDataSpace(dev, args[i]);
    }
}

Buf In(std::vector<float>& v) { return {v.data(), v.size() * sizeof(float), false}; }
Buf Out(std::vector<float>& v) { return {v.data(), v.size() * sizeof(float), true}; }

using kxc::relay::Op;

void Binary(const char* op, std::vector<float> expect) {
    kxc::Var x("x", kxc::TensorType({2, 3}, "float32"));
    kxc::Var y("y", kxc::TensorType({3}, "float32"));
    kxc::Call call(Op::Get(op), {x, y});
    kxc::Function func({x, y}, call);
    std::vector<float> xd = {1, 2, 3, 4, 5, 6}, yd = {10, 20, 30}, out(6, 0.0f);
    CompileAndRun(op, func, {In(xd), In(yd), Out(out)});
    ExpectNear(out, expect);
}
void TestAdd() { Binary("add", {11, 22, 33, 14, 25, 36}); }
void TestSubtract() { Binary("subtract", {-9, -18, -27, -6, -15, -24}); }
void TestMul() { Binary("mul", {10, 40, 90, 40, 100, 180}); }
void TestDivide() { Binary("divide", {0.1f, 0.1f, 0.1f, 0.4f, 0.25f, 0.2f}); }

void TestSqrt() {
    kxc::Var x("x", kxc::TensorType({4}, "float32"));
    kxc::Function func({x}, kxc::Call(Op::Get("sqrt"), {x}));
    std::vector<float> xd = {1, 4, 9, 16}, out(4, 0.0f);
    CompileAndRun("sqrt", func, {In(xd), Out(out)});
    ExpectNear(out, {1, 2, 3, 4});
}

void TestMatmul() {
    kxc::Var a("a", kxc::TensorType({2, 3}, "float32"));
    kxc::Var b("b", kxc::TensorType({3, 2}, "float32"));
    kxc::Function func({a, b}, kxc::Call(Op::Get("matmul"), {a, b}));
    std::vector<float> ad = {1, 2, 3, 4, 5, 6}, bd = {1, 2, 3, 4, 5, 6}, out(4, 0.0f);
    CompileAndRun("matmul", func, {In(ad), In(bd), Out(out)});
    ExpectNear(out, {22, 28, 49, 64});
}

void TestDense() {
    kxc::Var data("data", kxc::TensorType({2, 3}, "float32"));
    kxc::Var weight("weight", kxc::TensorType({2, 3}, "float32"));
    kxc::Call call(Op::Get("nn_dense"), {data, weight}, kxc::relay::DenseAttrs::Create(2, ""));
    kxc::Function func({data, weight}, call);
    std::vector<float> d = {1, 2, 3, 4, 5, 6}, w = {1, 0, 1, 0, 1, 1}, out(4, 0.0f);
    CompileAndRun("nn_dense", func, {In(d), In(w), Out(out)});
    ExpectNear(out, {4, 5, 10, 11});
}

void TestGemm() {
    kxc::Var a("a", kxc::TensorType({2, 3}, "float32"));
    kxc::Var b("b", kxc::TensorType({4, 3}, "float32"));
    kxc::Var c("c", kxc::TensorType({4}, "float32"));
    kxc::Call call(Op::Get("nn_gemm"), {a, b, c}, kxc::relay::GemmAttrs::Create(1.0f, 1.0f, 0, 1));
    kxc::Function func({a, b, c}, call);
    std::vector<float> ad = {1, 2, 3, 4, 5, 6}, bd = {1, 0, 0, 0, 1, 0, 0, 0, 1, 1, 1, 1}, cd = {10, 20, 30, 40}, out(8, 0.0f);
    CompileAndRun("nn_gemm", func, {In(ad), In(bd), In(cd), Out(out)});
    ExpectNear(out, {11, 22, 33, 46, 14, 25, 36, 55});
}

void TestRelu() {
    kxc::Var x("x", kxc::TensorType({6}, "float32"));
    kxc::Function func({x}, kxc::Call(Op::Get("nn_relu"), {x}, kxc::relay::ReluAttrs::Create()));
    std::vector<float> xd = {-2, -0.5f, 0, 1, 2, -3}, out(6, 0.0f);
    CompileAndRun("nn_relu", func, {In(xd), Out(out)});
    ExpectNear(out, {0, 0, 0, 1, 2, 0});
}

void TestConv2D() {
    kxc::Var data("data", kxc::TensorType({1, 1, 3, 3}, "float32"));
    kxc::Var weight("weight", kxc::TensorType({1, 1, 2, 2}, "float32"));
    auto attrs = kxc::relay::Conv2DAttrs::Create({1, 1}, {0, 0, 0, 0}, {1, 1}, 1, 1, {2, 2}, "NCHW", "OIHW", "", "");
    kxc::Function func({data, weight}, kxc::Call(Op::Get("nn_conv2d"), {data, weight}, attrs));
    std::vector<float> d = {1, 2, 3, 4, 5, 6, 7, 8, 9}, w = {1, 0, 0, 1}, out(4, 0.0f);
    CompileAndRun("nn_conv2d", func, {In(d), In(w), Out(out)});
    ExpectNear(out, {6, 8, 12, 14});
}

void Pool(const char* op, std::vector<float> expect) {
    kxc::Var data("data", kxc::TensorType({1, 1, 4, 4}, "float32"));
    auto attrs = kxc::relay::MaxPool2DAttrs::Create({2, 2}, {0, 0, 0, 0}, {1, 1}, {2, 2}, "NCHW", false);
    kxc::Function func({data}, kxc::Call(Op::Get(op), {data}, attrs));
    std::vector<float> d = {1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15, 16}, out(4, 0.0f);
    CompileAndRun(op, func, {In(d), Out(out)});
    ExpectNear(out, expect);
}
void TestMaxPool2D() { Pool("nn_max_pool2d", {6, 8, 14, 16}); }
void TestAvgPool2D() { Pool("nn_avg_pool2d", {3.5f, 5.5f, 11.5f, 13.5f}); }

void TestGlobalAvgPool2D() {
    kxc::Var data("data", kxc::TensorType({1, 2, 2, 2}, "float32"));
    kxc::Function func({data}, kxc::Call(Op::Get("nn_global_avg_pool2d"), {data}, kxc::relay::GlobalAvgPool2DAttrs::Create()));
    std::vector<float> d = {1, 2, 3, 4, 10, 20, 30, 40}, out(2, 0.0f);
    CompileAndRun("nn_global_avg_pool2d", func, {In(d), Out(out)});
    ExpectNear(out, {2.5f, 25.0f});
}

void TestFlatten() {
    kxc::Var data("data", kxc::TensorType({1, 2, 2, 3}, "float32"));
    kxc::Function func({data}, kxc::Call(Op::Get("nn_flatten"), {data}, kxc::relay::FlattenAttrs::Create(1)));
    std::vector<float> d = {1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12}, out(12, 0.0f);
    CompileAndRun("nn_flatten", func, {In(d), Out(out)});
    ExpectNear(out, d);
}

void TestReshape() {
    kxc::Var data("data", kxc::TensorType({2, 3}, "float32"));
    kxc::Function func({data}, kxc::Call(Op::Get("reshape"), {data}, kxc::relay::ReshapeAttrs::Create({3, 2})));
    std::vector<float> d = {1, 2, 3, 4, 5, 6}, out(6, 0.0f);
    CompileAndRun("reshape", func, {In(d), Out(out)});
    ExpectNear(out, d);
}

void TestTranspose() {
    kxc::Var data("data", kxc::TensorType({2, 3}, "float32"));
    kxc::Function func({data}, kxc::Call(Op::Get("transpose"), {data}, kxc::relay::TransposeAttrs::Create({1, 0})));
    std::vector<float> d = {1, 2, 3, 4, 5, 6}, out(6, 0.0f);
    CompileAndRun("transpose", func, {In(d), Out(out)});
    ExpectNear(out, {1, 4, 2, 5, 3, 6});
}

void TestReduceMean() {
    kxc::Var data("data", kxc::TensorType({2, 3}, "float32"));
    kxc::Function func({data}, kxc::Call(Op::Get("reduce_mean"), {data}, kxc::relay::ReduceMeanAttrs::Create({1}, 0)));
    std::vector<float> d = {1, 2, 3, 4, 5, 6}, out(2, 0.0f);
    CompileAndRun("reduce_mean", func, {In(d), Out(out)});
    ExpectNear(out, {2.0f, 5.0f});
}

// softmax over the last axis against the formula (test/op_numeric_llvm_test.cpp:271-293)
void TestSoftmax() {
    kxc::Var data("data", kxc::TensorType({2, 3}, "float32"));
    kxc::Function func({data}, kxc::Call(Op::Get("softmax"), {data}, kxc::relay::SoftmaxAttrs::Create(1)));
    std::vector<float> d = {1, 2, 3, 1, 3, 5}, out(6, 0.0f), expect(6, 0.0f);
    CompileAndRun("softmax", func, {In(d), Out(out)});
    for (int row = 0; row < 2; ++row) {
        float denom = 0.0f;
        for (int col = 0; col < 3; ++col) denom += std::exp(d[row * 3 + col]);
        for (int col = 0; col < 3; ++col) expect[row * 3 + col] = std::exp(d[row * 3 + col]) / denom;
    }
    ExpectNear(out, expect);
    // axis 0 of a rank-3 tensor, negative axis spelling: every column of the leading axis sums to 1
    kxc::Var t("t", kxc::TensorType({3, 2, 2}, "float32"));
    kxc::Function f2({t}, kxc::Call(Op::Get("softmax"), {t}, kxc::relay::SoftmaxAttrs::Create(-3)));
    std::vector<float> td = {0.5f, -1, 2, 0, 1, 1, -2, 3, 0.25f, 0, 1, -1}, to(12, 0.0f);
    CompileAndRun("softmax axis 0", f2, {In(td), Out(to)});
    for (int i = 0; i < 4; ++i) {
        float denom = std::exp(td[i]) + std::exp(td[4 + i]) + std::exp(td[8 + i]);
        ExpectNear({to[i], to[4 + i], to[8 + i]}, {std::exp(td[i]) / denom, std::exp(td[4 + i]) / denom, std::exp(td[8 + i]) / denom});
    }
}

// float32 -> int32 truncates toward zero (test/op_numeric_llvm_test.cpp:295-305)
void TestCast() {
    kxc::Var data("data", kxc::TensorType({4}, "float32"));
    kxc::Function func({data}, kxc::Call(Op::Get("cast"), {data}, kxc::relay::CastAttrs::Create(1)));
    std::vector<float> d = {1.9f, -2.2f, 3.0f, 4.8f};
    std::vector<int32_t> out(4, 0);
    CompileAndRun("cast", func, {In(d), Buf{out.data(), out.size() * sizeof(int32_t), true}});
    if (out != std::vector<int32_t>({1, -2, 3, 4})) throw std::runtime_error("cast: wrong result");
    // int32 -> float32 and back through a chain
    kxc::Var iv("iv", kxc::TensorType({3}, "int32"));
    kxc::Function f2({iv}, kxc::Call(Op::Get("cast"), {iv}, kxc::relay::CastAttrs::Create(0)));
    std::vector<int32_t> id = {-7, 0, 12};
    std::vector<float> fo(3, 0.0f);
    CompileAndRun("cast to float", f2, {Buf{id.data(), id.size() * sizeof(int32_t), false}, Out(fo)});
    ExpectNear(fo, {-7.0f, 0.0f, 12.0f});
    bool threw = false;
    try { kxc::relay::CastAttrs::Create(9); kxc::relay::CastDTypeFromCode(9); } catch (const std::exception& e) {
        threw = std::string(e.what()) == "cast has unsupported dtype code: 9";
    }
    if (!threw) throw std::runtime_error("cast: bad dtype code was not refused");
}

void TestModelAddChain() {
    kxc::Var x("x", kxc::TensorType({4}, "float32"));
    kxc::Var y("y", kxc::TensorType({4}, "float32"));
    kxc::Call first(Op::Get("add"), {x, y});
    kxc::Call second(Op::Get("add"), {first, y});
    kxc::Function func({x, y}, second);
    std::vector<float> xd = {1, 2, 3, 4}, yd = {10, 20, 30, 40}, out(4, 0.0f);
    CompileAndRun("model_add_chain", func, {In(xd), In(yd), Out(out)});
    ExpectNear(out, {21, 42, 63, 84});
}

void TestModelMLP() {
    kxc::Var x("x", kxc::TensorType({1, 2}, "float32"));
    kxc::Var w1("w1", kxc::TensorType({3, 2}, "float32"));
    kxc::Var w2("w2", kxc::TensorType({2, 3}, "float32"));
    kxc::Call hidden(Op::Get("nn_dense"), {x, w1}, kxc::relay::DenseAttrs::Create(3, ""));
    kxc::Call relu(Op::Get("nn_relu"), {hidden}, kxc::relay::ReluAttrs::Create());
    kxc::Call out_call(Op::Get("nn_dense"), {relu, w2}, kxc::relay::DenseAttrs::Create(2, ""));
    kxc::Function func({x, w1, w2}, out_call);
    std::vector<float> xd = {1, 2}, w1d = {1, 0, 0, 1, 1, 1}, w2d = {1, 1, 1, 1, 0, -1}, out(2, 0.0f);
    CompileAndRun("model_mlp", func, {In(xd), In(w1d), In(w2d), Out(out)});
    ExpectNear(out, {6, -2});
}

void TestModelCNN() {
    kxc::Var data("data", kxc::TensorType({1, 1, 3, 3}, "float32"));
    kxc::Var conv_weight("conv_weight", kxc::TensorType({1, 1, 2, 2}, "float32"));
    kxc::Var dense_weight("dense_weight", kxc::TensorType({2, 1}, "float32"));
    auto conv_attrs = kxc::relay::Conv2DAttrs::Create({1, 1}, {0, 0, 0, 0}, {1, 1}, 1, 1, {2, 2}, "NCHW", "OIHW", "", "");
    kxc::Call conv(Op::Get("nn_conv2d"), {data, conv_weight}, conv_attrs);
    kxc::Call relu(Op::Get("nn_relu"), {conv}, kxc::relay::ReluAttrs::Create());
    kxc::Call pool(Op::Get("nn_global_avg_pool2d"), {relu}, kxc::relay::GlobalAvgPool2DAttrs::Create());
    kxc::Call flatten(Op::Get("nn_flatten"), {pool}, kxc::relay::FlattenAttrs::Create(1));
    kxc::Call logits(Op::Get("nn_dense"), {flatten, dense_weight}, kxc::relay::DenseAttrs::Create(2, ""));
    kxc::Function func({data, conv_weight, dense_weight}, logits);
    std::vector<float> d = {1, 2, 3, 4, 5, 6, 7, 8, 9}, cw = {1, 0, 0, 1}, dw = {1, 2}, out(2, 0.0f);
    CompileAndRun("model_cnn", func, {In(d), In(cw), In(dw), Out(out)});
    ExpectNear(out, {10, 20});
}

// Error behaviour: the messages a user of the reference sees.
void TestErrors() {
    auto expect_throw = [](const std::function<void()>& fn, const std::string& needle) {
        try { fn(); } catch (const std::exception& e) {
            Check(std::string(e.what()).find(needle) != std::string::npos, std::string("unexpected message: ") + e.what());
            return;
        }
        throw std::runtime_error("no exception, expected: " + needle);
    };
    expect_throw([] {
        kxc::Var d("d", kxc::TensorType({1, 4, 3, 3}, "float32")), w("w", kxc::TensorType({8, 4, 5, 5}, "float32"));
        auto a = kxc::relay::Conv2DAttrs::Create({1, 1}, {0, 0, 0, 0}, {1, 1}, 1, 8, {5, 5}, "NCHW", "OIHW", "", "");
        kxc::relay::InferTypePass(kxc::Function({d, w}, kxc::Call(Op::Get("nn_conv2d"), {d, w}, a)));
    }, "window is larger than input");
    expect_throw([] {
        kxc::Var d("d", kxc::TensorType({1, 4, 8, 8}, "float32")), w("w", kxc::TensorType({8, 3, 3, 3}, "float32"));
        auto a = kxc::relay::Conv2DAttrs::Create({1, 1}, {1, 1, 1, 1}, {1, 1}, 1, 8, {3, 3}, "NCHW", "OIHW", "", "");
        kxc::relay::InferTypePass(kxc::Function({d, w}, kxc::Call(Op::Get("nn_conv2d"), {d, w}, a)));
    }, "input channel mismatch");
    expect_throw([] {
        kxc::Var a("a", kxc::TensorType({2, 3}, "float32")), b("b", kxc::TensorType({4, 5}, "float32"));
        kxc::relay::InferTypePass(kxc::Function({a, b}, kxc::Call(Op::Get("nn_dense"), {a, b}, kxc::relay::DenseAttrs::Create(4, ""))));
    }, "nn_dense input dimension mismatch");
    expect_throw([] {
        kxc::Var a("a", kxc::TensorType({2, 3}, "float32"));
        kxc::relay::InferTypePass(kxc::Function({a}, kxc::Call(Op::Get("no_such_op"), {a})));
    }, "No FInferType registered for op: no_such_op");
    expect_throw([] {
        kxc::Var a("a", kxc::TensorType({4}, "float32"));
        auto m = kxc::api::Compiler::Compile(kxc::Function({a}, kxc::Call(Op::Get("nn_relu"), {a})),
                                             kxc::api::CompileConfig::JIT(kxc::BuildTarget(kxc::kCPU)));
        m.Run({nullptr});
    }, "expected 2 packed arguments");
}

int RunOpNumeric() {
    const std::vector<std::pair<std::string, void (*)()>> tests = {
        {"add", TestAdd}, {"subtract", TestSubtract}, {"mul", TestMul}, {"divide", TestDivide}, {"sqrt", TestSqrt},
        {"matmul", TestMatmul}, {"nn_dense", TestDense}, {"nn_gemm", TestGemm}, {"nn_relu", TestRelu},
        {"nn_conv2d", TestConv2D}, {"nn_max_pool2d", TestMaxPool2D}, {"nn_avg_pool2d", TestAvgPool2D},
        {"nn_global_avg_pool2d", TestGlobalAvgPool2D}, {"nn_flatten", TestFlatten}, {"reshape", TestReshape},
        {"transpose", TestTranspose}, {"reduce_mean", TestReduceMean}, {"softmax", TestSoftmax}, {"cast", TestCast},
        {"model_add_chain", TestModelAddChain},
        {"model_mlp", TestModelMLP}, {"model_cnn", TestModelCNN}, {"errors", TestErrors},
    };
    for (const auto& t : tests) {
        try {
            t.second();
        } catch (const std::exception& e) {
            std::cerr << "[FAIL] " << t.first << ": " << e.what() << "\n";
            return 1;
        }
        std::cout << "[PASS] " << t.first << std::endl;
    }
    std::cout << "All operator numeric tests passed (" << g_mode << ").\n";
    return 0;
}

// ------------------------------------------------------------------ device info (test/device_info_test.cpp)
int RunDeviceInfo() {
    auto cpu = kxc::BuildTarget(kxc::kCPU);
    Check(cpu->kind == "llvm", "CPU target kind should be llvm");
    auto infos = kxc::GetAllDeviceInfo();
    bool saw_gpu = false;
    for (const auto& d : infos) {
        if (d.device_type != kxc::kGPU) continue;
        saw_gpu = true;
        Check(d.device_type_name == "hip" && d.target_kind == "hip", "GPU entry should be named hip");
        Check(!d.status.empty(), "GPU entry should carry a status text");
        Check(d.attrs.warp_size == 64, "wavefront size should be 64");
        Check(d.attrs.arch.rfind("gfx", 0) == 0, "arch should be a gfx name");
        std::cout << "gpu " << d.device_id << " available=" << d.available << " status=" << d.status << " arch=" << d.attrs.arch
                  << " cus=" << d.attrs.multi_processor_count << " lds=" << d.attrs.max_shared_memory_per_block << "\n";
    }
    Check(saw_gpu, "the GPU entry must always be listed");
    auto gpu = kxc::BuildTarget(kxc::kGPU);       // never throws: attributes are queryable without a runtime
    Check(gpu->kind == "hip", "GPU target kind should be hip");
    Check(kxc::GetAllDeviceInfoJSON().find("\"target_kind\":\"hip\"") != std::string::npos, "JSON should list the hip target");
    std::cout << "device info ok\n";
    return 0;
}

// ------------------------------------------------------------------ ResNet-18 (test/resnet18_ir_dump.cpp:191-452)
std::vector<char> ReadFile(const std::string& path, size_t expect) {
    std::ifstream in(path, std::ios::binary);
    if (!in) throw std::runtime_error("cannot open " + path);
    std::vector<char> data((std::istreambuf_iterator<char>(in)), std::istreambuf_iterator<char>());
    if (data.size() != expect) throw std::runtime_error(path + ": expected " + std::to_string(expect) + " bytes, got " + std::to_string(data.size()));
    return data;
}

int RunResNet18(const std::string& dir, int64_t batch, int64_t hw) {
    std::vector<kxc::runtime::NDArray> net_consts;
    kxc::Function func = kxc::models::BuildResNet18(batch, hw, &net_consts);
    auto config = MakeConfig();
    auto module = kxc::api::Compiler::Compile(func, config);
    std::cout << "status: " << module.GetStatus() << "\n";
    Check(module.input_count() == 1 && module.constant_count() == 42, "ResNet-18 should lower to 1 input and 42 constants");
    Check(module.GetPrimFunc()->params.size() == 44, "the lowered function should have 44 parameters");
    // the constants come back in parameter order, which is the graph's depth-first argument order
    const auto& consts = module.GetConstants();
    for (size_t k = 0; k < consts.size(); ++k)
        Check(consts[k].get() == net_consts[k].get(), "constant " + std::to_string(k) + " is out of lowering order");
    {
        std::ofstream plan(dir + "/plan.json");
        plan << module.ExecutionPlanJSON();
    }
    std::cout << "launches: " << module.GetKernelExecs().size() << "\n";
    for (const auto& e : module.GetKernelExecs()) std::cout << "  " << e.op_name << " -> " << e.kernel_symbol << "\n";
    if (!module.IsReady()) {
        std::cout << "module not loadable here (no GPU); plan and sources were generated\n";
        return 0;
    }
    std::vector<std::vector<char>> host;
    host.push_back(ReadFile(dir + "/input.bin", static_cast<size_t>(batch * 3 * hw * hw) * 4));
    for (size_t k = 0; k < consts.size(); ++k) host.push_back(ReadFile(dir + "/const_" + std::to_string(k) + ".bin", consts[k].nbytes()));
    std::vector<float> logits(static_cast<size_t>(batch) * 1000, 0.0f);
    std::vector<Buf> bufs;
    for (auto& h : host) bufs.push_back({h.data(), h.size(), false});
    bufs.push_back(Out(logits));
    std::vector<void*> args;
    if (g_mode == "cpu") {
        for (auto& b : bufs) args.push_back(b.host);
        module.Run(args);
    } else {
        kxc::DeviceAPI* api = kxc::GetDeviceAPI(kxc::kGPU);
        kxc::Device dev(kxc::kGPU, 0), cpu(kxc::kCPU, 0);
        for (auto& b : bufs) {
            void* d = api->AllocDataSpace(dev, b.bytes, 256);
            if (!b.out) api->CopyDataFromTo(cpu, b.host, dev, d, b.bytes);
            args.push_back(d);
        }
        module.Run(args);
        module.Run(args);      // a second run reuses the plan and its workspace
        api->CopyDataFromTo(dev, args.back(), cpu, logits.data(), logits.size() * sizeof(float));
        // the saved execution plan runs again without the graph and without compiling it
        std::ifstream saved(dir + "/plan.json");
        std::stringstream text;
        text << saved.rdbuf();
        auto replay = kxc::api::Compiler::LoadExecutionPlan(text.str(), config);
        Check(replay.IsReady() && replay.GetKernelExecs().size() == module.GetKernelExecs().size(), "replayed module");
        std::vector<float> zeros(logits.size(), 0.0f), again(logits.size(), -1.0f);
        api->CopyDataFromTo(cpu, zeros.data(), dev, args.back(), zeros.size() * sizeof(float));
        replay.Run(args);
        api->CopyDataFromTo(dev, args.back(), cpu, again.data(), again.size() * sizeof(float));
        Check(std::memcmp(again.data(), logits.data(), logits.size() * sizeof(float)) == 0,
              "replayed execution plan must reproduce the compiled module bit for bit");
        Check(replay.ExecutionPlanJSON() == text.str(), "a loaded plan serialises to the same JSON");
        std::cout << "execution plan replayed: " << replay.GetKernelExecs().size() << " launches, identical output\n";
        for (auto* p : args) api->FreeDataSpace(dev, p);
    }
    std::ofstream out(dir + "/logits.bin", std::ios::binary);
    out.write(reinterpret_cast<const char*>(logits.data()), static_cast<std::streamsize>(logits.size() * sizeof(float)));
    std::cout << "wrote " << dir << "/logits.bin\n";
    return 0;
}

// ------------------------------------------------------------------ lowering / code generators (no GPU)
int RunCodegen() {
    // config 1 of the benchmark: conv 3x3 + bias + relu lowers to the three loop nests of the reference
    kxc::Var data("data", kxc::TensorType({1, 64, 56, 56}, "float32"));
    kxc::Var weight("weight", kxc::TensorType({64, 64, 3, 3}, "float32"));
    kxc::Var bias("bias", kxc::TensorType({64}, "float32"));
    auto attrs = kxc::relay::Conv2DAttrs::Create({1, 1}, {1, 1, 1, 1}, {1, 1}, 1, 64, {3, 3}, "NCHW", "OIHW", "", "");
    kxc::Call conv(Op::Get("nn_conv2d"), {data, weight, bias}, attrs);
    kxc::Call relu(Op::Get("nn_relu"), {conv}, kxc::relay::ReluAttrs::Create());
    kxc::Function func({data, weight, bias}, relu);
    kxc::tir::PrimFunc pf = kxc::relay::LowerToTIR(kxc::relay::InferTypePass(func));
    Check(pf->params.size() == 4, "data, weight, bias, T_relu_out");
    Check(pf->params[3].name_hint() == "T_relu_out", "output parameter name: " + pf->params[3].name_hint());
    Check(pf->int_attrs.at("kxc.input_count") == 3 && pf->int_attrs.at("kxc.output_param_start") == 3, "kxc.* attrs");
    const std::string text = kxc::tir::ToString(pf);
    Check(text.find("allocate T_conv2d[") != std::string::npos && text.find("allocate T_conv2d_bias_add[") != std::string::npos,
          "intermediates are Allocate nodes");
    Check(text.find("for (rc, 0, 64)") != std::string::npos && text.find("for (rw, 0, 3)") != std::string::npos, "reduce loops");
    kxc::codegen::CodeGenC cgc;
    const std::string c_text = cgc.Generate(pf, "kxc_kernel_main");
    Check(c_text.find("int32_t kxc_kernel_main(void** packed_args)") != std::string::npos, "C entry point");
    Check(c_text.find("return 0;") != std::string::npos, "C returns 0");
    kxc::codegen::CodeGenHIP cgh;
    auto hip = cgh.Generate(pf, "kxc_t");
    Check(hip.kernels.size() == 3, "one kernel per compute stage");
    Check(hip.source.find("extern \"C\" __global__ void __launch_bounds__(256) kxc_t_s0_T_conv2d(") != std::string::npos, "kernel symbol");
    // 200 704 outputs: blocks of two output channels still leave 65 536 threads; the input window is read once per block
    Check(hip.kernels[0].schedule == "reg_tile", "conv stage takes the register-tiled schedule: " + hip.kernels[0].schedule);
    Check(hip.source.find("acc10 = acc10 + (u0 * weight[") != std::string::npos && hip.source.find("acc01") == std::string::npos &&
              hip.source.find("acc20") == std::string::npos,
          "blocks of 2 x 1 outputs sharing the input term");
    Check(hip.kernels[0].grid[0] == 392, "100 352 threads in workgroups of 256");
    Check(hip.kernels[1].schedule == "flat" && hip.kernels[2].schedule == "flat", "bias add and relu are flat");
    {
        // with no lower bound on the thread count the same stage takes 4 x 4 blocks (output channels x rows): the padded
        // window term is evaluated once per row of the block, the weight once per channel, 16 accumulators, guarded stores
        setenv("KXC_HIPGEN_TILE_MIN_UNITS", "1", 1);
        auto tiled = cgh.Generate(pf, "kxc_t");
        unsetenv("KXC_HIPGEN_TILE_MIN_UNITS");
        const std::string& src = tiled.source;
        Check(tiled.kernels[0].schedule == "reg_tile" && tiled.kernels[0].grid[0] == 49, "4 x 4 blocks: 12 544 threads");
        for (const char* piece : {"const auto u0_3 = (", "const auto u1_3 = weight[", "acc33 = acc33 + (u0_3 * u1_3);", "float acc00 = ",
                                  "if (ta_base + 3 < 64 && tb_base + 3 < 56) T_conv2d["})
            Check(src.find(piece) != std::string::npos, std::string("register-tiled source holds: ") + piece);
        Check(src.find("? data[") != std::string::npos && src.find("u0_0 = ((((") != std::string::npos,
              "the input load stays behind its bounds test inside the shared term");
    }
    {
        // a padded window at least 16 taps wide: the input load sits behind the padding select and must stay a lazy
        // global load (staged for a whole tile of rows it would read before the buffer and past its end); the weight
        // load, unguarded and contiguous along rw, may be staged
        kxc::Var xd("x", kxc::TensorType({1, 2, 4, 40}, "float32")), wd("w", kxc::TensorType({3, 2, 1, 17}, "float32"));
        auto wide = kxc::relay::Conv2DAttrs::Create({1, 1}, {0, 8, 0, 8}, {1, 1}, 1, 3, {1, 17}, "NCHW", "OIHW", "", "");
        kxc::Function fw({xd, wd}, kxc::Call(Op::Get("nn_conv2d"), {xd, wd}, wide));
        auto wide_hip = cgh.Generate(kxc::relay::LowerToTIR(kxc::relay::InferTypePass(fw)), "kxc_wide");
        Check(wide_hip.kernels.size() == 1, "one stage for a convolution without bias");
        const std::string& src = wide_hip.source;
        Check(src.find("= x[rowbase") == std::string::npos, "the padded input is never staged by row base:\n" + src);
        if (wide_hip.kernels[0].schedule == "lds_k_stage")
            Check(src.find("= w[rowbase") != std::string::npos && src.find("? x[") != std::string::npos,
                  "only the weights are staged; the input stays behind its select:\n" + src);
    }
    // global average pool: contiguous rows -> LDS staged reduction
    kxc::Var x("x", kxc::TensorType({4, 32, 7, 7}, "float32"));
    kxc::Function gap({x}, kxc::Call(Op::Get("nn_global_avg_pool2d"), {x}, kxc::relay::GlobalAvgPool2DAttrs::Create()));
    auto gap_hip = cgh.Generate(kxc::relay::LowerToTIR(kxc::relay::InferTypePass(gap)), "kxc_gap");
    Check(gap_hip.kernels.size() == 2 && gap_hip.kernels[0].schedule == "lds_row_reduce", "gap sum is LDS staged");
    Check(gap_hip.source.find("__shared__ float tile[") != std::string::npos, "LDS tile declared");
    Check(gap_hip.source.find("/ ((long long)49LL)") != std::string::npos || gap_hip.source.find("49") != std::string::npos, "division by H*W");
    // dense against a [units, k] weight: every thread walks a row of the weight -> staged through LDS in chunks of k,
    // still added in k order; a short reduction (k = 8) stays flat
    {
        kxc::Var dx("x", kxc::TensorType({8, 64}, "float32")), dw("w", kxc::TensorType({40, 64}, "float32"));
        kxc::Function dense({dx, dw}, kxc::Call(Op::Get("nn_dense"), {dx, dw}, kxc::relay::DenseAttrs::Create(40, "")));
        auto dense_hip = cgh.Generate(kxc::relay::LowerToTIR(kxc::relay::InferTypePass(dense)), "kxc_dense");
        Check(dense_hip.kernels.size() == 1 && dense_hip.kernels[0].schedule == "lds_k_stage",
              "dense is LDS staged along k, got " + dense_hip.kernels[0].schedule);
        Check(dense_hip.source.find("__shared__ float tile0[") != std::string::npos &&
                  dense_hip.source.find("acc = acc + ") != std::string::npos, "staged tile and ordered accumulation");
        if (const char* dump = std::getenv("KXC_DUMP_DENSE_HIP")) std::ofstream(dump) << dense_hip.source;
        kxc::Var sx("x", kxc::TensorType({8, 8}, "float32")), sw("w", kxc::TensorType({4, 8}, "float32"));
        kxc::Function small({sx, sw}, kxc::Call(Op::Get("nn_dense"), {sx, sw}, kxc::relay::DenseAttrs::Create(4, "")));
        auto small_hip = cgh.Generate(kxc::relay::LowerToTIR(kxc::relay::InferTypePass(small)), "kxc_small");
        Check(small_hip.kernels[0].schedule == "flat", "a reduction of 8 stays flat");
    }
    // a ResNet-18 compile for the hip target without a GPU: plan and fusion are built, nothing is loaded
    g_mode = "hip";
    auto module = kxc::api::Compiler::Compile(kxc::models::BuildResNet18(1, 224), MakeConfig());
    Check(module.GetKernelExecs().size() == 20, "49 Relay calls become 20 launches, got " + std::to_string(module.GetKernelExecs().size()));
    int fused_add = 0, fused_relu = 0;
    for (const auto& e : module.GetKernelExecs()) {
        if (e.kernel_symbol.find("kxc_conv2d") == 0 && e.input_values.size() == 4) ++fused_add;
        (void)fused_relu;
    }
    Check(fused_add == 8, "8 residual adds are folded into convolutions");
    Check(module.ExecutionPlanJSON().find("\"kernel_symbol\":\"kxc_conv2d_nchw_f32.mfma_k7x7") != std::string::npos, "plan JSON carries kernel symbols");
    std::cout << "codegen ok\n";
    return 0;
}

}  // namespace

// onnx <cpu|hip|hipgen> <dir>: loads <dir>/model.import.json + <dir>/model.params.bin (the reference's ONNX import
// wire format), compiles the imported function for the target and runs it on the input pattern of the
// reference's acceptance test (test/onnx_importer_test.cpp:138-144); writes <dir>/logits.bin.
int RunOnnx(const std::string& dir) {
    kxc::frontend::ImportedONNXModel imported =
        kxc::frontend::LoadONNXImportSpec(dir + "/model.import.json", dir + "/model.params.bin");
    Check(imported.function.defined(), "importer should construct a Relay Function");
    Check(imported.input_names.size() == 1 && imported.output_names.size() == 1, "one input, one output");
    Check(imported.params.size() == imported.param_order.size(), "every parameter is kept");
    std::cout << "imported: " << imported.param_order.size() << " params, input " << imported.input_names[0] << ", output "
              << imported.output_names[0] << "\n";
    auto config = MakeConfig();
    auto module = kxc::api::Compiler::Compile(imported.function, config);
    Check(module.input_count() == 1, "one function input");
    Check(static_cast<size_t>(module.constant_count()) == imported.param_order.size(), "every parameter becomes a constant argument");
    if (!module.IsReady()) { std::cout << "module not loadable here (no GPU)\n"; return 0; }
    // shapes of the input and the output come from the typed function
    kxc::Function typed = kxc::relay::InferTypePass(imported.function);
    auto elements = [](const kxc::Type& t) {
        size_t n = 1;
        for (auto d : static_cast<const kxc::TensorTypeNode*>(t.get())->shape) n *= static_cast<size_t>(d);
        return n;
    };
    const size_t in_elems = elements(typed->params[0]->type_annotation), out_elems = elements(typed->body.checked_type());
    std::vector<float> input(in_elems), output(out_elems, 0.0f);
    for (size_t i = 0; i < in_elems; ++i) input[i] = (static_cast<float>(i % 251) - 125.0f) / 125.0f;
    std::vector<std::vector<char>> consts;
    for (const auto& c : module.GetConstants()) {
        std::vector<char> bytes(c.nbytes());
        c.CopyToBytes(bytes.data(), bytes.size());
        consts.push_back(std::move(bytes));
    }
    std::vector<Buf> bufs;
    bufs.push_back(In(input));
    for (auto& c : consts) bufs.push_back({c.data(), c.size(), false});
    bufs.push_back(Out(output));
    std::vector<void*> args;
    if (g_mode == "cpu") {
        for (auto& b : bufs) args.push_back(b.host);
        module.Run(args);
    } else {
        kxc::DeviceAPI* api = kxc::GetDeviceAPI(kxc::kGPU);
        kxc::Device dev(kxc::kGPU, 0), cpu(kxc::kCPU, 0);
        for (auto& b : bufs) {
            void* d = api->AllocDataSpace(dev, b.bytes, 256);
            if (!b.out) api->CopyDataFromTo(cpu, b.host, dev, d, b.bytes);
            args.push_back(d);
        }
        module.Run(args);
        api->CopyDataFromTo(dev, args.back(), cpu, output.data(), output.size() * sizeof(float));
        for (auto* p : args) api->FreeDataSpace(dev, p);
    }
    std::ofstream out(dir + "/logits.bin", std::ios::binary);
    out.write(reinterpret_cast<const char*>(output.data()), static_cast<std::streamsize>(output.size() * sizeof(float)));
    std::cout << "launches: " << module.GetKernelExecs().size() << "; wrote " << dir << "/logits.bin\n";
    return 0;
}

// onnx_errors <dir>: malformed specs raise the reference's messages.
int RunOnnxErrors(const std::string& dir) {
    auto expect = [&](const std::string& file, const std::string& needle) {
        try {
            kxc::frontend::LoadONNXImportSpec(dir + "/" + file, dir + "/model.params.bin");
        } catch (const std::exception& e) {
            Check(std::string(e.what()).find(needle) != std::string::npos, file + ": expected '" + needle + "', got '" + e.what() + "'");
            return;
        }
        throw std::runtime_error(file + ": expected an error");
    };
    expect("bad_format.json", "Unsupported ONNX import spec format");
    expect("bad_op.json", "Unsupported Relay op in ONNX import spec: identity");
    expect("bad_input.json", "Missing input value 'nowhere' for node 'relu0'");
    expect("bad_range.json", "Param bytes range out of bounds for: conv1.weight");
    expect("bad_order.json", "param_order does not match params metadata");
    std::cout << "onnx error messages ok\n";
    return 0;
}

// adaptive <cpu|hip|hipgen> [bundle dir]: the adaptive runtime (kxc/runtime_session.h) -- cache rules, shape
// statistics, priority order of the background compiler, a session that goes miss -> fuzzy hit -> background
// compile -> exact hit, and compiles on worker threads concurrent with runs on this thread.
struct StagedArgs {                     // host vectors staged through DeviceAPI buffers when the target is the GPU
    std::vector<Buf> bufs;
    std::vector<void*> args;
    explicit StagedArgs(std::vector<Buf> b) : bufs(std::move(b)) {
        if (g_mode == "cpu") { for (auto& x : bufs) args.push_back(x.host); return; }
        kxc::DeviceAPI* api = kxc::GetDeviceAPI(kxc::kGPU);
        kxc::Device dev(kxc::kGPU, 0), cpu(kxc::kCPU, 0);
        for (auto& x : bufs) {
            void* d = api->AllocDataSpace(dev, x.bytes, 256);
            if (!x.out) api->CopyDataFromTo(cpu, x.host, dev, d, x.bytes);
            args.push_back(d);
        }
    }
    void Fetch() {
        if (g_mode == "cpu") return;
        kxc::DeviceAPI* api = kxc::GetDeviceAPI(kxc::kGPU);
        kxc::Device dev(kxc::kGPU, 0), cpu(kxc::kCPU, 0);
        for (size_t i = 0; i < bufs.size(); ++i)
            if (bufs[i].out) api->CopyDataFromTo(dev, args[i], cpu, bufs[i].host, bufs[i].bytes);
    }
    ~StagedArgs() {
        if (g_mode == "cpu") return;
        kxc::DeviceAPI* api = kxc::GetDeviceAPI(kxc::kGPU);
        for (void* d : args) api->FreeDataSpace(kxc::Device(kxc::kGPU, 0), d);
    }
};

int RunAdaptive(const std::string& bundle_dir) {
    using namespace kxc::runtime;
    // ---- KernelCache::ShapeDistance (kernel_cache.cc:54-73)
    auto sig = [](std::vector<std::vector<int64_t>> s) { return MakeShapeSignature(s); };
    Check(KernelCache::ShapeDistance(sig({{2, 3}}), sig({{2, 3}})) == 0, "identical shapes are at distance 0");
    Check(KernelCache::ShapeDistance(sig({{2, 3}}), sig({{4, 8}})) == 7, "distance is the summed difference");
    Check(KernelCache::ShapeDistance(sig({{2, 3}}), sig({{4, 2}})) == -1, "a smaller cached dimension cannot serve");
    Check(KernelCache::ShapeDistance(sig({{2, 3}}), sig({{2, 3, 1}})) == -1, "rank must agree");
    Check(KernelCache::ShapeDistance(sig({{2, 3}}), sig({{2, 3}, {1}})) == -1, "input count must agree");
    Check(sig({{2, 3}}).Hash() == sig({{2, 3}}).Hash() && !(sig({{2, 3}}) == sig({{3, 2}})), "signature equality / hash");
    // ---- ShapePredictor (shape_predictor.cc:17-66)
    {
        ShapePredictor p;
        for (int i = 0; i < 3; ++i) p.Record(sig({{8}}));
        p.Record(sig({{4}}));
        for (int i = 0; i < 2; ++i) p.Record(sig({{2}}));
        Check(p.TotalCount() == 6 && p.GetCount(sig({{8}})) == 3 && p.GetCount(sig({{9}})) == 0, "counts");
        auto top = p.PredictTopK(2);
        Check(top.size() == 2 && top[0] == sig({{8}}) && top[1] == sig({{2}}), "top-k is ordered by frequency");
        Check(p.ShouldCompile(sig({{2}})) && !p.ShouldCompile(sig({{4}})) && !p.ShouldCompile(sig({{9}})), "seen at least twice");
        Check(p.ShouldCompile(sig({{4}}), 1), "count threshold argument");
    }
    // ---- KernelRunner (kernel_runner.cc:13-34)
    {
        KernelRunner r;
        bool threw = false;
        try { r.Run({}); } catch (const std::exception& e) { threw = std::string(e.what()) == "KernelRunner: no kernel available"; }
        Check(threw && !r.HasKernel(), "an empty runner refuses to run");
    }

    auto make_add = [](int64_t rows) {
        kxc::Var x("x", kxc::TensorType({rows, 3}, "float32"));
        kxc::Var y("y", kxc::TensorType({3}, "float32"));
        return kxc::Function({x, y}, kxc::Call(Op::Get("add"), {x, y}));
    };
    // ---- BackgroundCompiler: one worker; while it is held inside the first task's callback four more tasks are
    // queued -- they must complete highest priority first (background_compiler.h:36, background_compiler.cc:54-58)
    {
        BackgroundCompiler bg(1);
        std::mutex mu;
        std::condition_variable cv;
        bool release = false;
        std::vector<int> order;
        auto task = [&](int priority, bool hold) {
            BackgroundCompiler::CompileTask t;
            t.relay_func = make_add(2);
            t.config = MakeConfig();
            t.priority = priority;
            t.on_complete = [&, priority, hold](kxc::api::CompiledModule m) {
                Check(m.IsReady() || g_mode == "cpu", "background module ready");
                std::unique_lock<std::mutex> lock(mu);
                if (hold) cv.wait(lock, [&] { return release; });
                order.push_back(priority);
            };
            return t;
        };
        bg.Submit(task(100, true));
        while (bg.PendingCount() != 0) std::this_thread::yield();          // the worker has taken it
        for (int p : {1, 7, 3, 5}) bg.Submit(task(p, false));
        Check(bg.PendingCount() == 4, "four tasks queued behind the running one");
        { std::lock_guard<std::mutex> lock(mu); release = true; }
        cv.notify_all();
        bg.WaitAll();
        Check(order == std::vector<int>({100, 7, 5, 3, 1}), "tasks complete in priority order");
        Check(bg.CompletedCount() == 5 && bg.PendingCount() == 0 && bg.FailedCount() == 0, "completed count");
        // a task whose compilation throws is counted as failed and does not stop the worker
        BackgroundCompiler::CompileTask bad;
        kxc::Var v("v", kxc::TensorType({2, 3}, "float32"));
        kxc::Var w("w", kxc::TensorType({4}, "float32"));
        bad.relay_func = kxc::Function({v, w}, kxc::Call(Op::Get("add"), {v, w}));     // shapes do not broadcast
        bad.config = MakeConfig();
        bg.Submit(bad);
        bg.WaitAll();
        Check(bg.FailedCount() == 1 && bg.CompletedCount() == 5, "a failing compile is contained");
    }

    // ---- RuntimeSession: warm up a larger shape, then ask for a smaller one three times
    std::shared_ptr<kxc::profiling::ProfileContext> ctx;
    if (!bundle_dir.empty()) {
        kxc::profiling::ProfileOptions options;
        options.enabled = true;
        options.bundle_dir = bundle_dir;
        ctx = kxc::profiling::ProfileContext::Create(options);
    }
    {
        std::unique_ptr<kxc::profiling::ActivationScope> scope;
        if (ctx) scope = std::make_unique<kxc::profiling::ActivationScope>(ctx, ctx->NextRunId("adaptive"));
        auto config = MakeConfig();
        config->background_threads = 2;
        RuntimeSession session(make_add(2), config, ctx);
        Check(session.CachedKernelCount() == 0 && session.GetStatus() == "RuntimeSession{cached=0, pending=0, completed=0, total_runs=0}",
              "fresh session status: " + session.GetStatus());
        session.WarmUp({{4, 3}, {3}});
        session.WarmUp({{4, 3}, {3}});                                    // second warm-up of a cached shape is a no-op
        Check(session.CachedKernelCount() == 1, "warm-up caches one module");
        std::vector<float> xd = {1, 2, 3, 4, 5, 6}, yd = {10, 20, 30}, out(6, 0.0f);
        StagedArgs staged({In(xd), In(yd), Out(out)});
        const std::vector<std::vector<int64_t>> small = {{2, 3}, {3}};
        const bool device = g_mode != "cpu";
        session.Run(staged.args, small);                                  // fuzzy hit, seen once: nothing scheduled
        session.WaitAll();
        // (on the hip target a module compiled for larger extents never runs on the caller's device buffers: the
        //  fuzzy candidate counts as a miss and the exact shape is compiled at once)
        Check(session.CachedKernelCount() == (device ? 2 : 1), "first run of the smaller shape");
        session.Run(staged.args, small);                                  // fuzzy hit, seen twice: background compile
        session.WaitAll();
        Check(session.CachedKernelCount() == 2, "second fuzzy hit compiles the exact shape in the background");
        session.Run(staged.args, small);                                  // exact hit
        session.Run(staged.args, small);
        session.WaitAll();
        staged.Fetch();
        ExpectNear(out, {11, 22, 33, 14, 25, 36});
        Check(session.GetStatus() == (device ? "RuntimeSession{cached=2, pending=0, completed=0, total_runs=4}"
                                             : "RuntimeSession{cached=2, pending=0, completed=1, total_runs=4}"),
              "status: " + session.GetStatus());
        Check(session.PendingCompileCount() == 0, "nothing pending");
        // a shape nothing cached can serve: compiled on the calling thread
        RuntimeSession cold(make_add(2), config, ctx);
        cold.Run(staged.args, small);
        Check(cold.CachedKernelCount() == 1 && cold.GetStatus() == "RuntimeSession{cached=1, pending=0, completed=0, total_runs=1}",
              "cold miss compiles synchronously: " + cold.GetStatus());
    }

    // ---- the same through the user-visible entry: CompileConfig::Adaptive + Compiler::Compile
    // (include/api/compile_config.h:62-68, src/api/compiler.cc:64-80,146-191)
    {
        auto base = MakeConfig();
        auto config = kxc::api::CompileConfig::Adaptive(base->target, {{4, 3}});
        config->hip_use_handwritten = base->hip_use_handwritten;
        config->hip_fuse = base->hip_fuse;
        config->background_threads = 1;
        Check(config->mode == kxc::api::CompileMode::kAdaptive && config->opt_level == 2 && config->enable_hot_swap, "Adaptive config");
        kxc::Var x("x", kxc::TensorType({2, 3}, "float32"));
        kxc::Function relu({x}, kxc::Call(Op::Get("nn_relu"), {x}));
        auto module = kxc::api::Compiler::Compile(relu, config);
        Check(module.IsReady(), "an adaptive module is ready at once");
        Check(module.GetStatus() == "RuntimeSession{cached=1, pending=0, completed=0, total_runs=0}",
              "the suggested shape was warmed up: " + module.GetStatus());
        std::vector<float> xd = {-1, 2, -3, 4, -5, 6}, out(6, 0.0f);
        StagedArgs staged({In(xd), Out(out)});
        bool threw = false;
        try { module.Run(staged.args); } catch (const std::exception& e) {
            threw = std::string(e.what()) == "Adaptive mode requires Run(args, input_shapes). Use the overload with input_shapes.";
        }
        Check(threw, "the plain Run of an adaptive module is refused");
        module.Run(staged.args, {{2, 3}});
        module.Run(staged.args, {{2, 3}});
        module.WaitAll();
        module.WarmUp({{8, 3}});
        staged.Fetch();
        ExpectNear(out, {0, 2, 0, 4, 0, 6});
        Check(module.GetStatus() == (g_mode != "cpu" ? "RuntimeSession{cached=3, pending=0, completed=0, total_runs=2}"
                                                     : "RuntimeSession{cached=3, pending=0, completed=1, total_runs=2}"),
              "adaptive module status: " + module.GetStatus());
        // a non-adaptive module accepts the shape overload and ignores the shapes
        auto plain = kxc::api::Compiler::Compile(relu, MakeConfig());
        std::fill(out.begin(), out.end(), 0.0f);
        StagedArgs staged2({In(xd), Out(out)});
        plain.Run(staged2.args, {{2, 3}});
        plain.WaitAll();
        staged2.Fetch();
        ExpectNear(out, {0, 2, 0, 4, 0, 6});
    }

    // ---- compiles on worker threads while this thread runs: the small CNN of the known-answer tests, compiled
    // eight times on four workers, each module run by the worker that built it, with the session above's kind of
    // run going on here in between
    {
        BackgroundCompiler bg(4);
        std::atomic<int> good{0};
        std::mutex print_mu;
        for (int i = 0; i < 8; ++i) {
            BackgroundCompiler::CompileTask t;
            t.relay_func = make_add(2 + i);
            t.config = MakeConfig();
            t.priority = i;
            const int rows = 2 + i;
            t.on_complete = [&, rows](kxc::api::CompiledModule m) {
                std::vector<float> xd(static_cast<size_t>(rows) * 3), yd = {1, 2, 3}, out(xd.size(), 0.0f);
                for (size_t k = 0; k < xd.size(); ++k) xd[k] = static_cast<float>(k);
                StagedArgs staged({In(xd), In(yd), Out(out)});
                m.Run(staged.args);
                staged.Fetch();
                bool ok = true;
                for (size_t k = 0; k < xd.size(); ++k) ok = ok && out[k] == xd[k] + yd[k % 3];
                if (ok) ++good;
            };
            bg.Submit(std::move(t));
        }
        auto module = kxc::api::Compiler::Compile(make_add(2), MakeConfig());
        std::vector<float> xd = {1, 2, 3, 4, 5, 6}, yd = {10, 20, 30}, out(6, 0.0f);
        StagedArgs staged({In(xd), In(yd), Out(out)});
        for (int it = 0; it < 50; ++it) module.Run(staged.args);
        bg.WaitAll();
        staged.Fetch();
        ExpectNear(out, {11, 22, 33, 14, 25, 36});
        Check(good.load() == 8 && bg.CompletedCount() == 8, "eight concurrent compiles ran correctly: " + std::to_string(good.load()));
    }
    if (ctx) {
        ctx->Flush();
        std::cout << "profile bundle: " << ctx->bundle_dir() << " events=" << ctx->event_count() << "\n";
    }
    std::cout << "adaptive runtime ok (" << g_mode << ")\n";
    return 0;
}

// profile <cpu|hip|hipgen> <bundle dir>: the CNN known-answer model under an active profiling context; the
// bundle lands in <bundle dir> (the Python tests read it back).
int RunProfile(const std::string& dir) {
    kxc::profiling::ProfileOptions options;
    options.enabled = true;
    options.bundle_dir = dir;
    options.ir_capture_mode = kxc::profiling::IRCaptureMode::kVerbose;
    options = kxc::profiling::ApplyEnvironmentOverrides(options);
    auto ctx = kxc::profiling::ProfileContext::Create(options);
    {
        kxc::profiling::ActivationScope scope(ctx, ctx->NextRunId("host_tests"));
        kxc::profiling::EventSpec spec;
        spec.component = "test";
        spec.event_type = "model_cnn";
        kxc::profiling::ScopedSpan span(ctx, spec);
        TestModelCNN();
        ctx->RecordLog(kxc::profiling::LogSeverity::kInfo, "test", "model_cnn passed",
                       kxc::profiling::MakeFields({{"mode", g_mode}}));
    }
    ctx->Flush();
    std::cout << "profile bundle: " << ctx->bundle_dir() << " events=" << ctx->event_count() << "\n";
    return 0;
}

// HIP counterpart of the reference's only GPU test (test/cupti_smoke_test.cpp:95-267): device API allocation,
// stream and copies, a fill, the kernel `scale_add` (y[i] = x[i] * alpha + 1, n = 64, block 128, grid 1, multiply and
// add rounded separately) compiled at run time and launched on the device API's stream, all inside a profiling
// context; the bundle must then hold backend.hip events of every kind: hip_runtime_api, hip_memcpy, hip_memset,
// hip_kernel.
// sdk: the activity records come from rocprofiler-sdk (ProfileOptions::enable_gpu_activity = 2), and the test itself
// calls hipMemcpyAsync -- outside the HIP library of this build, whose call sites the default mode instruments --
// and expects that copy in the bundle too.  The context is created before anything asks the HIP runtime a question:
// a rocprofiler-sdk tool can only be registered before the runtime initialises.
int RunHipSmoke(const std::string& dir, bool sdk = false) {
    namespace profiling = kxc::profiling;
    profiling::ProfileOptions options;
    options.enabled = true;
    options.bundle_dir = dir;
    options.enable_gpu_activity = sdk ? 2 : 1;
    auto ctx = profiling::ProfileContext::Create(options);
    auto target = kxc::BuildTarget(kxc::kGPU);
    Check(target->attrs.exists == 1, "hip_smoke needs a GPU: " + target->attrs.status);
    if (sdk) Check(ctx->gpu_activity_mode() == 2, std::string("rocprofiler-sdk tracing is not on: ") + kxc_hip_last_error());
    constexpr size_t kOutsideBytes = 200;       // a size nothing else in this test copies
    const std::string run_id = ctx->NextRunId("hip-smoke");
    {
        profiling::ActivationScope activation(ctx, run_id);
        profiling::EventSpec root_spec;
        root_spec.component = "test";
        root_spec.event_type = "hip_smoke";
        profiling::ScopedSpan root_span(ctx, std::move(root_spec), run_id);

        kxc::DeviceAPI* api = kxc::DeviceAPIManager::Global()->GetAPI(kxc::kGPU);
        const kxc::Device gpu(kxc::kGPU, 0), cpu(kxc::kCPU, 0);
        std::vector<float> host_in(64, 3.5f), host_out(64, -1.0f);
        const size_t nbytes = host_in.size() * sizeof(float);
        api->SetDevice(gpu);
        void* gpu_buf = api->AllocDataSpace(gpu, nbytes, 64);
        void* gpu_out = api->AllocDataSpace(gpu, nbytes, 64);
        kxc::StreamHandle stream = api->CreateStream(gpu);
        api->SetStream(gpu, stream);
        api->CopyDataFromTo(cpu, host_in.data(), gpu, gpu_buf, nbytes);
        Check(kxc_hip_memset(gpu_buf, 0, nbytes, 0, stream) == 0, std::string("memset: ") + kxc_hip_last_error());
        api->CopyDataFromTo(host_in.data(), 0, gpu_buf, 0, nbytes, cpu, gpu, stream);

        const char* source = R"(
extern "C" __global__ void scale_add(const float* x, float* y, float alpha, int n) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) {
    y[i] = x[i] * alpha + 1.0f;
  }
}
)";
        kxc_hip_module* module = nullptr;
        std::vector<char> log(4096, 0);
        Check(kxc_hip_module_compile(source, "scale_add.hip", &module, log.data(), log.size()) == 0,
              std::string("compile: ") + kxc_hip_last_error());
        void* kernel = nullptr;
        Check(kxc_hip_module_get_function(module, "scale_add", &kernel) == 0, std::string("get_function: ") + kxc_hip_last_error());
        float alpha = 2.0f;
        int n = static_cast<int>(host_in.size());
        void* kernel_args[] = {&gpu_buf, &gpu_out, &alpha, &n};
        const uint32_t block[3] = {128, 1, 1};
        const uint32_t grid[3] = {static_cast<uint32_t>((n + 127) / 128), 1, 1};
        Check(kxc_hip_module_launch(kernel, grid, block, 0, stream, kernel_args) == 0, std::string("launch: ") + kxc_hip_last_error());
        api->CopyDataFromTo(gpu_out, 0, host_out.data(), 0, nbytes, gpu, cpu, stream);
        if (sdk) {
            // a copy the application enqueues itself, straight through the HIP runtime
            using MemcpyAsync = int (*)(void*, const void*, size_t, int, void*);
            void* hip = dlopen("libamdhip64.so", RTLD_NOW);
            Check(hip != nullptr, "dlopen(libamdhip64.so)");
            auto copy = reinterpret_cast<MemcpyAsync>(dlsym(hip, "hipMemcpyAsync"));
            Check(copy != nullptr, "dlsym(hipMemcpyAsync)");
            Check(copy(gpu_buf, host_in.data(), kOutsideBytes, 1 /* hipMemcpyHostToDevice */, stream) == 0, "hipMemcpyAsync from the test");
        }
        api->StreamSync(gpu, stream);
        kxc_hip_module_free(module);
        for (float v : host_out) Check(v == 8.0f, "Kernel output verification failed");
        api->SetStream(gpu, nullptr);
        api->FreeStream(gpu, stream);
        api->FreeDataSpace(gpu, gpu_out);
        api->FreeDataSpace(gpu, gpu_buf);
        // single-attribute queries of the same back end
        Check(kxc::GetDeviceAttr(gpu, kxc::DeviceAttrKind::kWarpSize) == 64 && kxc::GetDeviceAttr(gpu, kxc::DeviceAttrKind::kExist) == 1,
              "GetAttr");
        Check(kxc::DeviceAPI::NeedSetDevice(kxc::kGPU) && !kxc::DeviceAPI::NeedSetDevice(kxc::kCPU), "NeedSetDevice");
    }
    if (sdk) std::this_thread::sleep_for(std::chrono::milliseconds(200));      // completion records are delivered by a profiler thread
    ctx->Flush();
    std::ifstream manifest(dir + "/manifest.json");
    std::string manifest_text((std::istreambuf_iterator<char>(manifest)), std::istreambuf_iterator<char>());
    Check(manifest_text.find("\"enable_gpu_activity\":true") != std::string::npos, "manifest marks GPU activity as on");
    Check(manifest_text.find(sdk ? "\"gpu_activity_source\":\"rocprofiler_sdk\"" : "\"gpu_activity_source\":\"hip_events\"") != std::string::npos,
          "manifest names the source of the activity records");
    bool saw_runtime = false, saw_memcpy = false, saw_memset = false, saw_kernel = false;
    bool saw_outside_call = !sdk, saw_outside_copy = !sdk;
    std::ifstream events(dir + "/events.jsonl");
    std::string line;
    while (std::getline(events, line)) {
        if (line.find("\"component\":\"backend.hip\"") == std::string::npos) continue;
        saw_runtime = saw_runtime || line.find("\"event_type\":\"hip_runtime_api\"") != std::string::npos;
        saw_memcpy = saw_memcpy || line.find("\"event_type\":\"hip_memcpy\"") != std::string::npos;
        saw_memset = saw_memset || line.find("\"event_type\":\"hip_memset\"") != std::string::npos;
        saw_kernel = saw_kernel || (line.find("\"event_type\":\"hip_kernel\"") != std::string::npos &&
                                    line.find("\"kernel_symbol\":\"scale_add\"") != std::string::npos &&
                                    (!sdk || line.find("\"backend.hip.timing_source\":\"rocprofiler_sdk\"") != std::string::npos));
        saw_outside_call = saw_outside_call || (line.find("\"event_type\":\"hip_runtime_api\"") != std::string::npos &&
                                                line.find("\"backend.hip.api\":\"hipMemcpyAsync\"") != std::string::npos);
        saw_outside_copy = saw_outside_copy || (line.find("\"event_type\":\"hip_memcpy\"") != std::string::npos &&
                                                line.find("\"bytes\":200") != std::string::npos);
    }
    Check(saw_runtime && saw_memcpy && saw_memset && saw_kernel, "Missing expected HIP activity events");
    Check(saw_outside_call && saw_outside_copy, "the copy the test enqueued itself is not in the bundle");
    std::cout << "HIP bundle generated at: " << dir << "\n";
    return 0;
}

// The device-side diagnosis rules on synthetic events: six module runs of 50 us, copies that make up most of the
// device API time, and synchronisation that makes up a third of everything.
int RunDiagnosis(const std::string& dir) {
    namespace profiling = kxc::profiling;
    profiling::ProfileOptions options;
    options.enabled = true;
    options.bundle_dir = dir;
    options.enable_gpu_activity = false;
    auto ctx = profiling::ProfileContext::Create(options);
    Check(ctx->DiagnoseDeviceOverheads().empty(), "an empty context has no findings");
    auto add = [&](const char* component, const char* type, std::int64_t start, std::int64_t dur) {
        profiling::EventSpec e;
        e.component = component;
        e.event_type = type;
        ctx->RecordCompletedSpan(e, "run-1", ctx->NextSpanId(), "", start, start + dur);
    };
    for (int i = 0; i < 6; ++i) add("runtime", "compiled_module_run", 1000 * i, 50000);
    add("device_api", "copy", 400000, 900000);
    add("device_api", "alloc_data_space", 1400000, 100000);
    add("device_api", "stream_sync", 1500000, 700000);
    const auto found = ctx->DiagnoseDeviceOverheads();
    auto has = [&](const char* c) { for (const auto& d : found) if (d.category == c) return true; return false; };
    Check(has("kernel_launch_overhead") && has("copy_dominance") && has("sync_overhead"), "all three rules fire");
    ctx->Flush();
    // one long module run and little copying: nothing fires
    auto calm = profiling::ProfileContext::Create(options);
    {
        profiling::EventSpec e;
        e.component = "runtime";
        e.event_type = "compiled_module_run";
        calm->RecordCompletedSpan(e, "run-1", calm->NextSpanId(), "", 0, 5000000);
        e.component = "device_api"; e.event_type = "alloc_data_space";
        calm->RecordCompletedSpan(e, "run-1", calm->NextSpanId(), "", 0, 1000);
    }
    Check(calm->DiagnoseDeviceOverheads().empty(), "a calm run has no findings");
    // (what a caller publishes is kept)
    ctx->PublishDiagnostics({{"pass_regression", "warn", "tir.transform", "published by a caller"}});
    ctx->Flush();
    std::ifstream f(dir + "/diagnosis.json");
    std::string text((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
    Check(text.find("pass_regression") != std::string::npos && text.find("copy_dominance") == std::string::npos, "published diagnosis is kept");
    ctx->PublishDiagnostics({});
    ctx->Flush();
    std::cout << "diagnosis rules ok\n";
    return 0;
}

// The compiled-kernel object and the compile-configuration surface (include/codegen/compiled_kernel.h:19-56,
// include/api/compile_config.h:40-50, include/api/compiler.h:88): fields, IsReady, the call operator with the
// reference's error texts, profile_options -> a module-owned context, GetProfileBundlePath.
int RunKernelObject(const std::string& dir) {
    using kxc::codegen::CodeGenBackend;
    kxc::Var x("x", kxc::TensorType({2, 3}, "float32"));
    kxc::Var y("y", kxc::TensorType({3}, "float32"));
    kxc::Function add({x, y}, kxc::Call(Op::Get("add"), {x, y}));
    auto config = MakeConfig();
    config->profile_options.enabled = !dir.empty();
    config->profile_options.bundle_dir = dir;
    config->cache_dir = "";
    auto module = kxc::api::Compiler::Compile(add, config);
    const kxc::codegen::CompiledKernel kernel = module.GetKernel();
    Check(kernel.defined() && kernel.IsReady() && module.IsReady(), "kernel is ready");
    Check(kernel->kernel_name == "kxc_kernel_main", "kernel name: " + kernel->kernel_name);
    Check(kernel->backend == (g_mode == "cpu" ? CodeGenBackend::kC : CodeGenBackend::kHIP), "kernel backend");
    Check(kernel->func_ptr != nullptr, "IsReady <=> func_ptr");
    Check(kernel->param_buffers.size() == 3 && kernel->param_buffers[0].shape == std::vector<int64_t>({2, 3}),
          "param_buffers carries the packed-argument signature");
    if (g_mode == "cpu") Check(kernel->lib_handle != nullptr && !kernel->so_path.empty(), "host back end owns its library");
    else Check(kernel->jit_resource != nullptr && kernel->lib_handle == nullptr, "hip back end owns its launch plan");
    std::vector<float> xd = {1, 2, 3, 4, 5, 6}, yd = {10, 20, 30}, out(6, 0.0f);
    {
        StagedArgs staged({In(xd), In(yd), Out(out)});
        kernel(staged.args);                                   // the kernel object is callable by itself
        staged.Fetch();
        ExpectNear(out, {11, 22, 33, 14, 25, 36});
    }
    {
        std::fill(out.begin(), out.end(), 0.0f);
        StagedArgs staged({In(xd), In(yd), Out(out)});
        module.Run(staged.args);
        staged.Fetch();
        ExpectNear(out, {11, 22, 33, 14, 25, 36});
    }
    bool threw = false;
    try { kxc::codegen::CompiledKernel()(std::vector<void*>{}); } catch (const std::exception& e) {
        threw = std::string(e.what()) == "CompiledKernel: not ready or func_ptr is null";
    }
    Check(threw, "an empty kernel refuses to run with the reference's message");
    Check(!kxc::codegen::CompiledKernel().IsReady(), "an empty kernel is not ready");
    if (g_mode != "cpu") {
        // a failing launch surfaces as the Run ABI's error: "Kernel <name> returned error code N"
        threw = false;
        try { kernel(std::vector<void*>{nullptr, nullptr, nullptr}); } catch (const std::exception& e) {
            threw = std::string(e.what()).rfind("Kernel kxc_kernel_main returned error code ", 0) == 0;
        }
        Check(threw, "kernel error text");
    }
    // a copy of the kernel handle keeps the resources alive after the module is gone
    module = kxc::api::CompiledModule();
    {
        std::fill(out.begin(), out.end(), 0.0f);
        StagedArgs staged({In(xd), In(yd), Out(out)});
        kernel(staged.args);
        staged.Fetch();
        ExpectNear(out, {11, 22, 33, 14, 25, 36});
    }
    if (!dir.empty()) {
        auto again = kxc::api::Compiler::Compile(add, config);
        Check(again.GetProfileBundlePath() == dir, "GetProfileBundlePath: " + again.GetProfileBundlePath());
        StagedArgs staged({In(xd), In(yd), Out(out)});
        again.Run(staged.args);
        std::ifstream events(dir + "/events.jsonl");
        std::string all((std::istreambuf_iterator<char>(events)), std::istreambuf_iterator<char>());
        Check(all.find("\"event_type\":\"compile\"") != std::string::npos, "the module's own context recorded the compile");
        Check(all.find("\"run_id\":\"execute") != std::string::npos, "Run activates the module's context under an execute run id");
        auto plain = MakeConfig();
        Check(kxc::api::Compiler::Compile(add, plain).GetProfileBundlePath().empty(), "no profiling: empty bundle path");
    }
    std::cout << "kernel object ok (" << g_mode << ")\n";
    return 0;
}

// Generated kernels against the host back end on shapes that exercise the LDS-staged schedules: ragged chunk counts,
// fewer outputs than a workgroup, operands that are and are not contiguous along the reduce axis.  Same loop order on
// both sides, no contraction: every output must be bit-identical.
int RunGeneratedNumeric() {
    auto fill = [](std::vector<float>& v, uint32_t seed) {
        for (float& x : v) { seed = seed * 1664525u + 1013904223u; x = static_cast<float>(static_cast<int32_t>(seed >> 8) % 2001 - 1000) / 997.0f; }
    };
    struct Case {
        std::string name; kxc::Function func; std::vector<std::vector<int64_t>> in_shapes; int64_t out_elems; std::string schedule;
        const char* tile_min_units = nullptr;      // KXC_HIPGEN_TILE_MIN_UNITS for this case (small shapes take the tiled schedule)
    };
    std::vector<Case> cases;
    {
        kxc::Var x("x", kxc::TensorType({5, 70}, "float32")), w("w", kxc::TensorType({37, 70}, "float32"));
        cases.push_back({"dense 5x70 . 37x70", kxc::Function({x, w}, kxc::Call(Op::Get("nn_dense"), {x, w}, kxc::relay::DenseAttrs::Create(37, ""))),
                         {{5, 70}, {37, 70}}, 5 * 37, "lds_k_stage"});
    }
    {
        kxc::Var x("x", kxc::TensorType({300, 16}, "float32")), w("w", kxc::TensorType({3, 16}, "float32"));
        cases.push_back({"dense 300x16 . 3x16", kxc::Function({x, w}, kxc::Call(Op::Get("nn_dense"), {x, w}, kxc::relay::DenseAttrs::Create(3, ""))),
                         {{300, 16}, {3, 16}}, 900, "lds_k_stage"});
    }
    {
        kxc::Var a("a", kxc::TensorType({9, 33}, "float32")), b("b", kxc::TensorType({33, 21}, "float32"));
        cases.push_back({"matmul 9x33 . 33x21", kxc::Function({a, b}, kxc::Call(Op::Get("matmul"), {a, b})), {{9, 33}, {33, 21}}, 9 * 21, "lds_k_stage"});
    }
    {
        kxc::Var d("d", kxc::TensorType({7, 100}, "float32"));
        cases.push_back({"reduce_mean 7x100", kxc::Function({d}, kxc::Call(Op::Get("reduce_mean"), {d}, kxc::relay::ReduceMeanAttrs::Create({1}, 0))),
                         {{7, 100}}, 7, "lds_k_stage"});
    }
    {
        kxc::Var d("d", kxc::TensorType({600, 40}, "float32"));
        cases.push_back({"reduce_mean 600x40", kxc::Function({d}, kxc::Call(Op::Get("reduce_mean"), {d}, kxc::relay::ReduceMeanAttrs::Create({1}, 0))),
                         {{600, 40}}, 600, "lds_row_reduce"});
    }
    {
        // a window 17 taps wide with padding 8: the weights are staged along rw, the padded input stays behind its select
        kxc::Var d("d", kxc::TensorType({1, 2, 4, 40}, "float32")), w("w", kxc::TensorType({3, 2, 1, 17}, "float32"));
        auto attrs = kxc::relay::Conv2DAttrs::Create({1, 1}, {0, 8, 0, 8}, {1, 1}, 1, 3, {1, 17}, "NCHW", "OIHW", "", "");
        cases.push_back({"conv2d 1x17 window, padding 8", kxc::Function({d, w}, kxc::Call(Op::Get("nn_conv2d"), {d, w}, attrs)),
                         {{1, 2, 4, 40}, {3, 2, 1, 17}}, 480, "lds_k_stage"});
    }
    // convolution-shaped nests: a thread owns a block of outputs along the output-channel axis and the row axis
    auto conv_case = [&](const std::string& name, std::vector<int64_t> xs, std::vector<int64_t> ws, std::vector<int64_t> strides,
                         std::vector<int64_t> pads, std::vector<int64_t> dil, const char* min_units, const std::string& schedule) {
        kxc::Var d("d", kxc::TensorType(xs, "float32")), w("w", kxc::TensorType(ws, "float32"));
        auto attrs = kxc::relay::Conv2DAttrs::Create(strides, pads, dil, 1, ws[0], {ws[2], ws[3]}, "NCHW", "OIHW", "", "");
        kxc::Function f({d, w}, kxc::Call(Op::Get("nn_conv2d"), {d, w}, attrs));
        const int64_t oh = (xs[2] + pads[0] + pads[2] - dil[0] * (ws[2] - 1) - 1) / strides[0] + 1;
        const int64_t ow = (xs[3] + pads[1] + pads[3] - dil[1] * (ws[3] - 1) - 1) / strides[1] + 1;
        cases.push_back({name, f, {xs, ws}, xs[0] * ws[0] * oh * ow, schedule, min_units});
    };
    conv_case("conv2d 3x3, 7 channels out, 9 rows (ragged blocks)", {2, 5, 9, 11}, {7, 5, 3, 3}, {1, 1}, {1, 1, 1, 1}, {1, 1}, "1", "reg_tile");
    conv_case("conv2d 3x3 stride 2 dilation 2", {1, 3, 13, 10}, {6, 3, 3, 3}, {2, 2}, {2, 2, 2, 2}, {2, 2}, "1", "reg_tile");
    conv_case("conv2d 1x1, two channels out", {3, 4, 5, 6}, {2, 4, 1, 1}, {1, 1}, {0, 0, 0, 0}, {1, 1}, "1", "reg_tile");
    conv_case("conv2d 5x5, padding 2 x 1, three channels in blocks of 2 x 1", {1, 2, 6, 7}, {3, 2, 5, 5}, {1, 1}, {2, 1, 2, 1}, {1, 1}, "40", "reg_tile");
    conv_case("conv2d 3x3 large enough for 4 x 4 blocks by default", {4, 8, 64, 64}, {64, 8, 3, 3}, {1, 1}, {1, 1, 1, 1}, {1, 1}, nullptr, "reg_tile");
    conv_case("conv2d 3x3 too small to give up threads", {1, 8, 14, 14}, {16, 8, 3, 3}, {1, 1}, {1, 1, 1, 1}, {1, 1}, nullptr, "flat");
    for (auto& c : cases) {
        if (c.tile_min_units) setenv("KXC_HIPGEN_TILE_MIN_UNITS", c.tile_min_units, 1);
        else unsetenv("KXC_HIPGEN_TILE_MIN_UNITS");
        std::vector<std::vector<float>> ins;
        uint32_t seed = 12345;
        for (const auto& shp : c.in_shapes) { ins.emplace_back(static_cast<size_t>(kxc::Product(shp))); fill(ins.back(), seed); seed += 7919; }
        std::vector<float> out_cpu(static_cast<size_t>(c.out_elems), -1.0f), out_gpu(static_cast<size_t>(c.out_elems), -2.0f);
        auto run = [&](const std::string& mode, std::vector<float>& out) {
            g_mode = mode;
            std::vector<Buf> bufs;
            for (auto& v : ins) bufs.push_back(In(v));
            bufs.push_back(Out(out));
            CompileAndRun(c.name, c.func, bufs);
        };
        run("cpu", out_cpu);
        run("hipgen", out_gpu);
        Check(std::memcmp(out_cpu.data(), out_gpu.data(), out_cpu.size() * sizeof(float)) == 0, c.name + ": generated kernel differs from the host loop nest");
        kxc::codegen::CodeGenHIP cgh;
        auto src = cgh.Generate(kxc::relay::LowerToTIR(kxc::relay::InferTypePass(c.func)), "kxc_t");
        bool found = false;
        for (const auto& k : src.kernels) found = found || k.schedule == c.schedule;
        Check(found, c.name + ": expected a " + c.schedule + " stage");
        std::cout << "[PASS] " << c.name << " (" << c.schedule << ")\n";
    }
    std::cout << "generated kernels ok\n";
    return 0;
}

// Quantised operators (qnn_quantize, qnn_conv2d, qnn_dense) through the compiler, bit-exact against hand-worked answers
// and against the C oracle loaded from the path given (its functions are bound by name, nothing else is linked).
int RunQnn(const std::string& oracle_path) {
    auto I8 = [](std::vector<int8_t>& v, bool out) { return Buf{v.data(), v.size(), out}; };
    auto I32 = [](std::vector<int32_t>& v) { return Buf{v.data(), v.size() * sizeof(int32_t), false}; };
    // ---- rounding: ties go to the even integer, NaN gives 0, saturation at +-127
    {
        kxc::Var x("x", kxc::TensorType({12}, "float32"));
        kxc::Function f({x}, kxc::Call(Op::Get("qnn_quantize"), {x}, kxc::relay::QnnQuantizeAttrs::Create(0.5)));
        std::vector<float> xd = {0.25f, 0.75f, 1.25f, -0.25f, -0.75f, 0.26f, 0.24f, 500.0f, -500.0f, std::nanf(""), 63.5f, -63.75f};
        std::vector<int8_t> q(12, 99);
        CompileAndRun("qnn_quantize", f, {In(xd), I8(q, true)});
        const std::vector<int8_t> expect = {0, 2, 2, 0, -2, 1, 0, 127, -127, 0, 127, -127};
        for (size_t i = 0; i < q.size(); ++i)
            Check(q[i] == expect[i], "qnn_quantize[" + std::to_string(i) + "] = " + std::to_string(q[i]) + ", expected " + std::to_string(expect[i]));
        std::cout << "[PASS] qnn_quantize rounding\n";
    }
    // ---- a 1x1x3x3 convolution worked by hand: 2x2 window of ones, bias 1, mult 0.25, residual weight 0.5
    {
        kxc::Var d("d", kxc::TensorType({1, 1, 3, 3}, "int8")), w("w", kxc::TensorType({1, 1, 2, 2}, "int8"));
        kxc::Var b("b", kxc::TensorType({1}, "int32")), m("m", kxc::TensorType({1}, "float32")), r("r", kxc::TensorType({1, 1, 2, 2}, "int8"));
        kxc::Function f({d, w, b, m, r}, kxc::Call(Op::Get("qnn_conv2d"), {d, w, b, m, r}, kxc::relay::QnnConv2DAttrs::Create({1, 1}, {0, 0}, true, 0.5)));
        std::vector<int8_t> dd = {1, 2, 3, 4, 5, 6, 7, 8, -100}, wd = {1, 1, 1, 1}, rd = {1, -20, 3, 0}, y(4, 99);
        std::vector<int32_t> bd = {1};
        std::vector<float> md = {0.25f};
        CompileAndRun("qnn_conv2d", f, {I8(dd, false), I8(wd, false), I32(bd), In(md), I8(rd, false), I8(y, true)});
        // sums 12 16 24 -81; +1 -> 13 17 25 -80; *0.25 -> 3.25 4.25 6.25 -20; + residual*0.5 -> 3.75 -5.75 7.75 -20; rint, relu
        const std::vector<int8_t> expect = {4, 0, 8, 0};
        Check(y == expect, "qnn_conv2d hand-worked case differs");
        std::cout << "[PASS] qnn_conv2d hand-worked\n";
    }
    void* lib = dlopen(oracle_path.c_str(), RTLD_NOW | RTLD_LOCAL);
    Check(lib != nullptr, "cannot load the oracle: " + oracle_path);
    using ConvFn = void (*)(const int8_t*, const int8_t*, const int32_t*, const float*, const int8_t*, float, int8_t*, int64_t, int64_t,
                            int64_t, int64_t, int64_t, int64_t, int64_t, int, int, int, int, int);
    using DenseFn = void (*)(const int8_t*, const int8_t*, const int32_t*, const float*, float*, int64_t, int64_t, int64_t);
    using QuantFn = void (*)(const float*, int8_t*, int64_t, float);
    auto oracle_conv = reinterpret_cast<ConvFn>(dlsym(lib, "kxc_oracle_qconv2d_nchw_i8"));
    auto oracle_dense = reinterpret_cast<DenseFn>(dlsym(lib, "kxc_oracle_qdense_i8"));
    auto oracle_quant = reinterpret_cast<QuantFn>(dlsym(lib, "kxc_oracle_quantize_f32_i8"));
    Check(oracle_conv && oracle_dense && oracle_quant, "oracle symbols missing");
    uint32_t seed = 2024;
    auto next = [&seed]() { seed = seed * 1664525u + 1013904223u; return seed >> 8; };
    auto fill_i8 = [&](std::vector<int8_t>& v) { for (auto& e : v) e = static_cast<int8_t>(static_cast<int>(next() % 255) - 127); };
    // ---- convolutions against the oracle: with and without residual / relu, strides 1 and 2, 1x1 / 3x3 / 7x7 windows
    struct CS { int64_t n, c, h, w, o, k; int s, p; bool relu, res; };
    const std::vector<CS> shapes = {{2, 5, 9, 7, 6, 3, 1, 1, true, true},   {1, 3, 8, 8, 4, 1, 2, 0, false, false},
                                    {1, 4, 10, 11, 8, 3, 2, 1, true, false}, {1, 3, 20, 20, 5, 7, 2, 3, false, true},
                                    {2, 16, 6, 6, 16, 3, 1, 1, true, true}};
    for (const auto& c : shapes) {
        const int64_t oh = (c.h + 2 * c.p - c.k) / c.s + 1, ow = (c.w + 2 * c.p - c.k) / c.s + 1;
        std::vector<int8_t> x(c.n * c.c * c.h * c.w), w(c.o * c.c * c.k * c.k), res(c.n * c.o * oh * ow), y(res.size(), 99), want(res.size(), 77);
        std::vector<int32_t> bias(c.o);
        std::vector<float> mult(c.o);
        fill_i8(x); fill_i8(w); fill_i8(res);
        for (auto& b : bias) b = static_cast<int32_t>(next() % 4001) - 2000;
        // multipliers sized so that outputs spread over the int8 range and some saturate
        for (auto& m : mult) m = (0.5f + static_cast<float>(next() % 1000) / 1000.0f) * 3.0f / (64.0f * std::sqrt(static_cast<float>(c.c * c.k * c.k)));
        const float res_mult = 0.37f;
        kxc::Var d("d", kxc::TensorType({c.n, c.c, c.h, c.w}, "int8")), wv("w", kxc::TensorType({c.o, c.c, c.k, c.k}, "int8"));
        kxc::Var b("b", kxc::TensorType({c.o}, "int32")), m("m", kxc::TensorType({c.o}, "float32")), r("r", kxc::TensorType({c.n, c.o, oh, ow}, "int8"));
        auto attrs = kxc::relay::QnnConv2DAttrs::Create({c.s, c.s}, {c.p, c.p}, c.relu, c.res ? res_mult : 0.0);
        std::vector<Buf> bufs = {I8(x, false), I8(w, false), I32(bias), In(mult)};
        kxc::Function f = c.res ? kxc::Function({d, wv, b, m, r}, kxc::Call(Op::Get("qnn_conv2d"), {d, wv, b, m, r}, attrs))
                                : kxc::Function({d, wv, b, m}, kxc::Call(Op::Get("qnn_conv2d"), {d, wv, b, m}, attrs));
        if (c.res) bufs.push_back(I8(res, false));
        bufs.push_back(I8(y, true));
        const std::string name = "qnn_conv2d " + std::to_string(c.c) + "x" + std::to_string(c.h) + "x" + std::to_string(c.w) + " k" +
                                 std::to_string(c.k) + " s" + std::to_string(c.s);
        CompileAndRun(name, f, bufs);
        oracle_conv(x.data(), w.data(), bias.data(), mult.data(), c.res ? res.data() : nullptr, res_mult, want.data(), c.n, c.c, c.h, c.w,
                    c.o, c.k, c.k, c.s, c.s, c.p, c.p, c.relu ? 1 : 0);
        int64_t saturated = 0, distinct[256] = {0}, kinds = 0;
        for (size_t i = 0; i < y.size(); ++i) {
            Check(y[i] == want[i], name + ": element " + std::to_string(i) + " = " + std::to_string(y[i]) + ", oracle " + std::to_string(want[i]));
            saturated += want[i] == 127;
            distinct[static_cast<uint8_t>(want[i])]++;
        }
        for (int64_t cnt : distinct) kinds += cnt > 0;
        Check(kinds > 20, name + ": the case does not spread over the int8 range");
        std::cout << "[PASS] " << name << " (" << kinds << " distinct values, " << saturated << " at +127)\n";
    }
    // ---- dense: float32 result compared as bits
    for (const auto& s : std::vector<std::array<int64_t, 3>>{{3, 10, 64}, {5, 7, 33}, {1, 1000, 512}}) {
        const int64_t M = s[0], N = s[1], K = s[2];
        std::vector<int8_t> a(M * K), bw(N * K);
        std::vector<int32_t> bias(N);
        std::vector<float> mult(N), y(M * N, -1.0f), want(M * N, -2.0f);
        fill_i8(a); fill_i8(bw);
        for (auto& b : bias) b = static_cast<int32_t>(next() % 20001) - 10000;
        for (auto& m : mult) m = static_cast<float>(1 + next() % 1000) / 65536.0f;
        kxc::Var av("a", kxc::TensorType({M, K}, "int8")), bv("b", kxc::TensorType({N, K}, "int8"));
        kxc::Var cv("c", kxc::TensorType({N}, "int32")), mv("m", kxc::TensorType({N}, "float32"));
        kxc::Function f({av, bv, cv, mv}, kxc::Call(Op::Get("qnn_dense"), {av, bv, cv, mv}));
        const std::string name = "qnn_dense " + std::to_string(M) + "x" + std::to_string(K) + " . " + std::to_string(N) + "x" + std::to_string(K);
        CompileAndRun(name, f, {I8(a, false), I8(bw, false), I32(bias), In(mult), Out(y)});
        oracle_dense(a.data(), bw.data(), bias.data(), mult.data(), want.data(), M, N, K);
        Check(std::memcmp(y.data(), want.data(), y.size() * sizeof(float)) == 0, name + " differs from the oracle");
        std::cout << "[PASS] " << name << "\n";
    }
    // ---- quantize against the oracle on values around every tie
    {
        const int64_t n = 4096;
        std::vector<float> x(n);
        for (int64_t i = 0; i < n; ++i) x[i] = (static_cast<float>(i) - 2048.0f) * 0.0625f * 0.0123f + (i % 3 == 0 ? 0.5f * 0.0123f : 0.0f);
        std::vector<int8_t> q(n, 99), want(n, 77);
        kxc::Var xv("x", kxc::TensorType({n}, "float32"));
        kxc::Function f({xv}, kxc::Call(Op::Get("qnn_quantize"), {xv}, kxc::relay::QnnQuantizeAttrs::Create(0.0123f)));
        CompileAndRun("qnn_quantize 4096", f, {In(x), I8(q, true)});
        oracle_quant(x.data(), want.data(), n, 0.0123f);
        Check(q == want, "qnn_quantize differs from the oracle");
        std::cout << "[PASS] qnn_quantize 4096\n";
    }
    // ---- a quantised chain: quantize -> conv (+relu) -> conv with the first as residual, each stage against the oracle
    {
        const int64_t N = 4, C = 8, H = 12, W = 12;
        std::vector<float> x(N * C * H * W), m1(C), m2(C);
        for (auto& v : x) v = static_cast<float>(static_cast<int>(next() % 2001) - 1000) / 400.0f;
        std::vector<int8_t> w1(C * C * 9), w2(C * C * 9), y(N * C * H * W, 99);
        std::vector<int32_t> b1(C), b2(C);
        fill_i8(w1); fill_i8(w2);
        for (int64_t i = 0; i < C; ++i) { b1[i] = static_cast<int32_t>(next() % 801) - 400; b2[i] = static_cast<int32_t>(next() % 801) - 400;
                                           m1[i] = 0.002f + 0.0001f * static_cast<float>(i); m2[i] = 0.003f - 0.0001f * static_cast<float>(i); }
        kxc::Var xv("x", kxc::TensorType({N, C, H, W}, "float32")), w1v("w1", kxc::TensorType({C, C, 3, 3}, "int8")), w2v("w2", kxc::TensorType({C, C, 3, 3}, "int8"));
        kxc::Var b1v("b1", kxc::TensorType({C}, "int32")), b2v("b2", kxc::TensorType({C}, "int32")), m1v("m1", kxc::TensorType({C}, "float32")), m2v("m2", kxc::TensorType({C}, "float32"));
        kxc::Call q(Op::Get("qnn_quantize"), {xv}, kxc::relay::QnnQuantizeAttrs::Create(0.02));
        kxc::Call c1(Op::Get("qnn_conv2d"), {q, w1v, b1v, m1v}, kxc::relay::QnnConv2DAttrs::Create({1, 1}, {1, 1}, true));
        kxc::Call c2(Op::Get("qnn_conv2d"), {c1, w2v, b2v, m2v, q}, kxc::relay::QnnConv2DAttrs::Create({1, 1}, {1, 1}, true, 0.75));
        kxc::Function f({xv, w1v, b1v, m1v, w2v, b2v, m2v}, c2);
        CompileAndRun("qnn chain", f, {In(x), I8(w1, false), I32(b1), In(m1), I8(w2, false), I32(b2), In(m2), I8(y, true)});
        std::vector<int8_t> xq(x.size()), t1(x.size()), want(x.size());
        oracle_quant(x.data(), xq.data(), static_cast<int64_t>(x.size()), 0.02f);
        oracle_conv(xq.data(), w1.data(), b1.data(), m1.data(), nullptr, 0.0f, t1.data(), N, C, H, W, C, 3, 3, 1, 1, 1, 1, 1);
        oracle_conv(t1.data(), w2.data(), b2.data(), m2.data(), xq.data(), 0.75f, want.data(), N, C, H, W, C, 3, 3, 1, 1, 1, 1, 1);
        Check(y == want, "qnn chain differs from the oracle");
        if (g_mode == "hip") {
            // the same graph as two shares of two images side by side (chains of the plan on halves of x and y)
            setenv("KXC_HIP_BATCH_LANES", "2", 1);
            std::vector<int8_t> y2(y.size(), 55);
            try {
                CompileAndRun("qnn chain in two shares", f, {In(x), I8(w1, false), I32(b1), In(m1), I8(w2, false), I32(b2), In(m2), I8(y2, true)});
                auto shares = kxc::api::Compiler::Compile(f, MakeConfig());
                Check(shares.GetKernelExecs().size() == 6 && shares.GetKernelExecs().back().kernel_symbol.find(" @share1") != std::string::npos,
                      "qnn chain: two shares expected");
            } catch (...) { unsetenv("KXC_HIP_BATCH_LANES"); throw; }
            unsetenv("KXC_HIP_BATCH_LANES");
            Check(y2 == want, "qnn chain in two shares differs from the oracle");
        }
        if (g_mode != "cpu") {
            // hip: the three operators dispatch to the hand-written int8 launches; hipgen: to generated kernels only
            int quant = 0, conv = 0;
            auto module = kxc::api::Compiler::Compile(f, MakeConfig());
            for (const auto& k : module.GetKernelExecs()) {
                quant += k.kernel_symbol.find("kxc_quantize_f32_i8") != std::string::npos;
                conv += k.kernel_symbol.find("kxc_qconv2d_nchw_i8") != std::string::npos;
            }
            Check(g_mode == "hip" ? (quant == 1 && conv == 2) : (quant == 0 && conv == 0),
                  "qnn chain: unexpected dispatch, quantize launches " + std::to_string(quant) + ", conv launches " + std::to_string(conv));
        }
        std::cout << "[PASS] qnn chain (quantize, conv, conv + residual)\n";
    }
    // ---- int8 max pool (padding candidate and reduce identity are the dtype's lowest value) and the requantising
    // global average pool, against the oracle; negative inputs everywhere so that a zero identity would show
    {
        using PoolFn = void (*)(const int8_t*, int8_t*, int64_t, int64_t, int64_t, int64_t, int, int, int, int, int, int, int, int);
        using GapFn = void (*)(const int8_t*, int8_t*, int64_t, int64_t, int64_t, int64_t, float);
        auto oracle_pool = reinterpret_cast<PoolFn>(dlsym(lib, "kxc_oracle_maxpool2d_i8"));
        auto oracle_gap = reinterpret_cast<GapFn>(dlsym(lib, "kxc_oracle_global_avg_pool2d_i8"));
        Check(oracle_pool && oracle_gap, "oracle pooling symbols missing");
        const int64_t N = 2, C = 5, H = 9, W = 11;
        std::vector<int8_t> x(N * C * H * W);
        for (auto& e : x) e = static_cast<int8_t>(-128 + static_cast<int>(next() % 100));       // all negative
        const int64_t OH = (H + 2 - 3) / 2 + 1, OW = (W + 2 - 3) / 2 + 1;
        std::vector<int8_t> y(N * C * OH * OW, 99), want(y.size(), 77);
        kxc::Var xv("x", kxc::TensorType({N, C, H, W}, "int8"));
        kxc::Function fp({xv}, kxc::Call(Op::Get("nn_max_pool2d"), {xv},
                                         kxc::relay::MaxPool2DAttrs::Create({2, 2}, {1, 1, 1, 1}, {1, 1}, {3, 3}, "NCHW", false)));
        CompileAndRun("int8 max pool", fp, {I8(x, false), I8(y, true)});
        oracle_pool(x.data(), want.data(), N, C, H, W, 3, 3, 2, 2, 1, 1, 1, 1);
        Check(y == want, "int8 nn_max_pool2d differs from the oracle");
        std::cout << "[PASS] int8 nn_max_pool2d on negative data\n";
        fill_i8(x);
        std::vector<int8_t> g(N * C, 99), gw(N * C, 77);
        const float mult = 0.0173f;
        kxc::Function fg({xv}, kxc::Call(Op::Get("qnn_global_avg_pool2d"), {xv}, kxc::relay::QnnRequantAttrs::Create(mult)));
        CompileAndRun("qnn_global_avg_pool2d", fg, {I8(x, false), I8(g, true)});
        oracle_gap(x.data(), gw.data(), N, C, H, W, mult);
        Check(g == gw, "qnn_global_avg_pool2d differs from the oracle");
        std::cout << "[PASS] qnn_global_avg_pool2d\n";
    }
    // ---- a chain wide enough for the int8 matrix cores: on the hip target the convolutions, the pool and the average
    // run channel-blocked with the weights packed by the plan, and converters appear only where NCHW tensors enter
    // (the int8 parameter, the residual parameter) -- same bytes as the oracle either way
    {
        using PoolFn = void (*)(const int8_t*, int8_t*, int64_t, int64_t, int64_t, int64_t, int, int, int, int, int, int, int, int);
        using GapFn = void (*)(const int8_t*, int8_t*, int64_t, int64_t, int64_t, int64_t, float);
        auto oracle_pool = reinterpret_cast<PoolFn>(dlsym(lib, "kxc_oracle_maxpool2d_i8"));
        auto oracle_gap = reinterpret_cast<GapFn>(dlsym(lib, "kxc_oracle_global_avg_pool2d_i8"));
        const int64_t N = 3, C = 24, H = 14, W = 10, O = 64;
        std::vector<int8_t> x(N * C * H * W), w1(O * C * 9), w2(O * O * 9), wd(O * C), res(N * O * 7 * 5);
        std::vector<int32_t> b1(O), b2(O), bd(O);
        std::vector<float> m1(O), m2(O), md(O);
        fill_i8(x); fill_i8(w1); fill_i8(w2); fill_i8(wd); fill_i8(res);
        for (int64_t i = 0; i < O; ++i) {
            b1[i] = static_cast<int32_t>(next() % 2001) - 1000; b2[i] = static_cast<int32_t>(next() % 2001) - 1000; bd[i] = static_cast<int32_t>(next() % 201) - 100;
            m1[i] = (0.5f + static_cast<float>(next() % 1000) / 1000.0f) / (64.0f * std::sqrt(static_cast<float>(C * 9)));
            m2[i] = (0.5f + static_cast<float>(next() % 1000) / 1000.0f) / (24.0f * std::sqrt(static_cast<float>(O * 9)));
            md[i] = (0.5f + static_cast<float>(next() % 1000) / 1000.0f) / (64.0f * std::sqrt(static_cast<float>(C)));
        }
        kxc::Var xv("x", kxc::TensorType({N, C, H, W}, "int8")), rv("r", kxc::TensorType({N, O, 7, 5}, "int8"));
        kxc::Var w1v("w1", kxc::TensorType({O, C, 3, 3}, "int8")), w2v("w2", kxc::TensorType({O, O, 3, 3}, "int8")), wdv("wd", kxc::TensorType({O, C, 1, 1}, "int8"));
        kxc::Var b1v("b1", kxc::TensorType({O}, "int32")), b2v("b2", kxc::TensorType({O}, "int32")), bdv("bd", kxc::TensorType({O}, "int32"));
        kxc::Var m1v("m1", kxc::TensorType({O}, "float32")), m2v("m2", kxc::TensorType({O}, "float32")), mdv("md", kxc::TensorType({O}, "float32"));
        // block: a = conv3x3/2(x) relu; idn = conv1x1/2(x); s = conv3x3(a) + idn, relu; t = conv3x3(s) + r (a parameter), relu;
        // p = maxpool(t); g = gap(p)
        kxc::Call a(Op::Get("qnn_conv2d"), {xv, w1v, b1v, m1v}, kxc::relay::QnnConv2DAttrs::Create({2, 2}, {1, 1}, true));
        kxc::Call idn(Op::Get("qnn_conv2d"), {xv, wdv, bdv, mdv}, kxc::relay::QnnConv2DAttrs::Create({2, 2}, {0, 0}, false));
        kxc::Call sum(Op::Get("qnn_conv2d"), {a, w2v, b2v, m2v, idn}, kxc::relay::QnnConv2DAttrs::Create({1, 1}, {1, 1}, true, 0.6));
        kxc::Call t(Op::Get("qnn_conv2d"), {sum, w2v, b2v, m2v, rv}, kxc::relay::QnnConv2DAttrs::Create({1, 1}, {1, 1}, true, 0.4));
        kxc::Call pool(Op::Get("nn_max_pool2d"), {t}, kxc::relay::MaxPool2DAttrs::Create({2, 2}, {1, 1, 1, 1}, {1, 1}, {3, 3}, "NCHW", false));
        kxc::Call gap(Op::Get("qnn_global_avg_pool2d"), {pool}, kxc::relay::QnnRequantAttrs::Create(0.21));
        std::vector<int8_t> ya(N * O * 7 * 5), yi(ya.size()), ys(ya.size()), yt(ya.size()), yp(N * O * 4 * 3), yg(N * O);
        oracle_conv(x.data(), w1.data(), b1.data(), m1.data(), nullptr, 0.0f, ya.data(), N, C, H, W, O, 3, 3, 2, 2, 1, 1, 1);
        oracle_conv(x.data(), wd.data(), bd.data(), md.data(), nullptr, 0.0f, yi.data(), N, C, H, W, O, 1, 1, 2, 2, 0, 0, 0);
        oracle_conv(ya.data(), w2.data(), b2.data(), m2.data(), yi.data(), 0.6f, ys.data(), N, O, 7, 5, O, 3, 3, 1, 1, 1, 1, 1);
        oracle_conv(ys.data(), w2.data(), b2.data(), m2.data(), res.data(), 0.4f, yt.data(), N, O, 7, 5, O, 3, 3, 1, 1, 1, 1, 1);
        oracle_pool(yt.data(), yp.data(), N, O, 7, 5, 3, 3, 2, 2, 1, 1, 1, 1);
        oracle_gap(yp.data(), yg.data(), N, O, 4, 3, 0.21f);
        const std::vector<kxc::Var> params = {xv, rv, w1v, b1v, m1v, w2v, b2v, m2v, wdv, bdv, mdv};
        auto bufs = [&](std::vector<int8_t>& out) {
            return std::vector<Buf>{I8(x, false), I8(res, false), I8(w1, false), I32(b1), In(m1), I8(w2, false), I32(b2), In(m2), I8(wd, false), I32(bd), In(md), I8(out, true)};
        };
        struct Cut { const char* name; kxc::Expr value; std::vector<int8_t>* want; };
        for (const Cut& c : {Cut{"t", t, &yt}, Cut{"pool", pool, &yp}, Cut{"gap", gap, &yg}, Cut{"idn", idn, &yi}}) {
            std::vector<int8_t> got(c.want->size(), 99);
            kxc::Function f(params, c.value);
            CompileAndRun(std::string("wide qnn chain cut at ") + c.name, f, bufs(got));
            Check(got == *c.want, std::string("wide qnn chain cut at ") + c.name + " differs from the oracle");
        }
        if (g_mode == "hip") {
            auto module = kxc::api::Compiler::Compile(kxc::Function(params, gap), MakeConfig());
            std::string all;
            int c16 = 0, to_c16 = 0, to_nchw = 0;
            for (const auto& k : module.GetKernelExecs()) {
                all += k.kernel_symbol + "; ";
                c16 += k.kernel_symbol.find("kxc_qconv2d_c16_i8") != std::string::npos;
                to_c16 += k.kernel_symbol == "kxc_i8_nchw_to_c16";
                to_nchw += k.kernel_symbol == "kxc_i8_c16_to_nchw";
            }
            // pair (a + idn), sum, t on the matrix cores; x and r converted on the way in; the pool and the average blocked
            Check(c16 == 3 && to_c16 == 2 && to_nchw == 0 && all.find("|qconv1x1+bias") != std::string::npos &&
                      all.find("kxc_max_pool2d_c16_i8") != std::string::npos && all.find("kxc_global_avg_pool2d_c16_i8") != std::string::npos,
                  "wide qnn chain: unexpected launches: " + all);
        }
        std::cout << "[PASS] wide qnn chain (matrix-core layouts on hip)\n";
    }
    // ---- type rules
    {
        auto expect_throw = [](const std::function<void()>& fn, const std::string& needle) {
            try { fn(); } catch (const std::exception& e) {
                Check(std::string(e.what()).find(needle) != std::string::npos, std::string("unexpected message: ") + e.what());
                return;
            }
            throw std::runtime_error("no exception, expected: " + needle);
        };
        expect_throw([] {
            kxc::Var d("d", kxc::TensorType({1, 4, 8, 8}, "float32")), w("w", kxc::TensorType({8, 4, 3, 3}, "int8"));
            kxc::Var b("b", kxc::TensorType({8}, "int32")), m("m", kxc::TensorType({8}, "float32"));
            kxc::relay::InferTypePass(kxc::Function({d, w, b, m}, kxc::Call(Op::Get("qnn_conv2d"), {d, w, b, m}, kxc::relay::QnnConv2DAttrs::Create({1, 1}, {1, 1}, false))));
        }, "int8");
        expect_throw([] {
            kxc::Var d("d", kxc::TensorType({1, 4, 8, 8}, "int8")), w("w", kxc::TensorType({8, 4, 3, 3}, "int8"));
            kxc::Var b("b", kxc::TensorType({7}, "int32")), m("m", kxc::TensorType({8}, "float32"));
            kxc::relay::InferTypePass(kxc::Function({d, w, b, m}, kxc::Call(Op::Get("qnn_conv2d"), {d, w, b, m}, kxc::relay::QnnConv2DAttrs::Create({1, 1}, {1, 1}, false))));
        }, "bias");
        expect_throw([] {
            kxc::Var d("d", kxc::TensorType({4}, "int8"));
            kxc::relay::InferTypePass(kxc::Function({d}, kxc::Call(Op::Get("qnn_quantize"), {d}, kxc::relay::QnnQuantizeAttrs::Create(1.0))));
        }, "float32");
        std::cout << "[PASS] qnn type rules\n";
    }
    dlclose(lib);
    std::cout << "quantised operators ok (" << g_mode << ")\n";
    return 0;
}

// relay::SplitBatch: graphs whose samples are independent split into shares, everything else is refused.
int RunSplitBatch() {
    using kxc::relay::SplitBatch; using kxc::relay::InferTypePass;
    auto shape0 = [](const kxc::Function& f) { return f->body.checked_type().As<kxc::TensorTypeNode>()->shape; };
    // ---- the ResNet-18 graph at batch 8 splits into 2 and 4 shares, not into 3
    {
        kxc::Function net = InferTypePass(kxc::models::BuildResNet18(8, 64));
        kxc::Function half = SplitBatch(net, 2), quarter = SplitBatch(net, 4);
        Check(half.defined() && quarter.defined(), "ResNet-18 should split along the batch");
        Check(shape0(half) == std::vector<int64_t>({4, 1000}) && shape0(quarter) == std::vector<int64_t>({2, 1000}), "share output shape");
        Check(half->params.size() == net->params.size(), "a share keeps the parameters");
        Check(!SplitBatch(net, 3).defined(), "8 samples do not divide into 3 shares");
        Check(!SplitBatch(net, 16).defined(), "more shares than samples");
        // constants are shared, calls are cloned
        std::set<const kxc::RelayExprNode*> c_full, c_half;
        std::function<void(const kxc::Expr&, std::set<const kxc::RelayExprNode*>*)> walk = [&](const kxc::Expr& e, std::set<const kxc::RelayExprNode*>* out) {
            if (e.As<kxc::ConstantNode>()) { out->insert(e.get()); return; }
            if (const auto* c = e.As<kxc::CallNode>()) for (const auto& a : c->args) walk(a, out);
        };
        walk(net->body, &c_full); walk(half->body, &c_half);
        Check(!c_full.empty() && c_full == c_half, "the shares read the graph's own constants");
        std::cout << "[PASS] ResNet-18 splits into shares\n";
    }
    auto var = [](const char* n, std::vector<int64_t> shape, const char* dt = "float32") { return kxc::Var(n, kxc::TensorType(shape, dt)); };
    auto splits = [&](kxc::Function f) { return SplitBatch(InferTypePass(f), 2).defined(); };
    // ---- accepted
    {
        kxc::Var x = var("x", {4, 6}), w = var("w", {5, 6}), b = var("b", {5});
        Check(splits(kxc::Function({x, w}, kxc::Call(Op::Get("nn_dense"), {x, w}, kxc::relay::DenseAttrs::Create(5, "")))), "dense");
        Check(splits(kxc::Function({x, w, b}, kxc::Call(Op::Get("nn_gemm"), {x, w, b}, kxc::relay::GemmAttrs::Create(1, 1, 0, 1)))), "gemm");
        Check(splits(kxc::Function({x}, kxc::Call(Op::Get("softmax"), {x}, kxc::relay::SoftmaxAttrs::Create(-1)))), "softmax over the last axis");
        Check(splits(kxc::Function({x}, kxc::Call(Op::Get("reduce_mean"), {x}, kxc::relay::ReduceMeanAttrs::Create({1}, 0)))), "reduce_mean over axis 1");
        kxc::Var y = var("y", {6});
        Check(splits(kxc::Function({x, y}, kxc::Call(Op::Get("add"), {x, y}))), "add with a broadcast row");
        Check(splits(kxc::Function({x}, kxc::Call(Op::Get("add"), {x, x}))), "add of two batched values");
        kxc::Var t = var("t", {4, 2, 3});
        Check(splits(kxc::Function({t}, kxc::Call(Op::Get("transpose"), {t}, kxc::relay::TransposeAttrs::Create({0, 2, 1})))), "transpose that keeps axis 0");
        kxc::Var q = var("q", {4, 3, 8, 8});
        Check(splits(kxc::Function({q}, kxc::Call(Op::Get("qnn_quantize"), {q}, kxc::relay::QnnQuantizeAttrs::Create(0.5)))), "qnn_quantize");
        std::cout << "[PASS] separable graphs are accepted\n";
    }
    // ---- refused: an operator that mixes samples, or a value that would have to be cut without being parameter 0
    {
        kxc::Var x = var("x", {4, 6}), w = var("w", {5, 6});
        Check(!splits(kxc::Function({x}, kxc::Call(Op::Get("softmax"), {x}, kxc::relay::SoftmaxAttrs::Create(0)))), "softmax over the batch");
        Check(!splits(kxc::Function({x}, kxc::Call(Op::Get("softmax"), {x}, kxc::relay::SoftmaxAttrs::Create(-2)))), "softmax over the batch, negative axis");
        Check(!splits(kxc::Function({x}, kxc::Call(Op::Get("reduce_mean"), {x}, kxc::relay::ReduceMeanAttrs::Create({0}, 0)))), "reduce_mean over the batch");
        Check(!splits(kxc::Function({x}, kxc::Call(Op::Get("transpose"), {x}, kxc::relay::TransposeAttrs::Create({1, 0})))), "transpose moves the batch");
        Check(!splits(kxc::Function({x}, kxc::Call(Op::Get("reshape"), {x}, kxc::relay::ReshapeAttrs::Create({2, 12})))), "reshape");
        Check(!splits(kxc::Function({x}, kxc::Call(Op::Get("nn_flatten"), {x}, kxc::relay::FlattenAttrs::Create(0)))), "flatten from axis 0");
        // the batch on the right-hand operand of a product
        kxc::Var w4 = var("w4", {4, 6});
        Check(!splits(kxc::Function({w4, x}, kxc::Call(Op::Get("nn_dense"), {x, w4}, kxc::relay::DenseAttrs::Create(4, "")))), "batched weight");
        kxc::Var a = var("a", {4, 4}), b2 = var("b", {4, 4});
        Check(!splits(kxc::Function({a, b2}, kxc::Call(Op::Get("matmul"), {b2, a}))), "matmul with the batch on the right");
        // a second operand of the batch's full shape that is not derived from parameter 0
        kxc::Var y = var("y", {4, 6});
        Check(!splits(kxc::Function({x, y}, kxc::Call(Op::Get("add"), {x, y}))), "add with an unbatched operand of batch extent");
        // the result does not carry the batch
        Check(!splits(kxc::Function({x, w}, kxc::Call(Op::Get("nn_relu"), {w}, kxc::relay::ReluAttrs::Create()))), "result independent of parameter 0");
        // shares must divide
        kxc::Var odd = var("odd", {5, 6});
        Check(!splits(kxc::Function({odd}, kxc::Call(Op::Get("nn_relu"), {odd}, kxc::relay::ReluAttrs::Create()))), "5 samples in 2 shares");
        std::cout << "[PASS] inseparable graphs are refused\n";
    }
    // ---- an explicit request the graph does not allow makes Compile throw (dry hip target: no GPU needed up to loading)
    {
        kxc::Var x = var("x", {4, 8});
        kxc::Function f({x}, kxc::Call(Op::Get("softmax"), {x}, kxc::relay::SoftmaxAttrs::Create(0)));
        auto cfg = kxc::api::CompileConfig::JIT(kxc::BuildTarget(kxc::kGPU));
        cfg->hip_batch_lanes = 2;
        bool threw = false;
        try { kxc::api::Compiler::Compile(f, cfg); } catch (const std::exception& e) {
            threw = std::string(e.what()).find("cannot be split along the batch") != std::string::npos;
        }
        Check(threw, "hip_batch_lanes = 2 on an inseparable graph should throw");
        std::cout << "[PASS] explicit request on an inseparable graph throws\n";
    }
    std::cout << "split batch ok\n";
    return 0;
}

// Shares of a batch on the GPU for a graph that mixes hand-written launches and generated kernels (softmax has no
// hand-written kernel): the shares reuse one compiled module per step, and give the one-share result bit for bit.
int RunSharesGenerated() {
    g_mode = "hip";
    const int64_t N = 8, C = 4, H = 6, O = 8;
    kxc::Var x("x", kxc::TensorType({N, C, H, H}, "float32"));
    kxc::Var w("w", kxc::TensorType({O, C, 3, 3}, "float32"));
    auto attrs = kxc::relay::Conv2DAttrs::Create({1, 1}, {1, 1, 1, 1}, {1, 1}, 1, O, {3, 3}, "NCHW", "OIHW", "", "");
    kxc::Call conv(Op::Get("nn_conv2d"), {x, w}, attrs);
    kxc::Call relu(Op::Get("nn_relu"), {conv}, kxc::relay::ReluAttrs::Create());
    kxc::Call gap(Op::Get("nn_global_avg_pool2d"), {relu}, kxc::relay::GlobalAvgPool2DAttrs::Create());
    kxc::Call flat(Op::Get("nn_flatten"), {gap}, kxc::relay::FlattenAttrs::Create(1));
    kxc::Call sm(Op::Get("softmax"), {flat}, kxc::relay::SoftmaxAttrs::Create(-1));
    kxc::Function f({x, w}, sm);
    std::vector<float> xd(N * C * H * H), wd(O * C * 9);
    uint32_t seed = 99;
    for (auto* v : {&xd, &wd})
        for (float& e : *v) { seed = seed * 1664525u + 1013904223u; e = static_cast<float>(static_cast<int32_t>(seed >> 8) % 2001 - 1000) / 1000.0f; }
    std::vector<std::vector<float>> outs;
    for (int lanes : {1, 2, 4}) {
        auto cfg = MakeConfig();
        cfg->hip_batch_lanes = lanes;
        auto module = kxc::api::Compiler::Compile(f, cfg);
        Check(module.IsReady(), "module should be ready: " + module.GetStatus());
        const auto& execs = module.GetKernelExecs();
        const size_t per_share = execs.size() / static_cast<size_t>(lanes);
        Check(execs.size() == per_share * static_cast<size_t>(lanes), "launch count is a multiple of the shares");
        size_t generated = 0;
        for (const auto& e : execs) generated += e.kernel_symbol.find("[generated:") != std::string::npos;
        Check(generated >= static_cast<size_t>(lanes), "softmax runs through generated kernels in every share");
        if (lanes > 1) Check(execs.back().kernel_symbol.find(" @share" + std::to_string(lanes - 1)) != std::string::npos, "last launch belongs to the last share");
        kxc::DeviceAPI* api = kxc::GetDeviceAPI(kxc::kGPU);
        kxc::Device dev(kxc::kGPU, 0), cpu(kxc::kCPU, 0);
        std::vector<float> out(N * O, -1.0f);
        void* dx = api->AllocDataSpace(dev, xd.size() * 4, 256);
        void* dw = api->AllocDataSpace(dev, wd.size() * 4, 256);
        void* dy = api->AllocDataSpace(dev, out.size() * 4, 256);
        api->CopyDataFromTo(cpu, xd.data(), dev, dx, xd.size() * 4);
        api->CopyDataFromTo(cpu, wd.data(), dev, dw, wd.size() * 4);
        for (int rep = 0; rep < 3; ++rep) module.Run({dx, dw, dy});
        api->CopyDataFromTo(dev, dy, cpu, out.data(), out.size() * 4);
        // the saved plan rebuilds (generated modules compiled again from the saved source, once per distinct source)
        auto again = kxc::api::Compiler::LoadExecutionPlan(module.ExecutionPlanJSON(), cfg);
        std::vector<float> out2(N * O, -2.0f);
        again.Run({dx, dw, dy});
        api->CopyDataFromTo(dev, dy, cpu, out2.data(), out2.size() * 4);
        Check(std::memcmp(out.data(), out2.data(), out.size() * 4) == 0, "rebuilt plan differs");
        for (void* p : {dx, dw, dy}) api->FreeDataSpace(dev, p);
        for (int64_t n = 0; n < N; ++n) {
            float sum = 0.0f;
            for (int64_t o = 0; o < O; ++o) sum += out[n * O + o];
            Check(std::fabs(sum - 1.0f) < 1e-5f, "softmax rows sum to 1");
        }
        outs.push_back(out);
        std::cout << "[PASS] " << lanes << " share(s): " << execs.size() << " launches\n";
    }
    Check(std::memcmp(outs[0].data(), outs[1].data(), outs[0].size() * 4) == 0, "two shares differ from one");
    Check(std::memcmp(outs[0].data(), outs[2].data(), outs[0].size() * 4) == 0, "four shares differ from one");
    std::cout << "shares with generated kernels ok\n";
    return 0;
}

// Random small convolutional graphs (plain and strided convolutions, pools, residual blocks with and without a
// downsample branch, a dense head, sometimes a softmax) at batch 4 or 8: the hip back end in one share and in two
// shares of the batch against the host back end (operator tolerance) and against each other.
int RunSharesRandom() {
    uint32_t seed = 4242;
    auto next = [&seed]() { seed = seed * 1664525u + 1013904223u; return seed >> 8; };
    auto uniform = [&](float lo, float hi) { return lo + (hi - lo) * static_cast<float>(next() % 100001) / 100000.0f; };
    auto constant = [&](std::vector<int64_t> shape, float scale) {
        kxc::runtime::NDArray a(shape, "float32");
        std::vector<float> v(static_cast<size_t>(kxc::Product(shape)));
        for (float& e : v) e = uniform(-scale, scale);
        a.CopyFromBytes(v.data(), v.size() * sizeof(float));
        return kxc::Constant(a);
    };
    auto conv = [&](kxc::Expr x, int64_t c, int64_t o, int k, int s, int p, bool bias) {
        auto attrs = kxc::relay::Conv2DAttrs::Create({s, s}, {p, p, p, p}, {1, 1}, 1, static_cast<int>(o), {k, k}, "NCHW", "OIHW", "", "");
        const float scale = std::sqrt(3.0f / static_cast<float>(c * k * k));
        if (bias) return kxc::Expr(kxc::Call(Op::Get("nn_conv2d"), {x, constant({o, c, k, k}, scale), constant({o}, 0.1f)}, attrs));
        return kxc::Expr(kxc::Call(Op::Get("nn_conv2d"), {x, constant({o, c, k, k}, scale)}, attrs));
    };
    auto relu = [](kxc::Expr x) { return kxc::Expr(kxc::Call(Op::Get("nn_relu"), {x}, kxc::relay::ReluAttrs::Create())); };
    auto add = [](kxc::Expr a, kxc::Expr b) { return kxc::Expr(kxc::Call(Op::Get("add"), {a, b})); };
    const int trials = 8;
    for (int trial = 0; trial < trials; ++trial) {
        const int64_t N = (trial % 2) ? 8 : 4;
        int64_t c = 3 + static_cast<int64_t>(next() % 6), h = 12 + 4 * static_cast<int64_t>(next() % 4);
        kxc::Var x("x", kxc::TensorType({N, c, h, h}, "float32"));
        std::vector<float> xd(static_cast<size_t>(N * c * h * h));
        for (float& e : xd) e = uniform(-1.0f, 1.0f);
        kxc::Expr e = x;
        std::string recipe;
        const int layers = 4 + static_cast<int>(next() % 4);
        for (int l = 0; l < layers; ++l) {
            const int kind = static_cast<int>(next() % 5);
            if (kind == 0) {
                const int64_t o = 8 * (1 + static_cast<int64_t>(next() % 4));
                e = conv(e, c, o, 3, 1, 1, next() % 2 == 0);
                if (next() % 2) e = relu(e);
                c = o; recipe += "c";
            } else if (kind == 1 && h >= 8) {
                const int64_t o = 8 * (1 + static_cast<int64_t>(next() % 4));
                e = relu(conv(e, c, o, 3, 2, 1, true));
                c = o; h = (h + 2 - 3) / 2 + 1; recipe += "s";
            } else if (kind == 2 && h >= 8) {
                const bool is_max = next() % 2 == 0;
                auto attrs = kxc::relay::MaxPool2DAttrs::Create({2, 2}, {1, 1, 1, 1}, {1, 1}, {3, 3}, "NCHW", false);
                e = kxc::Expr(kxc::Call(Op::Get(is_max ? "nn_max_pool2d" : "nn_avg_pool2d"), {e}, attrs));
                h = (h + 2 - 3) / 2 + 1; recipe += is_max ? "m" : "a";
            } else if (kind == 3) {
                kxc::Expr a = relu(conv(e, c, c, 3, 1, 1, true));
                e = relu(add(conv(a, c, c, 3, 1, 1, true), e));
                recipe += "r";
            } else if (h >= 8) {
                const int64_t o = 2 * c;
                kxc::Expr a = relu(conv(e, c, o, 3, 2, 1, true));
                kxc::Expr id = conv(e, c, o, 1, 2, 0, true);
                e = relu(add(conv(a, o, o, 3, 1, 1, true), id));
                c = o; h = (h + 2 - 3) / 2 + 1; recipe += "d";
            }
        }
        e = kxc::Expr(kxc::Call(Op::Get("nn_global_avg_pool2d"), {e}, kxc::relay::GlobalAvgPool2DAttrs::Create()));
        e = kxc::Expr(kxc::Call(Op::Get("nn_flatten"), {e}, kxc::relay::FlattenAttrs::Create(1)));
        const int64_t classes = 12;
        e = kxc::Expr(kxc::Call(Op::Get("nn_gemm"), {e, constant({classes, c}, 0.3f), constant({classes}, 0.1f)}, kxc::relay::GemmAttrs::Create(1.0f, 1.0f, 0, 1)));
        if (trial % 3 == 0) { e = kxc::Expr(kxc::Call(Op::Get("softmax"), {e}, kxc::relay::SoftmaxAttrs::Create(-1))); recipe += "+softmax"; }
        kxc::Function f({x}, e);
        auto run = [&](bool gpu, int lanes, size_t* launches) {
            auto cfg = kxc::api::CompileConfig::JIT(kxc::BuildTarget(gpu ? kxc::kGPU : kxc::kCPU));
            cfg->opt_level = 0;
            cfg->hip_batch_lanes = lanes;
            auto module = kxc::api::Compiler::Compile(f, cfg);
            Check(module.IsReady(), "module should be ready: " + module.GetStatus());
            *launches = module.GetKernelExecs().size();
            std::vector<float> out(static_cast<size_t>(N * classes), -7.0f);
            const auto& consts = module.GetConstants();
            std::vector<void*> args;
            if (!gpu) {
                args.push_back(xd.data());
                for (const auto& k : consts) args.push_back(const_cast<void*>(k->data()));
                args.push_back(out.data());
                module.Run(args);
                return out;
            }
            kxc::DeviceAPI* api = kxc::GetDeviceAPI(kxc::kGPU);
            kxc::Device dev(kxc::kGPU, 0), cpu(kxc::kCPU, 0);
            auto up = [&](const void* src, size_t bytes) {
                void* d = api->AllocDataSpace(dev, bytes, 256);
                api->CopyDataFromTo(cpu, const_cast<void*>(src), dev, d, bytes);
                return d;
            };
            args.push_back(up(xd.data(), xd.size() * 4));
            for (const auto& k : consts) args.push_back(up(k->data(), k.nbytes()));
            args.push_back(api->AllocDataSpace(dev, out.size() * 4, 256));
            for (int rep = 0; rep < 2; ++rep) module.Run(args);      // twice: the workspace is reused
            api->CopyDataFromTo(dev, args.back(), cpu, out.data(), out.size() * 4);
            for (void* p : args) api->FreeDataSpace(dev, p);
            return out;
        };
        size_t l_cpu = 0, l_one = 0, l_two = 0;
        const std::vector<float> want = run(false, 1, &l_cpu), one = run(true, 1, &l_one), two = run(true, 2, &l_two);
        Check(l_two == 2 * l_one, "two shares should hold twice the launches of one (" + std::to_string(l_two) + " vs " + std::to_string(l_one) + ")");
        float scale = 0.0f;
        for (float v : want) scale = std::max(scale, std::fabs(v));
        Check(scale > 0.0f && std::isfinite(scale), "degenerate case");
        for (size_t i = 0; i < want.size(); ++i) {
            Check(std::fabs(one[i] - want[i]) <= 1e-3f * std::max(scale, 1.0f), "trial " + std::to_string(trial) + " [" + recipe + "]: one share differs from the host back end at " + std::to_string(i));
            Check(std::fabs(two[i] - one[i]) <= 1e-4f * std::max(scale, 1.0f), "trial " + std::to_string(trial) + " [" + recipe + "]: two shares differ from one at " + std::to_string(i));
        }
        std::cout << "[PASS] trial " << trial << " batch " << N << " [" << recipe << "]: " << l_one << " launches per share\n";
    }
    std::cout << "random graphs in shares ok\n";
    return 0;
}

// The registry face of the device API and of the plan functions (include/base/registry.h, src/base/device_api.cc:442-658).
int RunPackedFunc(const std::string& mode) {
    using kxc::PackedFunc; using kxc::Registry; using kxc::RetValue;
    Registry& reg = Registry::Global();
    Check(!reg.Get("no.such.function").defined(), "an absent name gives an empty function");
    bool threw = false;
    try { RetValue rv; reg.Get("no.such.function")(kxc::Args(), &rv); } catch (const std::runtime_error& e) { threw = std::string(e.what()) == "PackedFunc is empty"; }
    Check(threw, "calling an empty function throws");
    threw = false;
    try { reg.Set("device_api.GetAttr", PackedFunc()); } catch (const std::runtime_error& e) {
        threw = std::string(e.what()) == "Function device_api.GetAttr is already registered.";
    }
    Check(threw, "a name registers once");
    for (const char* name : {"device_api.AllocDataSpace", "device_api.FreeDataSpace", "device_api.AllocWorkspace", "device_api.FreeWorkspace",
                             "device_api.CopyDataFromTo", "device_api.CopyDataFromToEx", "device_api.GetAttr", "device_api.CreateStream",
                             "device_api.FreeStream", "device_api.StreamSync", "device_api.SyncStreamFromTo", "device_api.SetStream",
                             "device_api.GetCurrentStream", "device_api.NeedSetDevice", "device_api.ListDevices", "device_api.ListDevicesJSON",
                             "device_api.GetAllDeviceInfo", "device_api.GetAllDeviceInfoJSON", "device_api.GetTargetKind",
                             "device_api.GetTargetArch", "target.Build", "device.DetectAndRegister",
                             "kxc.relay.transform.lower_to_exec_plan_json", "kxc.relay.transform.lower_to_exec_plan_json_file",
                             "kxc.hip.execute_plan_json", "kxc.hip.execute_plan_json_file"})
        Check(reg.Get(name).defined(), std::string(name) + " is registered");
    const kxc::Device cpu(kxc::kCPU, 0), gpu(kxc::kGPU, 0);
    Check(static_cast<int64_t>(reg.Get("device_api.NeedSetDevice")(0)) == 0 && static_cast<int64_t>(reg.Get("device_api.NeedSetDevice")(1)) == 1,
          "NeedSetDevice: every type but the CPU");
    Check(static_cast<std::string>(reg.Get("device_api.GetTargetKind")(cpu)) == "llvm", "CPU target kind");
    Check(static_cast<std::string>(reg.Get("device_api.ListDevicesJSON")()).find("\"cpu\"") != std::string::npos, "the CPU is always listed");
    threw = false;
    try { reg.Get("device_api.AllocDataSpace")(std::string("cpu"), 16, 16); } catch (const std::runtime_error& e) {
        threw = std::string(e.what()).find("Type mismatch") == 0;
    }
    Check(threw, "a wrong argument type is refused");
    // allocate, copy and free through the registry on the host back end
    std::vector<float> src = {1.5f, -2.0f, 3.25f, 4.0f}, dst(4, 0.0f);
    auto I = [](const void* p) { return static_cast<int64_t>(reinterpret_cast<uintptr_t>(p)); };
    const int64_t hbuf = reg.Get("device_api.AllocDataSpace")(cpu, 16, 64);
    Check(hbuf != 0, "host allocation");
    reg.Get("device_api.CopyDataFromTo")(cpu, I(src.data()), cpu, hbuf, 16);
    reg.Get("device_api.CopyDataFromTo")(cpu, hbuf, cpu, I(dst.data()), 16);
    Check(dst == src, "host copy round trip");
    reg.Get("device_api.FreeDataSpace")(cpu, hbuf);
    if (mode == "hip") {
        Check(static_cast<std::string>(reg.Get("device_api.GetTargetKind")(gpu)) == "hip" &&
                  static_cast<std::string>(reg.Get("device_api.GetTargetArch")(gpu)).find("gfx") == 0, "GPU target kind and arch");
        Check(static_cast<int64_t>(reg.Get("device_api.GetAttr")(gpu, static_cast<int>(kxc::DeviceAttrKind::kWarpSize))) == 64, "wave size 64");
        kxc::ObjectRef target = reg.Get("target.Build")(gpu);
        Check(target.defined() && target.As<kxc::TargetNode>() && target.As<kxc::TargetNode>()->kind == "hip", "target.Build gives a Target");
        reg.Get("device.DetectAndRegister")();
        // (the marketing name comes from the driver's id table and may be empty where that table is not installed)
        Check(reg.Get("device_info.hip.0.name").defined() && static_cast<int64_t>(reg.Get("device_info.hip.0.memory")()) > (1LL << 30) &&
                  !static_cast<std::string>(reg.Get("device_info.hip.0.compute_capability")()).empty(), "device_info.hip.0.*");
        (void)static_cast<std::string>(reg.Get("device_info.hip.0.name")());
        const int64_t stream = reg.Get("device_api.CreateStream")(gpu);
        const int64_t dbuf = reg.Get("device_api.AllocDataSpace")(gpu, 16, 256);
        std::fill(dst.begin(), dst.end(), 0.0f);
        reg.Get("device_api.CopyDataFromToEx")(cpu, I(src.data()), 0, gpu, dbuf, 0, 16, stream);
        reg.Get("device_api.CopyDataFromToEx")(gpu, dbuf, 8, cpu, I(dst.data()), 8, 8, stream);      // the second half only
        reg.Get("device_api.StreamSync")(gpu, stream);
        Check(dst[0] == 0.0f && dst[1] == 0.0f && dst[2] == src[2] && dst[3] == src[3], "device copy with offsets on a stream");
        // a Relay function -> plan JSON -> run from the JSON, all through the registry
        kxc::Var a("a", kxc::TensorType({2, 3}, "float32")), b("b", kxc::TensorType({2, 3}, "float32"));
        kxc::Function func({a, b}, kxc::Call(Op::Get("add"), {a, b}));
        const std::string json = reg.Get("kxc.relay.transform.lower_to_exec_plan_json")(func);
        Check(json.find("\"kernel_symbol\"") != std::string::npos && json.find("\"kxc_hip\"") != std::string::npos, "plan JSON from the registry");
        std::vector<float> av = {1, 2, 3, 4, 5, 6}, bv = {10, 20, 30, 40, 50, 60}, out(6, 0.0f);
        const int64_t da = reg.Get("device_api.AllocDataSpace")(gpu, 24, 256), db = reg.Get("device_api.AllocDataSpace")(gpu, 24, 256),
                      dout = reg.Get("device_api.AllocDataSpace")(gpu, 24, 256);
        reg.Get("device_api.CopyDataFromTo")(cpu, I(av.data()), gpu, da, 24);
        reg.Get("device_api.CopyDataFromTo")(cpu, I(bv.data()), gpu, db, 24);
        void* packed[3] = {reinterpret_cast<void*>(da), reinterpret_cast<void*>(db), reinterpret_cast<void*>(dout)};
        Check(static_cast<int64_t>(reg.Get("kxc.hip.execute_plan_json")(json, static_cast<void*>(packed), 3)) == 0, "plan run");
        reg.Get("device_api.StreamSync")(gpu, 0);
        reg.Get("device_api.CopyDataFromTo")(gpu, dout, cpu, I(out.data()), 24);
        Check(out == std::vector<float>({11, 22, 33, 44, 55, 66}), "plan run from JSON adds");
        for (int64_t p : {da, db, dout, dbuf}) reg.Get("device_api.FreeDataSpace")(gpu, p);
        reg.Get("device_api.FreeStream")(gpu, stream);
    }
    std::cout << "packed functions ok (" << mode << ")\n";
    return 0;
}

// Non-finite inputs through a 3x3 stride-1 convolution with constant weights on the hip target.  With
// CompileConfig::hip_winograd = false the special values spread exactly as in the CPU back end's direct sum (an Inf or
// NaN reaches the nine outputs per channel whose window holds it, and an Inf stays an Inf of the product's sign); with
// the default (Winograd F(2x2,3x3)) the input transform forms differences inside 4x4 patches, so a special value may
// reach up to sixteen outputs per channel (the 2x2 blocks of the four patches that hold it), an Inf may come out as
// NaN there, and every other output is unaffected.
int RunNonFinite() {
    const int64_t C = 8, H = 12, W = 12, O = 32;
    std::vector<float> x(C * H * W), w(O * C * 9), b(O);
    uint32_t seed = 99;
    auto next = [&seed]() { seed = seed * 1664525u + 1013904223u; return static_cast<float>(seed >> 8) / 16777216.0f - 0.5f; };
    for (auto& v : x) v = next();
    for (auto& v : w) { v = next(); if (std::fabs(v) < 0.01f) v = 0.25f; }     // no zero weight: Inf * 0 would be NaN on both sides
    for (auto& v : b) v = 0.1f * next();
    struct Special { int64_t c, h, w; float value; };
    const std::vector<Special> specials = {{2, 5, 6, INFINITY}, {5, 9, 2, NAN}};
    for (const auto& sp : specials) x[(sp.c * H + sp.h) * W + sp.w] = sp.value;
    kxc::runtime::NDArray wn({O, C, 3, 3}, "float32"), bn({O}, "float32");
    wn.CopyFromBytes(w.data(), w.size() * sizeof(float));
    bn.CopyFromBytes(b.data(), b.size() * sizeof(float));
    kxc::Var xv("x", kxc::TensorType({1, C, H, W}, "float32"));
    auto attrs = kxc::relay::Conv2DAttrs::Create({1, 1}, {1, 1, 1, 1}, {1, 1}, 1, static_cast<int>(O), {3, 3}, "NCHW", "OIHW", "", "");
    kxc::Function f({xv}, kxc::Call(Op::Get("nn_conv2d"), {xv, kxc::Constant(wn), kxc::Constant(bn)}, attrs));
    // the CPU back end's answer
    std::vector<float> want(O * H * W, 0.0f);
    {
        g_mode = "cpu";
        auto module = kxc::api::Compiler::Compile(f, MakeConfig());
        module.Run({x.data(), w.data(), b.data(), want.data()});
    }
    g_mode = "hip";
    kxc::DeviceAPI* api = kxc::GetDeviceAPI(kxc::kGPU);
    kxc::Device dev(kxc::kGPU, 0), cpu(kxc::kCPU, 0);
    auto run = [&](bool winograd, std::vector<float>* out, std::string* symbol) {
        auto config = MakeConfig();
        config->hip_winograd = winograd;
        auto module = kxc::api::Compiler::Compile(f, config);
        *symbol = module.GetKernelExecs().at(0).kernel_symbol;
        std::vector<std::pair<void*, size_t>> host = {{x.data(), x.size() * 4}, {w.data(), w.size() * 4}, {b.data(), b.size() * 4}, {out->data(), out->size() * 4}};
        std::vector<void*> args;
        for (auto& h : host) {
            void* d = api->AllocDataSpace(dev, h.second, 256);
            api->CopyDataFromTo(cpu, h.first, dev, d, h.second);
            args.push_back(d);
        }
        module.Run(args);
        api->CopyDataFromTo(dev, args[3], cpu, out->data(), out->size() * 4);
        for (void* d : args) api->FreeDataSpace(dev, d);
    };
    auto close = [](float got, float ref) { return std::fabs(got - ref) <= 1e-3f * std::max(1.0f, std::fabs(ref)); };
    // ---- switch off: the reference's propagation, value class by value class
    std::vector<float> direct(want.size(), 0.0f), wino(want.size(), 0.0f);
    std::string symbol;
    run(false, &direct, &symbol);
    Check(symbol.find("winograd") == std::string::npos, "hip_winograd = false still chose " + symbol);
    int64_t inf_count = 0, nan_count = 0;
    for (size_t i = 0; i < want.size(); ++i) {
        if (std::isnan(want[i])) { Check(std::isnan(direct[i]), "direct: NaN expected at " + std::to_string(i)); ++nan_count; }
        else if (std::isinf(want[i])) { Check(direct[i] == want[i], "direct: Inf of the same sign expected at " + std::to_string(i)); ++inf_count; }
        else Check(close(direct[i], want[i]), "direct: finite value differs at " + std::to_string(i));
    }
    Check(inf_count == 9 * O && nan_count == 9 * O, "the CPU back end spreads each special value over its nine windows per channel");
    // ---- default: Winograd
    run(true, &wino, &symbol);
    Check(symbol.find("winograd") != std::string::npos, "a 3x3 stride-1 convolution with constant weights should take the Winograd kernel: " + symbol);
    std::vector<int64_t> affected(O, 0);
    for (int64_t o = 0; o < O; ++o)
        for (int64_t h = 0; h < H; ++h)
            for (int64_t ww = 0; ww < W; ++ww) {
                const size_t i = static_cast<size_t>((o * H + h) * W + ww);
                // the 2x2 output blocks of the patches that hold a special value: rows / columns 2*floor((p-1)/2) .. +3
                bool in_reach = false;
                for (const auto& sp : specials) {
                    const int64_t h0 = 2 * ((sp.h - 1) / 2), w0 = 2 * ((sp.w - 1) / 2);
                    in_reach = in_reach || (h >= h0 && h < h0 + 4 && ww >= w0 && ww < w0 + 4);
                }
                if (!in_reach) {
                    Check(std::isfinite(want[i]) && close(wino[i], want[i]),
                          "winograd: an output outside the patches of the special values differs at " + std::to_string(i));
                    continue;
                }
                if (!std::isfinite(wino[i])) ++affected[o];
                // where the direct sum is non-finite, so is the Winograd result (an Inf may have become NaN)
                if (!std::isfinite(want[i])) Check(!std::isfinite(wino[i]), "winograd: a non-finite output came out finite at " + std::to_string(i));
                else if (std::isfinite(wino[i])) Check(close(wino[i], want[i]), "winograd: finite value differs at " + std::to_string(i));
            }
    for (int64_t o = 0; o < O; ++o)
        Check(affected[o] >= 18 && affected[o] <= 32, "winograd: a special value reaches at most 16 outputs per channel, got " +
                                                        std::to_string(affected[o]) + " for two of them in channel " + std::to_string(o));
    std::cout << "[PASS] non-finite inputs: reference propagation with hip_winograd = false, at most 16 outputs per special value with Winograd\n";
    std::cout << "non-finite ok\n";
    return 0;
}

int main(int argc, char** argv) {
    try {
        const std::string cmd = argc > 1 ? argv[1] : "";
        if (cmd == "op_numeric") { g_mode = argc > 2 ? argv[2] : "cpu"; return RunOpNumeric(); }
        if (cmd == "device_info") return RunDeviceInfo();
        if (cmd == "adaptive") { g_mode = argc > 2 ? argv[2] : "cpu"; return RunAdaptive(argc > 3 ? argv[3] : ""); }
        if (cmd == "codegen") return RunCodegen();
        if (cmd == "nonfinite") return RunNonFinite();
        if (cmd == "packed_func") return RunPackedFunc(argc > 2 ? argv[2] : "cpu");
        if (cmd == "generated_numeric") return RunGeneratedNumeric();
        if (cmd == "split_batch") return RunSplitBatch();
        if (cmd == "shares_generated") return RunSharesGenerated();
        if (cmd == "shares_random") return RunSharesRandom();
        if (cmd == "qnn" && argc >= 4) { g_mode = argv[2]; return RunQnn(argv[3]); }
        if (cmd == "onnx" && argc >= 4) { g_mode = argv[2]; return RunOnnx(argv[3]); }
        if (cmd == "onnx_errors" && argc >= 3) return RunOnnxErrors(argv[2]);
        if (cmd == "hip_smoke" && argc >= 3) return RunHipSmoke(argv[2]);
        if (cmd == "hip_smoke_sdk" && argc >= 3) return RunHipSmoke(argv[2], true);
        if (cmd == "diagnosis" && argc >= 3) return RunDiagnosis(argv[2]);
        if (cmd == "kernel_object") { g_mode = argc > 2 ? argv[2] : "cpu"; return RunKernelObject(argc > 3 ? argv[3] : ""); }
        if (cmd == "profile" && argc >= 4) { g_mode = argv[2]; return RunProfile(argv[3]); }
        if (cmd == "resnet18" && argc >= 6) { g_mode = argv[2]; return RunResNet18(argv[3], std::atoll(argv[4]), std::atoll(argv[5])); }
        std::cerr << "usage: host_tests op_numeric <cpu|hip|hipgen> | device_info | codegen | resnet18 <cpu|hip|hipgen> <dir> <batch> <hw>\n";
        return 2;
    } catch (const std::exception& e) {
        std::cerr << "[FAIL] " << e.what() << "\n";
        return 1;
    }
}
