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
#include <cmath>
#include <sstream>
#include <cstdio>
#include <cstring>
#include <fstream>
#include <functional>
#include <iostream>

#include "kxc/compiler.h"
#include "kxc/models.h"
#include "kxc/onnx_importer.h"
#include "kxc/profiling.h"
#include "kxc/topi.h"

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
        {"transpose", TestTranspose}, {"reduce_mean", TestReduceMean}, {"model_add_chain", TestModelAddChain},
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
    Check(hip.kernels[0].schedule == "flat", "conv stage is a flat schedule");
    // global average pool: contiguous rows -> LDS staged reduction
    kxc::Var x("x", kxc::TensorType({4, 32, 7, 7}, "float32"));
    kxc::Function gap({x}, kxc::Call(Op::Get("nn_global_avg_pool2d"), {x}, kxc::relay::GlobalAvgPool2DAttrs::Create()));
    auto gap_hip = cgh.Generate(kxc::relay::LowerToTIR(kxc::relay::InferTypePass(gap)), "kxc_gap");
    Check(gap_hip.kernels.size() == 2 && gap_hip.kernels[0].schedule == "lds_row_reduce", "gap sum is LDS staged");
    Check(gap_hip.source.find("__shared__ float tile[") != std::string::npos, "LDS tile declared");
    Check(gap_hip.source.find("/ ((long long)49LL)") != std::string::npos || gap_hip.source.find("49") != std::string::npos, "division by H*W");
    // a ResNet-18 compile for the hip target without a GPU: plan and fusion are built, nothing is loaded
    g_mode = "hip";
    auto module = kxc::api::Compiler::Compile(kxc::models::BuildResNet18(1, 224), MakeConfig());
    Check(module.GetKernelExecs().size() == 23, "49 Relay calls become 23 launches, got " + std::to_string(module.GetKernelExecs().size()));
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

int main(int argc, char** argv) {
    try {
        const std::string cmd = argc > 1 ? argv[1] : "";
        if (cmd == "op_numeric") { g_mode = argc > 2 ? argv[2] : "cpu"; return RunOpNumeric(); }
        if (cmd == "device_info") return RunDeviceInfo();
        if (cmd == "codegen") return RunCodegen();
        if (cmd == "onnx" && argc >= 4) { g_mode = argv[2]; return RunOnnx(argv[3]); }
        if (cmd == "onnx_errors" && argc >= 3) return RunOnnxErrors(argv[2]);
        if (cmd == "profile" && argc >= 4) { g_mode = argv[2]; return RunProfile(argv[3]); }
        if (cmd == "resnet18" && argc >= 6) { g_mode = argv[2]; return RunResNet18(argv[3], std::atoll(argv[4]), std::atoll(argv[5])); }
        std::cerr << "usage: host_tests op_numeric <cpu|hip|hipgen> | device_info | codegen | resnet18 <cpu|hip|hipgen> <dir> <batch> <hw>\n";
        return 2;
    } catch (const std::exception& e) {
        std::cerr << "[FAIL] " << e.what() << "\n";
        return 1;
    }
}
