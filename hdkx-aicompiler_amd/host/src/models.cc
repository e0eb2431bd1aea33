// models.cc -- see models.h.
#include "kxc/models.h"

#include <unordered_map>

namespace kxc {
namespace models {

namespace {
using relay::Op;

struct Builder {
    std::vector<runtime::NDArray>* consts;
    Expr Conv(Expr x, int64_t c, int64_t o, int k, int s, int p) {
        runtime::NDArray w({o, c, k, k}, "float32"), b({o}, "float32");
        if (consts) { consts->push_back(w); consts->push_back(b); }
        auto attrs = relay::Conv2DAttrs::Create({s, s}, {p, p, p, p}, {1, 1}, 1, static_cast<int>(o), {k, k}, "NCHW", "OIHW", "", "");
        return Call(Op::Get("nn_conv2d"), {x, Constant(w), Constant(b)}, attrs);
    }
    static Expr Relu(Expr x) { return Call(Op::Get("nn_relu"), {x}, relay::ReluAttrs::Create()); }
    // BasicBlock: conv-relu-conv, add(conv_out, identity), relu; identity = input or its 1x1/2 convolution
    Expr Block(Expr x, int64_t c, int64_t o, int stride, bool down) {
        Expr a = Relu(Conv(x, c, o, 3, stride, 1));
        Expr b = Conv(a, o, o, 3, 1, 1);
        Expr id = down ? Conv(x, c, o, 1, stride, 0) : x;
        return Relu(Call(Op::Get("add"), {b, id}, relay::AddAttrs::Create()));
    }
};
}  // namespace

Function BuildResNet18(int64_t batch, int64_t hw, std::vector<runtime::NDArray>* consts) {
    Builder b{consts};
    Var input("input", TensorType({batch, 3, hw, hw}, "float32"));
    Expr x = Builder::Relu(b.Conv(input, 3, 64, 7, 2, 3));
    x = Call(Op::Get("nn_max_pool2d"), {x}, relay::MaxPool2DAttrs::Create({2, 2}, {1, 1, 1, 1}, {1, 1}, {3, 3}, "NCHW", false));
    const int64_t ch[4] = {64, 128, 256, 512};
    int64_t cin = 64;
    for (int st = 0; st < 4; ++st) {
        x = b.Block(x, cin, ch[st], st == 0 ? 1 : 2, st != 0);
        x = b.Block(x, ch[st], ch[st], 1, false);
        cin = ch[st];
    }
    x = Call(Op::Get("nn_global_avg_pool2d"), {x}, relay::GlobalAvgPool2DAttrs::Create());
    x = Call(Op::Get("nn_flatten"), {x}, relay::FlattenAttrs::Create(1));
    runtime::NDArray fw({1000, 512}, "float32"), fb({1000}, "float32");
    if (consts) { consts->push_back(fw); consts->push_back(fb); }
    x = Call(Op::Get("nn_gemm"), {x, Constant(fw), Constant(fb)}, relay::GemmAttrs::Create(1.0f, 1.0f, 0, 1));
    return Function({input}, x);
}

namespace {
struct QBuilder {
    std::vector<runtime::NDArray>* consts;
    std::vector<std::string>* names;
    std::unordered_map<std::string, Expr> taps;
    Array<Expr> Weights(const std::string& layer, std::vector<int64_t> wshape) {
        const int64_t o = wshape[0];
        runtime::NDArray w(wshape, "int8"), b({o}, "int32"), m({o}, "float32");
        if (consts) { consts->push_back(w); consts->push_back(b); consts->push_back(m); }
        if (names) { names->push_back(layer + ".w"); names->push_back(layer + ".b"); names->push_back(layer + ".m"); }
        return {Constant(w), Constant(b), Constant(m)};
    }
    Expr Conv(const std::string& layer, Expr x, Array<Expr> wbm, int s, int p, bool relu, Expr residual = Expr(), double res_mult = 0.0) {
        Array<Expr> args{x, wbm[0], wbm[1], wbm[2]};
        if (residual.defined()) args.push_back(residual);
        Expr y = Call(Op::Get("qnn_conv2d"), args, relay::QnnConv2DAttrs::Create({s, s}, {p, p}, relu, res_mult));
        taps[layer] = y;
        return y;
    }
    // constants are created in depth-first argument order: first convolution, second convolution, downsample
    Expr Block(const std::string& name, Expr x, int64_t c, int64_t o, int stride, bool down, double res_mult) {
        Expr a = Conv(name + ".conv1", x, Weights(name + ".conv1", {o, c, 3, 3}), stride, 1, true);
        Array<Expr> second = Weights(name + ".conv2", {o, o, 3, 3});
        Expr id = down ? Conv(name + ".down", x, Weights(name + ".down", {o, c, 1, 1}), stride, 0, false) : x;
        return Conv(name + ".conv2", a, second, 1, 1, true, id, res_mult);
    }
};
}  // namespace

Function BuildQResNet18(int64_t batch, int64_t hw, const QResNet18Scales& scales, std::vector<runtime::NDArray>* consts,
                        std::vector<std::string>* const_names, const std::string& result) {
    QBuilder b{consts, const_names, {}};
    Var input("input", TensorType({batch, 3, hw, hw}, "float32"));
    Expr x = Call(Op::Get("qnn_quantize"), {input}, relay::QnnQuantizeAttrs::Create(scales.input_scale));
    b.taps["input"] = x;
    x = b.Conv("conv1", x, b.Weights("conv1", {64, 3, 7, 7}), 2, 3, true);
    x = Call(Op::Get("nn_max_pool2d"), {x}, relay::MaxPool2DAttrs::Create({2, 2}, {1, 1, 1, 1}, {1, 1}, {3, 3}, "NCHW", false));
    b.taps["maxpool"] = x;
    const int64_t ch[4] = {64, 128, 256, 512};
    int64_t cin = 64;
    for (int st = 0; st < 4; ++st) {
        const std::string stage = "l" + std::to_string(st + 1);
        x = b.Block(stage + ".0", x, cin, ch[st], st == 0 ? 1 : 2, st != 0, scales.res_mult[2 * st]);
        x = b.Block(stage + ".1", x, ch[st], ch[st], 1, false, scales.res_mult[2 * st + 1]);
        cin = ch[st];
    }
    x = Call(Op::Get("qnn_global_avg_pool2d"), {x}, relay::QnnRequantAttrs::Create(scales.gap_mult));
    b.taps["gap"] = x;
    x = Call(Op::Get("nn_flatten"), {x}, relay::FlattenAttrs::Create(1));
    Array<Expr> fc = b.Weights("fc", {1000, 512});
    x = Call(Op::Get("qnn_dense"), {x, fc[0], fc[1], fc[2]});
    if (!result.empty()) {
        auto it = b.taps.find(result);
        if (it == b.taps.end()) throw std::runtime_error("BuildQResNet18: no activation named " + result);
        x = it->second;
    }
    return Function({input}, x);
}

}  // namespace models
}  // namespace kxc
