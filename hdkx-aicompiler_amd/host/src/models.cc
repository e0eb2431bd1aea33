// models.cc -- see models.h.
#include "kxc/models.h"

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

}  // namespace models
}  // namespace kxc
