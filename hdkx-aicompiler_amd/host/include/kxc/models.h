// models.h -- graph builders for the benchmark networks.
#pragma once

#include "kxc/op.h"

namespace kxc {
namespace models {

// ResNet-18 with the topology of the reference's test/resnet18_ir_dump.cpp:191-452 (batch-norm folded
// into convolution biases): 49 Relay calls, 42 constants created in depth-first argument order.
// consts (optional) receives the constant tensors in that order.
Function BuildResNet18(int64_t batch, int64_t hw = 224, std::vector<runtime::NDArray>* consts = nullptr);

// The same topology with every convolution and the fully connected layer quantised (qnn_quantize, qnn_conv2d with the
// residual and the ReLU inside, int8 max pool, qnn_global_avg_pool2d, qnn_dense): 24 calls, 63 constants in
// depth-first argument order -- per convolution int8 weights [O,C,K,K], int32 bias [O], float32 multiplier [O]
// (a block's first convolution, then its second, then its 1x1 downsample), last the dense layer's three.  What the
// calibration fixes beside the constants goes into the attributes: the input scale, one residual multiplier per
// block (s_residual / s_out of the block's second convolution) and the pool's multiplier s_in / (H * W * s_out).
struct QResNet18Scales {
    double input_scale = 1.0;
    double res_mult[8] = {1, 1, 1, 1, 1, 1, 1, 1};
    double gap_mult = 1.0;
};
// const_names (optional) receives one name per entry of consts ("conv1.w", "l2.0.down.b", "fc.m" ...).  result names
// the value the function returns: "" = the logits, else an int8 activation -- "input" (the quantised input), "conv1",
// "maxpool", "l<stage>.<block>.conv1" / ".conv2" / ".down" -- so that every layer can be compared on its own; such a
// function reaches only the constants of the layers before it.
Function BuildQResNet18(int64_t batch, int64_t hw, const QResNet18Scales& scales, std::vector<runtime::NDArray>* consts = nullptr,
                        std::vector<std::string>* const_names = nullptr, const std::string& result = "");

}  // namespace models
}  // namespace kxc
