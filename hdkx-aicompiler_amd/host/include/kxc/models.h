// models.h -- graph builders for the benchmark networks.
#pragma once

#include "kxc/op.h"

namespace kxc {
namespace models {

// ResNet-18 with the topology of the reference's test/resnet18_ir_dump.cpp:191-452 (batch-norm folded
// into convolution biases): 49 Relay calls, 42 constants created in depth-first argument order.
// consts (optional) receives the constant tensors in that order.
Function BuildResNet18(int64_t batch, int64_t hw = 224, std::vector<runtime::NDArray>* consts = nullptr);

}  // namespace models
}  // namespace kxc
