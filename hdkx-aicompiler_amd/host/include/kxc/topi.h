// topi.h -- compute definitions of the operators, with the arithmetic of the reference's TOPI layer
// (include/te/topi/nn.h, broadcast.h, elemwise.h, transform.h): these define what every backend,
// CPU or GPU, has to reproduce.
#pragma once

#include "kxc/te.h"

namespace kxc {
namespace te {
namespace topi {

constexpr const char* kElementWise = "elemwise";
constexpr const char* kBroadcast = "broadcast";
constexpr const char* kMatMul = "matmul";
constexpr const char* kConv2d = "conv2d";
constexpr const char* kPool = "pool";
constexpr const char* kInjective = "injective";

PrimExpr make_const(tir::DataType t, double value);

// include/te/topi/nn.h:19-30
Tensor relu(const Tensor& x, std::string name = "relu");
// include/te/topi/nn.h:48-80 (B is [N, K])
Tensor dense(const Tensor& A, const Tensor& B, std::string name = "dense");
// include/te/topi/nn.h:84-101 (B is [K, N])
Tensor matmul(const Tensor& A, const Tensor& B, std::string name = "matmul");
// include/te/topi/nn.h:107-158
Tensor conv2d_nchw(const Tensor& data, const Tensor& kernel, int stride_h, int stride_w, int pad_h, int pad_w,
                   int dilation_h, int dilation_w, std::string name = "conv2d_nchw");
// include/te/topi/nn.h:161-258; padding = {top, left, bottom, right}
Tensor pool2d(const Tensor& data, std::vector<int> kernel_size, std::vector<int> stride, std::vector<int> padding,
              const std::string& pool_type, bool ceil_mode = false, std::string name = "pool2d");
// include/te/topi/nn.h:260-287
Tensor global_avg_pool2d(const Tensor& data, std::string name = "global_avg_pool2d");
// include/te/topi/broadcast.h:90-113; op: 0 add, 1 subtract, 2 multiply, 3 divide
Tensor broadcast_binary(int op, const Tensor& A, const Tensor& B, std::string name);
inline Tensor add(const Tensor& A, const Tensor& B, std::string name = "add") { return broadcast_binary(0, A, B, name); }
inline Tensor subtract(const Tensor& A, const Tensor& B, std::string name = "subtract") { return broadcast_binary(1, A, B, name); }
inline Tensor multiply(const Tensor& A, const Tensor& B, std::string name = "multiply") { return broadcast_binary(2, A, B, name); }
inline Tensor divide(const Tensor& A, const Tensor& B, std::string name = "divide") { return broadcast_binary(3, A, B, name); }
// elementwise intrinsic call (exp, log, sqrt, floor, ceil, fabs): include/te/topi/elemwise.h
Tensor unary_call(const Tensor& x, const std::string& intrinsic, std::string name);
// src/relay/op/tensor/transform.cc:70-182: index remap of a row-major reshape (flatten, reshape)
Tensor reshape(const Tensor& x, std::vector<int64_t> new_shape, std::string name);
Tensor transpose(const Tensor& x, std::vector<int> axes, std::string name);
// mean over trailing/selected axes: sum then division by the element count
Tensor reduce_mean(const Tensor& x, std::vector<int> axes, bool keepdims, std::string name);
// exp(x) / sum over `axis` of exp(x), as three stages named <name>_exp, <name>_sum (axis kept with extent 1) and
// <name> (src/relay/op/nn/softmax.cc: no max subtraction, like the reference)
Tensor softmax(const Tensor& x, int axis, std::string name);
// Call(dtype, "cast", {x}) per element (include/te/topi/elemwise.h:113-122): C conversion rules
Tensor cast(const Tensor& x, tir::DataType dtype, std::string name);

// Quantised operators (see QnnConv2DAttrsNode in op.h for the arithmetic).  residual may be an undefined Tensor.
Tensor qnn_quantize(const Tensor& x, double scale, std::string name);
Tensor qnn_conv2d_nchw(const Tensor& data, const Tensor& kernel, const Tensor& bias, const Tensor& mult, const Tensor& residual,
                       int stride_h, int stride_w, int pad_h, int pad_w, bool relu, double res_mult, std::string name);
Tensor qnn_dense(const Tensor& A, const Tensor& B, const Tensor& bias, const Tensor& mult, std::string name);
Tensor qnn_global_avg_pool2d(const Tensor& data, double mult, std::string name);

}  // namespace topi
}  // namespace te
}  // namespace kxc
