// onnx_importer.h -- loader of the "kxc.onnx_import.v1" wire format: a JSON function spec plus a flat binary
// file of parameter bytes, as written by the reference's Python exporter (python/kxc_onnx/spec.py:61-103,
// docs/ONNX_IMPORTER.md:64-83) and read by its C++ reifier (include/frontend/onnx_importer.h:13-22,
// src/frontend/onnx_importer.cc:410-527).  Same result type, same operator set (nn_conv2d, nn_relu,
// nn_max_pool2d, add, nn_global_avg_pool2d, nn_flatten, nn_gemm), same attribute keys and error texts, so a
// model exported for the reference loads here and runs on the HIP target.
#pragma once

#include <string>
#include <unordered_map>
#include <vector>

#include "kxc/relay.h"

namespace kxc {
namespace frontend {

struct ImportedONNXModel {
    Function function;
    std::unordered_map<std::string, runtime::NDArray> params;
    std::vector<std::string> param_order;
    std::vector<std::string> input_names;
    std::vector<std::string> output_names;
};

ImportedONNXModel LoadONNXImportSpec(const std::string& json_path, const std::string& params_path);

}  // namespace frontend
}  // namespace kxc
