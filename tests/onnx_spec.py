"""Writer of the "kxc.onnx_import.v1" wire format (JSON function spec + flat parameter bytes) for tests.

The layout follows the reference's exporter (python/kxc_onnx/spec.py:61-103, docs/ONNX_IMPORTER.md:64-83):
`format`, `function.{inputs,outputs,nodes}`, `params` records {name, shape, dtype, offset, nbytes} and
`param_order`; the binary file is the parameters' bytes in that order.  Node attribute keys are the ones the
reference's C++ reifier reads (src/frontend/onnx_importer.cc:361-407).
"""
import json
import os

import numpy as np


def resnet18_spec(batch, hw, consts):
    """The ResNet-18 graph of test/resnet18_ir_dump.cpp:191-452 with ONNX-style value and parameter names.
    consts: the 42 fp32 arrays in lowering order.  Returns (spec dict, parameter bytes)."""
    nodes, params = [], []
    names = iter(range(10 ** 6))
    k = [0]

    def param(name, arr):
        params.append((name, np.ascontiguousarray(arr, np.float32)))
        return name

    def conv(x, prefix, ksz, stride, pad):
        w, b = consts[k[0]], consts[k[0] + 1]
        k[0] += 2
        out = "%s_out" % prefix
        nodes.append({"name": prefix, "op_name": "nn_conv2d",
                      "inputs": [x, param(prefix + ".weight", w), param(prefix + ".bias", b)], "outputs": [out],
                      "attrs": {"strides": [stride, stride], "pads": [pad, pad, pad, pad], "dilations": [1, 1], "group": 1,
                                "channels": int(w.shape[0]), "kernel_size": [ksz, ksz], "data_layout": "NCHW",
                                "kernel_layout": "OIHW", "out_layout": "", "out_dtype": ""}})
        return out

    def unary(x, op, attrs=None):
        name = "%s_%d" % (op, next(names))
        nodes.append({"name": name, "op_name": op, "inputs": [x], "outputs": [name + "_out"], "attrs": attrs or {}})
        return name + "_out"

    x = unary(conv("input", "conv1", 7, 2, 3), "nn_relu")
    x = unary(x, "nn_max_pool2d", {"strides": [2, 2], "pads": [1, 1, 1, 1], "dilations": [1, 1], "pool_size": [3, 3],
                                   "layout": "NCHW", "ceil_mode": False})
    for stage in range(4):
        for blk in range(2):
            first = blk == 0 and stage > 0
            s = 2 if first else 1
            p = "layer%d.%d" % (stage + 1, blk)
            a = unary(conv(x, p + ".conv1", 3, s, 1), "nn_relu")
            b = conv(a, p + ".conv2", 3, 1, 1)
            idn = conv(x, p + ".downsample", 1, s, 0) if first else x
            name = p + ".add"
            nodes.append({"name": name, "op_name": "add", "inputs": [b, idn], "outputs": [name + "_out"], "attrs": {}})
            x = unary(name + "_out", "nn_relu")
    x = unary(x, "nn_global_avg_pool2d")
    x = unary(x, "nn_flatten", {"axis": 1})
    nodes.append({"name": "fc", "op_name": "nn_gemm",
                  "inputs": [x, param("fc.weight", consts[k[0]]), param("fc.bias", consts[k[0] + 1])], "outputs": ["logits"],
                  "attrs": {"alpha": 1.0, "beta": 1.0, "transA": 0, "transB": 1}})
    records, blob, offset = [], [], 0
    for name, arr in params:
        data = arr.tobytes()
        records.append({"name": name, "shape": list(arr.shape), "dtype": "float32", "offset": offset, "nbytes": len(data)})
        blob.append(data)
        offset += len(data)
    spec = {"format": "kxc.onnx_import.v1",
            "function": {"inputs": [{"name": "input", "shape": [batch, 3, hw, hw], "dtype": "float32"}],
                         "outputs": [{"name": "logits", "shape": [batch, 1000], "dtype": "float32"}], "nodes": nodes},
            "params": records, "param_order": [n for n, _ in params]}
    return spec, b"".join(blob)


def write(d, spec, blob, name="model"):
    with open(os.path.join(d, name + ".import.json"), "w") as f:
        f.write(json.dumps(spec, indent=2) + "\n")
    with open(os.path.join(d, name + ".params.bin"), "wb") as f:
        f.write(blob)


def reference_input(batch, hw):
    """Input pattern of the reference's acceptance test (test/onnx_importer_test.cpp:138-144)."""
    i = np.arange(batch * 3 * hw * hw, dtype=np.int64)
    return (((i % 251).astype(np.float32) - np.float32(125.0)) / np.float32(125.0)).reshape(batch, 3, hw, hw)
