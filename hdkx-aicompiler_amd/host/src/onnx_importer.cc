// onnx_importer.cc -- see kxc/onnx_importer.h.
#include "kxc/onnx_importer.h"

#include <fstream>
#include <sstream>
#include <stdexcept>

#include "json_reader.h"
#include "kxc/op.h"

namespace kxc {
namespace frontend {

namespace {

using json::Value;

[[noreturn]] void Bad(const std::string& what) { throw std::runtime_error(what); }

const Value& Field(const Value& obj, const std::string& key, const std::string& ctx) {
    if (obj.kind != Value::kObject) Bad(ctx + " must be an object");
    auto it = obj.object.find(key);
    if (it == obj.object.end()) Bad("Missing field '" + key + "' in " + ctx);
    return it->second;
}
std::string Str(const Value& v, const std::string& ctx) {
    if (v.kind != Value::kString) Bad(ctx + " must be a string");
    return v.string;
}
int64_t Int(const Value& v, const std::string& ctx) {
    if (v.kind != Value::kNumber || v.number != static_cast<double>(v.integer)) Bad(ctx + " must be an integer");
    return v.integer;
}
double Num(const Value& v, const std::string& ctx) {
    if (v.kind != Value::kNumber) Bad(ctx + " must be a number");
    return v.number;
}
bool Bool(const Value& v, const std::string& ctx) {
    if (v.kind == Value::kBool) return v.boolean;
    if (v.kind == Value::kNumber) return v.integer != 0;
    Bad(ctx + " must be a boolean");
}
std::vector<int64_t> Ints(const Value& v, const std::string& ctx) {
    if (v.kind != Value::kArray) Bad(ctx + " must be an array");
    std::vector<int64_t> out;
    for (size_t i = 0; i < v.array.size(); ++i) out.push_back(Int(v.array[i], ctx + "[" + std::to_string(i) + "]"));
    return out;
}
std::vector<std::string> Strs(const Value& v, const std::string& ctx) {
    if (v.kind != Value::kArray) Bad(ctx + " must be an array");
    std::vector<std::string> out;
    for (size_t i = 0; i < v.array.size(); ++i) out.push_back(Str(v.array[i], ctx + "[" + std::to_string(i) + "]"));
    return out;
}
Array<int64_t> ToArray(const std::vector<int64_t>& v) {
    Array<int64_t> a;
    for (int64_t d : v) a.push_back(d);
    return a;
}

std::string ReadText(const std::string& path) {
    std::ifstream in(path, std::ios::binary);
    if (!in) Bad("Failed to open ONNX import spec: " + path);
    std::ostringstream os;
    os << in.rdbuf();
    return os.str();
}
std::vector<char> ReadBinary(const std::string& path) {
    std::ifstream in(path, std::ios::binary);
    if (!in) Bad("Failed to open ONNX params file: " + path);
    return std::vector<char>((std::istreambuf_iterator<char>(in)), std::istreambuf_iterator<char>());
}

// Attribute objects per operator, with the key names of the exporter (src/frontend/onnx_importer.cc:361-407).
Attrs MakeAttrs(const std::string& op, const Value& a) {
    if (a.kind != Value::kObject) Bad("attrs for " + op + " must be an object");
    if (op == "nn_conv2d") {
        return relay::Conv2DAttrs::Create(Ints(Field(a, "strides", "conv attrs"), "conv attrs.strides"),
                                          Ints(Field(a, "pads", "conv attrs"), "conv attrs.pads"),
                                          Ints(Field(a, "dilations", "conv attrs"), "conv attrs.dilations"),
                                          static_cast<int>(Int(Field(a, "group", "conv attrs"), "conv attrs.group")),
                                          static_cast<int>(Int(Field(a, "channels", "conv attrs"), "conv attrs.channels")),
                                          Ints(Field(a, "kernel_size", "conv attrs"), "conv attrs.kernel_size"),
                                          Str(Field(a, "data_layout", "conv attrs"), "conv attrs.data_layout"),
                                          Str(Field(a, "kernel_layout", "conv attrs"), "conv attrs.kernel_layout"),
                                          Str(Field(a, "out_layout", "conv attrs"), "conv attrs.out_layout"),
                                          Str(Field(a, "out_dtype", "conv attrs"), "conv attrs.out_dtype"));
    }
    if (op == "nn_relu") return relay::ReluAttrs::Create();
    if (op == "nn_max_pool2d") {
        return relay::MaxPool2DAttrs::Create(Ints(Field(a, "strides", "pool attrs"), "pool attrs.strides"),
                                             Ints(Field(a, "pads", "pool attrs"), "pool attrs.pads"),
                                             Ints(Field(a, "dilations", "pool attrs"), "pool attrs.dilations"),
                                             Ints(Field(a, "pool_size", "pool attrs"), "pool attrs.pool_size"),
                                             Str(Field(a, "layout", "pool attrs"), "pool attrs.layout"),
                                             Bool(Field(a, "ceil_mode", "pool attrs"), "pool attrs.ceil_mode"));
    }
    if (op == "add") return relay::AddAttrs::Create();
    if (op == "nn_global_avg_pool2d") return relay::GlobalAvgPool2DAttrs::Create();
    if (op == "nn_flatten") return relay::FlattenAttrs::Create(static_cast<int>(Int(Field(a, "axis", "flatten attrs"), "flatten attrs.axis")));
    if (op == "nn_gemm") {
        return relay::GemmAttrs::Create(static_cast<float>(Num(Field(a, "alpha", "gemm attrs"), "gemm attrs.alpha")),
                                        static_cast<float>(Num(Field(a, "beta", "gemm attrs"), "gemm attrs.beta")),
                                        static_cast<int>(Int(Field(a, "transA", "gemm attrs"), "gemm attrs.transA")),
                                        static_cast<int>(Int(Field(a, "transB", "gemm attrs"), "gemm attrs.transB")));
    }
    Bad("Unsupported Relay op in ONNX import spec: " + op);
}

}  // namespace

ImportedONNXModel LoadONNXImportSpec(const std::string& json_path, const std::string& params_path) {
    const std::string text = ReadText(json_path);
    const Value root = json::Reader(text).Parse();
    const std::string format = Str(Field(root, "format", "root"), "root.format");
    if (format != "kxc.onnx_import.v1") Bad("Unsupported ONNX import spec format: " + format);
    const Value& fn = Field(root, "function", "root");
    const Value& inputs = Field(fn, "inputs", "function");
    const Value& outputs = Field(fn, "outputs", "function");
    const Value& nodes = Field(fn, "nodes", "function");
    const Value& params = Field(root, "params", "root");
    if (inputs.kind != Value::kArray) Bad("function.inputs must be an array");
    if (outputs.kind != Value::kArray) Bad("function.outputs must be an array");
    if (nodes.kind != Value::kArray) Bad("function.nodes must be an array");
    if (params.kind != Value::kArray) Bad("root.params must be an array");

    ImportedONNXModel result;
    std::unordered_map<std::string, Expr> values;
    Array<Var> fparams;
    for (size_t i = 0; i < inputs.array.size(); ++i) {
        const std::string ctx = "function.inputs[" + std::to_string(i) + "]";
        const std::string name = Str(Field(inputs.array[i], "name", ctx), ctx + ".name");
        const std::vector<int64_t> shape = Ints(Field(inputs.array[i], "shape", ctx), ctx + ".shape");
        const std::string dtype = Str(Field(inputs.array[i], "dtype", ctx), ctx + ".dtype");
        Var var(name, TensorType(ToArray(shape), dtype));
        fparams.push_back(var);
        values[name] = var;
        result.input_names.push_back(name);
    }

    const std::vector<char> bytes = ReadBinary(params_path);
    for (size_t i = 0; i < params.array.size(); ++i) {
        const Value& p = params.array[i];
        const std::string ctx = "root.params[" + std::to_string(i) + "]";
        const std::string name = Str(Field(p, "name", ctx), ctx + ".name");
        const std::vector<int64_t> shape = Ints(Field(p, "shape", ctx), ctx + ".shape");
        const std::string dtype = Str(Field(p, "dtype", ctx), ctx + ".dtype");
        const int64_t offset = Int(Field(p, "offset", ctx), ctx + ".offset");
        const int64_t nbytes = Int(Field(p, "nbytes", ctx), ctx + ".nbytes");
        if (offset < 0 || nbytes < 0 || static_cast<uint64_t>(offset) + static_cast<uint64_t>(nbytes) > bytes.size())
            Bad("Param bytes range out of bounds for: " + name);
        runtime::NDArray array(ToArray(shape), dtype);
        if (array.nbytes() != static_cast<size_t>(nbytes)) Bad("Param byte count does not match its shape and dtype: " + name);
        array.CopyFromBytes(bytes.data() + offset, static_cast<size_t>(nbytes));
        result.params.emplace(name, array);
        result.param_order.push_back(name);
        values[name] = Constant(array);
    }
    if (root.has("param_order") && Strs(root.at("param_order"), "root.param_order") != result.param_order)
        Bad("ONNX import spec param_order does not match params metadata");

    for (size_t i = 0; i < nodes.array.size(); ++i) {
        const Value& n = nodes.array[i];
        const std::string ctx = "function.nodes[" + std::to_string(i) + "]";
        const std::string node_name = Str(Field(n, "name", ctx), ctx + ".name");
        const std::string op_name = Str(Field(n, "op_name", ctx), ctx + ".op_name");
        const std::vector<std::string> in_names = Strs(Field(n, "inputs", ctx), ctx + ".inputs");
        const std::vector<std::string> out_names = Strs(Field(n, "outputs", ctx), ctx + ".outputs");
        if (out_names.size() != 1) Bad("ONNX import node must have one output: " + node_name);
        Array<Expr> args;
        for (const std::string& in : in_names) {
            auto it = values.find(in);
            if (it == values.end()) Bad("Missing input value '" + in + "' for node '" + node_name + "'");
            args.push_back(it->second);
        }
        Attrs attrs = MakeAttrs(op_name, Field(n, "attrs", ctx));
        values[out_names[0]] = Call(relay::Op::Get(op_name), args, attrs);
    }

    std::vector<Expr> outs;
    for (size_t i = 0; i < outputs.array.size(); ++i) {
        const std::string ctx = "function.outputs[" + std::to_string(i) + "]";
        const std::string name = Str(Field(outputs.array[i], "name", ctx), ctx + ".name");
        auto it = values.find(name);
        if (it == values.end()) Bad("Missing graph output value in ONNX import spec: " + name);
        outs.push_back(it->second);
        result.output_names.push_back(name);
    }
    if (outs.empty()) Bad("ONNX import spec has no graph outputs");
    if (outs.size() != 1) Bad("ONNX import spec with several graph outputs: tuples are outside this layer's operator path");
    result.function = Function(fparams, outs[0]);
    return result;
}

}  // namespace frontend
}  // namespace kxc
