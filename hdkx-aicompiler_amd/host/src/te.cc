// te.cc -- tensor expression constructors and the operator compute definitions.
#include "kxc/te.h"
#include "kxc/topi.h"

#include <algorithm>

namespace kxc {
namespace te {

using tir::DataType;
using tir::ExprKind;
using tir::ExprNode;
using tir::Var;

PrimExpr Tensor::operator()(const std::vector<PrimExpr>& indices) const {
    if (!defined()) throw std::runtime_error("access to an undefined tensor");
    if (indices.size() != ptr_->shape.size())
        throw std::runtime_error("tensor '" + ptr_->name + "' accessed with " + std::to_string(indices.size()) +
                                 " indices, rank is " + std::to_string(ptr_->shape.size()));
    auto n = std::make_shared<ExprNode>();
    n->kind = ExprKind::kProducerLoad;
    n->dtype = ptr_->dtype;
    n->args = indices;
    n->tensor = ptr_;
    return PrimExpr(n);
}

PrimExpr Tensor::operator()(const Array<Var>& indices) const {
    std::vector<PrimExpr> idx(indices.begin(), indices.end());
    return (*this)(idx);
}

std::vector<int64_t> Tensor::const_shape() const {
    std::vector<int64_t> out;
    for (auto& d : ptr_->shape) {
        int64_t v;
        if (!tir::GetConstInt(d, &v)) throw std::runtime_error("tensor '" + ptr_->name + "' has a non-constant shape");
        out.push_back(v);
    }
    return out;
}

Tensor placeholder(std::vector<PrimExpr> shape, DataType dtype, std::string name) {
    auto n = std::make_shared<tir::TensorNode>();
    n->shape = std::move(shape);
    n->dtype = dtype;
    n->name = std::move(name);
    n->is_placeholder = true;
    return Tensor(n);
}

Tensor compute(std::vector<PrimExpr> shape, std::function<PrimExpr(const Array<Var>&)> fcompute, std::string name,
               std::string tag) {
    auto n = std::make_shared<tir::TensorNode>();
    n->shape = std::move(shape);
    n->name = std::move(name);
    n->tag = std::move(tag);
    n->is_placeholder = false;
    Array<Var> axis;
    for (size_t i = 0; i < n->shape.size(); ++i) axis.push_back(Var("ax" + std::to_string(i), DataType::Int(32)));
    n->axis = axis;
    n->body = fcompute(axis);
    if (!n->body.defined()) throw std::runtime_error("ComputeOp body is empty");
    n->dtype = n->body.dtype();
    return Tensor(n);
}

IterVar reduce_axis(PrimExpr min, PrimExpr extent, std::string name) {
    return IterVar{Var(std::move(name), DataType::Int(32)), min, extent};
}

static PrimExpr MakeReduce(int type, PrimExpr source, const std::vector<IterVar>& axes) {
    auto n = std::make_shared<ExprNode>();
    n->kind = ExprKind::kReduce;
    n->dtype = source.dtype();
    n->args = {source};
    n->reduce_type = type;
    for (auto& a : axes) {
        n->reduce_vars.push_back(a.var);
        n->reduce_min.push_back(a.dom_min);
        n->reduce_extent.push_back(a.dom_extent);
    }
    return PrimExpr(n);
}
PrimExpr sum(PrimExpr source, std::vector<IterVar> axes) { return MakeReduce(kSum, source, axes); }
PrimExpr max(PrimExpr source, std::vector<IterVar> axes) { return MakeReduce(kMax, source, axes); }
PrimExpr min(PrimExpr source, std::vector<IterVar> axes) { return MakeReduce(kMin, source, axes); }

namespace topi {

static int64_t ConstDim(const PrimExpr& e) {
    int64_t v;
    if (!tir::GetConstInt(e, &v)) throw std::runtime_error("non-constant dimension");
    return v;
}
static PrimExpr I64(int64_t v) { return tir::IntImm(v, DataType::Int(64)); }

PrimExpr make_const(DataType t, double value) {
    if (t.is_float()) return tir::FloatImm(value, t);
    return tir::IntImm(static_cast<int64_t>(value), t);
}

Tensor relu(const Tensor& x, std::string name) {
    return compute(x->shape, [&](const Array<Var>& i) { return tir::Max(x(i), make_const(x->dtype, 0)); }, name,
                   kElementWise);
}

Tensor dense(const Tensor& A, const Tensor& B, std::string name) {
    IterVar k = reduce_axis(0, A->shape[1], "k");
    return compute({A->shape[0], B->shape[0]},
                   [&](const Array<Var>& i) { return sum(A(i[0], k.var) * B(i[1], k.var), {k}); },
                   name + "_matmul", kMatMul);
}

Tensor matmul(const Tensor& A, const Tensor& B, std::string name) {
    IterVar k = reduce_axis(0, A->shape[1], "k");
    return compute({A->shape[0], B->shape[1]},
                   [&](const Array<Var>& i) { return sum(A(i[0], k.var) * B(k.var, i[1]), {k}); }, name, kMatMul);
}

Tensor conv2d_nchw(const Tensor& data, const Tensor& kernel, int stride_h, int stride_w, int pad_h, int pad_w,
                   int dilation_h, int dilation_w, std::string name) {
    const int64_t H = ConstDim(data->shape[2]), W = ConstDim(data->shape[3]);
    const int64_t KH = ConstDim(kernel->shape[2]), KW = ConstDim(kernel->shape[3]);
    // OH = (H + 2*pad - ((KH-1)*dilation + 1)) / stride + 1
    const int64_t OH = (H + 2 * pad_h - ((KH - 1) * dilation_h + 1)) / stride_h + 1;
    const int64_t OW = (W + 2 * pad_w - ((KW - 1) * dilation_w + 1)) / stride_w + 1;
    IterVar rc = reduce_axis(0, data->shape[1], "rc");
    IterVar rh = reduce_axis(0, kernel->shape[2], "rh");
    IterVar rw = reduce_axis(0, kernel->shape[3], "rw");
    return compute(
        {data->shape[0], kernel->shape[0], I64(OH), I64(OW)},
        [&](const Array<Var>& i) {
            PrimExpr h_in = i[2] * stride_h + rh.var * dilation_h - pad_h;
            PrimExpr w_in = i[3] * stride_w + rw.var * dilation_w - pad_w;
            PrimExpr in_val = tir::Select((h_in >= 0) && (h_in < data->shape[2]) && (w_in >= 0) && (w_in < data->shape[3]),
                                          data(i[0], rc.var, h_in, w_in), make_const(data->dtype, 0));
            return sum(in_val * kernel(i[1], rc.var, rh.var, rw.var), {rc, rh, rw});
        },
        name, kConv2d);
}

Tensor pool2d(const Tensor& data, std::vector<int> kernel_size, std::vector<int> stride, std::vector<int> padding,
              const std::string& pool_type, bool ceil_mode, std::string name) {
    if (kernel_size.size() < 2) throw std::runtime_error("topi::pool2d expects kernel_size with at least 2 elements");
    if (stride.size() < 2) throw std::runtime_error("topi::pool2d expects stride with at least 2 elements");
    if (pool_type != "max" && pool_type != "avg") throw std::runtime_error("topi::pool2d only supports pool_type=max/avg");
    const int64_t H = ConstDim(data->shape[2]), W = ConstDim(data->shape[3]);
    const int KH = kernel_size[0], KW = kernel_size[1], SH = stride[0], SW = stride[1];
    int pt = 0, pl = 0, pb = 0, pr = 0;
    if (padding.size() >= 4) { pt = padding[0]; pl = padding[1]; pb = padding[2]; pr = padding[3]; }
    else if (padding.size() >= 2) { pt = pb = padding[0]; pl = pr = padding[1]; }
    const int64_t hn = H + pt + pb - KH, wn = W + pl + pr - KW;
    const int64_t OH = ceil_mode ? (hn + SH - 1) / SH + 1 : hn / SH + 1;
    const int64_t OW = ceil_mode ? (wn + SW - 1) / SW + 1 : wn / SW + 1;
    IterVar rh = reduce_axis(0, KH, "rh");
    IterVar rw = reduce_axis(0, KW, "rw");
    const bool is_max = pool_type == "max";
    auto window = [&](const Array<Var>& i, double pad_value) {
        PrimExpr h_in = i[2] * SH + rh.var - pt;
        PrimExpr w_in = i[3] * SW + rw.var - pl;
        return tir::Select((h_in >= 0) && (h_in < data->shape[2]) && (w_in >= 0) && (w_in < data->shape[3]),
                           data(i[0], i[1], h_in, w_in), make_const(data->dtype, pad_value));
    };
    std::vector<PrimExpr> oshape = {data->shape[0], data->shape[1], I64(OH), I64(OW)};
    // (the padding candidate of the reference, nn.h:225, is the float -1e30; an integer tensor takes its dtype's
    // smallest value instead -- the reference converts -1e30 out of range there, which is undefined)
    const double lowest = data->dtype.is_float() ? -1e30
                          : data->dtype.is_uint() ? 0.0 : -static_cast<double>(int64_t{1} << (data->dtype.bits - 1));
    if (is_max)
        return compute(oshape, [&](const Array<Var>& i) { return max(window(i, lowest), {rh, rw}); }, name, kPool);
    Tensor sum_out = compute(oshape, [&](const Array<Var>& i) { return sum(window(i, 0), {rh, rw}); }, name + "_sum", kPool);
    return compute(oshape, [&](const Array<Var>& i) { return sum_out(i) / make_const(sum_out->dtype, KH * KW); }, name,
                   kPool);
}

Tensor global_avg_pool2d(const Tensor& data, std::string name) {
    IterVar rh = reduce_axis(0, data->shape[2], "rh");
    IterVar rw = reduce_axis(0, data->shape[3], "rw");
    Tensor sum_out = compute({data->shape[0], data->shape[1], I64(1), I64(1)},
                             [&](const Array<Var>& i) { return sum(data(i[0], i[1], rh.var, rw.var), {rh, rw}); },
                             name + "_sum", kPool);
    // the divisor is the integer expression H*W; the code generators promote it to float
    return compute(sum_out->shape, [&](const Array<Var>& i) { return sum_out(i) / (data->shape[2] * data->shape[3]); }, name,
                   kPool);
}

Tensor broadcast_binary(int op, const Tensor& A, const Tensor& B, std::string name) {
    const size_t na = A->shape.size(), nb = B->shape.size(), n = std::max(na, nb);
    std::vector<PrimExpr> oshape;
    for (size_t i = 0; i < n; ++i) {
        const int64_t da = i >= n - na ? ConstDim(A->shape[i - (n - na)]) : 1;
        const int64_t db = i >= n - nb ? ConstDim(B->shape[i - (n - nb)]) : 1;
        if (da != db && da != 1 && db != 1)
            throw std::runtime_error("broadcast shapes are incompatible: " + std::to_string(da) + " vs " + std::to_string(db));
        oshape.push_back(I64(da == 1 ? db : da));
    }
    auto index = [&](const Tensor& t, const Array<Var>& out) {
        std::vector<PrimExpr> idx;
        const size_t nt = t->shape.size(), off = n - nt;
        for (size_t i = 0; i < nt; ++i) {
            if (ConstDim(t->shape[i]) == 1) idx.push_back(PrimExpr(0));
            else idx.push_back(out[i + off]);
        }
        return t(idx);
    };
    return compute(oshape, [&](const Array<Var>& i) {
        PrimExpr a = index(A, i), b = index(B, i);
        switch (op) {
            case 0: return a + b;
            case 1: return a - b;
            case 2: return a * b;
            default: return a / b;
        }
    }, name, kBroadcast);
}

Tensor unary_call(const Tensor& x, const std::string& intrinsic, std::string name) {
    return compute(x->shape, [&](const Array<Var>& i) { return tir::Call(x->dtype, intrinsic, {x(i)}); }, name, kElementWise);
}

Tensor reshape(const Tensor& x, std::vector<int64_t> new_shape, std::string name) {
    std::vector<int64_t> in_shape = x.const_shape();
    std::vector<PrimExpr> oshape;
    for (auto d : new_shape) oshape.push_back(I64(d));
    return compute(oshape, [&](const Array<Var>& i) {
        // flatten the output index, then unflatten with % and / (transform.cc:70-82)
        PrimExpr lin = i.empty() ? PrimExpr(0) : PrimExpr(i[0]);
        for (size_t d = 1; d < new_shape.size(); ++d) lin = lin * I64(new_shape[d]) + i[d];
        std::vector<PrimExpr> idx(in_shape.size());
        for (int d = static_cast<int>(in_shape.size()) - 1; d >= 0; --d) {
            idx[d] = lin % I64(in_shape[d]);
            lin = lin / I64(in_shape[d]);
        }
        return x(idx);
    }, name, kInjective);
}

Tensor transpose(const Tensor& x, std::vector<int> axes, std::string name) {
    std::vector<PrimExpr> oshape;
    for (int a : axes) oshape.push_back(x->shape[a]);
    return compute(oshape, [&](const Array<Var>& i) {
        std::vector<PrimExpr> idx(axes.size());
        for (size_t d = 0; d < axes.size(); ++d) idx[axes[d]] = i[d];
        return x(idx);
    }, name, kInjective);
}

Tensor reduce_mean(const Tensor& x, std::vector<int> axes, bool keepdims, std::string name) {
    std::vector<int64_t> in_shape = x.const_shape();
    const int nd = static_cast<int>(in_shape.size());
    std::vector<bool> reduced(nd, false);
    int64_t count = 1;
    for (int a : axes) {
        if (a < 0) a += nd;
        reduced[a] = true;
        count *= in_shape[a];
    }
    std::vector<IterVar> raxes;
    std::vector<PrimExpr> oshape;
    for (int d = 0; d < nd; ++d) {
        if (reduced[d]) {
            raxes.push_back(reduce_axis(0, I64(in_shape[d]), "r" + std::to_string(d)));
            if (keepdims) oshape.push_back(I64(1));
        } else {
            oshape.push_back(I64(in_shape[d]));
        }
    }
    Tensor s = compute(oshape, [&](const Array<Var>& i) {
        std::vector<PrimExpr> idx;
        size_t o = 0, r = 0;
        for (int d = 0; d < nd; ++d) {
            if (reduced[d]) { idx.push_back(raxes[r++].var); if (keepdims) ++o; }
            else idx.push_back(i[o++]);
        }
        return sum(x(idx), raxes);
    }, name + "_sum", kInjective);
    return compute(oshape, [&](const Array<Var>& i) { return s(i) / make_const(s->dtype, static_cast<double>(count)); }, name,
                   kInjective);
}

Tensor softmax(const Tensor& x, int axis, std::string name) {
    std::vector<int64_t> in_shape = x.const_shape();
    const int nd = static_cast<int>(in_shape.size());
    Tensor e = unary_call(x, "exp", name + "_exp");
    IterVar r = reduce_axis(0, I64(in_shape[axis]), "k");
    std::vector<PrimExpr> sshape;
    for (int d = 0; d < nd; ++d) sshape.push_back(I64(d == axis ? 1 : in_shape[d]));
    Tensor s = compute(sshape, [&](const Array<Var>& i) {
        std::vector<PrimExpr> idx;
        for (int d = 0; d < nd; ++d) idx.push_back(d == axis ? PrimExpr(r.var) : PrimExpr(i[d]));
        return sum(e(idx), {r});
    }, name + "_sum", kInjective);
    return compute(x->shape, [&](const Array<Var>& i) {
        std::vector<PrimExpr> den;
        for (int d = 0; d < nd; ++d) den.push_back(d == axis ? I64(0) : PrimExpr(i[d]));
        return e(i) / s(den);
    }, name, kInjective);
}

Tensor cast(const Tensor& x, tir::DataType dtype, std::string name) {
    return compute(x->shape, [&](const Array<Var>& i) { return tir::Call(dtype, "cast", {x(i)}); }, name, kElementWise);
}

// ---- quantised operators: int32 accumulation, one rounded fp32 multiply (and add) per output, rint = round to
// nearest with ties to even, NaN -> 0, clamp, convert
namespace {
PrimExpr RintClampToI8(PrimExpr v, double lo, double hi) {
    const DataType f32 = DataType::Float(32);
    PrimExpr r = tir::Call(f32, "rint", {v});
    r = tir::Select(tir::EQ(v, v), r, make_const(f32, 0.0));
    r = tir::Min(tir::Max(r, make_const(f32, lo)), make_const(f32, hi));
    return tir::Call(DataType::Int(8), "cast", {r});
}
}  // namespace

Tensor qnn_quantize(const Tensor& x, double scale, std::string name) {
    return compute(x->shape, [&](const Array<Var>& i) { return RintClampToI8(x(i) / make_const(x->dtype, scale), -127.0, 127.0); },
                   name, kElementWise);
}

Tensor qnn_conv2d_nchw(const Tensor& data, const Tensor& kernel, const Tensor& bias, const Tensor& mult, const Tensor& residual,
                       int stride_h, int stride_w, int pad_h, int pad_w, bool relu, double res_mult, std::string name) {
    const DataType i32 = DataType::Int(32), f32 = DataType::Float(32);
    const int64_t H = ConstDim(data->shape[2]), W = ConstDim(data->shape[3]);
    const int64_t KH = ConstDim(kernel->shape[2]), KW = ConstDim(kernel->shape[3]);
    const int64_t OH = (H + 2 * pad_h - KH) / stride_h + 1, OW = (W + 2 * pad_w - KW) / stride_w + 1;
    IterVar rc = reduce_axis(0, data->shape[1], "rc");
    IterVar rh = reduce_axis(0, kernel->shape[2], "rh");
    IterVar rw = reduce_axis(0, kernel->shape[3], "rw");
    const std::vector<PrimExpr> oshape = {data->shape[0], kernel->shape[0], I64(OH), I64(OW)};
    Tensor acc = compute(oshape, [&](const Array<Var>& i) {
        PrimExpr h_in = i[2] * stride_h + rh.var - pad_h;
        PrimExpr w_in = i[3] * stride_w + rw.var - pad_w;
        PrimExpr x = tir::Select((h_in >= 0) && (h_in < data->shape[2]) && (w_in >= 0) && (w_in < data->shape[3]),
                                 tir::Call(i32, "cast", {data(i[0], rc.var, h_in, w_in)}), make_const(i32, 0));
        return sum(x * tir::Call(i32, "cast", {kernel(i[1], rc.var, rh.var, rw.var)}), {rc, rh, rw});
    }, name + "_acc", kConv2d);
    return compute(oshape, [&](const Array<Var>& i) {
        PrimExpr v = tir::Call(f32, "cast", {acc(i) + bias(i[1])}) * mult(i[1]);
        if (residual.defined()) v = v + tir::Call(f32, "cast", {residual(i)}) * make_const(f32, static_cast<double>(static_cast<float>(res_mult)));
        return RintClampToI8(v, relu ? 0.0 : -128.0, 127.0);
    }, name, kElementWise);
}

Tensor qnn_global_avg_pool2d(const Tensor& data, double mult, std::string name) {
    const DataType i32 = DataType::Int(32), f32 = DataType::Float(32);
    IterVar rh = reduce_axis(0, data->shape[2], "rh");
    IterVar rw = reduce_axis(0, data->shape[3], "rw");
    Tensor acc = compute({data->shape[0], data->shape[1], I64(1), I64(1)},
                         [&](const Array<Var>& i) { return sum(tir::Call(i32, "cast", {data(i[0], i[1], rh.var, rw.var)}), {rh, rw}); },
                         name + "_sum", kPool);
    return compute(acc->shape, [&](const Array<Var>& i) {
        return RintClampToI8(tir::Call(f32, "cast", {acc(i)}) * make_const(f32, static_cast<double>(static_cast<float>(mult))), -128.0, 127.0);
    }, name, kElementWise);
}

Tensor qnn_dense(const Tensor& A, const Tensor& B, const Tensor& bias, const Tensor& mult, std::string name) {
    const DataType i32 = DataType::Int(32), f32 = DataType::Float(32);
    IterVar k = reduce_axis(0, A->shape[1], "k");
    Tensor acc = compute({A->shape[0], B->shape[0]}, [&](const Array<Var>& i) {
        return sum(tir::Call(i32, "cast", {A(i[0], k.var)}) * tir::Call(i32, "cast", {B(i[1], k.var)}), {k});
    }, name + "_acc", kMatMul);
    return compute(acc->shape, [&](const Array<Var>& i) { return tir::Call(f32, "cast", {acc(i) + bias(i[1])}) * mult(i[1]); },
                   name, kElementWise);
}

}  // namespace topi
}  // namespace te
}  // namespace kxc
