"""ctypes binding of include/kxc_hip.h.

Every wrapper takes torch tensors that already live on the GPU and passes their device pointers
through the C ABI; a non-zero status raises KxcHipError carrying kxc_hip_last_error(), the way the
reference's C++ layers throw std::runtime_error.  There is no CPU fallback: if the library is
missing, loading fails loudly.
"""
import ctypes as C
import os

PKG = os.path.dirname(os.path.abspath(__file__))
# KXC_HIP_LIB points at an alternative build of the same library (kernel experiments).
_LIB_PATH = os.environ.get("KXC_HIP_LIB") or os.path.join(PKG, "lib", "libkxc_hip.so")
_lib = None

CONV_BIAS, CONV_RESIDUAL, CONV_RELU, CONV_HPOOL, CONV_FORCE_DIRECT = 1, 2, 4, 0x10, 0x100
BUF_ARG, BUF_WORKSPACE, BUF_NONE, BUF_ARG_OFFSET = 0, 1, 2, 3


class KxcHipError(RuntimeError):
    pass


class ConvDesc(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("n", "c", "h", "w", "o", "kh", "kw", "stride_h", "stride_w",
                                         "pad_h", "pad_w", "dil_h", "dil_w")] + [("flags", C.c_uint32)]


class QConvDesc(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("n", "c", "h", "w", "o", "kh", "kw", "stride_h", "stride_w",
                                         "pad_h", "pad_w")] + [("flags", C.c_uint32), ("res_mult", C.c_float)]


class PoolDesc(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("n", "c", "h", "w", "kh", "kw", "stride_h", "stride_w",
                                         "pad_top", "pad_left", "pad_bottom", "pad_right", "ceil_mode", "is_avg")]


class Buf(C.Structure):
    _fields_ = [("kind", C.c_int32), ("index_or_offset", C.c_int64)]

    @staticmethod
    def arg(i):
        return Buf(BUF_ARG, i)

    @staticmethod
    def ws(offset):
        return Buf(BUF_WORKSPACE, offset)

    @staticmethod
    def none():
        return Buf(BUF_NONE, 0)

    @staticmethod
    def arg_offset(i, nbytes):
        """packed argument i plus a byte offset (a multiple of 16): one share of a batched argument"""
        return Buf(BUF_ARG_OFFSET, (i << 48) | nbytes)


class DeviceAttrs(C.Structure):
    _fields_ = [("exists", C.c_int32), ("warp_size", C.c_int32),
                ("max_threads_per_block", C.c_int64), ("max_shared_memory_per_block", C.c_int64),
                ("max_shared_memory_per_multiprocessor", C.c_int64), ("multi_processor_count", C.c_int64),
                ("max_clock_rate_khz", C.c_int64), ("max_registers_per_block", C.c_int64),
                ("l2_cache_size_bytes", C.c_int64), ("total_global_memory", C.c_int64),
                ("available_global_memory", C.c_int64), ("max_threads_per_multiprocessor", C.c_int64),
                ("compute_version_major", C.c_int32), ("compute_version_minor", C.c_int32),
                ("api_version", C.c_int32), ("driver_version", C.c_int32),
                ("device_name", C.c_char * 128), ("arch", C.c_char * 32), ("status", C.c_char * 128)]


def library_path():
    return _LIB_PATH


def lib():
    """The loaded C-ABI library.  Builds it first only when no built library exists."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            from . import build as _build
            _build.build(verbose=False)
        _lib = C.CDLL(_LIB_PATH)
        _lib.kxc_hip_last_error.restype = C.c_char_p
        _lib.kxc_hip_target_kind.restype = C.c_char_p
        _lib.kxc_hip_conv2d_variant.restype = C.c_char_p
        _lib.kxc_hip_conv2d_winograd_variant.restype = C.c_char_p
        _lib.kxc_hip_conv2d_pair_variant.restype = C.c_char_p
        _lib.kxc_hip_qconv2d_c16_variant.restype = C.c_char_p
        _lib.kxc_hip_plan_node_symbol.restype = C.c_char_p
        _lib.kxc_hip_plan_workspace.restype = C.c_void_p
        _lib.kxc_hip_conv2d_noalloc_scratch_bytes.restype = C.c_size_t
    return _lib


def _check(rc):
    if rc != 0:
        raise KxcHipError(lib().kxc_hip_last_error().decode())


def _p(t):
    return C.c_void_p(t.data_ptr()) if t is not None else C.c_void_p(0)


def _stream():
    import torch
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _need(t, dtype, name):
    import torch
    if t is None:
        return
    if not (t.is_cuda and t.is_contiguous() and t.dtype == dtype):
        raise KxcHipError("%s must be a contiguous %s tensor on the GPU" % (name, dtype))


def device_attributes(device_id=0):
    a = DeviceAttrs()
    _check(lib().kxc_hip_device_attributes(C.c_int32(device_id), C.byref(a)))
    return a


def conv_desc(x_shape, w_shape, stride, pad, dil=1, flags=0):
    n, c, h, w = x_shape
    o, _, kh, kw = w_shape
    return ConvDesc(n, c, h, w, o, kh, kw, stride, stride, pad, pad, dil, dil, flags)


def conv_out_shape(d):
    oh = (d.h + 2 * d.pad_h - ((d.kh - 1) * d.dil_h + 1)) // d.stride_h + 1
    ow = (d.w + 2 * d.pad_w - ((d.kw - 1) * d.dil_w + 1)) // d.stride_w + 1
    return (d.n, d.o, oh, ow // 2 if d.flags & CONV_HPOOL else ow)


def conv2d_hpool_supported(x_shape, w_shape, stride, pad, dil=1, flags=CONV_BIAS | CONV_RELU, preferred=False):
    d = conv_desc(x_shape, w_shape, stride, pad, dil, flags)
    f = lib().kxc_hip_conv2d_hpool_preferred if preferred else lib().kxc_hip_conv2d_hpool_supported
    return bool(f(C.byref(d)))


def conv2d_variant(x_shape, w_shape, stride, pad, dil=1, flags=0):
    d = conv_desc(x_shape, w_shape, stride, pad, dil, flags)
    return lib().kxc_hip_conv2d_variant(C.byref(d)).decode()


def conv2d(x, w, bias=None, residual=None, stride=1, pad=0, dil=1, relu=False, force_direct=False, out=None,
           no_alloc=False, hpool=False):
    """nn_conv2d through kxc_hip_conv2d_nchw_f32, or (no_alloc, with `out` given) through the entry point that
    allocates nothing.  hpool: KXC_HIP_CONV_HPOOL, the result max-pooled along W (window 3, stride 2, padding 1)."""
    import torch
    _need(x, torch.float32, "x"); _need(w, torch.float32, "w")
    _need(bias, torch.float32, "bias"); _need(residual, torch.float32, "residual")
    if x.shape[1] != w.shape[1]:
        raise KxcHipError("nn_conv2d input channel mismatch")
    flags = (CONV_BIAS if bias is not None else 0) | (CONV_RESIDUAL if residual is not None else 0) | \
            (CONV_RELU if relu else 0) | (CONV_FORCE_DIRECT if force_direct else 0) | (CONV_HPOOL if hpool else 0)
    d = conv_desc(tuple(x.shape), tuple(w.shape), stride, pad, dil, flags)
    if out is not None:
        _check_out(out, conv_out_shape(d))
    y = out if out is not None else torch.empty(conv_out_shape(d), dtype=torch.float32, device=x.device)
    entry = lib().kxc_hip_conv2d_nchw_f32_noalloc if no_alloc else lib().kxc_hip_conv2d_nchw_f32
    _check(entry(C.byref(d), _p(x), _p(w), _p(bias), _p(residual), _p(y), _stream()))
    return y


def _check_out(out, shape, name="out"):
    import torch
    _need(out, torch.float32, name)
    if tuple(out.shape) != tuple(shape):
        raise KxcHipError("%s has shape %s, the operator writes %s" % (name, tuple(out.shape), tuple(shape)))


def conv2d_pair_supported(x_shape, w_shape, stride, pad, dil=1):
    d = conv_desc(x_shape, w_shape, stride, pad, dil, 0)
    return bool(lib().kxc_hip_conv2d_pair_supported(C.byref(d)))


def conv2d_pair_variant(x_shape, w_shape, stride, pad, dil=1):
    d = conv_desc(x_shape, w_shape, stride, pad, dil, 0)
    return lib().kxc_hip_conv2d_pair_variant(C.byref(d)).decode()


def conv2d_pair(x, w, bias, residual, w2, bias2, stride=1, pad=0, dil=1, relu=False):
    """(conv(x, w) [+bias] [+residual] [relu], conv1x1(x, w2, same stride, no padding) [+bias2]) in one launch."""
    import torch
    for t, nm in ((x, "x"), (w, "w"), (bias, "bias"), (residual, "residual"), (w2, "w2"), (bias2, "bias2")):
        _need(t, torch.float32, nm)
    if x.shape[1] != w.shape[1] or tuple(w2.shape) != (w.shape[0], w.shape[1], 1, 1):
        raise KxcHipError("conv2d_pair: w2 must be [o, c, 1, 1] for w [o, c, kh, kw]")
    flags = (CONV_BIAS if bias is not None else 0) | (CONV_RESIDUAL if residual is not None else 0) | (CONV_RELU if relu else 0)
    d = conv_desc(tuple(x.shape), tuple(w.shape), stride, pad, dil, flags)
    y = torch.empty(conv_out_shape(d), dtype=torch.float32, device=x.device)
    y2 = torch.empty_like(y)
    _check(lib().kxc_hip_conv2d_pair_nchw_f32(C.byref(d), _p(x), _p(w), _p(bias), _p(residual), _p(y), _p(w2), _p(bias2), _p(y2),
                                              _stream()))
    return y, y2


def conv2d_winograd_supported(x_shape, w_shape, stride, pad, dil=1):
    d = conv_desc(x_shape, w_shape, stride, pad, dil, 0)
    return bool(lib().kxc_hip_conv2d_winograd_supported(C.byref(d)))


def conv2d_winograd_preferred(x_shape, w_shape, stride=1, pad=1, dil=1):
    d = conv_desc(x_shape, w_shape, stride, pad, dil, 0)
    return bool(lib().kxc_hip_conv2d_winograd_preferred(C.byref(d)))


def conv2d_winograd_weight_bytes(x_shape, w_shape, pad=1):
    d = conv_desc(x_shape, w_shape, 1, pad, 1, 0)
    nbytes = C.c_size_t(0)
    _check(lib().kxc_hip_conv2d_winograd_weight_bytes(C.byref(d), C.byref(nbytes)))
    return nbytes.value


def set_select_lanes(lanes):
    """Variant selection of this thread's stand-alone launches and queries assumes `lanes` equal launches side by
    side (kxc_hip_set_select_lanes); returns the previous value."""
    return int(lib().kxc_hip_set_select_lanes(C.c_int32(lanes)))


def conv2d_winograd_variant(x_shape, w_shape, stride=1, pad=1, dil=1):
    d = conv_desc(x_shape, w_shape, stride, pad, dil, 0)
    return lib().kxc_hip_conv2d_winograd_variant(C.byref(d)).decode()


def conv2d_winograd_transform_weights(x_shape, w, pad=1):
    """OIHW 3x3 weights -> the transformed, packed form kxc_hip_conv2d_winograd_nchw_f32 reads."""
    import torch
    _need(w, torch.float32, "w")
    d = conv_desc(tuple(x_shape), tuple(w.shape), 1, pad, 1, 0)
    nbytes = C.c_size_t(0)
    _check(lib().kxc_hip_conv2d_winograd_weight_bytes(C.byref(d), C.byref(nbytes)))
    u = torch.empty(nbytes.value // 4, dtype=torch.float32, device=w.device)
    _check(lib().kxc_hip_conv2d_winograd_transform_weights(C.byref(d), _p(w), _p(u), _stream()))
    return u


def conv2d_winograd(x, u, w_shape, bias=None, residual=None, pad=1, relu=False, out=None):
    import torch
    _need(x, torch.float32, "x"); _need(u, torch.float32, "u")
    _need(bias, torch.float32, "bias"); _need(residual, torch.float32, "residual")
    flags = (CONV_BIAS if bias is not None else 0) | (CONV_RESIDUAL if residual is not None else 0) | \
            (CONV_RELU if relu else 0)
    d = conv_desc(tuple(x.shape), tuple(w_shape), 1, pad, 1, flags)
    if out is not None:
        _check_out(out, conv_out_shape(d))
    y = out if out is not None else torch.empty(conv_out_shape(d), dtype=torch.float32, device=x.device)
    _check(lib().kxc_hip_conv2d_winograd_nchw_f32(C.byref(d), _p(x), _p(u), _p(bias), _p(residual), _p(y), _stream()))
    return y


def relu(x):
    import torch
    _need(x, torch.float32, "x")
    y = torch.empty_like(x)
    _check(lib().kxc_hip_relu_f32(_p(x), _p(y), C.c_int64(x.numel()), _stream()))
    return y


def binary(op, a, b, relu=False, out=None):
    import torch
    _need(a, torch.float32, "a"); _need(b, torch.float32, "b")
    shape = torch.broadcast_shapes(a.shape, b.shape)
    y = out if out is not None else torch.empty(shape, dtype=torch.float32, device=a.device)
    _need(y, torch.float32, "out")
    if tuple(y.shape) != tuple(shape):
        raise ValueError("binary: out has shape %s, expected %s" % (tuple(y.shape), tuple(shape)))
    sa = (C.c_int64 * max(1, a.dim()))(*a.shape); sb = (C.c_int64 * max(1, b.dim()))(*b.shape)
    _check(lib().kxc_hip_broadcast_binary_f32(C.c_int32(op), _p(a), sa, C.c_int32(a.dim()), _p(b), sb,
                                              C.c_int32(b.dim()), _p(y), C.c_int32(int(relu)), _stream()))
    return y


def bias_add(x, bias, relu=False):
    import torch
    _need(x, torch.float32, "x"); _need(bias, torch.float32, "bias")
    y = torch.empty_like(x)
    n, o = x.shape[:2]
    hw = x.numel() // max(1, n * o)
    _check(lib().kxc_hip_bias_add_nchw_f32(_p(x), _p(bias), _p(y), C.c_int64(n), C.c_int64(o), C.c_int64(hw),
                                           C.c_int32(int(relu)), _stream()))
    return y


def pool_desc(x_shape, k, s, pad, ceil_mode=False, avg=False):
    n, c, h, w = x_shape
    if isinstance(pad, int):
        pad = (pad, pad, pad, pad)
    kh, kw = (k, k) if isinstance(k, int) else k
    sh, sw = (s, s) if isinstance(s, int) else s
    return PoolDesc(n, c, h, w, kh, kw, sh, sw, pad[0], pad[1], pad[2], pad[3], int(ceil_mode), int(avg))


def pool_out_shape(d):
    hn = d.h + d.pad_top + d.pad_bottom - d.kh
    wn = d.w + d.pad_left + d.pad_right - d.kw
    if d.ceil_mode:
        return (d.n, d.c, (hn + d.stride_h - 1) // d.stride_h + 1, (wn + d.stride_w - 1) // d.stride_w + 1)
    return (d.n, d.c, hn // d.stride_h + 1, wn // d.stride_w + 1)


def pool2d(x, k, s, pad, ceil_mode=False, avg=False, out=None):
    import torch
    _need(x, torch.float32, "x")
    d = pool_desc(tuple(x.shape), k, s, pad, ceil_mode, avg)
    if out is not None:
        _check_out(out, pool_out_shape(d))
    y = out if out is not None else torch.empty(pool_out_shape(d), dtype=torch.float32, device=x.device)
    _check(lib().kxc_hip_pool2d_f32(C.byref(d), _p(x), _p(y), _stream()))
    return y


def global_avg_pool2d(x, out=None):
    import torch
    _need(x, torch.float32, "x")
    n, c, h, w = x.shape
    y = out if out is not None else torch.empty((n, c, 1, 1), dtype=torch.float32, device=x.device)
    _need(y, torch.float32, "out")
    if y.numel() != n * c:
        raise ValueError("global_avg_pool2d: out has %d elements, expected %d" % (y.numel(), n * c))
    _check(lib().kxc_hip_global_avg_pool2d_f32(_p(x), _p(y), C.c_int64(n), C.c_int64(c), C.c_int64(h), C.c_int64(w),
                                               _stream()))
    return y


def gemm(a, b, c=None, alpha=1.0, beta=1.0, transB=1, out=None):
    import torch
    _need(a, torch.float32, "a"); _need(b, torch.float32, "b"); _need(c, torch.float32, "c")
    m, k = a.shape
    n = b.shape[0] if transB else b.shape[1]
    y = out if out is not None else torch.empty((m, n), dtype=torch.float32, device=a.device)
    _need(y, torch.float32, "out")
    if y.numel() != m * n:
        raise ValueError("gemm: out has %d elements, expected %d" % (y.numel(), m * n))
    _check(lib().kxc_hip_gemm_f32(_p(a), _p(b), _p(c), _p(y), C.c_int64(m), C.c_int64(n), C.c_int64(k),
                                  C.c_float(alpha), C.c_float(beta), C.c_int32(transB),
                                  C.c_int64(c.numel() if c is not None else 0), _stream()))
    return y


def flatten(x):
    import torch
    _need(x, torch.float32, "x")
    y = torch.empty((x.shape[0], x.numel() // max(1, x.shape[0])), dtype=torch.float32, device=x.device)
    _check(lib().kxc_hip_flatten_f32(_p(x), _p(y), C.c_int64(x.numel()), _stream()))
    return y


def quantize(x, scale):
    import torch
    _need(x, torch.float32, "x")
    q = torch.empty(x.shape, dtype=torch.int8, device=x.device)
    _check(lib().kxc_hip_quantize_f32_i8(_p(x), _p(q), C.c_int64(x.numel()), C.c_float(scale), _stream()))
    return q


def absmax(x):
    """max |x| of a GPU fp32 tensor, as a Python float (synchronises)."""
    import torch
    _need(x, torch.float32, "x")
    out = torch.empty((1,), dtype=torch.float32, device=x.device)
    _check(lib().kxc_hip_absmax_f32(_p(x), C.c_int64(x.numel()), _p(out), _stream()))
    return float(out.item())


def qconv2d(x, w, bias, mult, residual=None, res_mult=0.0, stride=1, pad=0, relu=True, force_direct=False):
    import torch
    _need(x, torch.int8, "x"); _need(w, torch.int8, "w"); _need(bias, torch.int32, "bias")
    _need(mult, torch.float32, "mult"); _need(residual, torch.int8, "residual")
    n, c, h, wd = x.shape
    o, _, kh, kw = w.shape
    flags = (CONV_BIAS if bias is not None else 0) | (CONV_RESIDUAL if residual is not None else 0) | \
            (CONV_RELU if relu else 0) | (CONV_FORCE_DIRECT if force_direct else 0)
    d = QConvDesc(n, c, h, wd, o, kh, kw, stride, stride, pad, pad, flags, res_mult)
    oh = (h + 2 * pad - kh) // stride + 1; ow = (wd + 2 * pad - kw) // stride + 1
    y = torch.empty((n, o, oh, ow), dtype=torch.int8, device=x.device)
    _check(lib().kxc_hip_qconv2d_nchw_i8(C.byref(d), _p(x), _p(w), _p(bias), _p(mult), _p(residual), _p(y), _stream()))
    return y


def qdense(a, b, bias, mult):
    import torch
    _need(a, torch.int8, "a"); _need(b, torch.int8, "b"); _need(bias, torch.int32, "bias"); _need(mult, torch.float32, "mult")
    m, k = a.shape
    n = b.shape[0]
    y = torch.empty((m, n), dtype=torch.float32, device=a.device)
    _check(lib().kxc_hip_qdense_i8(_p(a), _p(b), _p(bias), _p(mult), _p(y), C.c_int64(m), C.c_int64(n), C.c_int64(k),
                                   _stream()))
    return y


def maxpool2d_i8(x, k, s, pad):
    import torch
    _need(x, torch.int8, "x")
    d = pool_desc(tuple(x.shape), k, s, pad)
    y = torch.empty(pool_out_shape(d), dtype=torch.int8, device=x.device)
    _check(lib().kxc_hip_maxpool2d_i8(C.byref(d), _p(x), _p(y), _stream()))
    return y


def global_avg_pool2d_i8(x, mult):
    import torch
    _need(x, torch.int8, "x")
    n, c, h, w = x.shape
    y = torch.empty((n, c, 1, 1), dtype=torch.int8, device=x.device)
    _check(lib().kxc_hip_global_avg_pool2d_i8(_p(x), _p(y), C.c_int64(n), C.c_int64(c), C.c_int64(h), C.c_int64(w),
                                              C.c_float(mult), _stream()))
    return y


# ---- int8 on the channel-blocked "c16" layout ([N][ceil(C/16)][H][W][16])

def c16_shape(n, c, h, w):
    return (n, (c + 15) // 16, h, w, 16)


def i8_nchw_to_c16(x):
    import torch
    _need(x, torch.int8, "x")
    n, c, h, w = x.shape
    y = torch.empty(c16_shape(n, c, h, w), dtype=torch.int8, device=x.device)
    _check(lib().kxc_hip_i8_nchw_to_c16(_p(x), _p(y), C.c_int64(n), C.c_int64(c), C.c_int64(h * w), _stream()))
    return y


def i8_c16_to_nchw(x, c):
    import torch
    _need(x, torch.int8, "x")
    n, cb, h, w, _ = x.shape
    y = torch.empty((n, c, h, w), dtype=torch.int8, device=x.device)
    _check(lib().kxc_hip_i8_c16_to_nchw(_p(x), _p(y), C.c_int64(n), C.c_int64(c), C.c_int64(h * w), _stream()))
    return y


def quantize_to_c16(x, scale):
    import torch
    _need(x, torch.float32, "x")
    n, c, h, w = x.shape
    y = torch.empty(c16_shape(n, c, h, w), dtype=torch.int8, device=x.device)
    _check(lib().kxc_hip_quantize_f32_nchw_to_c16_i8(_p(x), _p(y), C.c_int64(n), C.c_int64(c), C.c_int64(h * w),
                                                     C.c_float(scale), _stream()))
    return y


def qconv_desc(n, c, h, w, o, kh, kw, stride, pad, flags=0, res_mult=0.0):
    return QConvDesc(n, c, h, w, o, kh, kw, stride, stride, pad, pad, flags, res_mult)


def qconv2d_c16_variant(d):
    return lib().kxc_hip_qconv2d_c16_variant(C.byref(d)).decode()


def qconv2d_c16_pack_weights(w):
    """OIHW int8 weights (GPU) -> the packed order the matrix-core kernel reads."""
    import torch
    _need(w, torch.int8, "w")
    o, c, kh, kw = w.shape
    d = qconv_desc(1, c, kh, kw, o, kh, kw, 1, 0)
    nbytes = C.c_size_t()
    _check(lib().kxc_hip_qconv2d_c16_packed_bytes(C.byref(d), C.byref(nbytes)))
    packed = torch.empty((nbytes.value,), dtype=torch.int8, device=w.device)
    _check(lib().kxc_hip_qconv2d_c16_pack_weights(C.byref(d), _p(w), _p(packed), _stream()))
    return packed


def qconv2d_c16(x, c, w_packed, w_shape, bias, mult, residual=None, res_mult=0.0, stride=1, pad=0, relu=True):
    """x: c16 tensor of logical channel count c; returns the c16 output."""
    import torch
    _need(x, torch.int8, "x"); _need(w_packed, torch.int8, "w_packed"); _need(bias, torch.int32, "bias")
    _need(mult, torch.float32, "mult"); _need(residual, torch.int8, "residual")
    n, cb, h, wd, _ = x.shape
    o, _, kh, kw = w_shape
    flags = (CONV_BIAS if bias is not None else 0) | (CONV_RESIDUAL if residual is not None else 0) | \
            (CONV_RELU if relu else 0)
    d = qconv_desc(n, c, h, wd, o, kh, kw, stride, pad, flags, res_mult)
    oh = (h + 2 * pad - kh) // stride + 1; ow = (wd + 2 * pad - kw) // stride + 1
    y = torch.empty(c16_shape(n, o, oh, ow), dtype=torch.int8, device=x.device)
    _check(lib().kxc_hip_qconv2d_c16_i8(C.byref(d), _p(x), _p(w_packed), _p(bias), _p(mult), _p(residual), _p(y),
                                        _stream()))
    return y


def qconv2d_c16_pair_supported(n, c, h, w, o, k, stride, pad):
    d = qconv_desc(n, c, h, w, o, k, k, stride, pad, 0)
    return bool(lib().kxc_hip_qconv2d_c16_pair_supported(C.byref(d)))


def qconv2d_c16_pair_pack_weights(w2, k):
    """[o, c, 1, 1] int8 weights (GPU) of the second output -> packed in the chunking of the k x k convolution."""
    import torch
    _need(w2, torch.int8, "w2")
    o, c = w2.shape[0], w2.shape[1]
    d = qconv_desc(1, c, k, k, o, k, k, 1, 0)
    nbytes = C.c_size_t()
    _check(lib().kxc_hip_qconv2d_c16_pair_packed_bytes(C.byref(d), C.byref(nbytes)))
    packed = torch.empty((nbytes.value,), dtype=torch.int8, device=w2.device)
    _check(lib().kxc_hip_qconv2d_c16_pair_pack_weights(C.byref(d), _p(w2), _p(packed), _stream()))
    return packed


def qconv2d_c16_pair(x, c, w_packed, w_shape, bias, mult, w2_packed, bias2, mult2, residual=None, res_mult=0.0, stride=1,
                     pad=0, relu=True):
    """(qconv2d_c16(x, w ...), the 1x1 convolution with the same strides and no padding, bias2 + requantise) in one launch."""
    import torch
    _need(x, torch.int8, "x"); _need(w_packed, torch.int8, "w_packed"); _need(bias, torch.int32, "bias")
    _need(mult, torch.float32, "mult"); _need(residual, torch.int8, "residual")
    _need(w2_packed, torch.int8, "w2_packed"); _need(bias2, torch.int32, "bias2"); _need(mult2, torch.float32, "mult2")
    n, cb, h, wd, _ = x.shape
    o, _, kh, kw = w_shape
    flags = (CONV_BIAS if bias is not None else 0) | (CONV_RESIDUAL if residual is not None else 0) | \
            (CONV_RELU if relu else 0)
    d = qconv_desc(n, c, h, wd, o, kh, kw, stride, pad, flags, res_mult)
    oh = (h + 2 * pad - kh) // stride + 1; ow = (wd + 2 * pad - kw) // stride + 1
    y = torch.empty(c16_shape(n, o, oh, ow), dtype=torch.int8, device=x.device)
    y2 = torch.empty_like(y)
    _check(lib().kxc_hip_qconv2d_c16_pair_i8(C.byref(d), _p(x), _p(w_packed), _p(bias), _p(mult), _p(residual), _p(y),
                                             _p(w2_packed), _p(bias2), _p(mult2), _p(y2), _stream()))
    return y, y2


def quantize_to_c4(x, scale):
    """fp32 NCHW (at most 4 channels) -> int8 [N][H][W][4]."""
    import torch
    _need(x, torch.float32, "x")
    n, c, h, w = x.shape
    y = torch.empty((n, h, w, 4), dtype=torch.int8, device=x.device)
    _check(lib().kxc_hip_quantize_f32_nchw_to_c4_i8(_p(x), _p(y), C.c_int64(n), C.c_int64(c), C.c_int64(h * w),
                                                    C.c_float(scale), _stream()))
    return y


def qconv2d_c4_pack_weights(w):
    import torch
    _need(w, torch.int8, "w")
    o, c, kh, kw = w.shape
    d = qconv_desc(1, c, kh, kw, o, kh, kw, 2, 3)
    nbytes = C.c_size_t()
    _check(lib().kxc_hip_qconv2d_c4_packed_bytes(C.byref(d), C.byref(nbytes)))
    packed = torch.empty((nbytes.value,), dtype=torch.int8, device=w.device)
    _check(lib().kxc_hip_qconv2d_c4_pack_weights(C.byref(d), _p(w), _p(packed), _stream()))
    return packed


def qconv2d_c4(x, c, w_packed, w_shape, bias, mult, relu=True):
    """First layer: x in c4 ([N][H][W][4]), 7x7 / stride 2 / padding 3; returns the c16 output."""
    import torch
    _need(x, torch.int8, "x"); _need(w_packed, torch.int8, "w_packed"); _need(bias, torch.int32, "bias")
    _need(mult, torch.float32, "mult")
    n, h, wd, _ = x.shape
    o = w_shape[0]
    flags = (CONV_BIAS if bias is not None else 0) | (CONV_RELU if relu else 0)
    d = qconv_desc(n, c, h, wd, o, 7, 7, 2, 3, flags)
    oh = (h + 6 - 7) // 2 + 1; ow = (wd + 6 - 7) // 2 + 1
    y = torch.empty(c16_shape(n, o, oh, ow), dtype=torch.int8, device=x.device)
    _check(lib().kxc_hip_qconv2d_c4_i8(C.byref(d), _p(x), _p(w_packed), _p(bias), _p(mult), _p(y), _stream()))
    return y


def qconv2d_c4_maxpool_supported(x_shape, o, c=3, relu=True):
    n, h, wd, _ = x_shape
    d = qconv_desc(n, c, h, wd, o, 7, 7, 2, 3, CONV_BIAS | (CONV_RELU if relu else 0))
    return bool(lib().kxc_hip_qconv2d_c4_maxpool_supported(C.byref(d)))


def qconv2d_c4_maxpool(x, c, w_packed, w_shape, bias, mult, relu=True):
    """First layer and the 3x3 / stride 2 / padding 1 max pool behind it in one kernel; returns the pooled c16 map."""
    import torch
    _need(x, torch.int8, "x"); _need(w_packed, torch.int8, "w_packed"); _need(bias, torch.int32, "bias")
    _need(mult, torch.float32, "mult")
    n, h, wd, _ = x.shape
    o = w_shape[0]
    flags = (CONV_BIAS if bias is not None else 0) | (CONV_RELU if relu else 0)
    d = qconv_desc(n, c, h, wd, o, 7, 7, 2, 3, flags)
    oh = (h + 6 - 7) // 2 + 1; ow = (wd + 6 - 7) // 2 + 1
    y = torch.empty(c16_shape(n, o, (oh - 1) // 2 + 1, (ow - 1) // 2 + 1), dtype=torch.int8, device=x.device)
    _check(lib().kxc_hip_qconv2d_c4_maxpool_i8(C.byref(d), _p(x), _p(w_packed), _p(bias), _p(mult), _p(y), _stream()))
    return y


def maxpool2d_c16_i8(x, c, k, s, pad):
    import torch
    _need(x, torch.int8, "x")
    n, cb, h, w, _ = x.shape
    d = pool_desc((n, c, h, w), k, s, pad)
    _, _, oh, ow = pool_out_shape(d)
    y = torch.empty(c16_shape(n, c, oh, ow), dtype=torch.int8, device=x.device)
    _check(lib().kxc_hip_maxpool2d_c16_i8(C.byref(d), _p(x), _p(y), _stream()))
    return y


def global_avg_pool2d_c16_i8(x, c, mult):
    import torch
    _need(x, torch.int8, "x")
    n, cb, h, w, _ = x.shape
    y = torch.empty((n, cb * 16), dtype=torch.int8, device=x.device)
    _check(lib().kxc_hip_global_avg_pool2d_c16_i8(_p(x), _p(y), C.c_int64(n), C.c_int64(c), C.c_int64(h), C.c_int64(w),
                                                  C.c_float(mult), _stream()))
    return y


QPACK_C16, QPACK_C4, QPACK_C16_PAIR = 1, 2, 3


class Plan:
    """kxc_hip_plan: a list of launches over packed arguments and one workspace."""

    def __init__(self, num_args, device_id=0):
        self._h = C.c_void_p()
        _check(lib().kxc_hip_plan_create(C.c_int32(device_id), C.c_int32(num_args), C.byref(self._h)))
        self.num_args = num_args

    def close(self):
        if self._h:
            lib().kxc_hip_plan_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def add_conv2d(self, desc, x, w, bias, residual, y):
        _check(lib().kxc_hip_plan_add_conv2d(self._h, C.byref(desc), x, w, bias, residual, y))

    def add_conv2d_winograd(self, desc, x, w, bias, residual, y, u):
        _check(lib().kxc_hip_plan_add_conv2d_winograd(self._h, C.byref(desc), x, w, bias, residual, y, u))

    def add_conv2d_pair(self, desc, x, w, bias, residual, y, w2, bias2, y2):
        _check(lib().kxc_hip_plan_add_conv2d_pair(self._h, C.byref(desc), x, w, bias, residual, y, w2, bias2, y2))

    def invalidate_constants(self):
        _check(lib().kxc_hip_plan_invalidate_constants(self._h))

    def freeze_constants(self, frozen=True):
        _check(lib().kxc_hip_plan_freeze_constants(self._h, C.c_int32(1 if frozen else 0)))

    def add_pool2d(self, desc, x, y):
        _check(lib().kxc_hip_plan_add_pool2d(self._h, C.byref(desc), x, y))

    def add_global_avg_pool2d(self, n, c, h, w, x, y):
        _check(lib().kxc_hip_plan_add_global_avg_pool2d(self._h, C.c_int64(n), C.c_int64(c), C.c_int64(h), C.c_int64(w), x, y))

    def add_gemm(self, m, n, k, alpha, beta, transB, c_len, a, b, c, y):
        _check(lib().kxc_hip_plan_add_gemm(self._h, C.c_int64(m), C.c_int64(n), C.c_int64(k), C.c_float(alpha),
                                           C.c_float(beta), C.c_int32(transB), C.c_int64(c_len), a, b, c, y))

    def add_binary(self, op, a_shape, b_shape, relu, a, b, y):
        sa = (C.c_int64 * max(1, len(a_shape)))(*a_shape); sb = (C.c_int64 * max(1, len(b_shape)))(*b_shape)
        _check(lib().kxc_hip_plan_add_binary(self._h, C.c_int32(op), sa, C.c_int32(len(a_shape)), sb,
                                             C.c_int32(len(b_shape)), C.c_int32(int(relu)), a, b, y))

    def add_relu(self, n, x, y):
        _check(lib().kxc_hip_plan_add_relu(self._h, C.c_int64(n), x, y))

    def add_copy(self, nbytes, x, y):
        _check(lib().kxc_hip_plan_add_copy(self._h, C.c_int64(nbytes), x, y))

    def add_qconv2d(self, desc, x, w, bias, mult, residual, y):
        _check(lib().kxc_hip_plan_add_qconv2d(self._h, C.byref(desc), x, w, bias, mult, residual, y))

    def add_quantize(self, n, scale, x, q):
        _check(lib().kxc_hip_plan_add_quantize(self._h, C.c_int64(n), C.c_float(scale), x, q))

    def add_maxpool2d_i8(self, desc, x, y):
        _check(lib().kxc_hip_plan_add_maxpool2d_i8(self._h, C.byref(desc), x, y))

    def add_global_avg_pool2d_i8(self, n, c, h, w, mult, x, y):
        _check(lib().kxc_hip_plan_add_global_avg_pool2d_i8(self._h, C.c_int64(n), C.c_int64(c), C.c_int64(h),
                                                           C.c_int64(w), C.c_float(mult), x, y))

    def add_qconv2d_c16(self, desc, x, w_packed, bias, mult, residual, y):
        _check(lib().kxc_hip_plan_add_qconv2d_c16(self._h, C.byref(desc), x, w_packed, bias, mult, residual, y))

    def add_qconv2d_c16_pair(self, desc, x, w_packed, bias, mult, residual, y, w2_packed, bias2, mult2, y2):
        _check(lib().kxc_hip_plan_add_qconv2d_c16_pair(self._h, C.byref(desc), x, w_packed, bias, mult, residual, y,
                                                       w2_packed, bias2, mult2, y2))

    def add_qconv2d_c4(self, desc, x, w_packed, bias, mult, y):
        _check(lib().kxc_hip_plan_add_qconv2d_c4(self._h, C.byref(desc), x, w_packed, bias, mult, y))

    def add_quantize_c4(self, n, c, hw, scale, x, q):
        _check(lib().kxc_hip_plan_add_quantize_c4(self._h, C.c_int64(n), C.c_int64(c), C.c_int64(hw), C.c_float(scale), x, q))

    def add_quantize_c16(self, n, c, hw, scale, x, q):
        _check(lib().kxc_hip_plan_add_quantize_c16(self._h, C.c_int64(n), C.c_int64(c), C.c_int64(hw), C.c_float(scale), x, q))

    def add_maxpool2d_c16_i8(self, desc, x, y):
        _check(lib().kxc_hip_plan_add_maxpool2d_c16_i8(self._h, C.byref(desc), x, y))

    def add_global_avg_pool2d_c16_i8(self, n, c, h, w, mult, x, y):
        _check(lib().kxc_hip_plan_add_global_avg_pool2d_c16_i8(self._h, C.c_int64(n), C.c_int64(c), C.c_int64(h),
                                                               C.c_int64(w), C.c_float(mult), x, y))

    def add_i8_layout(self, to_c16, n, c, hw, x, y):
        _check(lib().kxc_hip_plan_add_i8_layout(self._h, C.c_int32(1 if to_c16 else 0), C.c_int64(n), C.c_int64(c), C.c_int64(hw), x, y))

    def add_qconv_weight_pack(self, kind, desc, w_oihw, w_packed, every_run=False):
        """kind: QPACK_C16 / QPACK_C4 / QPACK_C16_PAIR.  w_oihw must be a packed argument, w_packed a workspace region."""
        _check(lib().kxc_hip_plan_add_qconv_weight_pack(self._h, C.c_int32(kind), C.byref(desc), w_oihw, w_packed,
                                                        C.c_int32(1 if every_run else 0)))

    def num_weight_packs(self):
        return int(lib().kxc_hip_plan_num_weight_packs(self._h))

    def add_qdense(self, m, n, k, a, b, bias, mult, y):
        _check(lib().kxc_hip_plan_add_qdense(self._h, C.c_int64(m), C.c_int64(n), C.c_int64(k), a, b, bias, mult, y))

    def enable_graph(self, enable=True):
        _check(lib().kxc_hip_plan_enable_graph(self._h, C.c_int32(1 if enable else 0)))

    def set_chain(self, node, chain):
        """Node `node` runs on the plan's chain stream `chain` (1-7), beside the main lane (kxc_hip_plan_set_chain)."""
        _check(lib().kxc_hip_plan_set_chain(self._h, C.c_int32(node), C.c_int32(chain)))

    def interleave_chains(self):
        """Reorders the nodes so that the streams are fed at the same pace (kxc_hip_plan_interleave_chains); returns
        the new index of every old node index."""
        n = self.num_nodes()
        idx = (C.c_int32 * max(n, 1))()
        _check(lib().kxc_hip_plan_interleave_chains(self._h, idx, C.c_int32(n)))
        return [int(idx[i]) for i in range(n)]

    def set_select_lanes(self, lanes):
        _check(lib().kxc_hip_plan_set_select_lanes(self._h, C.c_int32(lanes)))

    def num_nodes(self):
        return int(lib().kxc_hip_plan_num_nodes(self._h))

    def finalize(self, workspace_bytes):
        _check(lib().kxc_hip_plan_finalize(self._h, C.c_size_t(workspace_bytes)))

    def run(self, tensors, stream=None):
        """tensors: the packed arguments (inputs, constants, outputs) as GPU tensors."""
        args = (C.c_void_p * len(tensors))(*[t.data_ptr() for t in tensors])
        s = C.c_void_p(stream) if stream is not None else _stream()
        _check(lib().kxc_hip_plan_run(self._h, args, s))

    def packed(self, tensors):
        return (C.c_void_p * len(tensors))(*[t.data_ptr() for t in tensors])

    def run_packed(self, args, stream):
        _check(lib().kxc_hip_plan_run(self._h, args, C.c_void_p(stream)))

    def serialize(self):
        """The finalized plan as text (kxc_hip_plan_serialize)."""
        need = C.c_size_t(0)
        _check(lib().kxc_hip_plan_serialize(self._h, None, C.c_size_t(0), C.byref(need)))
        buf = C.create_string_buffer(need.value)
        _check(lib().kxc_hip_plan_serialize(self._h, buf, C.c_size_t(need.value), C.byref(need)))
        return buf.value.decode()

    @classmethod
    def deserialize(cls, text, device_id=0):
        """A plan without generated-kernel nodes rebuilt from serialize() output, finalized."""
        self = cls.__new__(cls)
        self._h = C.c_void_p()
        _check(lib().kxc_hip_plan_deserialize(text.encode(), C.c_int32(device_id), None, C.c_int32(0), C.byref(self._h)))
        self.num_args = None
        return self

    def node_symbol(self, i):
        return lib().kxc_hip_plan_node_symbol(self._h, C.c_int32(i)).decode()

    def symbols(self):
        n = lib().kxc_hip_plan_num_nodes(self._h)
        return [lib().kxc_hip_plan_node_symbol(self._h, C.c_int32(i)).decode() for i in range(n)]

    def workspace_ptr(self):
        return lib().kxc_hip_plan_workspace(self._h)
