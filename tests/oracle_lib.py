"""ctypes binding of the CPU checker in oracle/ (test infrastructure).

Only tests, the smoke check and the benchmark's cpu_baseline leg import this.
"""
import ctypes as C
import os
import subprocess
import threading

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")

_f32p = C.POINTER(C.c_float)
_i8p = C.POINTER(C.c_int8)
_i32p = C.POINTER(C.c_int32)
_i64 = C.c_int64
_int = C.c_int


def _ptr(a, ty):
    return a.ctypes.data_as(ty)


def _build_if_missing(name):
    path = os.path.join(ORACLE_DIR, name)
    if not os.path.exists(path):
        subprocess.check_call(["make", "-C", ORACLE_DIR, name])
    return path


class Oracle:
    def __init__(self, fast=False):
        self.lib = C.CDLL(_build_if_missing("libkxc_oracle_o3.so" if fast else "libkxc_oracle.so"))

    # ---- fp32 ----
    def conv2d(self, x, w, stride=1, pad=0, dil=1):
        x = np.ascontiguousarray(x, np.float32); w = np.ascontiguousarray(w, np.float32)
        N, Cc, H, W = x.shape; O, _, KH, KW = w.shape
        OH = (H + 2 * pad - ((KH - 1) * dil + 1)) // stride + 1
        OW = (W + 2 * pad - ((KW - 1) * dil + 1)) // stride + 1
        y = np.empty((N, O, OH, OW), np.float32)
        self.lib.kxc_oracle_conv2d_nchw_f32(_ptr(x, _f32p), _ptr(w, _f32p), _ptr(y, _f32p),
                                            _i64(N), _i64(Cc), _i64(H), _i64(W), _i64(O), _i64(KH), _i64(KW),
                                            _int(stride), _int(stride), _int(pad), _int(pad), _int(dil), _int(dil))
        return y

    def bias_add(self, x, b):
        x = np.ascontiguousarray(x, np.float32); b = np.ascontiguousarray(b, np.float32)
        N, O = x.shape[:2]; HW = int(np.prod(x.shape[2:]))
        y = np.empty_like(x)
        self.lib.kxc_oracle_bias_add_nchw_f32(_ptr(x, _f32p), _ptr(b, _f32p), _ptr(y, _f32p), _i64(N), _i64(O), _i64(HW))
        return y

    def relu(self, x):
        x = np.ascontiguousarray(x, np.float32); y = np.empty_like(x)
        self.lib.kxc_oracle_relu_f32(_ptr(x, _f32p), _ptr(y, _f32p), _i64(x.size))
        return y

    def binary(self, op, a, b):
        a = np.ascontiguousarray(a, np.float32); b = np.ascontiguousarray(b, np.float32)
        oshape = np.broadcast_shapes(a.shape, b.shape)
        y = np.empty(oshape, np.float32)
        sh = lambda s: (C.c_int64 * len(s))(*s)
        self.lib.kxc_oracle_broadcast_binary_f32(_int(op), _ptr(a, _f32p), sh(a.shape), _int(a.ndim),
                                                 _ptr(b, _f32p), sh(b.shape), _int(b.ndim),
                                                 _ptr(y, _f32p), sh(oshape), _int(len(oshape)))
        return y

    def add(self, a, b):
        return self.binary(0, a, b)

    def conv_chain(self, x, w, b=None, stride=1, pad=0, skip=None, relu=False):
        """The unfused operator chain the reference lowers: conv, bias add, add(skip), relu."""
        y = self.conv2d(x, w, stride, pad)
        if b is not None:
            y = self.bias_add(y, b)
        if skip is not None:
            y = self.add(y, skip)
        if relu:
            y = self.relu(y)
        return y

    def pool2d(self, x, k, s, pad, ceil_mode=False, avg=False):
        x = np.ascontiguousarray(x, np.float32)
        N, Cc, H, W = x.shape
        if np.isscalar(pad):
            pad = (pad, pad, pad, pad)
        kh, kw = (k, k) if np.isscalar(k) else k                  # (window and stride: one number or (rows, columns))
        sh, sw = (s, s) if np.isscalar(s) else s
        hn = H + pad[0] + pad[2] - kh; wn = W + pad[1] + pad[3] - kw
        OH = (hn + sh - 1) // sh + 1 if ceil_mode else hn // sh + 1
        OW = (wn + sw - 1) // sw + 1 if ceil_mode else wn // sw + 1
        y = np.empty((N, Cc, OH, OW), np.float32)
        self.lib.kxc_oracle_pool2d_f32(_ptr(x, _f32p), _ptr(y, _f32p), _i64(N), _i64(Cc), _i64(H), _i64(W),
                                       _int(kh), _int(kw), _int(sh), _int(sw),
                                       _int(pad[0]), _int(pad[1]), _int(pad[2]), _int(pad[3]),
                                       _int(int(ceil_mode)), _int(int(avg)))
        return y

    def gap(self, x):
        x = np.ascontiguousarray(x, np.float32)
        N, Cc, H, W = x.shape
        y = np.empty((N, Cc, 1, 1), np.float32)
        self.lib.kxc_oracle_global_avg_pool2d_f32(_ptr(x, _f32p), _ptr(y, _f32p), _i64(N), _i64(Cc), _i64(H), _i64(W))
        return y

    def dense(self, a, b):
        a = np.ascontiguousarray(a, np.float32); b = np.ascontiguousarray(b, np.float32)
        M, K = a.shape; N = b.shape[0]
        y = np.empty((M, N), np.float32)
        self.lib.kxc_oracle_dense_f32(_ptr(a, _f32p), _ptr(b, _f32p), _ptr(y, _f32p), _i64(M), _i64(N), _i64(K))
        return y

    def matmul(self, a, b):
        a = np.ascontiguousarray(a, np.float32); b = np.ascontiguousarray(b, np.float32)
        M, K = a.shape; N = b.shape[1]
        y = np.empty((M, N), np.float32)
        self.lib.kxc_oracle_matmul_f32(_ptr(a, _f32p), _ptr(b, _f32p), _ptr(y, _f32p), _i64(M), _i64(N), _i64(K))
        return y

    def gemm(self, a, b, c, alpha=1.0, beta=1.0, transB=1):
        a = np.ascontiguousarray(a, np.float32); b = np.ascontiguousarray(b, np.float32)
        c = np.ascontiguousarray(c, np.float32)
        M, K = a.shape; N = b.shape[0] if transB else b.shape[1]
        y = np.empty((M, N), np.float32)
        self.lib.kxc_oracle_gemm_f32(_ptr(a, _f32p), _ptr(b, _f32p), _ptr(c, _f32p), _ptr(y, _f32p),
                                     _i64(M), _i64(N), _i64(K), C.c_float(alpha), C.c_float(beta),
                                     _int(transB), _i64(c.size))
        return y

    # ---- int8 ----
    def quantize(self, x, scale):
        x = np.ascontiguousarray(x, np.float32); q = np.empty(x.shape, np.int8)
        self.lib.kxc_oracle_quantize_f32_i8(_ptr(x, _f32p), _ptr(q, _i8p), _i64(x.size), C.c_float(scale))
        return q

    def qconv_acc(self, x, w, stride=1, pad=0):
        x = np.ascontiguousarray(x, np.int8); w = np.ascontiguousarray(w, np.int8)
        N, Cc, H, W = x.shape; O, _, KH, KW = w.shape
        OH = (H + 2 * pad - KH) // stride + 1; OW = (W + 2 * pad - KW) // stride + 1
        y = np.empty((N, O, OH, OW), np.int32)
        self.lib.kxc_oracle_qconv2d_nchw_i8_acc(_ptr(x, _i8p), _ptr(w, _i8p), _ptr(y, _i32p),
                                                _i64(N), _i64(Cc), _i64(H), _i64(W), _i64(O), _i64(KH), _i64(KW),
                                                _int(stride), _int(stride), _int(pad), _int(pad))
        return y

    def qconv(self, x, w, bias, mult, stride=1, pad=0, residual=None, res_mult=0.0, relu=True):
        x = np.ascontiguousarray(x, np.int8); w = np.ascontiguousarray(w, np.int8)
        mult = np.ascontiguousarray(mult, np.float32)
        N, Cc, H, W = x.shape; O, _, KH, KW = w.shape
        OH = (H + 2 * pad - KH) // stride + 1; OW = (W + 2 * pad - KW) // stride + 1
        y = np.empty((N, O, OH, OW), np.int8)
        bp = _ptr(np.ascontiguousarray(bias, np.int32), _i32p) if bias is not None else None
        if residual is not None:
            residual = np.ascontiguousarray(residual, np.int8)
        rp = _ptr(residual, _i8p) if residual is not None else None
        self.lib.kxc_oracle_qconv2d_nchw_i8(_ptr(x, _i8p), _ptr(w, _i8p), bp, _ptr(mult, _f32p), rp,
                                            C.c_float(res_mult), _ptr(y, _i8p),
                                            _i64(N), _i64(Cc), _i64(H), _i64(W), _i64(O), _i64(KH), _i64(KW),
                                            _int(stride), _int(stride), _int(pad), _int(pad), _int(int(relu)))
        return y

    def qdense(self, a, b, bias, mult):
        a = np.ascontiguousarray(a, np.int8); b = np.ascontiguousarray(b, np.int8)
        mult = np.ascontiguousarray(mult, np.float32)
        M, K = a.shape; N = b.shape[0]
        y = np.empty((M, N), np.float32)
        bp = _ptr(np.ascontiguousarray(bias, np.int32), _i32p) if bias is not None else None
        self.lib.kxc_oracle_qdense_i8(_ptr(a, _i8p), _ptr(b, _i8p), bp, _ptr(mult, _f32p), _ptr(y, _f32p),
                                      _i64(M), _i64(N), _i64(K))
        return y

    def qmaxpool(self, x, k, s, pad):
        x = np.ascontiguousarray(x, np.int8)
        N, Cc, H, W = x.shape
        OH = (H + 2 * pad - k) // s + 1; OW = (W + 2 * pad - k) // s + 1
        y = np.empty((N, Cc, OH, OW), np.int8)
        self.lib.kxc_oracle_maxpool2d_i8(_ptr(x, _i8p), _ptr(y, _i8p), _i64(N), _i64(Cc), _i64(H), _i64(W),
                                         _int(k), _int(k), _int(s), _int(s), _int(pad), _int(pad), _int(pad), _int(pad))
        return y

    def qgap(self, x, mult):
        x = np.ascontiguousarray(x, np.int8)
        N, Cc, H, W = x.shape
        y = np.empty((N, Cc, 1, 1), np.int8)
        self.lib.kxc_oracle_global_avg_pool2d_i8(_ptr(x, _i8p), _ptr(y, _i8p), _i64(N), _i64(Cc), _i64(H), _i64(W),
                                                 C.c_float(mult))
        return y

    def qresnet18(self, x, model, gap_mult):
        """Quantised ResNet-18 as a chain of the CPU int8 operators (NCHW).  `model` is the dict of quantised
        constants and scales the product's preparation step produced: both sides consume the same numbers.
        Returns (logits fp32, {tap name: int8 NCHW tensor})."""
        by = {L["name"]: L for L in model["layers"]}
        taps = {}

        def conv(t, name, res=None):
            L = by[name]
            y = self.qconv(t, L["wq"], L["bias_q"], L["mult"], L["stride"], L["pad"], res,
                           L["res_mult"] if res is not None else 0.0, L["relu"])
            taps[name] = y
            return y

        q = self.quantize(x, model["input_scale"])
        taps["input"] = q
        y = conv(q, "conv1")
        cur = self.qmaxpool(y, 3, 2, 1)
        taps["maxpool"] = cur
        for stage in range(4):
            for blk in range(2):
                first = blk == 0 and stage > 0
                name = "l%d.%d" % (stage + 1, blk)
                a = conv(cur, name + ".conv1")
                idn = conv(cur, name + ".down") if first else cur
                cur = conv(a, name + ".conv2", idn)
        g = self.qgap(cur, gap_mult)
        taps["gap"] = g
        fc = model["fc"]
        logits = self.qdense(g.reshape(g.shape[0], -1), fc["wq"], fc["bias_q"], fc["mult"])
        return logits, taps

    # ---- network ----
    TAP_NAMES = ("conv1_relu", "maxpool", "layer1", "layer2", "layer3", "layer4", "gap", "flatten", "logits")

    def resnet18(self, x, consts, taps=False):
        x = np.ascontiguousarray(x, np.float32)
        N, _, HW, _ = x.shape
        consts = [np.ascontiguousarray(c, np.float32) for c in consts]
        arr = (_f32p * 42)(*[_ptr(c, _f32p) for c in consts])
        logits = np.empty((N, 1000), np.float32)
        tap_ptrs = (_f32p * 9)() if taps else None
        self.lib.kxc_oracle_resnet18_f32(_i64(N), _i64(HW), _ptr(x, _f32p), arr, _ptr(logits, _f32p), tap_ptrs)
        if not taps:
            return logits
        h1 = (HW + 6 - 7) // 2 + 1; h2 = (h1 + 2 - 3) // 2 + 1
        shapes = [(N, 64, h1, h1), (N, 64, h2, h2), (N, 64, h2, h2)]
        h = h2
        for ch in (128, 256, 512):
            h = (h + 2 - 3) // 2 + 1
            shapes.append((N, ch, h, h))
        shapes += [(N, 512, 1, 1), (N, 512), (N, 1000)]
        libc = C.CDLL(None)
        libc.free.argtypes = [C.c_void_p]
        out = {}
        for name, shp, p in zip(self.TAP_NAMES, shapes, tap_ptrs):
            n = int(np.prod(shp))
            out[name] = np.ctypeslib.as_array(p, shape=(n,)).reshape(shp).copy()
            libc.free(C.cast(p, C.c_void_p))
        return logits, out


class RefCases:
    """oracle/_ref/libkxc_ref_cases.so: the reference's own lowering + C code generator output.

    Present only where it was built from the reference checkout (the build container); GPU machines get the
    committed fixtures written from it instead."""

    PATH = os.path.join(ORACLE_DIR, "_ref", "libkxc_ref_cases.so")

    @classmethod
    def available(cls):
        return os.path.exists(cls.PATH)

    def __init__(self):
        self.lib = C.CDLL(self.PATH)

    def run(self, name, arrays):
        """arrays: inputs, constants and outputs as contiguous numpy arrays in parameter order.

        The generated code keeps intermediates in stack arrays (src/codegen/codegen_c.cc:220-232),
        so run it on a thread with a large stack."""
        fn = getattr(self.lib, name)
        fn.restype = C.c_int32
        args = (C.c_void_p * len(arrays))(*[a.ctypes.data for a in arrays])
        rc = []
        old = threading.stack_size(512 * 1024 * 1024)
        try:
            t = threading.Thread(target=lambda: rc.append(fn(args)))
            t.start(); t.join()
        finally:
            threading.stack_size(old)
        if rc != [0]:
            raise RuntimeError(f"{name} returned {rc}")
