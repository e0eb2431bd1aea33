"""ctypes binding of the C++ host layer's C face (host/src/capi.cc): compile a Relay graph for a target
and run it with device pointers."""
import ctypes as C
import os

from . import hipabi

PKG = os.path.dirname(os.path.abspath(__file__))
_HOST_LIB = os.path.join(PKG, "lib", "libkxc_host.so")
_lib = None


def lib():
    global _lib
    if _lib is None:
        hipabi.lib()     # the C-ABI library must be loaded first (the host library links against it)
        if not os.path.exists(_HOST_LIB):
            import subprocess
            subprocess.check_call(["make", "-C", os.path.join(PKG, "host"), "-j8"])
        _lib = C.CDLL(_HOST_LIB, mode=C.RTLD_GLOBAL)
        _lib.kxc_host_last_error.restype = C.c_char_p
        _lib.kxc_host_module_status.restype = C.c_char_p
        _lib.kxc_host_module_symbols.restype = C.c_char_p
        _lib.kxc_host_module_plan_json.restype = C.c_char_p
        _lib.kxc_host_module_constant_names.restype = C.c_char_p
        _lib.kxc_host_module_workspace_bytes.restype = C.c_longlong
    return _lib


class CompiledModule:
    """A Relay graph compiled by Compiler::Compile for "hip" (or "cpu"); subclasses build the graph."""

    _h = None

    @property
    def ready(self):
        return bool(lib().kxc_host_module_is_ready(self._h))

    @property
    def status(self):
        return lib().kxc_host_module_status(self._h).decode()

    def launches(self):
        return [l for l in lib().kxc_host_module_symbols(self._h).decode().split("\n") if l]

    def plan_json(self):
        return lib().kxc_host_module_plan_json(self._h).decode()

    def workspace_bytes(self):
        return int(lib().kxc_host_module_workspace_bytes(self._h))

    def packed(self, tensors):
        return (C.c_void_p * len(tensors))(*[t.data_ptr() for t in tensors])

    def run_packed(self, args, stream=None):
        """Enqueue on `stream` (a hipStream_t as int), which is the thread's current stream for the call."""
        if stream is not None:
            hipabi.lib().kxc_hip_set_stream(0, C.c_void_p(stream))
        try:
            if lib().kxc_host_module_run(self._h, args, len(args)) != 0:
                raise hipabi.KxcHipError(lib().kxc_host_last_error().decode())
        finally:
            if stream is not None:
                hipabi.lib().kxc_hip_set_stream(0, C.c_void_p(0))     # do not leave it as the thread's current stream

    def enable_graph_replay(self, enable=True):
        """Later runs on a non-null stream with the same argument pointers replay a captured HIP graph."""
        if lib().kxc_host_module_enable_graph(self._h, 1 if enable else 0) != 0:
            raise hipabi.KxcHipError(lib().kxc_host_last_error().decode())

    def run_timed(self, args, stream=None):
        """One run with a HIP event between consecutive launches: [(kernel symbol, microseconds)] per launch."""
        n = len(self.launches())
        buf = (C.c_longlong * (n + 8))()
        count = C.c_int(0)
        if stream is not None:
            hipabi.lib().kxc_hip_set_stream(0, C.c_void_p(stream))
        try:
            if lib().kxc_host_module_run_timed(self._h, args, len(args), buf, n + 8, C.byref(count)) != 0:
                raise hipabi.KxcHipError(lib().kxc_host_last_error().decode())
        finally:
            if stream is not None:
                hipabi.lib().kxc_hip_set_stream(0, C.c_void_p(0))
        return [(self.launches()[i], buf[i] / 1e3) for i in range(count.value)]

    def freeze_constants(self, frozen=True):
        """Serving mode: the weights will not change behind the module's back, so Winograd layers transform their
        filters once instead of at the start of every run."""
        if lib().kxc_host_module_freeze_constants(self._h, 1 if frozen else 0) != 0:
            raise hipabi.KxcHipError(lib().kxc_host_last_error().decode())

    def invalidate_constants(self):
        if lib().kxc_host_module_invalidate_constants(self._h) != 0:
            raise hipabi.KxcHipError(lib().kxc_host_last_error().decode())

    def close(self):
        if self._h:
            lib().kxc_host_module_free(self._h)
            self._h = C.c_void_p()


class CompiledResNet18(CompiledModule):
    """The fp32 ResNet-18 graph (host/src/models.cc BuildResNet18): input, 42 constants, logits."""

    def __init__(self, batch, hw=224, target="hip", use_handwritten=True, fuse=True, sync_after_run=False):
        self._h = C.c_void_p()
        rc = lib().kxc_host_compile_resnet18(target.encode(), C.c_longlong(batch), C.c_longlong(hw),
                                             int(use_handwritten), int(fuse), int(sync_after_run), C.byref(self._h))
        if rc != 0:
            raise hipabi.KxcHipError(lib().kxc_host_last_error().decode())
        self.num_args = 44


class CompiledQResNet18(CompiledModule):
    """The quantised ResNet-18 graph (BuildQResNet18): fp32 input, 63 constants -- per convolution int8 OIHW weights,
    int32 bias, fp32 multiplier, in the order conv1, then per block first convolution, second convolution[, downsample],
    then the dense layer's three -- and fp32 logits.  `model` is what qresnet18.prepare returns; its tensors are the
    constants (see constants()), its scales become operator attributes."""

    def __init__(self, model, batch, hw=224, target="hip", lanes=0, sync_after_run=False, result=""):
        """result: "" for the logits, or the name of an int8 activation ("conv1", "maxpool", "l2.0.down" ...) that the
        compiled function returns instead (as int8 NCHW): the graph up to that layer."""
        import numpy as np
        self._h = C.c_void_p()
        res = [L["res_mult"] for L in model["layers"] if L["name"].endswith(".conv2")]
        assert len(res) == 8
        oh = (hw + 6 - 7) // 2 + 1                   # conv1
        for _ in range(4):                            # max pool and the three stride-2 stages
            oh = (oh + 2 - 3) // 2 + 1
        s_last = model["scale"][model["last"]]
        self.gap_mult = float(np.float32(s_last) / (np.float32(oh * oh) * np.float32(model["gap_scale_out"])))
        rc = lib().kxc_host_compile_qresnet18(target.encode(), C.c_longlong(batch), C.c_longlong(hw),
                                              C.c_double(model["input_scale"]), (C.c_double * 8)(*res), C.c_double(self.gap_mult),
                                              int(lanes), int(sync_after_run), result.encode(), C.byref(self._h))
        if rc != 0:
            raise hipabi.KxcHipError(lib().kxc_host_last_error().decode())
        self.constant_names = [n for n in lib().kxc_host_module_constant_names(self._h).decode().split("\n") if n]
        self.num_args = 1 + len(self.constant_names) + 1

    def constants(self, model):
        """The module's constants as numpy arrays in packed-argument order (63 for the whole network)."""
        by_name = {L["name"]: L for L in model["layers"]}
        by_name["fc"] = model["fc"]
        key = {"w": "wq", "b": "bias_q", "m": "mult"}
        out = []
        for name in self.constant_names:
            layer, kind = name.rsplit(".", 1)
            out.append(by_name[layer][key[kind]])
        return out
