"""The C-ABI library loads without a GPU and exports every symbol include/kxc_hip.h declares."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "kxc_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(kxc_hip_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_families():
    syms = declared_symbols()
    for s in ("kxc_hip_conv2d_nchw_f32", "kxc_hip_pool2d_f32", "kxc_hip_global_avg_pool2d_f32", "kxc_hip_gemm_f32",
              "kxc_hip_broadcast_binary_f32", "kxc_hip_qconv2d_nchw_i8", "kxc_hip_alloc", "kxc_hip_module_compile",
              "kxc_hip_plan_run"):
        assert s in syms
    assert len(syms) >= 45


def test_library_exports_every_declared_symbol(pkg):
    lib = ctypes.CDLL(pkg.library_path())
    missing = [s for s in declared_symbols() if not hasattr(lib, s)]
    assert not missing, missing


def test_device_queries_do_not_need_a_gpu(pkg):
    """Attribute query never fails: exists = 0 plus a reason when there is no device
    (the contract of the reference's test/device_info_test.cpp:110-125)."""
    a = pkg.device_attributes(0)
    assert a.arch.decode().startswith("gfx")
    assert a.warp_size == 64
    assert a.exists in (0, 1)
    if not a.exists:
        assert a.status.decode()
    assert pkg.lib().kxc_hip_target_kind() == b"hip"
    n = ctypes.c_int32(-1)
    assert pkg.lib().kxc_hip_device_count(ctypes.byref(n)) == 0 and n.value >= 0


def test_argument_errors_are_reported_not_crashed(pkg):
    import ctypes as C
    lib = pkg.lib()
    d = pkg.ConvDesc(1, 4, 3, 3, 8, 5, 5, 1, 1, 0, 0, 1, 1, 0)          # 5x5 window on a 3x3 input
    assert lib.kxc_hip_conv2d_nchw_f32(C.byref(d), None, None, None, None, None, None) == 1
    assert b"window is larger than input" in lib.kxc_hip_last_error()
    d = pkg.ConvDesc(1, 4, 8, 8, 8, 3, 3, 0, 1, 0, 0, 1, 1, 0)          # stride 0
    assert lib.kxc_hip_conv2d_nchw_f32(C.byref(d), None, None, None, None, None, None) == 1
    assert b"stride and dilation must be positive" in lib.kxc_hip_last_error()
    p = pkg.PoolDesc(1, 1, 2, 2, 3, 3, 1, 1, 0, 0, 0, 0, 0, 0)
    assert lib.kxc_hip_pool2d_f32(C.byref(p), None, None, None) == 1
    assert b"window is larger than input" in lib.kxc_hip_last_error()
    sa = (C.c_int64 * 2)(2, 3); sb = (C.c_int64 * 1)(4)
    one = C.c_void_p(1)
    assert lib.kxc_hip_broadcast_binary_f32(0, one, sa, 2, one, sb, 1, one, 0, None) == 1
    assert b"do not broadcast" in lib.kxc_hip_last_error()


def test_plan_builder_validates_on_the_host(pkg):
    import ctypes as C
    plan = pkg.Plan(3)
    d = pkg.ConvDesc(1, 4, 8, 8, 8, 3, 3, 1, 1, 1, 1, 1, 1, pkg.CONV_BIAS)
    try:
        plan.add_conv2d(d, pkg.Buf.arg(0), pkg.Buf.arg(1), pkg.Buf.none(), pkg.Buf.none(), pkg.Buf.arg(2))
        raise AssertionError("missing bias operand accepted")
    except pkg.KxcHipError as e:
        assert "required operand is absent" in str(e)
    try:
        plan.add_relu(4, pkg.Buf.arg(7), pkg.Buf.arg(2))
        raise AssertionError("argument index out of range accepted")
    except pkg.KxcHipError as e:
        assert "out of range" in str(e)
    try:
        plan.add_relu(4, pkg.Buf.ws(100), pkg.Buf.arg(2))
        raise AssertionError("unaligned workspace offset accepted")
    except pkg.KxcHipError as e:
        assert "multiples of 256" in str(e)
    plan.add_relu(4, pkg.Buf.arg(0), pkg.Buf.arg(2))
    assert plan.symbols() == ["kxc_relu_f32"]
    plan.close()
    # finalize checks every workspace operand's extent, not only where it starts, before it allocates anything
    plan = pkg.Plan(3)
    plan.add_relu(1000, pkg.Buf.arg(0), pkg.Buf.ws(256))                    # 4000 bytes at offset 256
    try:
        plan.finalize(4096)
        raise AssertionError("operand past the end of the workspace accepted")
    except pkg.KxcHipError as e:
        assert "does not fit" in str(e) and "4000 bytes" in str(e)
    plan.close()
    plan = pkg.Plan(3)
    d = pkg.ConvDesc(1, 4, 8, 8, 8, 3, 3, 1, 1, 1, 1, 1, 1, 0)             # y: 1 x 8 x 8 x 8 floats = 2048 bytes
    plan.add_conv2d(d, pkg.Buf.arg(0), pkg.Buf.arg(1), pkg.Buf.none(), pkg.Buf.none(), pkg.Buf.ws(1024))
    try:
        plan.finalize(2048)
        raise AssertionError("convolution output past the end of the workspace accepted")
    except pkg.KxcHipError as e:
        assert "does not fit" in str(e)
    plan.close()


def test_resnet18_plan_shape(pkg):
    """The plan builds on the host (no workspace allocation happens for a zero-size workspace only,
    so build it but skip finalize by checking the symbols through a dry builder)."""
    r = __import__("importlib").import_module("hdkx-aicompiler_amd.resnet18")
    assert r.flops_per_image() == 3628146688        # 2 x 1 814 073 344 multiply-accumulates per image (convolutions + FC)
