"""Source compatibility of the host layer: programs written against the reference's headers compile UNCHANGED against
the host layer through its forwarding include tree (host/include/compat) and run on its CPU back end.

Build-container only: the reference checkout is read where it lies and nothing of it is copied; the tests are
skipped where /root/reference does not exist (the GPU box).
"""
import os
import subprocess
import tempfile

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HOST = os.path.join(ROOT, "hdkx-aicompiler_amd", "host")
LIBDIR = os.path.join(ROOT, "hdkx-aicompiler_amd", "lib")
REF_TESTS = "/root/reference/test"

pytestmark = pytest.mark.skipif(not os.path.isdir(REF_TESTS), reason="the reference checkout is not present")


def _build(source, out, defines=()):
    if not os.path.exists(os.path.join(LIBDIR, "libkxc_host.so")):
        subprocess.check_call(["make", "-C", HOST, "-j8"])
    cmd = ["g++", "-std=c++17", "-O1"] + ["-D" + d for d in defines] + [
        "-I" + os.path.join(HOST, "include", "compat"), "-I" + os.path.join(HOST, "include"), "-I" + os.path.join(ROOT, "include"),
        os.path.join(REF_TESTS, source), "-o", out, "-L" + LIBDIR, "-lkxc_host", "-lkxc_hip", "-ldl", "-Wl,-rpath," + LIBDIR]
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-4000:]


def test_reference_operator_numeric_test_compiles_and_passes():
    """test/op_numeric_llvm_test.cpp (19 operators and 3 small models with literal expected vectors) with its
    compile-and-run branch switched on: CompileConfig::JIT(BuildTarget(kCPU)), Compiler::Compile, module.Run."""
    with tempfile.TemporaryDirectory() as d:
        exe = os.path.join(d, "op_numeric")
        _build("op_numeric_llvm_test.cpp", exe, defines=("KXC_USE_LLVM=1",))
        r = subprocess.run([exe], capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    assert "All MVP op LLVM numeric tests passed." in r.stdout
    assert r.stdout.count("[PASS]") >= 22 and "[SKIP]" not in r.stdout and "[FAIL]" not in r.stdout


def test_reference_resnet18_graph_builder_compiles_and_lowers():
    """test/resnet18_ir_dump.cpp: builds the ResNet-18 Relay graph with the reference's constructors and attribute
    factories, walks it, lowers it with LowerToTIR and dumps the PrimFunc: 44 parameters, 42 constants."""
    with tempfile.TemporaryDirectory() as d:
        exe = os.path.join(d, "resnet18_ir_dump")
        _build("resnet18_ir_dump.cpp", exe)
        r = subprocess.run([exe], capture_output=True, text=True, timeout=600, cwd=d)
        assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
        text = open(os.path.join(d, "resnet18_ir_dump.txt")).read()
    assert "Relay Graph Nodes(92)" in text
    assert text.count("[Call] nn_conv2d") == 20 and text.count("[Call] nn_relu") == 17 and text.count("[Call] add") == 8
    assert "params(44):" in text and "kxc.constant_count = 42" in text and "kxc.input_count = 1" in text
    assert "kxc.output_param_start = 43" in text
