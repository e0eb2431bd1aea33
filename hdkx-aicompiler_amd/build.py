"""Builds libkxc_hip.so (the C-ABI library of hand-written gfx950 kernels) with hipcc.

Usage: python build.py            (from anywhere; output goes to <package>/lib/libkxc_hip.so)
The benchmark, tests and smoke check load the built library and only call this when it is missing;
__graft_entry__.build() always calls it.
"""
import concurrent.futures
import os
import subprocess
import sys

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
LIBDIR = os.path.join(PKG, "lib")
OBJDIR = os.path.join(PKG, "build")
LIB = os.path.join(LIBDIR, "libkxc_hip.so")

SOURCES = ["device_api.hip", "activity.hip", "eltwise.hip", "pool.hip", "gemm.hip", "conv2d_f32.hip", "conv2d_wino_f32.hip", "split_reduce.hip", "qconv_i8.hip", "qconv_c16_i8.hip",
           "module.hip", "plan.hip"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = ["-O3", "--offload-arch=gfx950", "-fPIC", "-std=c++17", "-I" + os.path.join(ROOT, "include"),
         # packed fp32 instructions are kept out of every kernel
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         # no multiply-add contraction anywhere: the reference-order kernels must round every multiply
         # and add separately like the CPU backend (HIP's __fmul_rn/__fadd_rn do not prevent fusion)
         "-ffp-contract=off",
         "-Wall", "-Wno-unused-function"]


def _compile(src):
    obj = os.path.join(OBJDIR, src.replace(".hip", ".o"))
    cmd = [HIPCC] + FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, err))
    return obj, err


def build(verbose=True):
    os.makedirs(LIBDIR, exist_ok=True)
    os.makedirs(OBJDIR, exist_ok=True)
    with concurrent.futures.ThreadPoolExecutor(max_workers=8) as ex:
        results = list(ex.map(_compile, SOURCES))
    for obj, err in results:
        if verbose and err.strip():
            print(err, file=sys.stderr)
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + [o for o, _ in results] + ["-lhiprtc"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr)
    if verbose:
        print("built", LIB)
    build_rocprof_tool(verbose)
    return LIB


def build_rocprof_tool(verbose=True):
    """libkxc_hip_rocprof.so: the rocprofiler-sdk tool library behind kxc_hip_activity_enable(2).  Host code only;
    loaded on request, never linked into libkxc_hip.so."""
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    out = os.path.join(LIBDIR, "libkxc_hip_rocprof.so")
    cmd = [os.environ.get("CXX", "g++"), "-std=c++17", "-O2", "-fPIC", "-shared", "-Wall", "-D__HIP_PLATFORM_AMD__",
           "-I" + os.path.join(ROOT, "include"), "-I" + os.path.join(rocm, "include"),
           os.path.join(CSRC, "rocprof_tool.cpp"), "-o", out,
           "-L" + os.path.join(rocm, "lib"), "-lrocprofiler-sdk", "-Wl,-rpath," + os.path.join(rocm, "lib")]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("building libkxc_hip_rocprof.so failed:\n" + r.stderr)
    if verbose:
        print("built", out)
    return out


if __name__ == "__main__":
    build()
