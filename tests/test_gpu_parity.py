"""GPU parity: every hand-written operator, called through the C ABI, against the CPU checker.

Bit-exact where the arithmetic allows it (max pool, global average pool, elementwise, the direct
convolution / gemm kernels, all int8), within 1e-3 for the matrix-core kernels whose reduction order
differs.  Large (full-size) cases use properties that need no CPU run: agreement between the
matrix-core kernel and the bit-exact direct kernel, linearity, batch independence.
"""
import os

import numpy as np
import pytest
import torch

from gpu_util import assert_bit_exact, assert_close, dev, host
from oracle_lib import Oracle
from ref_case_table import CASES, case_inputs

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def orc():
    return Oracle()


@pytest.fixture(scope="module")
def fast_orc():
    return Oracle(fast=True)


# ------------------------------------------------------------------ reference-generated cases
CONV_CASES = {
    "kxc_ref_conv_cfg1": (1, 1, True, True, False), "kxc_ref_conv7x7s2": (2, 3, True, True, False),
    "kxc_ref_conv3x3s1": (1, 1, True, True, False), "kxc_ref_conv3x3s2": (2, 1, True, True, False),
    "kxc_ref_conv1x1s2": (2, 0, True, False, False), "kxc_ref_conv_nobias": (1, 1, False, False, False),
    "kxc_ref_conv_add_relu": (1, 1, True, True, True),
}


@pytest.mark.parametrize("name", sorted(CONV_CASES))
@pytest.mark.parametrize("direct", [True, False])
def test_conv_reference_cases(pkg, orc, name, direct):
    stride, pad, bias, relu, skip = CONV_CASES[name]
    ins = case_inputs(name)
    want = CASES[name][1](orc, ins)
    x, w = dev(ins[0]), dev(ins[1])
    b = dev(ins[2]) if bias else None
    r = dev(ins[3]) if skip else None
    got = host(pkg.conv2d(x, w, b, r, stride, pad, 1, relu, force_direct=direct))
    if direct or pkg.conv2d_variant(ins[0].shape, ins[1].shape, stride, pad) == "direct":
        assert_bit_exact(got, want, name)          # the direct kernel is the CPU loop nest
    else:
        assert_close(got, want, what=name)


def test_other_reference_cases(pkg, orc):
    for name in ("kxc_ref_maxpool3x3s2", "kxc_ref_maxpool_ceil", "kxc_ref_avgpool3x3s2"):
        ins = case_inputs(name)
        want = CASES[name][1](orc, ins)
        got = host(pkg.pool2d(dev(ins[0]), 3, 2, 1, ceil_mode="ceil" in name, avg="avg" in name))
        assert_bit_exact(got, want, name)
    ins = case_inputs("kxc_ref_gap7x7")
    assert_bit_exact(host(pkg.global_avg_pool2d(dev(ins[0]))), orc.gap(ins[0]), "gap")
    ins = case_inputs("kxc_ref_add_relu")
    assert_bit_exact(host(pkg.binary(0, dev(ins[0]), dev(ins[1]), relu=True)), orc.relu(orc.add(*ins)), "add_relu")
    ins = case_inputs("kxc_ref_add_bcast")
    assert_bit_exact(host(pkg.binary(0, dev(ins[0]), dev(ins[1]))), orc.add(*ins), "add_bcast")
    ins = case_inputs("kxc_ref_dense")
    assert_close(host(pkg.gemm(dev(ins[0]), dev(ins[1]))), orc.dense(*ins), what="dense")
    ins = case_inputs("kxc_ref_gemm_fc")
    assert_close(host(pkg.gemm(dev(ins[0]), dev(ins[1]), dev(ins[2]))), orc.gemm(*ins), what="gemm_fc")
    ins = case_inputs("kxc_ref_gemm_ab")
    assert_bit_exact(host(pkg.gemm(dev(ins[0]), dev(ins[1]), dev(ins[2]), 0.5, 2.0, 0)),
                     orc.gemm(ins[0], ins[1], ins[2], 0.5, 2.0, 0), "gemm_ab")


def test_reference_known_answers_through_the_abi(pkg):
    """The literals of the reference's test/op_numeric_llvm_test.cpp, computed on the GPU."""
    f = lambda v, s: dev(np.array(v, np.float32).reshape(s))
    assert host(pkg.binary(0, f([1, 2, 3, 4, 5, 6], (2, 3)), f([10, 20, 30], (3,)))).reshape(-1).tolist() == [11, 22, 33, 14, 25, 36]
    assert host(pkg.gemm(f([1, 2, 3, 4, 5, 6], (2, 3)), f([1, 0, 1, 0, 1, 1], (2, 3)))).reshape(-1).tolist() == [4, 5, 10, 11]
    y = pkg.gemm(f([1, 2, 3, 4, 5, 6], (2, 3)), f([1, 0, 0, 0, 1, 0, 0, 0, 1, 1, 1, 1], (4, 3)), f([10, 20, 30, 40], (4,)))
    assert host(y).reshape(-1).tolist() == [11, 22, 33, 46, 14, 25, 36, 55]
    assert host(pkg.relu(f([-2, -0.5, 0, 1, 2, -3], (6,)))).tolist() == [0, 0, 0, 1, 2, 0]
    y = pkg.conv2d(f(range(1, 10), (1, 1, 3, 3)), f([1, 0, 0, 1], (1, 1, 2, 2)))
    assert host(y).reshape(-1).tolist() == [6, 8, 12, 14]
    x = f(range(1, 17), (1, 1, 4, 4))
    assert host(pkg.pool2d(x, 2, 2, 0)).reshape(-1).tolist() == [6, 8, 14, 16]
    assert host(pkg.pool2d(x, 2, 2, 0, avg=True)).reshape(-1).tolist() == [3.5, 5.5, 11.5, 13.5]
    assert host(pkg.global_avg_pool2d(f([1, 2, 3, 4, 10, 20, 30, 40], (1, 2, 2, 2)))).reshape(-1).tolist() == [2.5, 25.0]
    assert host(pkg.flatten(f(range(1, 13), (1, 2, 2, 3)))).reshape(-1).tolist() == list(range(1, 13))
    # model_cnn: conv -> relu -> gap -> flatten -> dense = {10, 20}
    c = pkg.conv2d(f(range(1, 10), (1, 1, 3, 3)), f([1, 0, 0, 1], (1, 1, 2, 2)), relu=True)
    g = pkg.flatten(pkg.global_avg_pool2d(c))
    assert host(pkg.gemm(g, f([1, 2], (2, 1)))).reshape(-1).tolist() == [10, 20]


# ------------------------------------------------------------------ matrix-core convolution, every ResNet geometry
MFMA_SHAPES = [
    # n, c, h, w, o, k, s, p
    (2, 64, 56, 56, 64, 3, 1, 1),      # layer1
    (2, 64, 56, 56, 128, 3, 2, 1),     # layer2.0 conv1
    (3, 128, 28, 28, 128, 3, 1, 1),    # layer2
    (2, 128, 28, 28, 256, 3, 2, 1),    # layer3.0 conv1
    (5, 256, 14, 14, 256, 3, 1, 1),    # layer3: tiles cross image boundaries
    (3, 256, 14, 14, 512, 3, 2, 1),    # layer4.0 conv1
    (7, 512, 7, 7, 512, 3, 1, 1),      # layer4: several images per tile
    (2, 64, 56, 56, 128, 1, 2, 0),     # downsamples
    (3, 128, 28, 28, 256, 1, 2, 0),
    (5, 256, 14, 14, 512, 1, 2, 0),
    (2, 3, 224, 224, 64, 7, 2, 3),     # conv1
    (1, 3, 64, 64, 64, 7, 2, 3),
    (1, 30, 17, 19, 96, 3, 1, 1),      # ragged: odd sizes, channels not a multiple of the chunk
    (2, 7, 9, 33, 32, 3, 2, 1),
    (1, 5, 12, 12, 40, 1, 1, 0),       # output channels not a multiple of the tile
]


@pytest.mark.parametrize("shape", MFMA_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_conv_mfma_against_oracle(pkg, fast_orc, synth, shape):
    n, c, h, w, o, k, s, p = shape
    variant = pkg.conv2d_variant((n, c, h, w), (o, c, k, k), s, p)
    assert variant.startswith("mfma"), variant
    seed = 100 + MFMA_SHAPES.index(shape) * 7
    x = synth.uniform((n, c, h, w), seed)
    wt = synth.normal((o, c, k, k), seed + 1, float(np.sqrt(2.0 / (c * k * k))))
    b = synth.uniform((o,), seed + 2, -0.1, 0.1)
    oh, ow = (h + 2 * p - k) // s + 1, (w + 2 * p - k) // s + 1
    skip = synth.uniform((n, o, oh, ow), seed + 3)
    want = fast_orc.conv_chain(x, wt, b, s, p, skip, True)
    got = host(pkg.conv2d(dev(x), dev(wt), dev(b), dev(skip), s, p, 1, True))
    assert_close(got, want, what=variant)
    # no epilogue at all
    want = fast_orc.conv2d(x, wt, s, p)
    got = host(pkg.conv2d(dev(x), dev(wt), None, None, s, p, 1, False))
    assert_close(got, want, what=variant + " (bare)")


@pytest.mark.parametrize("shape,forced", [((1, 512, 7, 7, 512, 3, 1, 1), None), ((1, 256, 14, 14, 256, 3, 1, 1), None),
                                          ((1, 256, 14, 14, 512, 1, 2, 0), None), ((1, 256, 14, 14, 512, 3, 2, 1), None),
                                          ((2, 128, 28, 28, 128, 3, 1, 1), "3"), ((2, 128, 28, 28, 128, 3, 1, 1), "5"),
                                          ((1, 70, 9, 11, 64, 3, 1, 1), "2")],
                         ids=lambda v: "x".join(map(str, v)) if isinstance(v, tuple) else str(v))
def test_conv_reduction_split_over_workgroups(pkg, fast_orc, synth, monkeypatch, shape, forced):
    """Small launches with a long reduction (batch-1 deep layers) split the channels over workgroups and add the
    partial sums in a second kernel: same tolerance, bias / residual / ReLU applied once, deterministic."""
    n, c, h, w, o, k, s, p = shape
    if forced is not None:
        monkeypatch.setenv("KXC_HIP_CONV_GSPLIT", forced)
    x = synth.uniform((n, c, h, w), 6100)
    wt = synth.normal((o, c, k, k), 6101, float(np.sqrt(2.0 / (c * k * k))))
    b = synth.uniform((o,), 6102, -0.1, 0.1)
    oh, ow = (h + 2 * p - k) // s + 1, (w + 2 * p - k) // s + 1
    skip = synth.uniform((n, o, oh, ow), 6103)
    want = fast_orc.conv_chain(x, wt, b, s, p, skip=skip, relu=True)
    got1 = host(pkg.conv2d(dev(x), dev(wt), dev(b), dev(skip), s, p, 1, True))
    got2 = host(pkg.conv2d(dev(x), dev(wt), dev(b), dev(skip), s, p, 1, True))
    assert_close(got1, want, what="split reduction %s" % (shape,))
    assert_bit_exact(got2, got1, "split reduction is deterministic")


# ------------------------------------------------------------------ convolution pair (3x3 + 1x1 downsample)
PAIR_SHAPES = [
    # n, c, h, w, o, k, s, p
    (2, 64, 56, 56, 128, 3, 2, 1),     # layer2.0: conv1 + downsample
    (2, 128, 28, 28, 256, 3, 2, 1),    # layer3.0
    (3, 256, 14, 14, 512, 3, 2, 1),    # layer4.0 (tiles cross image boundaries)
    (8, 64, 56, 56, 128, 3, 2, 1),     # enough work for the unsplit tiles
    (16, 256, 14, 14, 512, 3, 2, 1),
    (1, 30, 17, 19, 96, 3, 2, 1),      # ragged: odd sizes, channels not a multiple of the chunk
    (2, 7, 9, 33, 40, 3, 1, 1),        # stride 1, output channels not a multiple of the tile
    (1, 12, 20, 20, 64, 5, 2, 2),      # no 5x5 matrix kernel: refused
]


@pytest.mark.parametrize("shape", PAIR_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_conv_pair_against_oracle(pkg, fast_orc, synth, monkeypatch, shape):
    """A block's first convolution and its 1x1 downsample in one launch: both outputs against the CPU path's two
    separate convolutions, and the first output bit for bit what the separate matrix-core launch gives."""
    n, c, h, w, o, k, s, p = shape
    if k == 5:
        assert not pkg.conv2d_pair_supported((n, c, h, w), (o, c, k, k), s, p)
        assert pkg.conv2d_pair_variant((n, c, h, w), (o, c, k, k), s, p) == "unsupported"
        return
    if not pkg.conv2d_pair_supported((n, c, h, w), (o, c, k, k), s, p):
        # a launch this small would rather split its reduction over workgroups: not paired unless that is ruled out
        assert _scratch_needed(pkg, (n, c, h, w), (o, c, k, k), s, p) > 0
        monkeypatch.setenv("KXC_HIP_CONV_GSPLIT", "1")
    assert pkg.conv2d_pair_supported((n, c, h, w), (o, c, k, k), s, p)
    variant = pkg.conv2d_pair_variant((n, c, h, w), (o, c, k, k), s, p)
    assert variant.endswith("_ds"), variant
    seed = 6300 + PAIR_SHAPES.index(shape) * 11
    x = synth.uniform((n, c, h, w), seed)
    w1 = synth.normal((o, c, k, k), seed + 1, float(np.sqrt(2.0 / (c * k * k))))
    b1 = synth.uniform((o,), seed + 2, -0.1, 0.1)
    w2 = synth.normal((o, c, 1, 1), seed + 3, float(np.sqrt(2.0 / c)))
    b2 = synth.uniform((o,), seed + 4, -0.1, 0.1)
    oh, ow = (h + 2 * p - k) // s + 1, (w + 2 * p - k) // s + 1
    skip = synth.uniform((n, o, oh, ow), seed + 5)
    want1 = fast_orc.conv_chain(x, w1, b1, s, p, None, True)
    want2 = fast_orc.conv_chain(x, w2, b2, s, 0, None, False)
    y1, y2 = pkg.conv2d_pair(dev(x), dev(w1), dev(b1), None, dev(w2), dev(b2), s, p, 1, True)
    assert_close(host(y1), want1, what=variant + " first output")
    assert_close(host(y2), want2, what=variant + " second output")
    # the first output is the single launch's, bit for bit (same tile, same order of sums)
    alone = pkg.conv2d(dev(x), dev(w1), dev(b1), None, s, p, 1, True)
    if pkg.conv2d_variant((n, c, h, w), (o, c, k, k), s, p) + "_ds" == variant and _scratch_needed(pkg, (n, c, h, w), (o, c, k, k), s, p) == 0:
        assert_bit_exact(host(y1), host(alone), "first output of the pair equals the single launch")
    # residual on the first output, no biases
    want1 = fast_orc.conv_chain(x, w1, None, s, p, skip, False)
    want2 = fast_orc.conv2d(x, w2, s, 0)
    y1, y2 = pkg.conv2d_pair(dev(x), dev(w1), None, dev(skip), dev(w2), None, s, p, 1, False)
    assert_close(host(y1), want1, what=variant + " first output (+residual)")
    assert_close(host(y2), want2, what=variant + " second output (bare)")


@pytest.mark.parametrize("shape", [(1, 64, 56, 56, 128), (1, 128, 28, 28, 256), (1, 256, 14, 14, 512), (2, 256, 14, 14, 512)],
                         ids=["l2.0", "l3.0", "l4.0", "l4.0-n2"])
def test_conv_pair_with_both_reductions_split_over_workgroups(pkg, fast_orc, synth, monkeypatch, shape):
    """The ResNet-18 stride-2 blocks at batch 1-2: the launch splits its input channels over workgroups, every part
    writes raw sums of both outputs and ONE adding launch finishes both (bias + ReLU on the first, bias on the
    second).  Both outputs against the CPU path's separate convolutions, run to run bit-identical (the parts are
    added in split order), and refused with KXC_HIP_PAIR_SPLIT=0."""
    n, c, h, w, o = shape
    xs, ws = (n, c, h, w), (o, c, 3, 3)
    assert _scratch_needed(pkg, xs, ws, 2, 1) > 0                  # the single-output launch of this shape splits
    assert pkg.conv2d_pair_supported(xs, ws, 2, 1)
    seed = 6800 + 13 * c + n
    x = synth.uniform(xs, seed)
    w1 = synth.normal(ws, seed + 1, float(np.sqrt(2.0 / (c * 9))))
    b1 = synth.uniform((o,), seed + 2, -0.1, 0.1)
    w2 = synth.normal((o, c, 1, 1), seed + 3, float(np.sqrt(2.0 / c)))
    b2 = synth.uniform((o,), seed + 4, -0.1, 0.1)
    want1 = fast_orc.conv_chain(x, w1, b1, 2, 1, None, True)
    want2 = fast_orc.conv_chain(x, w2, b2, 2, 0, None, False)
    y1, y2 = pkg.conv2d_pair(dev(x), dev(w1), dev(b1), None, dev(w2), dev(b2), 2, 1, 1, True)
    assert_close(host(y1), want1, what="split pair, first output")
    assert_close(host(y2), want2, what="split pair, second output")
    z1, z2 = pkg.conv2d_pair(dev(x), dev(w1), dev(b1), None, dev(w2), dev(b2), 2, 1, 1, True)
    assert_bit_exact(host(z1), host(y1), "first output, second run")
    assert_bit_exact(host(z2), host(y2), "second output, second run")
    # no bias on the second output, a residual on the first
    skip = synth.uniform(want1.shape, seed + 5)
    y1, y2 = pkg.conv2d_pair(dev(x), dev(w1), None, dev(skip), dev(w2), None, 2, 1, 1, False)
    assert_close(host(y1), fast_orc.conv_chain(x, w1, None, 2, 1, skip, False), what="split pair, first output (+residual)")
    assert_close(host(y2), fast_orc.conv2d(x, w2, 2, 0), what="split pair, second output (bare)")
    monkeypatch.setenv("KXC_HIP_PAIR_SPLIT", "0")
    assert not pkg.conv2d_pair_supported(xs, ws, 2, 1)


def _scratch_needed(pkg, xs, ws, s, p):
    import ctypes as C
    d = pkg.conv_desc(xs, ws, s, p, 1, 0)
    n = C.c_size_t(0)
    assert pkg.lib().kxc_hip_conv2d_scratch_needed(C.byref(d), C.byref(n)) == 0
    return n.value


@pytest.mark.parametrize("variant", ["mfma_k3x3_c4_o1x1_p4x1", "mfma_k3x3_c4_o1x1_p8x1", "mfma_k3x3_c2_o1x1_p4x1",
                                     "mfma_k3x3_c4_o1x1_p2x1", "mfma_k3x3_c4_o2x1_p8x1", "mfma_k3x3_c4_o1x1_p4x1_ks2",
                                     "mfma_k3x3_c4_o1x1_p2x1_ks4", "mfma_k3x3_c4_o1x1_p2x1_ks8", "mfma_k3x3_c4_o1x1_p7x1_ks2",
                                     "mfma_k3x3_c4_o2x1_p7x1"])
def test_conv_pair_every_tile(pkg, fast_orc, synth, monkeypatch, variant):
    """Every tile shape that exists with a second output, forced once (128 -> 256 channels)."""
    monkeypatch.setenv("KXC_HIP_CONV_VARIANT", variant)
    # (a forced tile must hold the shape's input patch: the first candidate shape it accepts is used)
    for n, c, h, o, s, p in ((2, 128, 28, 256, 2, 1), (3, 128, 12, 256, 1, 1)):
        if pkg.conv2d_pair_variant((n, c, h, h), (o, c, 3, 3), s, p) == variant + "_ds":
            break
    else:
        raise AssertionError("no candidate shape fits " + variant)
    x = synth.uniform((n, c, h, h), 6500)
    w1 = synth.normal((o, c, 3, 3), 6501, float(np.sqrt(2.0 / (c * 9))))
    b1 = synth.uniform((o,), 6502, -0.1, 0.1)
    w2 = synth.normal((o, c, 1, 1), 6503, float(np.sqrt(2.0 / c)))
    b2 = synth.uniform((o,), 6504, -0.1, 0.1)
    y1, y2 = pkg.conv2d_pair(dev(x), dev(w1), dev(b1), None, dev(w2), dev(b2), s, p, 1, True)
    assert_close(host(y1), fast_orc.conv_chain(x, w1, b1, s, p, None, True), what=variant + " first output")
    assert_close(host(y2), fast_orc.conv_chain(x, w2, b2, s, 0, None, False), what=variant + " second output")


def test_conv_pair_full_batch_properties(pkg, synth):
    """Batch 64 at the three ResNet-18 shapes: the pair launch against the two separate launches."""
    for c, h, o in ((64, 56, 128), (128, 28, 256), (256, 14, 512)):
        x = dev(synth.uniform((64, c, h, h), 6600 + c))
        w1 = dev(synth.normal((o, c, 3, 3), 6601 + c, float(np.sqrt(2.0 / (c * 9)))))
        b1 = dev(synth.uniform((o,), 6602 + c, -0.1, 0.1))
        w2 = dev(synth.normal((o, c, 1, 1), 6603 + c, float(np.sqrt(2.0 / c))))
        b2 = dev(synth.uniform((o,), 6604 + c, -0.1, 0.1))
        y1, y2 = pkg.conv2d_pair(x, w1, b1, None, w2, b2, 2, 1, 1, True)
        a1 = pkg.conv2d(x, w1, b1, None, 2, 1, 1, True)
        a2 = pkg.conv2d(x, w2, b2, None, 2, 0, 1, False)
        assert_close(host(y1), host(a1), tol=1e-4, what="pair vs single launch, first output, %d channels" % c)
        assert_close(host(y2), host(a2), tol=1e-4, what="pair vs single launch, second output, %d channels" % c)
        d2 = pkg.conv2d(x[5:6].contiguous(), w2, b2, None, 2, 0, 1, False, force_direct=True)
        assert_close(host(y2[5:6]), host(d2), what="second output vs the reference-order kernel, image 5")


# ------------------------------------------------------------------ Winograd F(2x2,3x3)
@pytest.mark.parametrize("shape", [(4, 64, 56, 56, 128, 3, 1), (3, 128, 28, 28, 256, 3, 1), (5, 256, 14, 14, 512, 3, 1),
                                   (2, 3, 64, 64, 64, 7, 3), (2, 8, 13, 17, 32, 3, 1), (2, 6, 12, 18, 40, 5, 2)])
def test_conv_stride2_phase_plane_layout_is_bit_identical(pkg, synth, monkeypatch, shape):
    """KXC_HIP_CONV_PHASE stages a stride-2 patch as four (row parity, column parity) planes.  Only where the patch
    sits in LDS changes, not the order of the products, so every output equals the default layout's bit for bit
    (the pair kernel's second output included); odd padded extents fall back to the default layout by themselves."""
    n, c, h, w, o, k, p = shape
    x = dev(synth.uniform((n, c, h, w), 7700))
    wt = dev(synth.normal((o, c, k, k), 7701, float(np.sqrt(2.0 / (c * k * k)))))
    b = dev(synth.uniform((o,), 7702, -0.1, 0.1))
    w2 = dev(synth.normal((o, c, 1, 1), 7703, float(np.sqrt(2.0 / c))))
    pair = k == 3 and pkg.conv2d_pair_supported((n, c, h, w), (o, c, k, k), 2, p)
    def run():
        outs = [pkg.conv2d(x, wt, b, None, 2, p, 1, True).clone()]
        if pair:
            outs += [t.clone() for t in pkg.conv2d_pair(x, wt, b, None, w2, None, 2, p, 1, True)]
        return outs
    monkeypatch.setenv("KXC_HIP_CONV_PHASE", "0")
    want = run()
    monkeypatch.setenv("KXC_HIP_CONV_PHASE", "2")
    got = run()
    assert len(got) == len(want)
    for g, t in zip(got, want):
        assert torch.equal(g, t), shape


WINOGRAD_SHAPES = [
    (2, 64, 56, 56, 64, 1),       # layer1
    (3, 128, 28, 28, 128, 1),     # layer2
    (5, 256, 14, 14, 256, 1),     # layer3: tile groups cross image boundaries
    (7, 512, 7, 7, 512, 1),       # layer4: odd output size, partial 2x2 blocks
    (1, 8, 9, 33, 40, 1),         # ragged: output channels not a multiple of 32, odd width
    (2, 12, 10, 6, 96, 0),        # no padding
    (1, 4, 5, 4, 16, 2),          # padding wider than the filter needs
    (3, 20, 1, 1, 32, 1),         # one pixel
]


@pytest.mark.parametrize("shape", WINOGRAD_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_conv_winograd_against_oracle(pkg, fast_orc, synth, shape):
    """The Winograd path of nn_conv2d (3x3, stride 1) against the CPU loop nest: fp32 tolerance, with and without
    the fused bias / residual / ReLU."""
    n, c, h, w, o, p = shape
    assert pkg.conv2d_winograd_supported((n, c, h, w), (o, c, 3, 3), 1, p)
    seed = 7000 + WINOGRAD_SHAPES.index(shape) * 5
    x = synth.uniform((n, c, h, w), seed)
    wt = synth.normal((o, c, 3, 3), seed + 1, float(np.sqrt(2.0 / (c * 9))))
    b = synth.uniform((o,), seed + 2, -0.1, 0.1)
    oh, ow = h + 2 * p - 2, w + 2 * p - 2
    skip = synth.uniform((n, o, oh, ow), seed + 3)
    u = pkg.conv2d_winograd_transform_weights((n, c, h, w), dev(wt), p)
    assert u.numel() * 4 == pkg.conv2d_winograd_weight_bytes((n, c, h, w), (o, c, 3, 3), p)
    want = fast_orc.conv_chain(x, wt, b, 1, p, skip, True)
    got = host(pkg.conv2d_winograd(dev(x), u, wt.shape, dev(b), dev(skip), p, True))
    assert_close(got, want, what="winograd %s" % (shape,))
    want = fast_orc.conv2d(x, wt, 1, p)
    got = host(pkg.conv2d_winograd(dev(x), u, wt.shape, None, None, p, False))
    assert_close(got, want, what="winograd bare %s" % (shape,))


def test_conv_winograd_exact_on_small_integers(pkg, orc):
    """Small integers keep every transformed value, product and partial sum exact (the filter transform's halves
    and quarters included), so the result must equal the direct loop nest bit for bit: isolates indexing."""
    rng = np.random.default_rng(12)
    for (n, c, h, w, o, p) in [(3, 16, 14, 14, 64, 1), (9, 8, 7, 7, 64, 1), (2, 4, 9, 12, 48, 0)]:
        x = rng.integers(-3, 4, (n, c, h, w)).astype(np.float32)
        wt = (4 * rng.integers(-2, 3, (o, c, 3, 3))).astype(np.float32)
        b = rng.integers(-5, 6, (o,)).astype(np.float32)
        want = orc.conv_chain(x, wt, b, 1, p, None, True)
        u = pkg.conv2d_winograd_transform_weights(x.shape, dev(wt), p)
        assert_bit_exact(host(pkg.conv2d_winograd(dev(x), u, wt.shape, dev(b), None, p, True)), want, str((n, c, h, w, o, p)))


@pytest.mark.parametrize("variant", ["winograd_f2k3_o2_t2_ks2", "winograd_f2k3_o2_t1_ks2", "winograd_f2k3_o2_t4", "winograd_f2k3_o1_t4",
                                     "winograd_f2k3_o1_t2", "winograd_f2k3_o2_t2"])
def test_conv_winograd_variants(pkg, fast_orc, orc, synth, monkeypatch, variant):
    """Every workgroup shape of the Winograd kernel, forced: the two-group channel split (accumulators added through
    LDS) and the larger / smaller tiles, on a ragged shape against the oracle and bit-exact on small integers."""
    monkeypatch.setenv("KXC_HIP_WINOGRAD_VARIANT", variant)
    n, c, h, w, o, p = 3, 24, 13, 10, 80, 1
    assert pkg.conv2d_winograd_variant((n, c, h, w), (o, c, 3, 3), 1, p) == variant
    x = synth.uniform((n, c, h, w), 7300)
    wt = synth.normal((o, c, 3, 3), 7301, float(np.sqrt(2.0 / (c * 9))))
    b = synth.uniform((o,), 7302, -0.1, 0.1)
    skip = synth.uniform((n, o, h, w), 7303)
    u = pkg.conv2d_winograd_transform_weights((n, c, h, w), dev(wt), p)
    got = host(pkg.conv2d_winograd(dev(x), u, wt.shape, dev(b), dev(skip), p, True))
    assert_close(got, fast_orc.conv_chain(x, wt, b, 1, p, skip, True), what=variant)
    rng = np.random.default_rng(13)
    xi = rng.integers(-3, 4, (2, 16, 9, 8)).astype(np.float32)
    wi = (4 * rng.integers(-2, 3, (64, 16, 3, 3))).astype(np.float32)
    bi = rng.integers(-5, 6, (64,)).astype(np.float32)
    ui = pkg.conv2d_winograd_transform_weights(xi.shape, dev(wi), 1)
    assert_bit_exact(host(pkg.conv2d_winograd(dev(xi), ui, wi.shape, dev(bi), None, 1, True)),
                     orc.conv_chain(xi, wi, bi, 1, 1, None, True), variant + " on small integers")


@pytest.mark.parametrize("forced", [None, "2", "3", "5"])
def test_conv_winograd_channel_split_over_workgroups(pkg, fast_orc, orc, synth, monkeypatch, forced):
    """Small launches split the input channels over workgroups (partial output transforms in a scratch buffer,
    added in order by a second kernel that applies the epilogue): batch-1 ResNet layers with the automatic split,
    a ragged shape with forced splits that leave a shorter last part, and small integers bit for bit."""
    if forced:
        monkeypatch.setenv("KXC_HIP_WINOGRAD_GSPLIT", forced)
    shapes = [(1, 512, 7, 7, 512, 1), (1, 128, 28, 28, 128, 1)] if forced is None else [(2, 44, 9, 11, 72, 1), (1, 64, 6, 5, 40, 0)]
    for (n, c, h, w, o, p) in shapes:
        x = synth.uniform((n, c, h, w), 7400)
        wt = synth.normal((o, c, 3, 3), 7401, float(np.sqrt(2.0 / (c * 9))))
        b = synth.uniform((o,), 7402, -0.1, 0.1)
        oh, ow = h + 2 * p - 2, w + 2 * p - 2
        skip = synth.uniform((n, o, oh, ow), 7403)
        assert pkg.conv2d_winograd_variant((n, c, h, w), (o, c, 3, 3), 1, p) == "winograd_f2k3_o2_t1"
        u = pkg.conv2d_winograd_transform_weights((n, c, h, w), dev(wt), p)
        got = host(pkg.conv2d_winograd(dev(x), u, wt.shape, dev(b), dev(skip), p, True))
        assert_close(got, fast_orc.conv_chain(x, wt, b, 1, p, skip, True), what="split %s %s" % (forced, (n, c, h, w, o, p)))
        got = host(pkg.conv2d_winograd(dev(x), u, wt.shape, None, None, p, False))
        assert_close(got, fast_orc.conv_chain(x, wt, None, 1, p, None, False), what="split, no epilogue")
    rng = np.random.default_rng(17)
    xi = rng.integers(-3, 4, (1, 64, 9, 8)).astype(np.float32)
    wi = (4 * rng.integers(-2, 3, (64, 64, 3, 3))).astype(np.float32)
    bi = rng.integers(-5, 6, (64,)).astype(np.float32)
    ui = pkg.conv2d_winograd_transform_weights(xi.shape, dev(wi), 1)
    assert_bit_exact(host(pkg.conv2d_winograd(dev(xi), ui, wi.shape, dev(bi), None, 1, True)),
                     orc.conv_chain(xi, wi, bi, 1, 1, None, True), "split on small integers")


@pytest.mark.parametrize("shape", [(1, 64, 56, 56, 64), (1, 128, 28, 28, 128), (1, 256, 14, 14, 256), (1, 512, 7, 7, 512), (2, 44, 9, 11, 72)])
def test_conv_winograd_last_part_finishes_the_reduction(pkg, synth, monkeypatch, shape):
    """KXC_HIP_SPLIT_FUSE_MAX lets the part that arrives last at its tile's counter add the parts and apply the
    epilogue instead of the adding kernel (off by default: measured slower).  Same order of additions, so the
    result equals the adding kernel's bit for bit -- on every one of 30 launches into an output pre-filled with NaN
    (a tile nobody finished, or one finished before all parts were visible, would show), with the counters left at
    zero for the next launch."""
    n, c, h, w, o = shape
    x = dev(synth.uniform((n, c, h, w), 7500))
    wt = dev(synth.normal((o, c, 3, 3), 7501, float(np.sqrt(2.0 / (c * 9)))))
    b = dev(synth.uniform((o,), 7502, -0.1, 0.1))
    skip = dev(synth.uniform((n, o, h, w), 7503))
    if n == 2:
        monkeypatch.setenv("KXC_HIP_WINOGRAD_GSPLIT", "3")
    u = pkg.conv2d_winograd_transform_weights((n, c, h, w), wt, 1)
    monkeypatch.setenv("KXC_HIP_SPLIT_FUSE_MAX", "0")
    want = pkg.conv2d_winograd(x, u, wt.shape, b, skip, 1, True).clone()
    want_plain = pkg.conv2d_winograd(x, u, wt.shape, None, None, 1, False).clone()
    monkeypatch.setenv("KXC_HIP_SPLIT_FUSE_MAX", "32")
    out = torch.empty_like(want)
    for it in range(30):
        out.fill_(float("nan"))
        got = pkg.conv2d_winograd(x, u, wt.shape, b, skip, 1, True, out=out)
        assert torch.equal(got, want), "launch %d of %s" % (it, shape)
    out.fill_(float("nan"))
    assert torch.equal(pkg.conv2d_winograd(x, u, wt.shape, None, None, 1, False, out=out), want_plain)


def test_split_reduction_from_two_host_threads(pkg, synth):
    """Two host threads enqueue split convolutions (parts + adding kernel, sharing the stream's scratch buffer) on
    the same stream at the same time: the pair of launches of one call is never interleaved with another call's,
    so every result equals the single-threaded one."""
    import threading
    shapes = [(1, 512, 7, 7, 512), (1, 128, 28, 28, 128)]
    cases = []
    for i, (n, c, h, w, o) in enumerate(shapes):
        x = dev(synth.uniform((n, c, h, w), 7600 + i))
        wt = dev(synth.normal((o, c, 3, 3), 7610 + i, float(np.sqrt(2.0 / (c * 9)))))
        u = pkg.conv2d_winograd_transform_weights((n, c, h, w), wt, 1)
        want_w = pkg.conv2d_winograd(x, u, wt.shape, None, None, 1, True).clone()
        want_g = pkg.conv2d(x, wt, None, None, 1, 1, 1, True).clone()
        cases.append((x, wt, u, want_w, want_g))
    torch.cuda.synchronize()
    stream = torch.cuda.current_stream()
    errors = []

    def worker(idx):
        x, wt, u, want_w, want_g = cases[idx]
        with torch.cuda.stream(stream):
            for it in range(40):
                got_w = pkg.conv2d_winograd(x, u, wt.shape, None, None, 1, True)
                got_g = pkg.conv2d(x, wt, None, None, 1, 1, 1, True)
                if it % 10 == 9:
                    stream.synchronize()
                    if not (torch.equal(got_w, want_w) and torch.equal(got_g, want_g)):
                        errors.append((idx, it))

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    assert not errors, errors


def test_conv_winograd_random_shapes_against_direct_kernel(pkg):
    """Seeded random geometries (batch, channels, height, width, output channels, padding; every epilogue mix):
    the Winograd kernel against the reference-order direct kernel on the same GPU tensors."""
    rng = np.random.default_rng(20240601)
    for case in range(24):
        n = int(rng.integers(1, 6)); c = 4 * int(rng.integers(1, 24)); o = int(rng.integers(1, 150))
        h = int(rng.integers(1, 40)); w = int(rng.integers(1, 40)); p = int(rng.integers(0, 3))
        if h + 2 * p < 3 or w + 2 * p < 3:
            continue
        x = torch.from_numpy(rng.uniform(-1, 1, (n, c, h, w)).astype(np.float32)).cuda()
        wt = torch.from_numpy((rng.standard_normal((o, c, 3, 3)) * np.sqrt(2.0 / (9 * c))).astype(np.float32)).cuda()
        b = torch.from_numpy(rng.uniform(-0.1, 0.1, (o,)).astype(np.float32)).cuda() if case % 2 == 0 else None
        oh, ow = h + 2 * p - 2, w + 2 * p - 2
        r = torch.from_numpy(rng.uniform(-1, 1, (n, o, oh, ow)).astype(np.float32)).cuda() if case % 3 == 0 else None
        relu = case % 4 != 3
        u = pkg.conv2d_winograd_transform_weights(x.shape, wt, p)
        got = pkg.conv2d_winograd(x, u, wt.shape, b, r, p, relu)
        want = pkg.conv2d(x, wt, b, r, 1, p, 1, relu, force_direct=True)
        assert_close(host(got), host(want), what="case %d: n=%d c=%d h=%d w=%d o=%d p=%d" % (case, n, c, h, w, o, p))


def test_conv_random_shapes_against_direct_kernel(pkg):
    """Seeded random geometries over every filter size the matrix-core kernels take (1x1, 3x3, 7x7; strides 1-3,
    paddings 0-3, dilations 1-2; ragged channel, output-channel and pixel counts; every epilogue mix): whatever
    kernel the library selects -- tiled, split over wave groups or workgroups, the small-launch 1x1 kernel --
    against the reference-order direct kernel on the same GPU tensors."""
    rng = np.random.default_rng(20240707)
    seen = set()
    for case in range(60):
        k = int(rng.choice([1, 1, 3, 3, 3, 7]))
        n = int(rng.integers(1, 5)); c = int(rng.choice([3, 8, 16, 24, 40, 64, 96, 128, 200, 256])); o = int(rng.integers(8, 200))
        h = int(rng.integers(4, 40)); w = int(rng.integers(4, 40))
        stride = int(rng.integers(1, 4)); p = int(rng.integers(0, 4)); dil = int(rng.integers(1, 3)) if k == 3 else 1
        if k == 1:
            p = int(rng.choice([0, 0, 1]))
        if h + 2 * p < dil * (k - 1) + 1 or w + 2 * p < dil * (k - 1) + 1:
            continue
        x = torch.from_numpy(rng.uniform(-1, 1, (n, c, h, w)).astype(np.float32)).cuda()
        wt = torch.from_numpy((rng.standard_normal((o, c, k, k)) * np.sqrt(2.0 / (k * k * c))).astype(np.float32)).cuda()
        b = torch.from_numpy(rng.uniform(-0.1, 0.1, (o,)).astype(np.float32)).cuda() if case % 2 == 0 else None
        oh = (h + 2 * p - (dil * (k - 1) + 1)) // stride + 1; ow = (w + 2 * p - (dil * (k - 1) + 1)) // stride + 1
        r = torch.from_numpy(rng.uniform(-1, 1, (n, o, oh, ow)).astype(np.float32)).cuda() if case % 3 == 0 else None
        relu = case % 4 != 3
        seen.add(pkg.conv2d_variant((n, c, h, w), (o, c, k, k), stride, p, dil))
        got = pkg.conv2d(x, wt, b, r, stride, p, dil, relu)
        want = pkg.conv2d(x, wt, b, r, stride, p, dil, relu, force_direct=True)
        assert_close(host(got), host(want), what="case %d: k=%d n=%d c=%d h=%d w=%d o=%d s=%d p=%d d=%d" % (case, k, n, c, h, w, o, stride, p, dil))
    assert "mfma_k1x1_small" in seen and any(v.startswith("mfma_k3x3") for v in seen) and any(v.startswith("mfma_k7x7") for v in seen), seen


def test_conv_pair_random_shapes_against_direct_kernel(pkg):
    """Seeded random geometries for the two-output kernel (3x3 filters, strides 1-3, padding 1 (0 and 2 are refused: the outputs' extents would differ), ragged channel,
    output-channel and pixel counts, with and without either bias, residual and ReLU on the main output): both
    outputs against the reference-order direct kernel run twice on the same GPU tensors."""
    rng = np.random.default_rng(20250101)
    ran = 0
    for case in range(90):
        n = int(rng.integers(1, 6)); c = int(rng.choice([4, 8, 16, 24, 40, 64, 96, 128])); o = int(rng.choice([32, 40, 64, 96, 128, 200]))
        h = int(rng.integers(5, 34)); w = int(rng.integers(5, 34)); stride = int(rng.integers(1, 4)); p = int(rng.choice([0, 1, 1, 1, 1, 2]))
        if p != 1:
            assert not pkg.conv2d_pair_supported((n, c, h, w), (o, c, 3, 3), stride, p)      # the two outputs would differ in extent
        if h + 2 * p < 3 or w + 2 * p < 3 or not pkg.conv2d_pair_supported((n, c, h, w), (o, c, 3, 3), stride, p):
            continue
        ran += 1
        x = torch.from_numpy(rng.uniform(-1, 1, (n, c, h, w)).astype(np.float32)).cuda()
        wt = torch.from_numpy((rng.standard_normal((o, c, 3, 3)) * np.sqrt(2.0 / (9 * c))).astype(np.float32)).cuda()
        w2 = torch.from_numpy((rng.standard_normal((o, c, 1, 1)) * np.sqrt(2.0 / c)).astype(np.float32)).cuda()
        b = torch.from_numpy(rng.uniform(-0.1, 0.1, (o,)).astype(np.float32)).cuda() if case % 2 == 0 else None
        b2 = torch.from_numpy(rng.uniform(-0.1, 0.1, (o,)).astype(np.float32)).cuda() if case % 3 != 0 else None
        oh = (h + 2 * p - 3) // stride + 1; ow = (w + 2 * p - 3) // stride + 1
        r = torch.from_numpy(rng.uniform(-1, 1, (n, o, oh, ow)).astype(np.float32)).cuda() if case % 4 == 0 else None
        relu = case % 5 != 4
        # the 1x1 convolution reads x[oh*stride + p - p, ...]: same strides, no padding, on the window's tap (p, p)
        y, y2 = pkg.conv2d_pair(x, wt, b, r, w2, b2, stride, p, 1, relu)
        want = pkg.conv2d(x, wt, b, r, stride, p, 1, relu, force_direct=True)
        xs = x[:, :, 0:(oh - 1) * stride + 1:stride, 0:(ow - 1) * stride + 1:stride].contiguous()
        want2 = pkg.conv2d(xs, w2, b2, None, 1, 0, 1, False, force_direct=True)
        what = "case %d: n=%d c=%d h=%d w=%d o=%d s=%d p=%d" % (case, n, c, h, w, o, stride, p)
        assert_close(host(y), host(want), what=what + " (main)")
        assert_close(host(y2), host(want2), what=what + " (second)")
    assert ran >= 20, ran


def test_conv_winograd_unsupported_shapes_are_refused(pkg):
    assert not pkg.conv2d_winograd_supported((1, 8, 8, 8), (16, 8, 3, 3), 2, 1)        # stride
    assert not pkg.conv2d_winograd_supported((1, 8, 8, 8), (16, 8, 1, 1), 1, 0)        # filter size
    assert not pkg.conv2d_winograd_supported((1, 6, 8, 8), (16, 6, 3, 3), 1, 1)        # channels not a multiple of 4
    assert not pkg.conv2d_winograd_supported((1, 8, 8, 8), (16, 8, 3, 3), 1, 1, 2)     # dilation
    assert pkg.conv2d_winograd_preferred((1, 512, 7, 7), (512, 512, 3, 3))             # small launches split their channels
    os.environ["KXC_HIP_WINOGRAD_MIN_WORK"] = "512"
    try:
        assert not pkg.conv2d_winograd_preferred((1, 512, 7, 7), (512, 512, 3, 3))     # 16 blocks * 512 < 512 * 512
    finally:
        del os.environ["KXC_HIP_WINOGRAD_MIN_WORK"]
    assert pkg.conv2d_winograd_variant((1, 64, 56, 56), (64, 64, 3, 3)).endswith("_t1")  # small launches: smaller groups
    assert pkg.conv2d_winograd_preferred((64, 64, 56, 56), (64, 64, 3, 3))
    x = torch.zeros((1, 6, 8, 8), device="cuda"); u = torch.zeros((1024,), device="cuda")
    with pytest.raises(pkg.KxcHipError):
        pkg.conv2d_winograd(x, u, (16, 6, 3, 3))


def test_conv_winograd_full_batch_properties(pkg, synth):
    """Full-size layers (batch 64): Winograd vs the implicit-GEMM kernel on the GPU, linearity in the weights
    and batch independence."""
    for (c, hw, o) in [(64, 56, 64), (512, 7, 512)]:
        x = dev(synth.uniform((64, c, hw, hw), 7100))
        w1 = dev(synth.normal((o, c, 3, 3), 7101, float(np.sqrt(2.0 / (9 * c)))))
        w2 = dev(synth.normal((o, c, 3, 3), 7102, float(np.sqrt(2.0 / (9 * c)))))
        b = dev(synth.uniform((o,), 7103, -0.1, 0.1))
        u1 = pkg.conv2d_winograd_transform_weights(x.shape, w1); u2 = pkg.conv2d_winograd_transform_weights(x.shape, w2)
        u12 = pkg.conv2d_winograd_transform_weights(x.shape, w1 + w2)
        fast = pkg.conv2d_winograd(x, u1, w1.shape, b, None, 1, True)
        other = pkg.conv2d(x, w1, b, None, 1, 1, 1, True)
        assert_close(host(fast), host(other), what="winograd vs implicit GEMM, batch 64")
        y12 = pkg.conv2d_winograd(x, u12, w1.shape); y1 = pkg.conv2d_winograd(x, u1, w1.shape); y2 = pkg.conv2d_winograd(x, u2, w1.shape)
        assert_close(host(y12), host(y1 + y2), what="linearity")
        one = pkg.conv2d_winograd(x[17:18].contiguous(), u1, w1.shape, b, None, 1, True)
        assert_close(host(one), host(fast[17:18]), tol=1e-4, what="batch independence")


def test_plan_winograd_node_constants(pkg, synth, fast_orc):
    """A plan's Winograd node takes the OIHW weights as a packed argument.  By default every run transforms them
    again (one launch per plan), so weights rewritten in place at the same address are seen, as the CPU backend
    would see them; with frozen constants they are transformed when a pointer is first seen, an in-place update
    needs invalidate_constants, and a run on another stream is ordered after the transform.  The serialised plan
    keeps the node."""
    n, c, h, o = 4, 16, 12, 64
    x = synth.uniform((n, c, h, h), 7200)
    w1 = synth.normal((o, c, 3, 3), 7201, 0.1); w2 = synth.normal((o, c, 3, 3), 7202, 0.1)
    b = synth.uniform((o,), 7203, -0.1, 0.1)
    d = pkg.ConvDesc(n, c, h, h, o, 3, 3, 1, 1, 1, 1, 1, 1, pkg.CONV_BIAS | pkg.CONV_RELU)
    ubytes = pkg.conv2d_winograd_weight_bytes((n, c, h, h), (o, c, 3, 3))
    plan = pkg.Plan(4)
    plan.add_conv2d_winograd(d, pkg.Buf.arg(0), pkg.Buf.arg(1), pkg.Buf.arg(2), pkg.Buf.none(), pkg.Buf.arg(3), pkg.Buf.ws(0))
    plan.finalize(ubytes)
    assert "winograd" in plan.node_symbol(0)
    xd, w1d, w2d, bd = dev(x), dev(w1), dev(w2), dev(b)
    y = torch.empty((n, o, h, h), device="cuda")
    want1 = fast_orc.conv_chain(x, w1, b, 1, 1, None, True)
    want2 = fast_orc.conv_chain(x, w2, b, 1, 1, None, True)
    for wd, want in ((w1d, want1), (w1d, want1), (w2d, want2)):
        plan.run([xd, wd, bd, y]); torch.cuda.synchronize()
        assert_close(host(y), want, what="plan winograd")
    # default: rewritten in place at the same pointer, nothing said -- the next run uses the new contents
    w2d.copy_(w1d)
    plan.run([xd, w2d, bd, y]); torch.cuda.synchronize()
    assert_close(host(y), want1, what="plan winograd after an in-place update")
    # the same through a captured graph: the transform is part of the replay
    stream = torch.cuda.Stream()
    plan.enable_graph(True)
    with torch.cuda.stream(stream):
        for k, (src, want) in enumerate(((w2, want2), (w2, want2), (w1, want1), (w2, want2))):
            w2d.copy_(dev(src)); y.zero_()
            plan.run([xd, w2d, bd, y], stream.cuda_stream); stream.synchronize()
            assert_close(host(y), want, what="graph replay %d sees the current weights" % k)
    plan.enable_graph(False)
    # frozen: transformed once per pointer
    plan.freeze_constants(True)
    w2d.copy_(dev(w2))
    plan.run([xd, w2d, bd, y]); torch.cuda.synchronize()
    assert_close(host(y), want2, what="frozen: first run transforms")
    w2d.copy_(w1d)                                        # behind the plan's back: stale by contract
    plan.run([xd, w2d, bd, y]); torch.cuda.synchronize()
    assert_close(host(y), want2, what="frozen: an unannounced in-place update is not seen")
    plan.invalidate_constants()
    other = torch.cuda.Stream()
    with torch.cuda.stream(other):                        # transform enqueued on this stream ...
        plan.run([xd, w2d, bd, y], other.cuda_stream)
    y2 = torch.empty_like(y)
    plan.run([xd, w2d, bd, y2])                           # ... and a run on another stream waits for it
    torch.cuda.synchronize()
    assert_close(host(y), want1, what="frozen: after invalidate")
    assert_bit_exact(host(y2), host(y), "frozen: run on a second stream after the transform")
    again = pkg.Plan.deserialize(plan.serialize(), 0)
    y3 = torch.empty_like(y)
    again.run([xd, w1d, bd, y3]); torch.cuda.synchronize()
    assert_bit_exact(host(y3), host(y), "deserialised winograd plan")


@pytest.mark.parametrize("shape", [(1, 64, 56, 56, 128, 2), (1, 256, 14, 14, 512, 2), (2, 8, 5, 7, 40, 1), (3, 24, 9, 6, 33, 2),
                                   (1, 40, 7, 7, 100, 3), (2, 272, 6, 6, 48, 1)], ids=lambda s: "x".join(map(str, s)))
def test_conv1x1_small_launch_kernel(pkg, fast_orc, orc, synth, shape):
    """Unpadded 1x1 filters on small launches (the downsample convolutions at batch 1-16) take a kernel of their
    own: four or eight waves split the input channels and feed the matrix cores straight from memory.  Channel
    counts that leave a short last batch of loads, output channels and pixels that do not fill a 32 x 32 tile,
    strides 1-3, every epilogue mix."""
    n, c, h, w, o, stride = shape
    assert pkg.conv2d_variant((n, c, h, w), (o, c, 1, 1), stride, 0) == "mfma_k1x1_small"
    x = synth.uniform((n, c, h, w), 7500)
    wt = synth.normal((o, c, 1, 1), 7501, float(np.sqrt(2.0 / c)))
    b = synth.uniform((o,), 7502, -0.1, 0.1)
    oh, ow = (h - 1) // stride + 1, (w - 1) // stride + 1
    skip = synth.uniform((n, o, oh, ow), 7503)
    for (bias, res, relu) in [(b, None, False), (b, skip, True), (None, None, True), (None, skip, False)]:
        got = host(pkg.conv2d(dev(x), dev(wt), None if bias is None else dev(bias), None if res is None else dev(res),
                              stride, 0, 1, relu))
        assert_close(got, fast_orc.conv_chain(x, wt, bias, stride, 0, res, relu), what="1x1 small %s" % (shape,))
    rng = np.random.default_rng(19)
    xi = rng.integers(-3, 4, (n, c, h, w)).astype(np.float32)
    wi = rng.integers(-2, 3, (o, c, 1, 1)).astype(np.float32)
    assert_bit_exact(host(pkg.conv2d(dev(xi), dev(wi), None, None, stride, 0, 1, False)),
                     orc.conv_chain(xi, wi, None, stride, 0, None, False), "1x1 small on small integers")


def test_conv_dilation(pkg, orc, synth):
    x = synth.uniform((1, 8, 20, 20), 300); w = synth.uniform((32, 8, 3, 3), 301)
    want = orc.conv2d(x, w, 1, 2, 2)
    assert_bit_exact(host(pkg.conv2d(dev(x), dev(w), stride=1, pad=2, dil=2, force_direct=True)), want, "dilated direct")
    assert_close(host(pkg.conv2d(dev(x), dev(w), stride=1, pad=2, dil=2)), want, what="dilated")


def test_conv_exact_on_small_integers(pkg, orc):
    """Small-integer data makes every product and partial sum exact, so any summation order must
    give identical bits: isolates indexing mistakes from rounding."""
    rng = np.random.default_rng(11)
    for (n, c, h, w, o, k, s, p) in [(3, 16, 14, 14, 64, 3, 1, 1), (2, 16, 15, 15, 32, 3, 2, 1), (9, 8, 7, 7, 64, 3, 1, 1),
                                     (2, 3, 40, 40, 64, 7, 2, 3), (2, 16, 14, 14, 64, 1, 2, 0)]:
        x = rng.integers(-3, 4, (n, c, h, w)).astype(np.float32)
        wt = rng.integers(-2, 3, (o, c, k, k)).astype(np.float32)
        b = rng.integers(-5, 6, (o,)).astype(np.float32)
        want = orc.conv_chain(x, wt, b, s, p, None, True)
        assert pkg.conv2d_variant(x.shape, wt.shape, s, p).startswith("mfma")
        assert_bit_exact(host(pkg.conv2d(dev(x), dev(wt), dev(b), None, s, p, 1, True)), want, str((n, c, h, w, o, k, s, p)))


def test_conv_full_batch_properties(pkg, synth):
    """Full-size layer (batch 64): matrix-core kernel vs the bit-exact direct kernel on the GPU,
    plus linearity in the weights and batch independence."""
    x = dev(synth.uniform((64, 64, 56, 56), 4100))
    w1 = dev(synth.normal((64, 64, 3, 3), 4101, float(np.sqrt(2.0 / 576))))
    w2 = dev(synth.normal((64, 64, 3, 3), 4102, float(np.sqrt(2.0 / 576))))
    b = dev(synth.uniform((64,), 4103, -0.1, 0.1))
    fast = pkg.conv2d(x, w1, b, None, 1, 1, 1, True)
    slow = pkg.conv2d(x, w1, b, None, 1, 1, 1, True, force_direct=True)
    assert_close(host(fast), host(slow), what="layer1 batch 64")
    y12 = pkg.conv2d(x, w1 + w2, None, None, 1, 1)
    y1 = pkg.conv2d(x, w1, None, None, 1, 1); y2 = pkg.conv2d(x, w2, None, None, 1, 1)
    assert_close(host(y12), host(y1 + y2), what="linearity")
    one = pkg.conv2d(x[17:18].contiguous(), w1, b, None, 1, 1, 1, True)
    assert_close(host(one), host(fast[17:18]), tol=1e-4, what="batch independence")


# ------------------------------------------------------------------ pooling / elementwise at full sizes
def test_maxpool_full_size_bit_exact(pkg, fast_orc, synth):
    x = synth.uniform((64, 64, 112, 112), 2000)
    xd = dev(x)
    got = pkg.pool2d(xd, 3, 2, 1)
    # the CPU checker on four images (first, last, two in between), bit for bit
    for n in (0, 21, 42, 63):
        assert_bit_exact(host(got[n:n + 1]), fast_orc.pool2d(x[n:n + 1], 3, 2, 1), "maxpool image %d" % n)
    # every image against torch's max pool (exact for inputs above -1e30)
    want = torch.nn.functional.max_pool2d(xd, 3, 2, 1)
    assert torch.equal(got, want)
    # small launches take one output row per thread instead of four: a batch-1 map and a ragged small one
    for i, shape in enumerate([(1, 64, 112, 112), (2, 3, 14, 24), (1, 5, 2, 8)]):
        xs = synth.uniform(shape, 2040 + i)
        assert_bit_exact(host(pkg.pool2d(dev(xs), 3, 2, 1)), fast_orc.pool2d(xs, 3, 2, 1), "maxpool %s" % (shape,))
    # idempotence-like property: pooling a constant plane returns the constant
    c = torch.full((2, 3, 16, 16), -7.5, device="cuda")
    assert torch.equal(pkg.pool2d(c, 3, 2, 1), torch.full((2, 3, 8, 8), -7.5, device="cuda"))


def test_pool_random_shapes_against_oracle(pkg, fast_orc):
    """Seeded random pooling geometries (window 1-4, stride 1-3, padding below the window) through the generic
    kernel, and 3x3/2/1 maps of every size class through the row-reusing kernel: max bit for bit against the CPU
    checker, average within the fp32 tolerance."""
    rng = np.random.default_rng(20240808)
    for case in range(24):
        k = int(rng.integers(1, 5)); s_ = int(rng.integers(1, 4)); p = int(rng.integers(0, (k + 1) // 2 + 1))
        p = min(p, k - 1) if k > 1 else 0
        n = int(rng.integers(1, 4)); c = int(rng.integers(1, 20)); h = int(rng.integers(k, 30)); w = int(rng.integers(k, 30))
        x = rng.uniform(-1, 1, (n, c, h, w)).astype(np.float32)
        what = "case %d: k=%d s=%d p=%d shape=%s" % (case, k, s_, p, (n, c, h, w))
        assert_bit_exact(host(pkg.pool2d(dev(x), k, s_, p)), fast_orc.pool2d(x, k, s_, p), what)
        assert_close(host(pkg.pool2d(dev(x), k, s_, p, avg=True)), fast_orc.pool2d(x, k, s_, p, avg=True), what=what + " avg")
    for shape in [(1, 3, 8, 8), (2, 5, 6, 16), (1, 64, 56, 56), (3, 7, 30, 24), (4, 64, 112, 112), (9, 128, 28, 32)]:
        x = rng.uniform(-1, 1, shape).astype(np.float32)
        assert_bit_exact(host(pkg.pool2d(dev(x), 3, 2, 1)), fast_orc.pool2d(x, 3, 2, 1), "3x3/2 %s" % (shape,))


def test_maxpool_edge_semantics(pkg, orc):
    x = np.full((1, 1, 8, 8), -3e30, np.float32)            # below the -1e30 pad candidate
    assert_bit_exact(host(pkg.pool2d(dev(x), 3, 2, 1)), orc.pool2d(x, 3, 2, 1), "pad candidate")
    rng = np.random.default_rng(12)
    x = rng.standard_normal((2, 3, 16, 24)).astype(np.float32)
    x[0, 0, 3, 5] = np.nan; x[1, 2, 0, 0] = np.nan; x[0, 1, 15, 23] = np.nan; x[1, 1, 7, 8] = -0.0
    assert_bit_exact(host(pkg.pool2d(dev(x), 3, 2, 1)), orc.pool2d(x, 3, 2, 1), "NaN select chain (fast kernel)")
    x = rng.standard_normal((2, 3, 9, 11)).astype(np.float32); x[0, 0, 4, 4] = np.nan
    for k, s, p in [(3, 2, 1), (2, 2, 0), (3, 1, 1), (5, 3, 2)]:
        assert_bit_exact(host(pkg.pool2d(dev(x), k, s, p)), orc.pool2d(x, k, s, p), "generic %s" % ((k, s, p),))
        assert_bit_exact(host(pkg.pool2d(dev(x), k, s, p, avg=True)), orc.pool2d(x, k, s, p, avg=True), "avg")


def test_column_maxpool_bit_exact(pkg, fast_orc, orc, synth):
    """The 3x1 window with stride (2,1) that finishes a 3x3/2 max pool whose column maxima were taken by the
    convolution before it: bit for bit against the CPU checker, on the first layer's half-width map (four rows per
    thread), small maps (one row per thread), odd heights, and values below the -1e30 pad candidate."""
    x = synth.uniform((4, 64, 112, 56), 2100)
    assert_bit_exact(host(pkg.pool2d(dev(x), (3, 1), (2, 1), (1, 0, 1, 0))), fast_orc.pool2d(x, (3, 1), (2, 1), (1, 0, 1, 0)), "column pool")
    for i, shape in enumerate([(1, 64, 112, 56), (2, 3, 14, 24), (1, 5, 7, 8), (3, 2, 9, 4), (1, 1, 2, 4)]):
        xs = synth.uniform(shape, 2110 + i)
        for pad in ((1, 0, 1, 0), (1, 0, 0, 0)):
            assert_bit_exact(host(pkg.pool2d(dev(xs), (3, 1), (2, 1), pad)), fast_orc.pool2d(xs, (3, 1), (2, 1), pad), "column pool %s %s" % (shape, pad))
    x = np.full((1, 2, 8, 8), -3e30, np.float32)
    x[0, 1, 3, 2] = np.nan
    assert_bit_exact(host(pkg.pool2d(dev(x), (3, 1), (2, 1), (1, 0, 1, 0))), orc.pool2d(x, (3, 1), (2, 1), (1, 0, 1, 0)), "pad candidate, NaN")
    # a width that is not a multiple of four takes the generic kernel
    xs = synth.uniform((2, 3, 10, 6), 2130)
    assert_bit_exact(host(pkg.pool2d(dev(xs), (3, 1), (2, 1), (1, 0, 1, 0))), fast_orc.pool2d(xs, (3, 1), (2, 1), (1, 0, 1, 0)), "generic")


HPOOL_SHAPES = [(2, 3, 224, 224, 64, 7, 2, 3), (2, 3, 112, 112, 48, 7, 2, 3), (7, 3, 64, 64, 64, 7, 2, 3), (1, 5, 31, 56, 80, 7, 2, 3)]


@pytest.mark.parametrize("shape", HPOOL_SHAPES, ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("variant", ["mfma_k7x7_t1_o2x1_p2x7", "mfma_k7x7_t1_o1x2_p7x1"])
def test_conv_with_column_maxima_in_the_epilogue(pkg, fast_orc, synth, monkeypatch, shape, variant):
    """KXC_HIP_CONV_HPOOL: conv -> bias -> relu with the maximum over the three columns of every 3x3/2 pooling window
    taken in the convolution's epilogue, then the 3x1 column pool: against the CPU checker's
    pool2d(relu(conv2d + bias)) within the matrix-core tolerance, and bit for bit against the same kernel family
    without the epilogue followed by the 3x3 pool (the maximum is exact, so only the convolution's rounding is in
    play and that is the same in both).  Both tiles that have the epilogue."""
    n, c, h, w, o, k, s, p = shape
    monkeypatch.setenv("KXC_HIP_CONV_HPOOL_VARIANT", variant)
    if not pkg.conv2d_hpool_supported((n, c, h, w), (o, c, k, k), s, p):
        pytest.skip("tile %s does not cover %s" % (variant, shape,))
    flags = pkg.CONV_BIAS | pkg.CONV_RELU | pkg.CONV_HPOOL
    assert pkg.conv2d_variant((n, c, h, w), (o, c, k, k), s, p, 1, flags) == variant
    seed = 2200 + HPOOL_SHAPES.index(shape) * 5
    x = synth.uniform((n, c, h, w), seed)
    wt = synth.normal((o, c, k, k), seed + 1, float(np.sqrt(2.0 / (c * k * k))))
    b = synth.uniform((o,), seed + 2, -0.1, 0.1)
    half = pkg.conv2d(dev(x), dev(wt), dev(b), None, s, p, 1, True, hpool=True)
    oh, ow = (h + 2 * p - k) // s + 1, (w + 2 * p - k) // s + 1
    assert tuple(half.shape) == (n, o, oh, ow // 2)
    got = pkg.pool2d(half, (3, 1), (2, 1), (1, 0, 1, 0))
    want = fast_orc.pool2d(fast_orc.conv_chain(x, wt, b, s, p, None, True), 3, 2, 1)
    assert_close(host(got), want, what=variant)
    # the same tile without the epilogue, then the whole 3x3 window (a 64-channel tile is not taken for fewer channels)
    if o < 64:
        return
    monkeypatch.setenv("KXC_HIP_CONV_VARIANT", variant)
    monkeypatch.setenv("KXC_HIP_CONV_GSPLIT", "1")        # (a small unpooled launch would split its reduction over workgroups)
    assert pkg.conv2d_variant((n, c, h, w), (o, c, k, k), s, p) == variant
    full = pkg.conv2d(dev(x), dev(wt), dev(b), None, s, p, 1, True)
    assert torch.equal(half, torch.nn.functional.max_pool2d(full, (1, 3), (1, 2), (0, 1)))
    assert torch.equal(got, pkg.pool2d(full, 3, 2, 1))


def test_conv_column_maxima_refusals_and_full_batch(pkg, synth):
    """Shapes the epilogue does not cover are reported and refused; at the benchmark's batch the two launches equal
    convolution + 3x3 pool bit for bit on every image (first-layer shape, both shares' batch)."""
    w7 = (64, 3, 7, 7)
    assert pkg.conv2d_hpool_supported((64, 3, 224, 224), w7, 2, 3)
    assert pkg.conv2d_hpool_supported((64, 3, 224, 224), w7, 2, 3, preferred=True)
    assert not pkg.conv2d_hpool_supported((2, 3, 224, 224), w7, 2, 3, preferred=True)       # too few tiles to pay
    assert not pkg.conv2d_hpool_supported((1, 3, 64, 64), w7, 2, 3)                          # 1024 pixels: not whole tiles
    assert not pkg.conv2d_hpool_supported((2, 3, 222, 222), w7, 2, 3)                        # 111 columns: odd
    assert not pkg.conv2d_hpool_supported((2, 3, 224, 224), (60, 3, 7, 7), 2, 3)             # channels are masked eight at a time
    assert not pkg.conv2d_hpool_supported((2, 64, 56, 56), (64, 64, 3, 3), 1, 1)             # no 3x3 kernel has it
    assert not pkg.conv2d_hpool_supported((2, 3, 224, 224), w7, 2, 3, flags=pkg.CONV_BIAS)   # needs the ReLU
    assert not pkg.conv2d_hpool_supported((2, 3, 224, 224), w7, 2, 3, flags=pkg.CONV_BIAS | pkg.CONV_RELU | pkg.CONV_RESIDUAL)
    x = dev(synth.uniform((1, 3, 64, 64), 2300)); w = dev(synth.normal(w7, 2301, 0.1)); b = dev(synth.uniform((64,), 2302))
    with pytest.raises(pkg.KxcHipError, match="pooling epilogue"):
        pkg.conv2d(x, w, b, None, 2, 3, 1, True, hpool=True)
    with pytest.raises(pkg.KxcHipError, match="pooling epilogue"):
        pkg.conv2d(dev(synth.uniform((2, 3, 224, 224), 2303)), w, b, None, 2, 3, 1, False, hpool=True)
    for batch in (32, 64):
        xb = dev(synth.uniform((batch, 3, 224, 224), 2310 + batch))
        got = pkg.pool2d(pkg.conv2d(xb, w, b, None, 2, 3, 1, True, hpool=True), (3, 1), (2, 1), (1, 0, 1, 0))
        want = pkg.pool2d(pkg.conv2d(xb, w, b, None, 2, 3, 1, True), 3, 2, 1)
        assert torch.equal(got, want)
        del got, want, xb


def test_add_relu_full_size(pkg, fast_orc, synth):
    a = synth.uniform((64, 128, 28, 28), 2010); b = synth.uniform((64, 128, 28, 28), 2011)
    got = host(pkg.binary(0, dev(a), dev(b), relu=True))
    assert_bit_exact(got, fast_orc.relu(fast_orc.add(a, b)), "add+relu")
    x = np.array([np.nan, -0.0, 0.0, -1.0, 2.0, np.inf, -np.inf, 5.0], np.float32)
    assert_bit_exact(host(pkg.relu(dev(x))), fast_orc.relu(x), "relu specials")
    assert_bit_exact(host(pkg.relu(dev(x)[1:])), fast_orc.relu(x[1:]), "relu unaligned")   # 4-byte aligned view


def test_broadcast_binary_random_shapes(pkg):
    """add / subtract / multiply / divide over seeded random right-aligned broadcast shapes (size-1 and missing
    leading dimensions on either side, lengths that leave a vector tail), with and without the fused ReLU: one
    rounded fp32 operation per element, so bit for bit against numpy."""
    rng = np.random.default_rng(20240909)
    ops = [np.add, np.subtract, np.multiply, np.divide]
    for case in range(40):
        nd = int(rng.integers(1, 5))
        full = [int(rng.integers(1, 9)) for _ in range(nd)]
        sa = [d if rng.random() < 0.7 else 1 for d in full][int(rng.integers(0, nd)):]
        sb = [d if rng.random() < 0.7 else 1 for d in full][int(rng.integers(0, nd)):]
        if case % 5 == 0:                       # same shape, long enough for the vector kernel and its tail
            sa = sb = [int(rng.integers(1, 4)), int(rng.integers(1000, 5000))]
        a = rng.uniform(-2, 2, sa).astype(np.float32); b = rng.uniform(0.5, 2, sb).astype(np.float32) * rng.choice([-1, 1], sb).astype(np.float32)
        op = case % 4; relu = case % 3 == 0
        want = ops[op](a, b).astype(np.float32)
        if relu:
            want = np.where(want > 0, want, np.float32(0))
        got = host(pkg.binary(op, dev(a), dev(b), relu=relu))
        assert got.shape == want.shape, (case, sa, sb)
        assert_bit_exact(got, want, "case %d: op %d %s %s relu=%s" % (case, op, sa, sb, relu))


def test_gap_full_size(pkg, fast_orc, synth):
    x = synth.uniform((64, 512, 7, 7), 2020)
    assert_bit_exact(host(pkg.global_avg_pool2d(dev(x))), fast_orc.gap(x), "gap 7x7")
    x = synth.uniform((3, 5, 2, 2), 2021)
    assert_bit_exact(host(pkg.global_avg_pool2d(dev(x))), fast_orc.gap(x), "gap 2x2")
    x = synth.uniform((2, 3, 40, 40), 2022)            # large plane: wave reduction, different order
    assert_close(host(pkg.global_avg_pool2d(dev(x))), fast_orc.gap(x), what="gap 40x40")
    # the staged kernel's limits: plane counts that do not fill a workgroup, planes of 1 and of 128 elements
    for i, shape in enumerate([(1, 17, 1, 1), (3, 11, 8, 16), (1, 33, 9, 14), (2, 16, 1, 127), (1, 5, 2, 64)]):
        x = synth.uniform(shape, 2030 + i)
        assert_bit_exact(host(pkg.global_avg_pool2d(dev(x))), fast_orc.gap(x), "gap %s" % (shape,))
    x = synth.uniform((1, 5, 3, 43), 2036)             # 129 elements: the first plane size of the wave reduction
    assert_close(host(pkg.global_avg_pool2d(dev(x))), fast_orc.gap(x), what="gap 3x43")


def test_dense_full_size(pkg, fast_orc, synth):
    a = synth.uniform((64, 512), 2030); w = synth.uniform((1000, 512), 2031); b = synth.uniform((1000,), 2032)
    want = fast_orc.gemm(a, w, b, 1.0, 1.0, 1)
    assert_close(host(pkg.gemm(dev(a), dev(w), dev(b))), want, what="fc")
    # odd sizes take the reference-order kernel: bit-exact
    a = synth.uniform((5, 33), 2033); w = synth.uniform((9, 33), 2034); b = synth.uniform((9,), 2035)
    assert_bit_exact(host(pkg.gemm(dev(a), dev(w), dev(b), 0.5, 2.0, 1)), fast_orc.gemm(a, w, b, 0.5, 2.0, 1), "gemm odd")
    assert_bit_exact(host(pkg.gemm(dev(a), dev(w))), fast_orc.dense(a, w), "dense odd")
    ai = np.arange(64 * 64, dtype=np.float32).reshape(64, 64) % 7
    assert_bit_exact(host(pkg.gemm(dev(ai), dev(np.eye(64, dtype=np.float32)))), ai, "identity weight (mfma)")


@pytest.mark.parametrize("m", [1, 2, 3, 4, 5])
def test_gemm_few_rows(pkg, m):
    """Up to four rows (a classifier at batch 1-4) take the kernel whose waves split k over their lanes; five take
    the matrix-core tile.  Against a float64 evaluation, with alpha / beta, a scalar bias and a column count that
    leaves the last wave's columns partly empty; run to run bit-identical."""
    rng = np.random.default_rng(4100 + m)
    for (n, k, alpha, beta, clen) in [(1000, 512, 1.0, 1.0, 1000), (1001, 96, 0.5, 2.0, 1), (3, 32, 1.0, 1.0, 0), (130, 2048, 1.0, 1.0, 130)]:
        a = rng.uniform(-1, 1, (m, k)).astype(np.float32)
        b = rng.uniform(-1, 1, (n, k)).astype(np.float32)
        c = None if clen == 0 else rng.uniform(-1, 1, (clen,)).astype(np.float32)
        want = alpha * (a.astype(np.float64) @ b.astype(np.float64).T)
        if c is not None:
            want = want + beta * c.astype(np.float64)
        got = host(pkg.gemm(dev(a), dev(b), None if c is None else dev(c), alpha, beta, 1))
        assert_close(got, want.astype(np.float32), what="m=%d n=%d k=%d" % (m, n, k))
        again = host(pkg.gemm(dev(a), dev(b), None if c is None else dev(c), alpha, beta, 1))
        assert_bit_exact(again, got, "second run")


def test_gemm_random_shapes(pkg):
    """nn_dense / nn_gemm over seeded random sizes (k a multiple of 32 takes the matrix-core kernel, anything
    else the reference-order kernel), both layouts of the second operand, alpha / beta scaling, bias of length n
    or 1: against a float64 evaluation within the fp32 tolerance."""
    rng = np.random.default_rng(20241010)
    for case in range(30):
        m = int(rng.integers(1, 70)); n = int(rng.integers(1, 130))
        k = 32 * int(rng.integers(1, 10)) if case % 2 == 0 else int(rng.integers(1, 200))
        trans_b = 1 if case % 3 != 2 else 0
        a = rng.uniform(-1, 1, (m, k)).astype(np.float32)
        b = rng.uniform(-1, 1, (n, k) if trans_b else (k, n)).astype(np.float32)
        c = None if case % 4 == 3 else rng.uniform(-1, 1, (1,) if case % 4 == 2 else (n,)).astype(np.float32)
        alpha = 1.0 if case % 5 else 0.5; beta = 1.0 if case % 7 else 2.0
        want = alpha * (a.astype(np.float64) @ (b.astype(np.float64).T if trans_b else b.astype(np.float64)))
        if c is not None:
            want = want + beta * c.astype(np.float64)
        got = host(pkg.gemm(dev(a), dev(b), None if c is None else dev(c), alpha, beta, trans_b))
        assert_close(got, want.astype(np.float32), what="case %d: m=%d n=%d k=%d transB=%d" % (case, m, n, k, trans_b))


def test_bias_add_and_flatten(pkg, orc, synth):
    x = synth.uniform((3, 6, 5, 7), 2040); b = synth.uniform((6,), 2041)
    assert_bit_exact(host(pkg.bias_add(dev(x), dev(b))), orc.bias_add(x, b), "bias_add")
    assert_bit_exact(host(pkg.bias_add(dev(x), dev(b), relu=True)), orc.relu(orc.bias_add(x, b)), "bias_add+relu")
    assert_bit_exact(host(pkg.flatten(dev(x))), x.reshape(3, -1), "flatten")


def test_empty_inputs(pkg):
    e = torch.empty((0, 4, 8, 8), device="cuda")
    w = torch.zeros((32, 4, 3, 3), device="cuda")
    assert pkg.conv2d(e, w, stride=1, pad=1).shape == (0, 32, 8, 8)
    assert pkg.pool2d(e, 3, 2, 1).shape == (0, 4, 4, 4)
    assert pkg.global_avg_pool2d(e).shape == (0, 4, 1, 1)
    assert pkg.relu(torch.empty((0,), device="cuda")).numel() == 0


# ------------------------------------------------------------------ int8 (bit-exact)
def test_int8_ops_bit_exact(pkg, orc, synth):
    rng = np.random.default_rng(13)
    xf = synth.normal((2, 16, 14, 14), 5000)
    scale = float(np.abs(xf).max() / 127.0)
    xq = orc.quantize(xf, scale)
    assert_bit_exact(host(pkg.quantize(dev(xf), scale)), xq, "quantize")
    ties = np.array([0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 126.5, 127.5, 1e9, -1e9, np.nan], np.float32)
    assert_bit_exact(host(pkg.quantize(dev(ties), 1.0)), orc.quantize(ties, 1.0), "quantize ties")
    for (o, k, s, p) in [(32, 3, 1, 1), (32, 3, 2, 1), (24, 1, 2, 0), (8, 7, 2, 3)]:
        w = rng.integers(-127, 128, (o, 16, k, k), dtype=np.int8)
        bias = rng.integers(-2000, 2000, o).astype(np.int32)
        mult = (rng.random(o).astype(np.float32) + 0.5) * np.float32(2e-4)
        oh = (14 + 2 * p - k) // s + 1
        res = rng.integers(-128, 128, (2, o, oh, oh), dtype=np.int8)
        want = orc.qconv(xq, w, bias, mult, s, p, res, 0.37, True)
        got = host(pkg.qconv2d(dev(xq), dev(w), dev(bias), dev(mult), dev(res), 0.37, s, p, True))
        assert_bit_exact(got, want, "qconv %s" % ((o, k, s, p),))
        want = orc.qconv(xq, w, None, mult, s, p, None, 0.0, False)
        got = host(pkg.qconv2d(dev(xq), dev(w), None, dev(mult), None, 0.0, s, p, False))
        assert_bit_exact(got, want, "qconv bare %s" % ((o, k, s, p),))
    a = rng.integers(-128, 128, (8, 512), dtype=np.int8); b = rng.integers(-128, 128, (100, 512), dtype=np.int8)
    bias = rng.integers(-500, 500, 100).astype(np.int32); mult = rng.random(100).astype(np.float32) * 0.01
    assert_bit_exact(host(pkg.qdense(dev(a), dev(b), dev(bias), dev(mult))), orc.qdense(a, b, bias, mult), "qdense")
    x = rng.integers(-128, 128, (2, 6, 16, 16), dtype=np.int8)
    assert_bit_exact(host(pkg.maxpool2d_i8(dev(x), 3, 2, 1)), orc.qmaxpool(x, 3, 2, 1), "maxpool i8")
    assert_bit_exact(host(pkg.global_avg_pool2d_i8(dev(x), 0.0123)), orc.qgap(x, 0.0123), "gap i8")


# ------------------------------------------------------------------ whole network through the launch plan
def _run_plan(pkg, batch, hw, config, fuse=True):
    import importlib
    r = importlib.import_module("hdkx-aicompiler_amd.resnet18")
    synth = importlib.import_module("hdkx-aicompiler_amd.synth")
    consts = synth.resnet18_consts(config)
    x = synth.resnet18_input(config, batch, hw)
    plan, info = r.build_plan(batch, hw, fuse)
    out = torch.empty((batch, 1000), device="cuda")
    tensors = [dev(x)] + [dev(c) for c in consts] + [out]
    plan.run(tensors)
    got = host(out)
    plan.close()
    return x, consts, got, info


def test_resnet18_small_image(pkg, fast_orc):
    x, consts, got, info = _run_plan(pkg, 2, 64, 3)
    want = fast_orc.resnet18(x, consts)
    assert_close(got, want, what="resnet18 64x64 logits", floor="scale")
    assert len(info["launches"]) == 23
    x, consts, got2, info2 = _run_plan(pkg, 2, 64, 3, fuse=False)
    assert_close(got2, want, what="resnet18 64x64 logits (unfused launches)", floor="scale")
    assert len(info2["launches"]) > 23


def test_resnet18_batch1_224(pkg, fast_orc):
    """Benchmark configuration 3: full ResNet-18 at batch 1, logits within 1e-3 of the CPU path."""
    x, consts, got, info = _run_plan(pkg, 1, 224, 3)
    want = fast_orc.resnet18(x, consts)
    assert_close(got, want, what="resnet18 224 logits", floor="scale")
    assert int(np.argmax(got)) == int(np.argmax(want))


def test_resnet18_batch64_properties(pkg, fast_orc):
    """Benchmark configuration 4 at full size: image 0 and image 63 of the batch against the CPU path
    run on those images alone (the graph is independent per image)."""
    import importlib
    synth = importlib.import_module("hdkx-aicompiler_amd.synth")
    x, consts, got, info = _run_plan(pkg, 64, 224, 4)
    assert np.isfinite(got).all()
    for n in (0, 63):
        want = fast_orc.resnet18(x[n:n + 1], consts)
        assert_close(got[n:n + 1], want, what="resnet18 batch 64, image %d" % n, floor="scale")


def test_plan_chains_run_shares_of_a_batch_side_by_side(pkg, synth, fast_orc):
    """Two chains of one plan run the same three launches (Winograd convolution + bias + ReLU with shared transformed
    weights, max pool, convolution with a residual) on the two halves of a batch, each on a stream of its own, on
    KXC_HIP_BUF_ARG_OFFSET shares of the arguments: bit-identical to the same nodes in one lane, to the plan rebuilt
    from its text (version 2 keeps chain and select_lanes) and to every replay of the captured graph; within the
    operator tolerance of the CPU path.  Wrong uses are refused."""
    n, c, h, o = 8, 16, 24, 64
    x = synth.uniform((n, c, h, h), 9100)
    w = synth.normal((o, c, 3, 3), 9101, 0.1); b = synth.uniform((o,), 9102, -0.1, 0.1)
    w2 = synth.normal((o, o, 3, 3), 9103, 0.05)
    half = n // 2
    d1 = pkg.ConvDesc(half, c, h, h, o, 3, 3, 1, 1, 1, 1, 1, 1, pkg.CONV_BIAS | pkg.CONV_RELU)
    dp = pkg.pool_desc((half, o, h, h), 3, 1, 1)
    d2 = pkg.ConvDesc(half, o, h, h, o, 3, 3, 1, 1, 1, 1, 1, 1, pkg.CONV_RESIDUAL)
    ubytes = pkg.conv2d_winograd_weight_bytes((half, c, h, h), (o, c, 3, 3))
    ubytes = (ubytes + 255) // 256 * 256
    act = half * o * h * h * 4                                       # bytes of one share's activation
    x_share, y_share = half * c * h * h * 4, act

    def build(chains, interleave=False):
        plan = pkg.Plan(5)                                           # x, w, b, w2, y
        plan.set_select_lanes(2)
        for k in range(2):
            xk, yk = pkg.Buf.arg_offset(0, k * x_share), pkg.Buf.arg_offset(4, k * y_share)
            t0, t1 = pkg.Buf.ws(ubytes + (2 * k) * act), pkg.Buf.ws(ubytes + (2 * k + 1) * act)
            first = plan.num_nodes()
            plan.add_conv2d_winograd(d1, xk, pkg.Buf.arg(1), pkg.Buf.arg(2), pkg.Buf.none(), t0, pkg.Buf.ws(0))
            plan.add_pool2d(dp, t0, t1)
            plan.add_conv2d(d2, t1, pkg.Buf.arg(3), pkg.Buf.none(), t0, yk)
            if chains and k == 1:
                for node in range(first, plan.num_nodes()):
                    plan.set_chain(node, 1)
        if interleave:
            # main lane and chain alternate; every stream keeps its own order
            assert plan.interleave_chains() == [0, 2, 4, 1, 3, 5]
            assert ["winograd" in plan.node_symbol(i) for i in range(6)] == [True, True, False, False, False, False]
        plan.finalize(ubytes + 4 * act)
        return plan

    tensors = [dev(x), dev(w), dev(b), dev(w2)]
    y_line, y_chain = torch.zeros((n, o, h, h), device="cuda"), torch.zeros((n, o, h, h), device="cuda")
    in_line, chained = build(False), build(True)
    in_line.run(tensors + [y_line]); torch.cuda.synchronize()
    chained.run(tensors + [y_chain]); torch.cuda.synchronize()
    assert_bit_exact(host(y_chain), host(y_line), "chains against the same nodes in one lane")
    mixed = build(True, interleave=True)
    y_mixed = torch.zeros_like(y_chain)
    mixed.run(tensors + [y_mixed]); torch.cuda.synchronize()
    assert_bit_exact(host(y_mixed), host(y_line), "chains with their launches interleaved")
    assert pkg.Plan.deserialize(mixed.serialize(), 0).serialize() == mixed.serialize()
    mixed.close()
    t = fast_orc.conv_chain(x, w, b, 1, 1, None, True)
    t1 = fast_orc.pool2d(t, 3, 1, 1)
    want = fast_orc.conv_chain(t1, w2, None, 1, 1, t, False)
    assert_close(host(y_chain), want, what="two chains, conv / pool / conv + residual")
    # the text form keeps the chains; the rebuilt plan gives the same bits
    text = chained.serialize()
    # header: version, arguments, workspace bytes, nodes, select lanes, weight packs
    assert text.startswith("kxc_hip_plan 3 5 ") and text.splitlines()[0].split()[-2:] == ["2", "0"]
    again = pkg.Plan.deserialize(text, 0)
    assert again.serialize() == text
    y2 = torch.zeros_like(y_chain)
    again.run(tensors + [y2]); torch.cuda.synchronize()
    assert_bit_exact(host(y2), host(y_line), "deserialised plan with chains")
    # graph replay: the chains are parallel branches of the captured graph
    stream = torch.cuda.Stream()
    chained.enable_graph(True)
    with torch.cuda.stream(stream):
        for replay in range(5):
            y_chain.zero_()
            chained.run(tensors + [y_chain], stream.cuda_stream)
            stream.synchronize()
            assert_bit_exact(host(y_chain), host(y_line), "graph replay %d of a plan with chains" % replay)
            z = pkg.relu(tensors[0]); torch.cuda.synchronize()          # eager work between the replays
            assert torch.isfinite(z).all()
    # back-to-back runs without waiting in between: a run's chains start after the previous run's end
    chained.enable_graph(False)
    for _ in range(4):
        chained.run(tensors + [y_chain])
    torch.cuda.synchronize()
    assert_bit_exact(host(y_chain), host(y_line), "four runs enqueued back to back")
    for p in (in_line, chained, again):
        p.close()
    # refused: a chain beyond the seventh, an offset that is not a multiple of 16, a chain on a side-lane node
    plan = pkg.Plan(2)
    plan.add_relu(64, pkg.Buf.arg(0), pkg.Buf.arg(1))
    with pytest.raises(pkg.KxcHipError, match="chain must be in"):
        plan.set_chain(0, 8)
    with pytest.raises(pkg.KxcHipError, match="multiple of 16"):
        plan.add_relu(64, pkg.Buf.arg_offset(0, 8), pkg.Buf.arg(1))
    with pytest.raises(pkg.KxcHipError, match="out of range"):
        plan.add_relu(64, pkg.Buf.arg_offset(2, 0), pkg.Buf.arg(1))
    with pytest.raises(pkg.KxcHipError, match="lanes must be in"):
        plan.set_select_lanes(0)
    plan.close()


def test_plan_text_versions_1_and_2_still_load(pkg, synth):
    """The plan text gained a select_lanes field in the header and a chain field per node (version 2), then a count
    of weight packs in the header and a line per pack (version 3); a version-2 and a version-1 text -- the same plan
    written without them -- still load and give the same bits."""
    n, c, h, o = 2, 8, 10, 32
    x = synth.uniform((n, c, h, h), 9300); w = synth.normal((o, c, 3, 3), 9301, 0.1); b = synth.uniform((o,), 9302, -0.1, 0.1)
    d = pkg.ConvDesc(n, c, h, h, o, 3, 3, 1, 1, 1, 1, 1, 1, pkg.CONV_BIAS | pkg.CONV_RELU)
    plan = pkg.Plan(4)
    plan.add_conv2d(d, pkg.Buf.arg(0), pkg.Buf.arg(1), pkg.Buf.arg(2), pkg.Buf.none(), pkg.Buf.ws(0))
    plan.add_pool2d(pkg.pool_desc((n, o, h, h), 2, 2, 0), pkg.Buf.ws(0), pkg.Buf.arg(3))
    plan.finalize(n * o * h * h * 4)
    tensors = [dev(x), dev(w), dev(b)]
    y2 = torch.zeros((n, o, h // 2, h // 2), device="cuda")
    plan.run(tensors + [y2]); torch.cuda.synchronize()
    lines = plan.serialize().splitlines()
    head = lines[0].split()
    assert head[:2] == ["kxc_hip_plan", "3"] and head[-2:] == ["1", "0"]
    v2 = pkg.Plan.deserialize("\n".join([" ".join(["kxc_hip_plan", "2"] + head[2:-1])] + lines[1:]) + "\n", 0)
    y0 = torch.zeros_like(y2)
    v2.run(tensors + [y0]); torch.cuda.synchronize()
    assert_bit_exact(host(y0), host(y2), "plan rebuilt from a version-2 text")
    assert v2.serialize() == plan.serialize()
    v2.close()
    old_lines = [" ".join(["kxc_hip_plan", "1"] + head[2:-2])]
    for line in lines[1:]:
        t = line.split()
        if not t or t[0] != "node":
            old_lines.append(line)
            continue
        # the node ends "... lane join chain np [kind offset]*np"; find np by walking back
        k = len(t) - 1
        while True:
            cand = int(t[k])
            if len(t) - 1 - k == 2 * cand:
                break
            k -= 2
        assert t[k - 1] == "0"                                   # chain
        old_lines.append(" ".join(t[:k - 1] + t[k:]))
    y1 = torch.zeros_like(y2)
    old = pkg.Plan.deserialize("\n".join(old_lines) + "\n", 0)
    old.run(tensors + [y1]); torch.cuda.synchronize()
    assert_bit_exact(host(y1), host(y2), "plan rebuilt from a version-1 text")
    assert old.serialize() == plan.serialize()                   # written back as the current version
    plan.close(); old.close()


def test_plan_hip_graph_replay(pkg):
    """A launch plan replayed as a captured HIP graph gives the eager result on every replay, with eager work and
    synchronisations in between, and re-captures when an argument pointer changes.  Batch 1 exercises the
    workgroup-split reduction (scratch buffer, second kernel) inside the graph."""
    import importlib
    r = importlib.import_module("hdkx-aicompiler_amd.resnet18")
    synth = importlib.import_module("hdkx-aicompiler_amd.synth")
    consts = [dev(c) for c in synth.resnet18_consts(3)]
    x = dev(synth.resnet18_input(3, 1, 224))
    plan, info = r.build_plan(1, 224, True)
    out = torch.empty((1, 1000), device="cuda")
    plan.run([x] + consts + [out])
    torch.cuda.synchronize()
    eager = host(out).copy()
    assert np.isfinite(eager).all() and np.abs(eager).max() > 0
    stream = torch.cuda.Stream()
    plan.enable_graph(True)
    with torch.cuda.stream(stream):
        for replay in range(5):
            out.zero_()
            plan.run([x] + consts + [out], stream.cuda_stream)     # run 0 eager, run 1 captures, runs 2.. replay
            stream.synchronize()
            assert_bit_exact(host(out), eager, "graph replay %d" % replay)
            # eager work of the program between replays
            y = pkg.conv2d(x, consts[0], consts[1], None, 2, 3, 1, True)
            torch.cuda.synchronize()
            assert torch.isfinite(y).all()
        other = torch.empty((1, 1000), device="cuda")             # different output pointer: captured again
        for replay in range(3):
            other.zero_()
            plan.run([x] + consts + [other], stream.cuda_stream)
            stream.synchronize()
            assert_bit_exact(host(other), eager, "graph replay with a new output buffer %d" % replay)
    # another stream: the captured kernels hold the first stream's scratch addresses, so the plan runs eagerly
    # once and captures again there
    second = torch.cuda.Stream()
    with torch.cuda.stream(second):
        for replay in range(4):
            other.zero_()
            second.synchronize()
            plan.run([x] + consts + [other], second.cuda_stream)
            second.synchronize()
            assert_bit_exact(host(other), eager, "graph replay on a second stream %d" % replay)
    plan.enable_graph(False)
    plan.run([x] + consts + [out])
    torch.cuda.synchronize()
    assert_bit_exact(host(out), eager, "eager again")
    plan.close()
