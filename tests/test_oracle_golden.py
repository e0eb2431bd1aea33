"""Pins the CPU checker (oracle/) before anything is compared with it.

Evidence, in decreasing strength:
  1. oracle/_ref (the reference's own lowering + C code generator, where built): bit-exact.
  2. tests/golden/ref_cases.npz, written from (1) by tests/golden/make_golden.py: bit-exact.
  3. The literal known answers of the reference's test/op_numeric_llvm_test.cpp.
  4. What the mathematics fixes: closed forms, order-sensitive sums, float64 brute force,
     torch CPU cross-checks.
The int8 functions have no reference counterpart (parity unpinned); they get (4) only.
"""
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle_lib import Oracle, RefCases
from ref_case_table import CASES, case_inputs

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "ref_cases.npz")


@pytest.fixture(scope="module")
def orc():
    return Oracle()


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


# ------------------------------------------------------------------ 1. the reference itself
@pytest.mark.skipif(not RefCases.available(), reason="oracle/_ref not built (no reference checkout)")
@pytest.mark.parametrize("name", sorted(CASES))
def test_oracle_equals_reference_codegen(orc, name):
    ref = RefCases()
    ins = case_inputs(name)
    want = CASES[name][1](orc, ins)
    got = np.zeros_like(want)
    ref.run(name, ins + [got])
    assert np.array_equal(bits(got), bits(want)), name


@pytest.mark.skipif(not RefCases.available(), reason="oracle/_ref not built (no reference checkout)")
def test_reference_codegen_known_answers():
    """The reference-generated code reproduces the reference test's literals (sanity of the build)."""
    ref = RefCases()
    f = lambda *v: np.array(v, np.float32)
    y = np.zeros(4, np.float32)
    ref.run("kxc_ref_conv_kat", [f(1, 2, 3, 4, 5, 6, 7, 8, 9), f(1, 0, 0, 1), y])
    assert y.tolist() == [6, 8, 12, 14]
    ref.run("kxc_ref_maxpool_kat", [np.arange(1, 17, dtype=np.float32), y])
    assert y.tolist() == [6, 8, 14, 16]
    ref.run("kxc_ref_avgpool_kat", [np.arange(1, 17, dtype=np.float32), y])
    assert y.tolist() == [3.5, 5.5, 11.5, 13.5]


# ------------------------------------------------------------------ 2. committed fixtures
@pytest.mark.parametrize("name", sorted(CASES))
def test_oracle_equals_golden_fixture(orc, name):
    g = np.load(GOLDEN)
    ins = case_inputs(name)
    got = CASES[name][1](orc, ins)
    if name in g.files:
        assert np.array_equal(bits(got), bits(g[name])), name
    else:
        flat = got.reshape(-1)
        assert np.array_equal(bits(flat[g[name + "__idx"]]), bits(g[name + "__sample"]))
        assert np.bitwise_xor.reduce(flat.view(np.uint32)) == g[name + "__xor"]
        assert np.float64(flat.astype(np.float64).sum()) == g[name + "__sum64"]


# ------------------------------------------------------------------ 3. reference test literals
def test_kat_add(orc):       # test/op_numeric_llvm_test.cpp:59-70
    y = orc.add(np.array([[1, 2, 3], [4, 5, 6]], np.float32), np.array([10, 20, 30], np.float32))
    assert y.reshape(-1).tolist() == [11, 22, 33, 14, 25, 36]


def test_kat_sub_mul_div(orc):  # :72-109
    x = np.array([[1, 2, 3], [4, 5, 6]], np.float32); y = np.array([10, 20, 30], np.float32)
    assert orc.binary(1, x, y).reshape(-1).tolist() == [-9, -18, -27, -6, -15, -24]
    assert orc.binary(2, x, y).reshape(-1).tolist() == [10, 40, 90, 40, 100, 180]
    np.testing.assert_allclose(orc.binary(3, x, y).reshape(-1), [0.1, 0.1, 0.1, 0.4, 0.25, 0.2], atol=1e-4)


def test_kat_matmul(orc):    # :122-133
    a = np.arange(1, 7, dtype=np.float32).reshape(2, 3); b = np.arange(1, 7, dtype=np.float32).reshape(3, 2)
    assert orc.matmul(a, b).reshape(-1).tolist() == [22, 28, 49, 64]


def test_kat_dense(orc):     # :135-147
    a = np.arange(1, 7, dtype=np.float32).reshape(2, 3)
    w = np.array([[1, 0, 1], [0, 1, 1]], np.float32)
    assert orc.dense(a, w).reshape(-1).tolist() == [4, 5, 10, 11]


def test_kat_gemm(orc):      # :149-163
    a = np.arange(1, 7, dtype=np.float32).reshape(2, 3)
    b = np.array([1, 0, 0, 0, 1, 0, 0, 0, 1, 1, 1, 1], np.float32).reshape(4, 3)
    c = np.array([10, 20, 30, 40], np.float32)
    assert orc.gemm(a, b, c, 1.0, 1.0, 1).reshape(-1).tolist() == [11, 22, 33, 46, 14, 25, 36, 55]


def test_kat_relu(orc):      # :165-174
    assert orc.relu(np.array([-2, -0.5, 0, 1, 2, -3], np.float32)).tolist() == [0, 0, 0, 1, 2, 0]


def test_kat_conv2d(orc):    # :176-189
    x = np.arange(1, 10, dtype=np.float32).reshape(1, 1, 3, 3)
    w = np.array([1, 0, 0, 1], np.float32).reshape(1, 1, 2, 2)
    assert orc.conv2d(x, w).reshape(-1).tolist() == [6, 8, 12, 14]


def test_kat_maxpool_avgpool_gap(orc):  # :191-229
    x = np.arange(1, 17, dtype=np.float32).reshape(1, 1, 4, 4)
    assert orc.pool2d(x, 2, 2, 0).reshape(-1).tolist() == [6, 8, 14, 16]
    assert orc.pool2d(x, 2, 2, 0, avg=True).reshape(-1).tolist() == [3.5, 5.5, 11.5, 13.5]
    g = np.array([1, 2, 3, 4, 10, 20, 30, 40], np.float32).reshape(1, 2, 2, 2)
    assert orc.gap(g).reshape(-1).tolist() == [2.5, 25.0]


def test_kat_model_mlp_cnn(orc):  # :327-371
    x = np.array([[1, 2]], np.float32)
    w1 = np.array([[1, 0], [0, 1], [1, 1]], np.float32); w2 = np.array([[1, 1, 1], [1, 0, -1]], np.float32)
    assert orc.dense(orc.relu(orc.dense(x, w1)), w2).reshape(-1).tolist() == [6, -2]
    d = np.arange(1, 10, dtype=np.float32).reshape(1, 1, 3, 3)
    cw = np.array([1, 0, 0, 1], np.float32).reshape(1, 1, 2, 2)
    gp = orc.gap(orc.relu(orc.conv2d(d, cw))).reshape(1, 1)
    assert orc.dense(gp, np.array([[1], [2]], np.float32)).reshape(-1).tolist() == [10, 20]


# ------------------------------------------------------------------ 4. mathematics
def test_conv_one_hot_weight_is_shifted_copy(orc):
    rng = np.random.default_rng(1)
    x = rng.standard_normal((2, 3, 6, 7)).astype(np.float32)
    for c in range(3):
        for rh in range(3):
            for rw in range(3):
                w = np.zeros((1, 3, 3, 3), np.float32); w[0, c, rh, rw] = 1
                y = orc.conv2d(x, w, 1, 1)
                xp = np.pad(x, ((0, 0), (0, 0), (1, 1), (1, 1)))
                assert np.array_equal(y[:, 0], xp[:, c, rh:rh + 6, rw:rw + 7])


def test_conv_tap_count_and_stride(orc):
    y = orc.conv2d(np.ones((1, 1, 5, 5), np.float32), np.ones((1, 1, 3, 3), np.float32), 1, 1)[0, 0]
    assert y[0, 0] == 4 and y[0, 2] == 6 and y[2, 2] == 9 and y[4, 4] == 4
    # stride 2, pad 1 on 5x5: centres at input rows 0,2,4 -> 3x3 output, corner sees 2x2 taps
    y = orc.conv2d(np.ones((1, 1, 5, 5), np.float32), np.ones((1, 1, 3, 3), np.float32), 2, 1)[0, 0]
    assert y.shape == (3, 3) and y[0, 0] == 4 and y[1, 1] == 9
    # dilation 2, 3x3 -> effective 5x5
    y = orc.conv2d(np.ones((1, 1, 7, 7), np.float32), np.ones((1, 1, 3, 3), np.float32), 1, 0, 2)
    assert y.shape == (1, 1, 3, 3) and np.all(y == 9)


def test_conv_reduction_order_is_rc_rh_rw_ascending(orc):
    """fp32 addition is not associative: (1e8 + 1) - 1e8 = 0 but (1e8 - 1e8) + 1 = 1."""
    big = np.float32(1e8)
    x = np.array([big, 1, -big], np.float32).reshape(1, 3, 1, 1)      # over rc
    assert orc.conv2d(x, np.ones((1, 3, 1, 1), np.float32))[0, 0, 0, 0] == 0.0
    x = np.array([big, -big, 1], np.float32).reshape(1, 3, 1, 1)
    assert orc.conv2d(x, np.ones((1, 3, 1, 1), np.float32))[0, 0, 0, 0] == 1.0
    x = np.array([[big, 1, -big]], np.float32).reshape(1, 1, 1, 3)     # over rw
    assert orc.conv2d(x, np.ones((1, 1, 1, 3), np.float32))[0, 0, 0, 0] == 0.0
    x = np.array([[big], [1], [-big]], np.float32).reshape(1, 1, 3, 1)  # over rh
    assert orc.conv2d(x, np.ones((1, 1, 3, 1), np.float32))[0, 0, 0, 0] == 0.0
    # rc is outside rh/rw: channel 0 holds (big, 1), channel 1 holds (-big, 0)
    x = np.array([[big, 1], [-big, 0]], np.float32).reshape(1, 2, 1, 2)
    assert orc.conv2d(x, np.ones((1, 2, 1, 2), np.float32))[0, 0, 0, 0] == 0.0


def test_conv_padded_taps_still_multiply(orc):
    """Out-of-bounds taps contribute 0.0f * w (a NaN for w = inf), they are not skipped."""
    w = np.zeros((1, 1, 3, 3), np.float32); w[0, 0, 0, 0] = np.inf
    y = orc.conv2d(np.ones((1, 1, 4, 4), np.float32), w, 1, 1)[0, 0]
    assert np.isnan(y[0, 0]) and np.isnan(y[0, 3]) and np.isnan(y[3, 0]) and np.isinf(y[1, 1])


def test_conv_mul_and_add_round_separately(orc):
    a = np.float32(1 + 2.0 ** -12)
    c = -np.float32(a * a)                      # the rounded product
    fused = float(np.float64(a) * np.float64(a) + np.float64(c))
    assert fused != 0.0                          # an FMA would leave the rounding residue
    x = np.array([a, 1], np.float32).reshape(1, 2, 1, 1)
    w = np.array([a, c], np.float32).reshape(1, 2, 1, 1)
    assert orc.conv2d(x, w)[0, 0, 0, 0] == 0.0
    assert orc.dense(np.array([[a, 1]], np.float32), np.array([[a, c]], np.float32))[0, 0] == 0.0


def test_conv_brute_force_float64(orc):
    rng = np.random.default_rng(2)
    for (n, c, h, w_, o, k, s, p) in [(2, 3, 7, 6, 4, 3, 1, 1), (1, 5, 9, 9, 3, 3, 2, 1), (1, 2, 11, 11, 2, 7, 2, 3),
                                      (2, 4, 6, 6, 5, 1, 2, 0)]:
        x = rng.standard_normal((n, c, h, w_)).astype(np.float32)
        wt = rng.standard_normal((o, c, k, k)).astype(np.float32)
        y = orc.conv2d(x, wt, s, p)
        ref = F.conv2d(torch.from_numpy(x).double(), torch.from_numpy(wt).double(), stride=s, padding=p).numpy()
        assert y.shape == ref.shape
        np.testing.assert_allclose(y, ref, rtol=1e-5, atol=1e-5)


def test_conv_linearity_and_batch_independence(orc):
    rng = np.random.default_rng(3)
    x = rng.integers(-4, 5, (3, 4, 8, 8)).astype(np.float32)      # small integers: exact arithmetic
    w1 = rng.integers(-3, 4, (6, 4, 3, 3)).astype(np.float32)
    w2 = rng.integers(-3, 4, (6, 4, 3, 3)).astype(np.float32)
    assert np.array_equal(orc.conv2d(x, w1 + w2, 1, 1), orc.conv2d(x, w1, 1, 1) + orc.conv2d(x, w2, 1, 1))
    assert np.array_equal(orc.conv2d(x, w1, 2, 1)[1:2], orc.conv2d(x[1:2], w1, 2, 1))


def test_bias_relu_add_semantics(orc):
    x = np.array([np.nan, -0.0, 0.0, -1.0, 2.0, np.inf, -np.inf], np.float32)
    y = orc.relu(x)
    assert y.tolist() == [0, 0, 0, 0, 2, np.inf, 0] and not np.signbit(y[1])   # NaN -> 0, -0 -> +0
    assert np.array_equal(orc.relu(orc.relu(x)), orc.relu(x))                 # idempotent
    t = np.arange(24, dtype=np.float32).reshape(1, 2, 3, 4)
    assert np.array_equal(orc.bias_add(t, np.array([10, 100], np.float32)),
                          t + np.array([10, 100], np.float32).reshape(1, 2, 1, 1))


def test_broadcast_matches_numpy(orc):
    rng = np.random.default_rng(4)
    for sa, sb in [((2, 3, 4), (3, 1)), ((4,), (3, 1, 4)), ((2, 1, 5), (1, 6, 1)), ((1,), (2, 2))]:
        a = rng.standard_normal(sa).astype(np.float32); b = rng.standard_normal(sb).astype(np.float32) + 3
        for op, fn in enumerate((np.add, np.subtract, np.multiply, np.divide)):
            assert np.array_equal(bits(orc.binary(op, a, b)), bits(fn(a, b)))


def test_maxpool_exact_against_torch_and_ramp(orc):
    rng = np.random.default_rng(5)
    x = rng.standard_normal((2, 3, 13, 17)).astype(np.float32)
    for k, s, p in [(3, 2, 1), (2, 2, 0), (3, 1, 1), (5, 3, 2)]:
        got = orc.pool2d(x, k, s, p)
        want = F.max_pool2d(torch.from_numpy(x), k, s, p).numpy()
        assert np.array_equal(bits(got), bits(want))
    got = orc.pool2d(x, 3, 2, 1, ceil_mode=True)
    assert got.shape == F.max_pool2d(torch.from_numpy(x), 3, 2, 1, ceil_mode=True).shape
    ramp = np.arange(8 * 8, dtype=np.float32).reshape(1, 1, 8, 8)              # max = bottom-right tap
    assert np.array_equal(orc.pool2d(ramp, 3, 2, 1)[0, 0], ramp[0, 0, 1::2, 1::2])


def test_maxpool_pad_value_is_minus_1e30(orc):
    x = np.full((1, 1, 4, 4), -3e30, np.float32)
    y = orc.pool2d(x, 3, 2, 1)[0, 0]
    assert y[0, 0] == np.float32(-1e30)        # window touches padding: the pad candidate wins
    x = np.full((1, 1, 5, 5), -3e30, np.float32)
    assert orc.pool2d(x, 3, 2, 1)[0, 0, 1, 1] == np.float32(-3e30)   # interior window: no padding


def test_maxpool_nan_follows_select_chain(orc):
    """old > src ? old : src : a NaN src replaces old, and is replaced by the next src."""
    x = np.array([[1, np.nan], [0, -5]], np.float32).reshape(1, 1, 2, 2)
    assert orc.pool2d(x, 2, 2, 0)[0, 0, 0, 0] == 0.0    # 1, NaN, then (NaN > 0) false -> 0, then 0 > -5
    x = np.array([[1, 2], [3, np.nan]], np.float32).reshape(1, 1, 2, 2)
    assert np.isnan(orc.pool2d(x, 2, 2, 0)[0, 0, 0, 0])


def test_avgpool_counts_padding(orc):
    y = orc.pool2d(np.ones((1, 1, 4, 4), np.float32), 3, 2, 1, avg=True)[0, 0]
    assert y[0, 0] == np.float32(4) / np.float32(9) and y[1, 1] == 1.0
    rng = np.random.default_rng(6)
    x = rng.standard_normal((2, 2, 9, 9)).astype(np.float32)
    want = F.avg_pool2d(torch.from_numpy(x), 3, 2, 1, count_include_pad=True).numpy()
    np.testing.assert_allclose(orc.pool2d(x, 3, 2, 1, avg=True), want, rtol=1e-5, atol=1e-6)


def test_gap_sequential_sum_then_true_division(orc):
    big = np.float32(1e8)
    x = np.array([big, 1, -big, 0], np.float32).reshape(1, 1, 2, 2)
    assert orc.gap(x)[0, 0, 0, 0] == 0.0                    # row-major order rh, rw
    x = np.full((1, 1, 7, 7), 3.0, np.float32)
    assert orc.gap(x)[0, 0, 0, 0] == np.float32(147.0) / np.float32(49.0)
    # division, not multiplication by a rounded reciprocal: find a sum where they differ
    s = np.arange(1, 2000, dtype=np.float32)
    differs = s[(s / np.float32(49.0)) != (s * (np.float32(1.0) / np.float32(49.0)))]
    assert differs.size > 0
    v = differs[0]
    x = np.zeros((1, 1, 7, 7), np.float32); x[0, 0, 0, 0] = v
    assert orc.gap(x)[0, 0, 0, 0] == v / np.float32(49.0)


def test_dense_gemm_against_float64_and_identity(orc):
    rng = np.random.default_rng(7)
    a = rng.standard_normal((5, 33)).astype(np.float32); b = rng.standard_normal((9, 33)).astype(np.float32)
    c = rng.standard_normal(9).astype(np.float32)
    np.testing.assert_allclose(orc.dense(a, b), a.astype(np.float64) @ b.astype(np.float64).T, rtol=1e-5, atol=1e-5)
    assert np.array_equal(orc.dense(a, np.eye(33, dtype=np.float32)), a)
    np.testing.assert_allclose(orc.gemm(a, b, c, 0.5, 2.0, 1), 0.5 * (a.astype(np.float64) @ b.T) + 2.0 * c,
                               rtol=1e-5, atol=1e-5)
    bt = np.ascontiguousarray(b.T)
    assert np.array_equal(bits(orc.gemm(a, bt, c, 1.0, 1.0, 0)), bits(orc.gemm(a, b, c, 1.0, 1.0, 1)))
    big = np.float32(1e8)
    assert orc.dense(np.array([[big, 1, -big]], np.float32), np.ones((1, 3), np.float32))[0, 0] == 0.0  # k ascending


def test_resnet18_composition_small(orc, synth):
    """The whole-network oracle equals a by-hand composition of the pinned operators (64x64 input)."""
    consts = synth.resnet18_consts(3)
    x = synth.resnet18_input(3, 1, 64)
    logits, taps = orc.resnet18(x, consts, taps=True)
    y = orc.relu(orc.bias_add(orc.conv2d(x, consts[0], 2, 3), consts[1]))
    assert np.array_equal(bits(y), bits(taps["conv1_relu"]))
    y = orc.pool2d(y, 3, 2, 1)
    assert np.array_equal(bits(y), bits(taps["maxpool"]))
    i = 2
    for stage in range(4):
        for blk in range(2):
            first = blk == 0 and stage > 0
            s = 2 if first else 1
            a = orc.relu(orc.bias_add(orc.conv2d(y, consts[i], s, 1), consts[i + 1]))
            b = orc.bias_add(orc.conv2d(a, consts[i + 2], 1, 1), consts[i + 3])
            idn = y
            if first:
                idn = orc.bias_add(orc.conv2d(y, consts[i + 4], s, 0), consts[i + 5])
            i += 6 if first else 4
            y = orc.relu(orc.add(b, idn))
        assert np.array_equal(bits(y), bits(taps["layer%d" % (stage + 1)]))
    g = orc.gap(y)
    want = orc.gemm(g.reshape(1, 512), consts[40], consts[41], 1.0, 1.0, 1)
    assert np.array_equal(bits(want), bits(logits))
    t = torch.from_numpy
    # and against torch in float64 end to end
    z = t(x).double()
    z = F.relu(F.conv2d(z, t(consts[0]).double(), t(consts[1]).double(), 2, 3)); z = F.max_pool2d(z, 3, 2, 1)
    i = 2
    for stage in range(4):
        for blk in range(2):
            first = blk == 0 and stage > 0
            s = 2 if first else 1
            a = F.relu(F.conv2d(z, t(consts[i]).double(), t(consts[i + 1]).double(), s, 1))
            b = F.conv2d(a, t(consts[i + 2]).double(), t(consts[i + 3]).double(), 1, 1)
            idn = F.conv2d(z, t(consts[i + 4]).double(), t(consts[i + 5]).double(), s, 0) if first else z
            i += 6 if first else 4
            z = F.relu(b + idn)
    z = F.linear(z.mean((2, 3)), t(consts[40]).double(), t(consts[41]).double()).numpy()
    err = np.abs(logits - z) / np.maximum(1.0, np.abs(z))
    assert err.max() < 1e-4


# ------------------------------------------------------------------ int8 (parity unpinned by the reference)
def test_quantize_half_even_and_saturation(orc):
    x = np.array([0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 126.5, 127.5, 1e9, -1e9, 0.49999997], np.float32)
    assert orc.quantize(x, 1.0).tolist() == [0, 2, 2, 0, -2, -2, 126, 127, 127, -127, 0]
    assert orc.quantize(np.array([1.0, -3.0], np.float32), 0.5).tolist() == [2, -6]


def test_qconv_all_ones_and_bruteforce(orc):
    x = np.ones((1, 8, 5, 5), np.int8); w = np.ones((4, 8, 3, 3), np.int8)
    acc = orc.qconv_acc(x, w, 1, 1)
    assert acc[0, 0, 2, 2] == 72 and acc[0, 0, 0, 0] == 32
    rng = np.random.default_rng(8)
    x = rng.integers(-128, 128, (2, 5, 7, 6), dtype=np.int8); w = rng.integers(-128, 128, (3, 5, 3, 3), dtype=np.int8)
    for s, p in [(1, 1), (2, 1), (1, 0)]:
        want = F.conv2d(torch.from_numpy(x).double(), torch.from_numpy(w).double(), stride=s, padding=p).numpy()
        assert np.array_equal(orc.qconv_acc(x, w, s, p), want.astype(np.int64))


def test_qconv_requant_definition(orc):
    rng = np.random.default_rng(9)
    x = rng.integers(-128, 128, (1, 4, 6, 6), dtype=np.int8); w = rng.integers(-128, 128, (3, 4, 3, 3), dtype=np.int8)
    bias = rng.integers(-1000, 1000, 3).astype(np.int32)
    res = rng.integers(-128, 128, (1, 3, 6, 6), dtype=np.int8)
    acc = orc.qconv_acc(x, w, 1, 1) + bias.reshape(1, 3, 1, 1)
    # power-of-two multipliers: the float product is exact, so requant is an exact shift + round-half-even
    mult = np.array([2.0 ** -7, 2.0 ** -9, 2.0 ** -8], np.float32)
    v = acc.astype(np.float64) * mult.reshape(1, 3, 1, 1).astype(np.float64)
    want = np.clip(np.rint(v), 0, 127).astype(np.int8)
    assert np.array_equal(orc.qconv(x, w, bias, mult, 1, 1, None, 0.0, True), want)
    v2 = v + res.astype(np.float64) * 0.25
    want = np.clip(np.rint(v2), -128, 127).astype(np.int8)
    assert np.array_equal(orc.qconv(x, w, bias, mult, 1, 1, res, 0.25, False), want)
    # general multiplier: fp32 product rounded once, then rint
    mult = np.array([0.0123, 0.0031, 0.0077], np.float32)
    vf = (acc.astype(np.float32) * mult.reshape(1, 3, 1, 1)).astype(np.float32)
    assert np.array_equal(orc.qconv(x, w, bias, mult, 1, 1, None, 0.0, True), np.clip(np.rint(vf), 0, 127).astype(np.int8))


def test_qdense_qpool(orc):
    rng = np.random.default_rng(10)
    a = rng.integers(-128, 128, (3, 40), dtype=np.int8); b = rng.integers(-128, 128, (7, 40), dtype=np.int8)
    bias = rng.integers(-500, 500, 7).astype(np.int32); mult = rng.random(7).astype(np.float32) * 0.01
    acc = a.astype(np.int64) @ b.astype(np.int64).T + bias
    assert np.array_equal(orc.qdense(a, b, bias, mult), acc.astype(np.float32) * mult)
    x = rng.integers(-128, 128, (2, 3, 9, 9), dtype=np.int8)
    want = F.max_pool2d(torch.from_numpy(x).float(), 3, 2, 1).numpy().astype(np.int8)
    assert np.array_equal(orc.qmaxpool(x, 3, 2, 1), want)
    s = x.astype(np.int64).sum((2, 3))
    want = np.clip(np.rint((s.astype(np.float32) * np.float32(0.0625)).astype(np.float32)), -128, 127).astype(np.int8)
    assert np.array_equal(orc.qgap(x, 0.0625).reshape(2, 3), want)
