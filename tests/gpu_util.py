"""Helpers shared by the GPU parity tests: error metrics as the reference's own acceptance check defines
them (test/onnx_importer_test.cpp:146-179) and host<->device shuttling."""
import numpy as np
import torch

FP32_TOL = 1e-3     # the stated tolerance: max relative error 1e-3 for fp32 operators and end-to-end logits


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    torch.cuda.synchronize()
    return t.detach().cpu().numpy()


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


def scaled_err(got, want):
    """max |a - r| / max(1, |r|), the reference's metric."""
    got = np.asarray(got, np.float64); want = np.asarray(want, np.float64)
    return float(np.max(np.abs(got - want) / np.maximum(1.0, np.abs(want))))


def rel_err(got, want, floor=1e-2):
    """plain max relative error over elements with |r| > floor."""
    got = np.asarray(got, np.float64); want = np.asarray(want, np.float64)
    m = np.abs(want) > floor
    if not m.any():
        return 0.0
    return float(np.max(np.abs(got[m] - want[m]) / np.abs(want[m])))


def assert_close(got, want, tol=FP32_TOL, what="", floor=1e-2):
    """Both the reference's metric and the plain relative error over elements above `floor` must be
    within tol.  floor is absolute (1e-2) for single operators; end-to-end logits pass
    floor="scale" = 1e-2 * max|want|, because a logit that happens to cancel to a value far below the
    tensor's scale carries the absolute error of the whole sum."""
    assert got.shape == want.shape, (what, got.shape, want.shape)
    assert np.isfinite(got).all(), what + ": non-finite output"
    if floor == "scale":
        floor = 1e-2 * float(np.max(np.abs(want)))
    e1, e2 = scaled_err(got, want), rel_err(got, want, floor)
    assert e1 <= tol and e2 <= tol, "%s: scaled err %.3g, rel err %.3g above %.3g (tol %g)" % (what, e1, e2, floor, tol)


def assert_bit_exact(got, want, what=""):
    assert got.shape == want.shape, (what, got.shape, want.shape)
    if got.dtype == np.float32:
        same = bits(got) == bits(want)
    else:
        same = got == want
    assert same.all(), "%s: %d of %d elements differ" % (what, int((~same).sum()), same.size)
