"""kxc_hip_conv2d_nchw_f32_noalloc -- the entry point that allocates nothing -- against kxc_hip_conv2d_nchw_f32.

Both run the same kernels, so the outputs must be identical bit for bit; the shapes are ones whose reduction is
split over workgroups (the launches that use scratch memory: the built-in device array here, a hipMalloc'ed
buffer there).  Two calls in a row, the second on a smaller input, so stale contents of the shared array from
the first call would show in the second.
"""
import ctypes as C
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _tensors(synth, torch, xs, ws, seed):
    x = torch.from_numpy(synth.normal(xs, seed, 1.0)).cuda()
    w = torch.from_numpy(synth.normal(ws, seed + 1, float(np.sqrt(2.0 / (ws[1] * ws[2] * ws[3]))))).cuda()
    b = torch.from_numpy(synth.uniform((ws[0],), seed + 2, -0.1, 0.1)).cuda()
    return x, w, b


def _needed(pkg, xs, ws, stride, pad):
    d = pkg.conv_desc(xs, ws, stride, pad, 1, 0)
    n = C.c_size_t(0)
    assert pkg.lib().kxc_hip_conv2d_scratch_needed(C.byref(d), C.byref(n)) == 0
    return n.value


# (x shape, w shape, stride, pad, with residual): batch-1 ResNet-18 layers with long reductions, larger one first
CASES = [((1, 512, 7, 7), (512, 512, 3, 3), 1, 1, True),
         ((1, 256, 14, 14), (256, 256, 3, 3), 2, 1, False)]


def test_noalloc_conv2d_matches_the_allocating_entry_point_twice_in_a_row(pkg, synth):
    import torch
    assert torch.cuda.is_available()
    capacity = pkg.lib().kxc_hip_conv2d_noalloc_scratch_bytes()
    assert capacity == 8 << 20
    needs = [_needed(pkg, xs, ws, s, p) for xs, ws, s, p, _ in CASES]
    # both launches use scratch, the second less than the first
    assert needs[0] > needs[1] > 0 and needs[0] <= capacity, needs
    allocations = pkg.lib().kxc_hip_debug_device_allocations
    allocations.restype = C.c_int64
    for i, (xs, ws, stride, pad, with_res) in enumerate(CASES):
        x, w, b = _tensors(synth, torch, xs, ws, 7100 + 10 * i)
        oshape = pkg.conv_out_shape(pkg.conv_desc(xs, ws, stride, pad, 1, 0))
        res = torch.from_numpy(synth.uniform(tuple(oshape), 7105 + 10 * i)).cuda() if with_res else None
        got = torch.full(tuple(oshape), float("nan"), dtype=torch.float32, device="cuda")
        print("no-alloc conv2d", xs, ws, "stride", stride, "scratch bytes", needs[i], flush=True)
        # the entry point that allocates nothing goes FIRST on each shape (a scratch buffer grown lazily for the shape
        # would show), and the library's own count of device allocations must not move
        before = allocations()
        pkg.conv2d(x, w, b, res, stride, pad, 1, True, out=got, no_alloc=True)
        torch.cuda.synchronize()
        assert allocations() == before, "the no-alloc entry point allocated device memory"
        want = pkg.conv2d(x, w, b, res, stride, pad, 1, True)
        torch.cuda.synchronize()
        assert torch.equal(got, want), float((got - want).abs().max())
        # and a third time on the same buffers: the array's leftovers from this very shape change nothing
        got.fill_(float("nan"))
        pkg.conv2d(x, w, b, res, stride, pad, 1, True, out=got, no_alloc=True)
        torch.cuda.synchronize()
        assert torch.equal(got, want)


def test_allocation_counter_sees_the_allocating_entry_point(pkg, synth):
    """The counter the test above relies on does move when the library allocates: a split shape on a fresh stream
    makes the allocating entry point create that stream's scratch buffer."""
    import torch
    allocations = pkg.lib().kxc_hip_debug_device_allocations
    allocations.restype = C.c_int64
    xs, ws, stride, pad, _ = CASES[0]
    x, w, b = _tensors(synth, torch, xs, ws, 7150)
    stream = torch.cuda.Stream()
    before = allocations()
    with torch.cuda.stream(stream):
        pkg.conv2d(x, w, b, None, stride, pad, 1, True)
        stream.synchronize()
    assert allocations() > before


def test_noalloc_conv2d_takes_launches_without_scratch(pkg, synth):
    """Shapes whose reduction is not split (the usual case) run exactly as through the other entry point."""
    import torch
    xs, ws = (8, 64, 56, 56), (64, 64, 3, 3)
    assert _needed(pkg, xs, ws, 1, 1) == 0
    x, w, b = _tensors(synth, torch, xs, ws, 7200)
    want = pkg.conv2d(x, w, b, None, 1, 1, 1, True)
    got = torch.empty_like(want)
    pkg.conv2d(x, w, b, None, 1, 1, 1, True, out=got, no_alloc=True)
    torch.cuda.synchronize()
    assert torch.equal(got, want)


def test_noalloc_conv2d_refuses_what_does_not_fit(pkg, synth):
    """A forced split whose partial sums exceed the built-in array is an error, and nothing is launched."""
    import torch
    xs, ws = (16, 128, 28, 28), (128, 128, 3, 3)           # 1.6 M outputs: 6.4 MB per part
    x, w, b = _tensors(synth, torch, xs, ws, 7300)
    y = torch.zeros((16, 128, 28, 28), dtype=torch.float32, device="cuda")
    os.environ["KXC_HIP_CONV_GSPLIT"] = "4"
    try:
        assert _needed(pkg, xs, ws, 1, 1) > 8 << 20
        with pytest.raises(pkg.KxcHipError, match="bytes of scratch"):
            pkg.conv2d(x, w, b, None, 1, 1, 1, True, out=y, no_alloc=True)
    finally:
        del os.environ["KXC_HIP_CONV_GSPLIT"]
    torch.cuda.synchronize()
    assert float(y.abs().max()) == 0.0
