"""ogle_hip_conv2d_noalloc (split-K scratch inside the library's device image) against
ogle_hip_conv2d with a caller workspace: same plan, so the outputs must be bit-identical.
Two calls in a row share the one scratch array; the second is the smaller problem."""
import ctypes

import numpy as np
import pytest

from ogle_amd import hip as H
import oracle as O
import util as U

pytestmark = pytest.mark.gpu


def _run(entry, x, w, b, stride, pad, with_workspace):
    import torch
    n, h, wd, c = x.shape
    o, _, k, _ = w.shape
    xd, bd = U.dev(x), U.dev(b)
    wdv = U.pack_filter(w, H.FILTER_OHWI)
    oh, ow = H.out_size(h, k, stride, pad), H.out_size(wd, k, stride, pad)
    y = torch.full((n, oh, ow, o), float("nan"), dtype=torch.float32, device="cuda")
    args = H.conv_args(xd.data_ptr(), wdv.data_ptr(), bd.data_ptr(), y.data_ptr(), n, h, wd, c, o,
                       k, stride, pad, act=H.ACT_RELU)
    need = H.lib().ogle_hip_conv_workspace_bytes(ctypes.byref(args))
    ws = None
    if with_workspace and need:
        ws = torch.empty(need, dtype=torch.uint8, device="cuda")
        args.workspace_dev, args.workspace_bytes = ws.data_ptr(), need
    H.check(getattr(H.lib(), entry)(ctypes.byref(args), U.stream_ptr()))
    torch.cuda.synchronize()
    return y.cpu().numpy(), need


# (n, h, w, c, o, k, stride, pad): split-K plans of decreasing scratch size, then one
# that needs no scratch at all
CASES = [
    (2, 5, 5, 512, 24, 3, 1, 1),
    (1, 3, 3, 256, 24, 3, 1, 1),
    (1, 19, 19, 64, 32, 1, 1, 0),
]


def test_noalloc_matches_workspace_entry_two_calls_in_a_row():
    r = U.rng(4242)
    needs = []
    for (n, h, w, c, o, k, s, p) in CASES:
        x = r.uniform(-1, 1, (n, h, w, c)).astype(np.float32)
        wt = r.normal(0, np.sqrt(2.0 / (k * k * c)), (o, c, k, k)).astype(np.float32)
        b = r.uniform(-0.1, 0.1, o).astype(np.float32)
        got, need = _run("ogle_hip_conv2d_noalloc", x, wt, b, s, p, False)
        ref, _ = _run("ogle_hip_conv2d", x, wt, b, s, p, True)
        needs.append(need)
        assert np.array_equal(got, ref), (n, h, w, c, o, k)
        ora = O.conv2d(x, wt, b, s, p, 1, 1, O.ACT_RELU)
        U.assert_conv_close(got, ora, O.conv2d_abs(x, wt, b, s, p, 1, 1), U.FP32_RTOL, "noalloc")
    assert needs[0] > needs[1] > 0 and needs[0] <= H.CONV_NOALLOC_SCRATCH_BYTES, needs


def _oversized_problem():
    """A convolution whose split-K plan wants more scratch than the built-in array holds: SSD
    class heads on the 19x19 map, the batch doubled until the plan is too large."""
    import torch
    h, c, o = 19, 512, 126
    for n in (64, 128, 256):
        x = torch.zeros((n, h, h, c), device="cuda")
        w = torch.zeros((o, 3, 3, c), device="cuda")
        y = torch.zeros((n, h, h, o), device="cuda")
        args = H.conv_args(x.data_ptr(), w.data_ptr(), None, y.data_ptr(), n, h, h, c, o, 3, 1, 1)
        need = H.lib().ogle_hip_conv_workspace_bytes(ctypes.byref(args))
        if need > H.CONV_NOALLOC_SCRATCH_BYTES:
            return args, need, (x, w, y)
    raise AssertionError("no plan exceeds the built-in scratch: pick another shape for this test")


def test_noalloc_refuses_oversized_and_caller_workspace():
    import torch
    args, need, keep = _oversized_problem()
    assert need > H.CONV_NOALLOC_SCRATCH_BYTES
    st = H.lib().ogle_hip_conv2d_noalloc(ctypes.byref(args), U.stream_ptr())
    assert st == H.ERR_INVALID_ARG
    assert str(need) in H.last_error() and str(H.CONV_NOALLOC_SCRATCH_BYTES) in H.last_error()
    # a caller workspace is refused: a pointer with a size, and a size without a pointer
    args.workspace_dev, args.workspace_bytes = keep[2].data_ptr(), 16
    assert H.lib().ogle_hip_conv2d_noalloc(ctypes.byref(args), U.stream_ptr()) == H.ERR_INVALID_ARG
    args.workspace_dev, args.workspace_bytes = None, 4096
    assert H.lib().ogle_hip_conv2d_noalloc(ctypes.byref(args), U.stream_ptr()) == H.ERR_INVALID_ARG
    torch.cuda.synchronize()
    # refused calls launched nothing and left the scratch alone: two good calls right after
    # them on the same stream still equal the workspace entry bit for bit
    r = U.rng(4243)
    for (n, h, w, c, o, k, s, p) in CASES[:2]:
        x = r.uniform(-1, 1, (n, h, w, c)).astype(np.float32)
        wt = r.normal(0, np.sqrt(2.0 / (k * k * c)), (o, c, k, k)).astype(np.float32)
        b = r.uniform(-0.1, 0.1, o).astype(np.float32)
        got, _ = _run("ogle_hip_conv2d_noalloc", x, wt, b, s, p, False)
        ref, _ = _run("ogle_hip_conv2d", x, wt, b, s, p, True)
        assert np.array_equal(got, ref), (n, h, w, c, o, k)
