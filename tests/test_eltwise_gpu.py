"""Elementwise ops and Gemm through the C ABI against the oracle (bit-exact for the
elementwise ops in fp32, contraction tolerance for Gemm)."""
import ctypes

import numpy as np
import pytest

import oracle as O
from ogle_amd import hip as H
from util import dev, rng, stream_ptr

pytestmark = pytest.mark.gpu


def _torch():
    import torch
    return torch


def gpu_unary(x, op, lo=0.0, hi=0.0, dtype=H.F32, in_place=False):
    torch = _torch()
    t = dev(x).to(torch.float16 if dtype == H.F16 else torch.float32).contiguous()
    y = t if in_place else torch.full_like(t, float("nan"))
    a = H.UnaryArgs(t.data_ptr(), y.data_ptr(), t.numel(), op, lo, hi, dtype)
    H.check(H.lib().ogle_hip_unary(ctypes.byref(a), stream_ptr()))
    torch.cuda.synchronize()
    return y.float().cpu().numpy()


SHAPES = [(1,), (3,), (4,), (5, 7), (2, 9, 9, 5), (4, 19, 19, 64), (1, 150, 150, 32), (1023,), (0,)]


@pytest.mark.parametrize("shape", SHAPES)
def test_relu_and_clip(shape):
    r = rng(11000 + len(shape) * 31 + shape[0])
    x = r.normal(0, 2, shape).astype(np.float32)
    np.testing.assert_array_equal(gpu_unary(x, H.UNARY_RELU), O.relu(x))
    np.testing.assert_array_equal(gpu_unary(x, H.UNARY_CLIP, -0.5, 1.25), O.clip(x, -0.5, 1.25))
    np.testing.assert_array_equal(gpu_unary(x, H.UNARY_CLIP, 0.0, 6.0, in_place=True), O.clip(x, 0.0, 6.0))
    # min above max: the last operation wins, as in the shader
    np.testing.assert_array_equal(gpu_unary(x, H.UNARY_CLIP, 2.0, 1.0), O.clip(x, 2.0, 1.0))
    xh = x.astype(np.float16).astype(np.float32)
    np.testing.assert_array_equal(gpu_unary(xh, H.UNARY_RELU, dtype=H.F16), O.relu(xh))


@pytest.mark.parametrize("shape", SHAPES)
def test_add(shape):
    torch = _torch()
    r = rng(11500 + len(shape) * 31 + shape[0])
    a = r.normal(0, 2, shape).astype(np.float32)
    b = r.normal(0, 2, shape).astype(np.float32)
    ad, bd = dev(a), dev(b)
    y = torch.full_like(ad, float("nan"))
    args = H.BinaryArgs(ad.data_ptr(), bd.data_ptr(), y.data_ptr(), ad.numel(), H.F32)
    H.check(H.lib().ogle_hip_add(ctypes.byref(args), stream_ptr()))
    torch.cuda.synchronize()
    np.testing.assert_array_equal(y.cpu().numpy(), O.add(a, b))
    # fp16 storage: fp32 sum rounded once
    ah, bh = ad.half(), bd.half()
    yh = torch.empty_like(ah)
    args = H.BinaryArgs(ah.data_ptr(), bh.data_ptr(), yh.data_ptr(), ah.numel(), H.F16)
    H.check(H.lib().ogle_hip_add(ctypes.byref(args), stream_ptr()))
    torch.cuda.synchronize()
    ref = (ah.float() + bh.float()).half()
    assert torch.equal(yh, ref)


@pytest.mark.parametrize("shape", [(1, 1, 1, 1), (2, 5, 7, 3), (2, 9, 9, 8), (4, 19, 19, 64), (3, 10),
                                   (1, 75, 75, 130)])
def test_batchnorm(shape):
    torch = _torch()
    r = rng(12000 + shape[-1])
    c = shape[-1]
    x = r.normal(0, 2, shape).astype(np.float32)
    gamma, beta = r.uniform(0.5, 1.5, c).astype(np.float32), r.normal(0, 0.1, c).astype(np.float32)
    mean, var = r.normal(0, 0.3, c).astype(np.float32), r.uniform(0.5, 1.5, c).astype(np.float32)
    xd, g, bt, mu, vr = dev(x), dev(gamma), dev(beta), dev(mean), dev(var)
    y = torch.full_like(xd, float("nan"))
    a = H.BatchNormArgs(xd.data_ptr(), g.data_ptr(), bt.data_ptr(), mu.data_ptr(), vr.data_ptr(),
                        y.data_ptr(), x.size // c, c, 1e-5, H.F32)
    H.check(H.lib().ogle_hip_batchnorm(ctypes.byref(a), stream_ptr()))
    torch.cuda.synchronize()
    np.testing.assert_array_equal(y.cpu().numpy(), O.batchnorm(x, gamma, beta, mean, var, 1e-5))


def gpu_gemm(a, b, c, alpha, beta, trans_b, workspace=True):
    torch = _torch()
    m, k = a.shape
    n = b.shape[0] if trans_b else b.shape[1]
    ad, bd = dev(a), dev(b)
    cd = dev(c) if c is not None else None
    y = torch.full((m, n), float("nan"), device="cuda")
    args = H.GemmArgs(ad.data_ptr(), bd.data_ptr(), cd.data_ptr() if cd is not None else None,
                      y.data_ptr(), m, n, k, int(trans_b), c.ndim if c is not None else 0, alpha, beta,
                      None, 0)
    need = H.lib().ogle_hip_gemm_workspace_bytes(ctypes.byref(args))
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
    if need and workspace:
        args.workspace_dev, args.workspace_bytes = ws.data_ptr(), need
    H.check(H.lib().ogle_hip_gemm(ctypes.byref(args), stream_ptr()))
    torch.cuda.synchronize()
    return y.cpu().numpy(), need


GEMM_CASES = [
    # m, n, k, trans_b, c ("row" | "full" | None), alpha, beta
    (1, 1000, 1024, True, "row", 1.0, 1.0),     # classifier head, batch 1 (MFMA path, split-K)
    (16, 1000, 1024, True, "row", 1.0, 1.0),    # batch 16
    (64, 1000, 2048, True, None, 1.0, 1.0),
    (5, 33, 20, True, "row", 1.0, 1.0),         # MFMA path, ragged
    (3, 10, 7, True, "row", 1.0, 1.0),          # K % 4 != 0 -> general kernel
    (4, 70, 36, False, "row", 1.0, 1.0),        # B not transposed
    (17, 65, 40, True, "full", 0.5, -2.0),      # alpha, beta, full addend
    (2, 3, 5, False, None, 2.0, 0.0),
]


@pytest.mark.parametrize("case", GEMM_CASES)
def test_gemm(case):
    m, n, k, trans_b, cmode, alpha, beta = case
    r = rng(13000 + GEMM_CASES.index(case))
    a = r.normal(0, 1, (m, k)).astype(np.float32)
    b = r.normal(0, 0.2, (n, k) if trans_b else (k, n)).astype(np.float32)
    c = None if cmode is None else r.normal(0, 1, n if cmode == "row" else (m, n)).astype(np.float32)
    ref = O.gemm(a, b, c, alpha, beta, trans_b)
    bm = np.abs(b.T if trans_b else b).astype(np.float64)
    scale = abs(alpha) * (np.abs(a).astype(np.float64) @ bm)
    if c is not None:
        scale = scale + abs(beta) * np.abs(c)
    for workspace in (True, False):
        got, need = gpu_gemm(a, b, c, alpha, beta, trans_b, workspace)
        assert np.all(np.abs(got - ref) <= 1e-4 * scale + 1e-30), case


def test_eltwise_argument_checks():
    torch = _torch()
    x = torch.zeros(64, device="cuda")
    a = H.UnaryArgs(x.data_ptr() + 4, x.data_ptr(), 8, H.UNARY_RELU, 0, 0, H.F32)
    assert H.lib().ogle_hip_unary(ctypes.byref(a), 0) == H.ERR_INVALID_ARG      # misaligned
    a = H.UnaryArgs(x.data_ptr(), x.data_ptr(), 8, 7, 0, 0, H.F32)
    assert H.lib().ogle_hip_unary(ctypes.byref(a), 0) == H.ERR_UNSUPPORTED      # unknown op
    g = H.GemmArgs(x.data_ptr(), x.data_ptr(), x.data_ptr(), x.data_ptr(), 2, 2, 2, 1, 3, 1.0, 1.0, None, 0)
    assert H.lib().ogle_hip_gemm(ctypes.byref(g), 0) == H.ERR_INVALID_ARG       # c_rank
