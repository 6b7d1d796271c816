"""Seeded random convolution shapes against the oracle: the launch plans (tile shape, K split,
wave-split kernels, direct kernels) are chosen from the shape, so shapes nobody picked by hand
are the check that no threshold hides a wrong path.  Every case runs with and without a
workspace, some with fp16 storage, some with the output images written apart
(OgleConvArgs.out_image_stride), some depthwise or grouped."""
import numpy as np
import pytest

import oracle as O
from ogle_amd import hip as H
from util import FP16_RTOL, FP32_RTOL, assert_conv_close, gpu_conv

pytestmark = pytest.mark.gpu


def _cases(seed, count):
    r = np.random.default_rng(seed)
    out = []
    while len(out) < count:
        k = int(r.choice([1, 1, 3, 3, 5]))
        s = int(r.choice([1, 1, 2]))
        p = int(r.integers(0, k // 2 + 2))
        d = 1 if k == 1 else int(r.choice([1, 1, 2]))
        n = int(r.choice([1, 1, 2, 3, 16]))
        h, w = int(r.integers(1, 40)), int(r.integers(1, 40))
        c = int(r.choice([3, 4, 8, 12, 16, 24, 32, 64, 100, 128, 256, 512, 1024]))
        o = int(r.choice([1, 3, 4, 12, 16, 21, 24, 32, 63, 64, 100, 126, 128, 256, 512]))
        kind = r.choice(["dense", "dense", "dense", "depthwise", "grouped"])
        g = 1
        if kind == "depthwise":
            o = g = c
        elif kind == "grouped":
            g = int(r.choice([2, 4]))
            if c % g or o % g:
                continue
        if n * h * w * c > 1_500_000 or (c // g) * o * k * k > 1_500_000:
            continue
        keff = k * d - d + 1
        if h + 2 * p < keff or w + 2 * p < keff:
            continue
        oh, ow = H.out_size(h, k, s, p, d), H.out_size(w, k, s, p, d)
        if n * oh * ow * o * (c // g) * k * k > 600_000_000:      # keeps the oracle to a second or so
            continue
        f16 = c % 8 == 0 and r.random() < 0.3
        apart = g == 1 and c % (8 if f16 else 4) == 0 and k * k * c >= 32 and r.random() < 0.4
        out.append((n, h, w, c, o, k, s, p, d, g, f16, apart, int(r.integers(0, 1 << 30))))
    return out


@pytest.mark.parametrize("seed", [11, 12, 13, 14, 15, 16])
def test_random_convolutions_match_the_oracle(seed):
    for case in _cases(seed, 60):
        n, h, w, c, o, k, s, p, d, g, f16, apart, sub = case
        r = np.random.default_rng(sub)
        x = r.uniform(-1, 1, (n, h, w, c)).astype(np.float32)
        wt = r.normal(0, 0.2, (o, c // g, k, k)).astype(np.float32)
        b = r.uniform(-0.1, 0.1, o).astype(np.float32) if r.random() < 0.8 else None
        dt = H.F16 if f16 else H.F32
        if f16:
            x = x.astype(np.float16).astype(np.float32)
            wt = wt.astype(np.float16).astype(np.float32)
        pw = k == 1 and s == 1 and p == 0 and g == 1
        variant = H.VARIANT_PW if pw else (H.VARIANT_ANY4 if 1 < g < c else H.VARIANT_NHWC4)
        act = int(r.choice([O.ACT_NONE, O.ACT_RELU, O.ACT_CLIP]))
        ref = O.conv2d(x, wt, b, s, p, d, g, act, 0.0, 6.0, variant)
        scale = O.conv2d_abs(x, wt, b, s, p, d, g)
        rtol = FP16_RTOL if f16 else FP32_RTOL
        if f16:
            # the result is rounded to fp16 once on the way out: half an fp16 ulp of the output
            # (subnormal outputs: half of 2^-24) on top of the bound, which matters where the
            # contraction is a single small term (a 1x1 depthwise convolution)
            a = np.maximum(np.abs(ref.astype(np.float64)), 2.0 ** -14)
            scale = scale + 0.5 * 2.0 ** (np.floor(np.log2(a)) - 10) / rtol
        for ws in (True, False):
            got = gpu_conv(x, wt, b, s, p, d, g, act, 0.0, 6.0, variant, dt, None, ws)
            assert_conv_close(got, ref, scale, rtol, "seed %d %s ws=%s" % (seed, case, ws),
                              min_abs=2.0 ** -14 if f16 else 0.0)
            if apart:
                image = got[0].size
                stride = image + 4 * int(r.integers(1, 9))
                flat = gpu_conv(x, wt, b, s, p, d, g, act, 0.0, 6.0, variant, dt, None, ws,
                                image_stride=stride, lead=8)
                rows = flat[8:].reshape(n, stride)
                np.testing.assert_array_equal(rows[:, :image].reshape(got.shape), got, err_msg=str(case))
                assert np.isnan(rows[:, image:]).all() and np.isnan(flat[:8]).all(), case
