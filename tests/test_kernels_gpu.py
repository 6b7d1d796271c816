"""GPU parity tests: every kernel is called through the C ABI (include/ogle_hip.h)
on seeded inputs and compared with the CPU oracle.

Tolerances (util.assert_conv_close): every output within 1e-5 (fp32) / 5e-3 (fp16 storage) of
the accumulated magnitude sum|x||w|, and BASELINE's literal max relative error 1e-4 / 5e-3 on
every output not dominated by cancellation (|ref| >= 1e-2 sum|x||w|); pooling,
concat and kept indices / class ids exact; box coordinates 1e-4.
The shape sweeps mirror the reference's DIFFERENT_SHAPE_LOOP
(ogl_runtime/opengl/nn/kernels/kernel_test_utils.h:59-65) and its conv tests
(conv2d_test.cc:220-354: any-format input, no bias, dilation 2, grouped, stride 2
at 320x320x3->32, depthwise).
"""
import numpy as np
import pytest

import oracle as O
from ogle_amd import hip as H
from util import (assert_conv_close, gpu_concat, gpu_conv, gpu_decode, gpu_detect, gpu_pool,
                  gpu_topk_nms, rng)

pytestmark = pytest.mark.gpu

from util import FP16_RTOL, FP32_RTOL


def check_conv(x, w, b, stride=1, pad=0, dil=1, groups=1, act=H.ACT_NONE, minv=0.0, maxv=0.0,
               variant=H.VARIANT_NHWC4, dtype=H.F32, entry=None, what=""):
    ref = O.conv2d(x, w, b, stride, pad, dil, groups, act, minv, maxv, variant)
    scale = O.conv2d_abs(x, w, b, stride, pad, dil, groups)
    got = gpu_conv(x, w, b, stride, pad, dil, groups, act, minv, maxv, variant, dtype, entry)
    return assert_conv_close(got, ref, scale, FP16_RTOL if dtype == H.F16 else FP32_RTOL, what)



def assert_same_detections(got, ora, logits, threshold, what=""):
    """Kept prior indices and class ids must be bit-exact; scores may differ in the last
    place because the host's expf is not correctly rounded on every input (the device's is).
    A prior whose decision a 1-ulp change of one exponential could flip (score within 2e-6 of
    the threshold, or its two best foreground classes within 2e-6 of each other) is excluded
    from the exact comparison and counted; none occurs with the seeds used here."""
    l64 = logits.astype(np.float64)
    e = np.exp(l64 - l64.max(-1, keepdims=True))
    sm = e / e.sum(-1, keepdims=True)
    fg = np.sort(sm[:, 1:], axis=-1)
    ambiguous = (np.abs(fg[:, -1] - threshold) < 2e-6) | ((fg[:, -1] - fg[:, -2]) < 2e-6 * fg[:, -1])
    amb = set(np.nonzero(ambiguous)[0].tolist())
    gp = [(int(p), int(c)) for p, c in zip(got["prior"], got["cls"]) if int(p) not in amb]
    op = [(int(p), int(c)) for p, c in zip(ora["prior"], ora["cls"]) if int(p) not in amb]
    assert gp == op, what
    if len(got["prior"]) == len(ora["prior"]) and np.array_equal(got["prior"], ora["prior"]):
        np.testing.assert_allclose(got["score"], ora["score"], rtol=3e-7, atol=0)
        np.testing.assert_array_equal(got["box"], ora["box"])
        np.testing.assert_array_equal(got["rect"], ora["rect"])
    return len(amb)


SMALL_CASES = [
    # n, h, w, c, o, k, s, p, d, g
    (1, 3, 3, 3, 1, 3, 1, 1, 1, 1),
    (2, 7, 5, 4, 6, 3, 1, 1, 1, 1),
    (1, 9, 9, 5, 7, 3, 2, 1, 1, 1),
    (1, 8, 8, 3, 4, 3, 1, 2, 2, 1),
    (2, 6, 6, 8, 8, 3, 1, 1, 1, 8),
    (1, 6, 7, 8, 12, 3, 2, 1, 1, 4),
    (3, 5, 5, 16, 9, 1, 1, 0, 1, 1),
    (1, 10, 10, 6, 4, 5, 1, 2, 1, 1),
    (1, 4, 4, 2, 3, 1, 2, 0, 1, 1),
    (1, 1, 1, 20, 5, 3, 1, 1, 1, 1),
    (2, 13, 11, 32, 40, 3, 1, 1, 1, 1),    # MFMA path, ragged M and N
    (1, 17, 17, 64, 130, 3, 2, 1, 1, 1),   # MFMA path, stride 2, N just over a tile
    (1, 9, 9, 36, 33, 3, 1, 1, 2, 1),      # MFMA path, dilation 2, K tail inside a slab
    (4, 19, 19, 128, 24, 3, 1, 1, 1, 1),   # SSD loc head shape
    (2, 10, 10, 64, 126, 3, 1, 1, 1, 1),   # SSD conf head shape
    (1, 5, 5, 48, 72, 1, 1, 0, 1, 1),      # pointwise, K not a multiple of the slab
    (2, 9, 7, 12, 12, 5, 2, 2, 1, 12),     # depthwise 5x5 stride 2 (general kernel)
    (1, 8, 8, 6, 6, 3, 1, 1, 1, 6),        # depthwise, C not a multiple of 4
    (1, 11, 9, 16, 16, 3, 2, 1, 1, 16),    # depthwise stride 2
]


@pytest.mark.parametrize("case", SMALL_CASES)
@pytest.mark.parametrize("use_bias", [False, True])
def test_conv_small_cases(case, use_bias):
    n, h, w, c, o, k, s, p, d, g = case
    r = rng(1000 + SMALL_CASES.index(case))
    x = r.uniform(-1, 1, (n, h, w, c)).astype(np.float32)
    wt = r.normal(0, 0.5, (o, c // g, k, k)).astype(np.float32)
    b = r.uniform(-0.1, 0.1, o).astype(np.float32) if use_bias else None
    check_conv(x, wt, b, s, p, d, g, what=str(case))


def test_conv_shape_sweep_dense_and_depthwise():
    """size 1,2,4..32 x channels 1..20, dense 3x3 p1 and depthwise, with bias + ReLU."""
    r = rng(2000)
    for size in (1, 2, 4, 8, 16, 32):
        for ch in range(1, 21):
            x = r.uniform(-1, 1, (2, size, size, ch)).astype(np.float32)
            wt = r.normal(0, 0.5, (ch + 1, ch, 3, 3)).astype(np.float32)
            b = r.uniform(-0.1, 0.1, ch + 1).astype(np.float32)
            check_conv(x, wt, b, 1, 1, act=H.ACT_RELU, what="dense %d %d" % (size, ch))
            wd = r.normal(0, 0.5, (ch, 1, 3, 3)).astype(np.float32)
            bd = r.uniform(-0.1, 0.1, ch).astype(np.float32)
            check_conv(x, wd, bd, 1, 1, 1, ch, act=H.ACT_CLIP, maxv=0.5,
                       entry="ogle_hip_dwconv2d", what="dw %d %d" % (size, ch))


STEM_CASES = [
    # n, h, w, c, o, k, s, p, d   (K = k*k*c <= 32 and >= 4096 output pixels: the MFMA stem kernel)
    (2, 96, 96, 3, 32, 3, 2, 1, 1),     # the RGB stem shape (pair loads: even stride, padding 1, even width)
    (3, 75, 78, 3, 64, 3, 2, 1, 1),     # RGB pair loads, odd height, ragged last tile, two channel tiles
    (2, 50, 90, 3, 32, 3, 4, 1, 1),     # RGB pair loads, stride 4, the right edge is padding
    (3, 75, 77, 3, 32, 3, 2, 1, 1),     # RGB, odd width: the general kernel
    (2, 66, 65, 3, 64, 3, 1, 1, 1),     # RGB, stride 1, two channel tiles
    (2, 71, 70, 3, 32, 3, 2, 0, 1),     # RGB, no padding
    (1, 131, 67, 3, 96, 3, 3, 1, 1),    # RGB, stride 3
    (1, 70, 67, 3, 20, 3, 1, 1, 1),     # ragged pixel count, fewer channels than a tile
    (1, 65, 66, 1, 40, 3, 1, 0, 1),     # one input channel, two channel tiles, no padding
    (1, 80, 80, 2, 33, 3, 1, 2, 2),     # dilation 2
    (1, 64, 70, 3, 8, 2, 1, 0, 1),      # even kernel, K = 12
    (1, 68, 68, 1, 5, 5, 1, 2, 1),      # 5x5 on one channel, K = 25
    (1, 64, 64, 8, 16, 2, 2, 0, 1),     # K = 32 exactly
]


@pytest.mark.parametrize("case", STEM_CASES)
@pytest.mark.parametrize("dtype", [H.F32, H.F16])
def test_conv_stem_kernel(case, dtype):
    n, h, w, c, o, k, s, p, d = case
    r = rng(1500 + STEM_CASES.index(case))
    x = r.uniform(-1, 1, (n, h, w, c)).astype(np.float32)
    wt = r.normal(0, 0.5, (o, c, k, k)).astype(np.float32)
    b = r.uniform(-0.1, 0.1, o).astype(np.float32)
    if dtype == H.F16:  # the oracle sees the values the device stores
        x = x.astype(np.float16).astype(np.float32)
        wt = wt.astype(np.float16).astype(np.float32)
    check_conv(x, wt, b, s, p, d, 1, act=H.ACT_CLIP, maxv=6.0, dtype=dtype, what=str(case))


WAVE_CASES = [
    # n, h, w, c, o, k, s, p, d   small problems with a long enough K: the wave-split kernel
    (1, 19, 19, 512, 512, 1, 1, 0, 1),    # 32x32 tiles, pointwise (a batch-1 MobileNet layer)
    (1, 38, 38, 256, 250, 1, 1, 0, 1),    # 32x32 tiles, ragged N with 2-element tail
    (2, 40, 40, 20, 64, 3, 1, 1, 1),      # 32x32 tiles, 3x3, C % 8 == 4 (half-filled last step)
    (1, 45, 41, 36, 33, 3, 2, 1, 1),      # 32x32 tiles, stride 2, N not a multiple of 4
    (1, 10, 10, 1024, 256, 1, 1, 0, 1),   # 16x16 tiles, pointwise
    (1, 3, 3, 128, 256, 3, 2, 1, 1),      # 16x16 tiles, one output pixel per image
    (3, 5, 5, 64, 21, 3, 1, 2, 2),        # 16x16 tiles, dilation 2, odd N
    (1, 1, 1, 1024, 1000, 1, 1, 0, 1),    # 16x16 tiles, M = 1 (a classifier head)
    (1, 7, 9, 128, 10, 3, 1, 1, 1),       # 16x16 tiles, fewer channels than a tile
    (1, 10, 10, 1024, 1024, 1, 1, 0, 1),  # 16x16 tiles, pointwise, two tiles per compute unit
    (1, 9, 11, 504, 130, 1, 1, 0, 1),     # 16x16 tiles, pointwise, ragged M, N and last K step
    (2, 10, 10, 1024, 1024, 1, 1, 0, 1),  # 32x32 tiles, pointwise, K = 1024
]


@pytest.mark.parametrize("case", WAVE_CASES)
@pytest.mark.parametrize("dtype", [H.F32, H.F16])
def test_conv_wave_split_kernel(case, dtype):
    n, h, w, c, o, k, s, p, d = case
    r = rng(1700 + WAVE_CASES.index(case))
    x = r.uniform(-1, 1, (n, h, w, c)).astype(np.float32)
    wt = r.normal(0, 0.2, (o, c, k, k)).astype(np.float32)
    b = r.uniform(-0.1, 0.1, o).astype(np.float32)
    if dtype == H.F16:
        if c % 8 != 0:
            pytest.skip("fp16 storage needs C % 8 == 0 for the MFMA kernels")
        x = x.astype(np.float16).astype(np.float32)
        wt = wt.astype(np.float16).astype(np.float32)
    variant = H.VARIANT_PW if (k == 1 and s == 1 and p == 0) else H.VARIANT_NHWC4
    # with and without a workspace: the plan must not depend on it
    for entry_ws in (True, False):
        ref = O.conv2d(x, wt, b, s, p, d, 1, O.ACT_CLIP, 0.0, 6.0, variant)
        scale = O.conv2d_abs(x, wt, b, s, p, d, 1)
        got = gpu_conv(x, wt, b, s, p, d, 1, H.ACT_CLIP, 0.0, 6.0, variant, dtype, None, entry_ws)
        assert_conv_close(got, ref, scale, FP16_RTOL if dtype == H.F16 else FP32_RTOL, str(case))


# (n, h, w, c, o, k, stride, pad, image stride beyond the image's own outputs, lead)
IMAGE_STRIDE_CASES = [
    (16, 19, 19, 512, 12, 3, 1, 1, 2000, 0),     # box head: split-K + reduce, 16-byte rows
    (16, 19, 19, 512, 63, 3, 1, 1, 40257 - 22743, 0),   # class head: odd stride, stores by element
    (4, 10, 10, 256, 24, 3, 1, 1, 36, 24),       # small map: wave-split kernel or short split
    (3, 5, 5, 64, 126, 3, 1, 1, 1, 7),           # 16x16 tiles, everything unaligned
    (2, 38, 38, 128, 64, 1, 1, 0, 64, 128),      # pointwise, no split: the tile kernel's row stores
    (64, 10, 10, 256, 24, 3, 1, 1, 5064, 0),     # batch 64: tile kernel without a split
    (5, 7, 9, 32, 40, 3, 2, 1, 0, 0),            # stride equal to the image: the dense case
]


@pytest.mark.parametrize("case", IMAGE_STRIDE_CASES)
@pytest.mark.parametrize("dtype", [H.F32, H.F16])
@pytest.mark.parametrize("workspace", [True, False])
def test_conv_out_image_stride(case, dtype, workspace):
    """OgleConvArgs.out_image_stride: every image's outputs equal the dense launch's bit for bit,
    land at lead + b * stride, and nothing between the images is written."""
    n, h, w, c, o, k, s, p, extra, lead = case
    r = rng(1800 + IMAGE_STRIDE_CASES.index(case))
    x = r.uniform(-1, 1, (n, h, w, c)).astype(np.float32)
    wt = r.normal(0, 0.2, (o, c, k, k)).astype(np.float32)
    b = r.uniform(-0.1, 0.1, o).astype(np.float32)
    variant = H.VARIANT_PW if (k == 1 and s == 1 and p == 0) else H.VARIANT_NHWC4
    dense = gpu_conv(x, wt, b, s, p, 1, 1, H.ACT_RELU, 0.0, 0.0, variant, dtype, None, workspace)
    image = dense[0].size
    stride = image + extra
    flat = gpu_conv(x, wt, b, s, p, 1, 1, H.ACT_RELU, 0.0, 0.0, variant, dtype, None, workspace,
                    image_stride=stride, lead=lead)
    assert flat.size == lead + n * stride
    assert np.isnan(flat[:lead]).all()
    rows = flat[lead:].reshape(n, stride)
    np.testing.assert_array_equal(rows[:, :image].reshape(dense.shape), dense)
    assert np.isnan(rows[:, image:]).all()
    if dtype == H.F32:
        ref = O.conv2d(x, wt, b, s, p, 1, 1, O.ACT_RELU, 0.0, 0.0, variant)
        assert_conv_close(dense, ref, O.conv2d_abs(x, wt, b, s, p, 1, 1), FP32_RTOL, "stride " + str(case))


def test_conv_out_image_stride_is_refused_off_the_mfma_path():
    r = rng(1850)
    x = r.uniform(-1, 1, (2, 6, 6, 3)).astype(np.float32)
    wt = r.normal(0, 0.2, (8, 3, 3, 3)).astype(np.float32)
    with pytest.raises(H.OgleError, match="out_image_stride"):
        gpu_conv(x, wt, None, 1, 1, image_stride=6 * 6 * 8 + 8)
    xd = r.uniform(-1, 1, (2, 6, 6, 16)).astype(np.float32)
    wd = r.normal(0, 0.2, (16, 1, 3, 3)).astype(np.float32)
    with pytest.raises(H.OgleError, match="out_image_stride"):
        gpu_conv(xd, wd, None, 1, 1, groups=16, image_stride=6 * 6 * 16 + 16)
    wt2 = r.normal(0, 0.2, (8, 16, 3, 3)).astype(np.float32)
    with pytest.raises(H.OgleError, match="less than one image"):
        gpu_conv(xd, wt2, None, 1, 1, image_stride=6 * 6 * 8 - 1)


# (n, h, w, c, o, k, stride, pad): at most 16 output channels on the MFMA path, i.e. the tile
# of 16x16 MFMA blocks: one tile row and many, ragged M, split K and not, ragged last K step
NARROW_CASES = [
    (16, 19, 19, 512, 12, 3, 1, 1),    # the 19x19 box head at batch 16 (split K + reduce)
    (1, 38, 38, 128, 16, 3, 1, 1),     # all 16 columns used, M = 1444
    (2, 9, 7, 24, 5, 3, 2, 1),         # tiny, M = 40 < one tile, C not a multiple of the K slab
    (3, 31, 17, 64, 1, 1, 1, 0),       # pointwise, one output channel
    (64, 10, 10, 64, 13, 1, 1, 0),     # pointwise, 50 tile rows, odd channel count
    (1, 150, 150, 32, 8, 3, 1, 1),     # many tile rows, short K
    (2, 5, 5, 1024, 16, 3, 1, 2),      # padding 2 (output 7x7), long K
]


@pytest.mark.parametrize("case", NARROW_CASES)
@pytest.mark.parametrize("dtype", [H.F32, H.F16])
def test_conv_narrow_tile(case, dtype):
    n, h, w, c, o, k, s, p = case
    r = rng(1900 + NARROW_CASES.index(case))
    x = r.uniform(-1, 1, (n, h, w, c)).astype(np.float32)
    wt = r.normal(0, 0.2, (o, c, k, k)).astype(np.float32)
    b = r.uniform(-0.1, 0.1, o).astype(np.float32)
    if dtype == H.F16:
        x = x.astype(np.float16).astype(np.float32)
        wt = wt.astype(np.float16).astype(np.float32)
    variant = H.VARIANT_PW if (k == 1 and s == 1 and p == 0) else H.VARIANT_NHWC4
    ref = O.conv2d(x, wt, b, s, p, 1, 1, O.ACT_CLIP, 0.0, 6.0, variant)
    scale = O.conv2d_abs(x, wt, b, s, p, 1, 1)
    for workspace in (True, False):
        got = gpu_conv(x, wt, b, s, p, 1, 1, H.ACT_CLIP, 0.0, 6.0, variant, dtype, None, workspace)
        assert_conv_close(got, ref, scale, FP16_RTOL if dtype == H.F16 else FP32_RTOL,
                          "narrow %s ws=%s" % (case, workspace))


def test_conv_shape_sweep_mfma_path():
    """Channel counts that take the implicit-GEMM kernel, ragged in every dimension."""
    r = rng(2100)
    for (h, w) in ((1, 1), (3, 5), (8, 8), (19, 19), (33, 9)):
        for c in (8, 12, 16, 20, 64, 100):
            for o in (1, 31, 32, 33, 64, 65, 129):
                x = r.uniform(-1, 1, (2, h, w, c)).astype(np.float32)
                wt = r.normal(0, 0.3, (o, c, 1, 1)).astype(np.float32)
                b = r.uniform(-0.1, 0.1, o).astype(np.float32)
                check_conv(x, wt, b, act=H.ACT_RELU, variant=H.VARIANT_PW,
                           what="pw %dx%d c%d o%d" % (h, w, c, o))
    for c in (8, 16, 36):
        for o in (4, 40, 70):
            x = r.uniform(-1, 1, (1, 7, 6, c)).astype(np.float32)
            wt = r.normal(0, 0.3, (o, c, 3, 3)).astype(np.float32)
            check_conv(x, wt, None, 1, 1, what="3x3 c%d o%d" % (c, o))


def test_activation_variants_on_device():
    r = rng(2200)
    x = r.uniform(-2, 2, (1, 6, 6, 16)).astype(np.float32)
    w1 = r.normal(0, 0.5, (16, 16, 1, 1)).astype(np.float32)
    w3 = r.normal(0, 0.3, (16, 16, 3, 3)).astype(np.float32)
    wd = r.normal(0, 0.5, (16, 1, 3, 3)).astype(np.float32)
    for variant in (H.VARIANT_NHWC4, H.VARIANT_PW, H.VARIANT_ANY4):
        for act, mn, mx in ((H.ACT_CLIP, -0.5, 1.0), (H.ACT_RELU, -0.25, 0.0), (H.ACT_CLIP, 0.0, 6.0)):
            check_conv(x, w1, None, act=act, minv=mn, maxv=mx, variant=variant, what="pw act")
            check_conv(x, w3, None, 1, 1, act=act, minv=mn, maxv=mx, variant=variant, what="3x3 act")
            check_conv(x, wd, None, 1, 1, 1, 16, act=act, minv=mn, maxv=mx, variant=variant,
                       what="dw act")


def test_stride2_stem_320():
    """conv2d_test.cc:324-337: 320x320x3 -> 32, 3x3 stride 2."""
    r = rng(2300)
    x = r.uniform(-1, 1, (1, 320, 320, 3)).astype(np.float32)
    w = r.normal(0, np.sqrt(2 / 27), (32, 3, 3, 3)).astype(np.float32)
    b = r.uniform(-0.1, 0.1, 32).astype(np.float32)
    check_conv(x, w, b, 2, 1, act=H.ACT_CLIP, maxv=6.0, what="stem")


# ----------------------------------------------------------- BASELINE configs --

def test_config1_dense_3x3():
    r = rng(20240001)
    x = r.uniform(-1, 1, (1, 112, 112, 32)).astype(np.float32)
    w = r.normal(0, np.sqrt(2 / 288), (64, 32, 3, 3)).astype(np.float32)
    b = r.uniform(-0.1, 0.1, 64).astype(np.float32)
    check_conv(x, w, b, 1, 1, act=H.ACT_RELU, what="C1")


@pytest.mark.parametrize("batch", [1, 8])
def test_config2_depthwise_separable_block(batch):
    r = rng(20240002)
    x = r.uniform(0, 6, (batch, 38, 38, 256)).astype(np.float32)
    wd = r.normal(0, np.sqrt(2 / 9), (256, 1, 3, 3)).astype(np.float32)
    wp = r.normal(0, np.sqrt(2 / 256), (512, 256, 1, 1)).astype(np.float32)

    def bn(c):
        return (r.uniform(0.5, 1.5, c).astype(np.float32), r.normal(0, 0.1, c).astype(np.float32),
                r.normal(0, 0.1, c).astype(np.float32), r.uniform(0.5, 1.5, c).astype(np.float32))

    wdf, bdf = O.fold_bn(wd, None, *bn(256))
    wpf, bpf = O.fold_bn(wp, None, *bn(512))
    ref1 = O.conv2d(x, wdf, bdf, 1, 1, 1, 256, O.ACT_CLIP, 0.0, 6.0)
    got1 = gpu_conv(x, wdf, bdf, 1, 1, 1, 256, H.ACT_CLIP, 0.0, 6.0)
    assert_conv_close(got1, ref1, O.conv2d_abs(x, wdf, bdf, 1, 1, 1, 256), FP32_RTOL, "C2 dw")
    ref2 = O.conv2d(ref1, wpf, bpf, act=O.ACT_CLIP, maxv=6.0, variant=O.VARIANT_PW)
    got2 = gpu_conv(ref1, wpf, bpf, act=H.ACT_CLIP, maxv=6.0, variant=H.VARIANT_PW)
    assert_conv_close(got2, ref2, O.conv2d_abs(ref1, wpf, bpf), FP32_RTOL, "C2 pw")


@pytest.mark.parametrize("dtype", [H.F32, H.F16])
def test_config3_pointwise_gemm(dtype):
    r = rng(20240003)
    x = r.uniform(0, 6, (32, 19, 19, 512)).astype(np.float32)
    w = r.normal(0, np.sqrt(2 / 512), (1024, 512, 1, 1)).astype(np.float32)
    b = r.uniform(-0.1, 0.1, 1024).astype(np.float32)
    # float64 matmul is the tight reference here (the scalar oracle takes minutes at this size);
    # the oracle itself is compared on the first image below.
    a64 = x.reshape(-1, 512).astype(np.float64)
    ref = np.maximum(a64 @ w.reshape(1024, 512).astype(np.float64).T + b, 0).astype(np.float32)
    scale = (np.abs(a64) @ np.abs(w.reshape(1024, 512)).astype(np.float64).T + np.abs(b))
    got = gpu_conv(x, w, b, act=H.ACT_RELU, variant=H.VARIANT_PW, dtype=dtype)
    rtol = FP16_RTOL if dtype == H.F16 else FP32_RTOL
    assert_conv_close(got.reshape(-1, 1024), ref, scale.astype(np.float32), rtol, "C3")
    ora = O.conv2d(x[:1], w, b, act=O.ACT_RELU, variant=O.VARIANT_PW)
    assert_conv_close(got[:1], ora, scale[:361].reshape(1, 19, 19, 1024).astype(np.float32), rtol,
                      "C3 vs oracle")


def test_conv_batch_equals_single_launches():
    """ogle_hip_conv2d_batch: several independent convolutions in grouped launches give exactly
    what one launch each gives (same kernels, same summation order)."""
    import ctypes
    import torch
    r = rng(2500)
    cases = [  # n, h, w, c, o, k, s, p
        (4, 19, 19, 128, 12, 3, 1, 1), (4, 19, 19, 128, 63, 3, 1, 1), (4, 10, 10, 256, 24, 3, 1, 1),
        (4, 10, 10, 256, 126, 3, 1, 1), (4, 5, 5, 128, 126, 3, 1, 1), (4, 3, 3, 64, 24, 3, 1, 1),
        (2, 7, 7, 64, 96, 1, 1, 0), (2, 9, 9, 32, 40, 1, 1, 0), (1, 8, 8, 3, 8, 3, 2, 1),
        (1, 6, 6, 6, 6, 3, 1, 1), (2, 9, 9, 32, 24, 1, 1, 0), (16, 19, 19, 64, 64, 1, 1, 0),
    ]
    keep, single, args = [], [], (H.ConvArgs * len(cases))()
    for i, (n, h, w, c, o, k, st, p) in enumerate(cases):
        x = torch.from_numpy(r.uniform(-1, 1, (n, h, w, c)).astype(np.float32)).cuda()
        wt = r.normal(0, 0.2, (o, c, k, k)).astype(np.float32)
        from util import pack_filter
        wd = pack_filter(wt, H.FILTER_OHWI)
        b = torch.from_numpy(r.uniform(-.1, .1, o).astype(np.float32)).cuda()
        oh, ow = H.out_size(h, k, st, p), H.out_size(w, k, st, p)
        y1 = torch.full((n, oh, ow, o), float("nan"), device="cuda")
        y2 = torch.full((n, oh, ow, o), float("nan"), device="cuda")
        a = H.conv_args(x.data_ptr(), wd.data_ptr(), b.data_ptr(), y1.data_ptr(), n, h, w, c, o, k,
                        st, p, 1, 1, H.ACT_RELU)
        need = H.lib().ogle_hip_conv_workspace_bytes(ctypes.byref(a))
        ws1 = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
        ws2 = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
        if need:
            a.workspace_dev, a.workspace_bytes = ws1.data_ptr(), need
        H.check(H.lib().ogle_hip_conv2d(ctypes.byref(a), 0))
        a.output_dev = y2.data_ptr()
        if need:
            a.workspace_dev = ws2.data_ptr()
        args[i] = a
        keep += [x, wd, b, ws1, ws2]
        single.append((y1, y2))
    H.check(H.lib().ogle_hip_conv2d_batch(args, len(cases), 0))
    torch.cuda.synchronize()
    for y1, y2 in single:
        assert torch.isfinite(y2).all()
        assert torch.equal(y1, y2)
    # dependent convolutions are refused
    args[1].input_dev = args[0].output_dev
    assert H.lib().ogle_hip_conv2d_batch(args, 2, 0) == H.ERR_INVALID_ARG


def ssd_anchors():
    """1917 center-size priors: 19/10/5/3/2/1 maps, 3,6,6,6,6,6 anchors, scales 0.2-0.95."""
    maps, counts = [19, 10, 5, 3, 2, 1], [3, 6, 6, 6, 6, 6]
    scales = [0.2 + (0.95 - 0.2) * i / 5 for i in range(6)] + [1.0]
    out = []
    for k, (m, a) in enumerate(zip(maps, counts)):
        ratios = [1.0, 2.0, 0.5] if a == 3 else [1.0, 2.0, 0.5, 3.0, 1.0 / 3.0]
        for y in range(m):
            for x in range(m):
                cx, cy = (x + 0.5) / m, (y + 0.5) / m
                for ar in ratios:
                    out.append([cx, cy, scales[k] * np.sqrt(ar), scales[k] / np.sqrt(ar)])
                if a == 6:
                    s = np.sqrt(scales[k] * scales[k + 1])
                    out.append([cx, cy, s, s])
    a = np.array(out, np.float32)
    assert a.shape == (1917, 4)
    return a


C4_MAPS = [(19, 512, 3), (10, 1024, 6), (5, 512, 6), (3, 256, 6), (2, 256, 6), (1, 128, 6)]


def _conv3x3_f64(x, w):
    """3x3 stride 1 pad 1 cross-correlation in float64 as an im2col matrix product (numpy only):
    the tight reference where the scalar oracle would take minutes.  x NHWC, w OIHW."""
    n, h, wd, c = x.shape
    o = w.shape[0]
    xp = np.zeros((n, h + 2, wd + 2, c), np.float64)
    xp[:, 1:-1, 1:-1] = x
    cols = np.empty((n, h, wd, 9, c), np.float64)
    for ky in range(3):
        for kx in range(3):
            cols[:, :, :, ky * 3 + kx] = xp[:, ky:ky + h, kx:kx + wd]
    wm = w.astype(np.float64).transpose(2, 3, 1, 0).reshape(9 * c, o)   # (ky, kx, c) x o
    return (cols.reshape(n * h * wd, 9 * c) @ wm).reshape(n, h, wd, o)


def test_config4_heads_batch64_single_and_grouped_calls():
    """The twelve SSD head convolutions at the full batch of 64 (a different launch plan from
    batch 4: long-K splits, grouped grids), each as its own call and all twelve as one
    ogle_hip_conv2d_batch call, against a float64 im2col product; image 0 also against the
    oracle.  Inputs are BASELINE config 4's: features U(0,6), weights N(0, 0.01)."""
    import ctypes
    import torch
    from util import pack_filter
    r = rng(20240004)
    batch = 64
    keep, checks = [], []
    args = (H.ConvArgs * 12)()
    for mi, (m, c, a) in enumerate(C4_MAPS):
        f = r.uniform(0, 6, (batch, m, m, c)).astype(np.float32)
        fd = torch.from_numpy(f).cuda()
        for hi, last in enumerate((4, 21)):
            o = a * last
            wt = r.normal(0, 0.01, (o, c, 3, 3)).astype(np.float32)
            ref = _conv3x3_f64(f, wt)
            scale = _conv3x3_f64(np.abs(f), np.abs(wt))
            wd = pack_filter(wt, H.FILTER_OHWI)
            y1 = torch.full((batch, m, m, o), float("nan"), device="cuda")
            y2 = torch.full((batch, m, m, o), float("nan"), device="cuda")
            ar = H.conv_args(fd.data_ptr(), wd.data_ptr(), None, y1.data_ptr(), batch, m, m, c, o, 3, 1, 1)
            need = H.lib().ogle_hip_conv_workspace_bytes(ctypes.byref(ar))
            ws1 = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
            ws2 = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
            if need:
                ar.workspace_dev, ar.workspace_bytes = ws1.data_ptr(), need
            H.check(H.lib().ogle_hip_conv2d(ctypes.byref(ar), 0))
            ar.output_dev = y2.data_ptr()
            if need:
                ar.workspace_dev = ws2.data_ptr()
            args[mi * 2 + hi] = ar
            keep += [fd, wd, ws1, ws2]
            ora = O.conv2d(f[:1], wt, None, 1, 1)
            checks.append((m, o, y1, y2, ref, scale, ora))
    H.check(H.lib().ogle_hip_conv2d_batch(args, 12, 0))
    torch.cuda.synchronize()
    for m, o, y1, y2, ref, scale, ora in checks:
        for tag, y in (("single", y1), ("grouped", y2)):
            got = y.cpu().numpy()
            what = "C4 b64 head %dx%d o%d %s" % (m, m, o, tag)
            assert_conv_close(got, ref.astype(np.float32), scale, FP32_RTOL, what)
            assert_conv_close(got[:1], ora, scale[:1], FP32_RTOL, what + " vs oracle")


@pytest.mark.parametrize("batch", [2, 16])
def test_heads_written_in_place_of_the_concat(batch):
    """The twelve SSD heads as one ogle_hip_conv2d_batch call (and as begin + finish) with
    out_image_stride set so that every head writes its images straight into box_preds /
    cls_logits: the two buffers equal the concatenation of the heads launched one by one, bit
    for bit, and the call still refuses two heads whose places overlap."""
    import ctypes
    import torch
    from util import pack_filter
    r = rng(20240016)
    priors = sum(m * m * a for m, _, a in C4_MAPS)
    outs = {4: torch.full((batch, priors, 4), float("nan"), device="cuda"),
            21: torch.full((batch, priors, 21), float("nan"), device="cuda")}
    outs2 = {k: torch.full_like(v, float("nan")) for k, v in outs.items()}
    args = (H.ConvArgs * 12)()
    args2 = (H.ConvArgs * 12)()
    keep, singles = [], {4: [], 21: []}
    at = 0
    for mi, (m, c, a) in enumerate(C4_MAPS):
        f = r.uniform(0, 6, (batch, m, m, c)).astype(np.float32)
        fd = torch.from_numpy(f).cuda()
        for hi, last in enumerate((4, 21)):
            o = a * last
            wt = r.normal(0, 0.01, (o, c, 3, 3)).astype(np.float32)
            b = r.uniform(-0.1, 0.1, o).astype(np.float32)
            singles[last].append(gpu_conv(f, wt, b, 1, 1).reshape(batch, m * m * a, last))
            wd = pack_filter(wt, H.FILTER_OHWI)
            bd = torch.from_numpy(b).cuda()
            for arr, dst in ((args, outs), (args2, outs2)):
                ar = H.conv_args(fd.data_ptr(), wd.data_ptr(), bd.data_ptr(),
                                 dst[last].data_ptr() + at * last * 4, batch, m, m, c, o, 3, 1, 1)
                ar.out_image_stride = priors * last
                need = H.lib().ogle_hip_conv_workspace_bytes(ctypes.byref(ar))
                if need:
                    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
                    ar.workspace_dev, ar.workspace_bytes = ws.data_ptr(), need
                    keep.append(ws)
                arr[mi * 2 + hi] = ar
            keep += [fd, wd, bd]
        at += m * m * a
    H.check(H.lib().ogle_hip_conv2d_batch(args, 12, 0))
    open_ = (ctypes.c_int32 * 12)()
    H.check(H.lib().ogle_hip_conv2d_batch_begin(args2, 12, open_, 0))
    H.check(H.lib().ogle_hip_conv2d_batch_finish(args2, 12, 0))
    torch.cuda.synchronize()
    for last in (4, 21):
        ref = np.concatenate(singles[last], axis=1)
        np.testing.assert_array_equal(outs[last].cpu().numpy(), ref)
        np.testing.assert_array_equal(outs2[last].cpu().numpy(), ref)
    # the second map's box head moved one element into the first one's place
    args[2].output_dev -= 4
    assert H.lib().ogle_hip_conv2d_batch(args, 12, 0) == H.ERR_INVALID_ARG
    assert "depend on each other" in H.last_error()
    torch.cuda.synchronize()


def test_fp16_storage_depthwise_and_pool():
    """fp16 storage (fp32 accumulation) of the bandwidth-bound kernels.  Inputs are rounded to
    fp16 first, so the oracle sees the values the device stores; the result is then rounded to
    fp16 once on the device, which adds up to half an fp16 ulp of the output (subnormal
    outputs: half of 2^-24) on top of the 5e-3 bound."""
    r = rng(2600)

    def half_ulp(v):
        a = np.maximum(np.abs(v.astype(np.float64)), 2.0 ** -14)
        return 0.5 * 2.0 ** (np.floor(np.log2(a)) - 10)

    for (n, h, w, c, s) in ((2, 38, 38, 256, 1), (1, 19, 19, 512, 2), (3, 9, 7, 24, 1), (1, 5, 5, 8, 2)):
        x = r.uniform(0, 6, (n, h, w, c)).astype(np.float16).astype(np.float32)
        wd = r.normal(0, np.sqrt(2 / 9), (c, 1, 3, 3)).astype(np.float16).astype(np.float32)
        b = r.normal(0, 0.1, c).astype(np.float32)
        ref = O.conv2d(x, wd, b, s, 1, 1, c, O.ACT_CLIP, 0.0, 6.0)
        scale = O.conv2d_abs(x, wd, b, s, 1, 1, c)
        got = gpu_conv(x, wd, b, s, 1, 1, c, H.ACT_CLIP, 0.0, 6.0, dtype=H.F16)
        assert_conv_close(got, ref, scale + half_ulp(ref) / FP16_RTOL, FP16_RTOL,
                          "fp16 dw %dx%dx%d s%d" % (h, w, c, s))
    # tiny weights: outputs in fp16's subnormal range
    x = r.uniform(0, 1, (1, 6, 6, 8)).astype(np.float16).astype(np.float32)
    wd = (r.normal(0, 1, (8, 1, 3, 3)) * 2.0 ** -20).astype(np.float16).astype(np.float32)
    ref = O.conv2d(x, wd, None, 1, 1, 1, 8)
    got = gpu_conv(x, wd, None, 1, 1, 1, 8, dtype=H.F16)
    assert np.all(np.abs(got.astype(np.float64) - ref) <= half_ulp(ref) + 1e-30)
    for (k, s, p, pt) in ((3, 2, 1, H.POOL_MAX), (2, 2, 0, H.POOL_MAX), (3, 1, 1, H.POOL_AVG),
                          (2, 2, 0, H.POOL_AVG), (0, 0, 0, H.POOL_GLOBAL_AVG)):
        x = r.normal(0, 2, (2, 14, 14, 24)).astype(np.float16).astype(np.float32)
        ref = O.pool2d(x, k, s, p, pt)
        got = gpu_pool(x, k, s, p, pt, dtype=H.F16)
        if pt == H.POOL_MAX:
            np.testing.assert_array_equal(got, ref)       # a max of fp16 values is one of them
        else:
            assert np.all(np.abs(got.astype(np.float64) - ref) <= half_ulp(ref) * 1.01 + 1e-6 * np.abs(ref))


def test_config4_heads_concat_decode():
    """SSD heads (3x3 convs) -> concat -> softmax-max/threshold -> decode, batch 4 for the
    oracle-checked part (the oracle's convs at batch 64 take minutes)."""
    r = rng(20240004)
    batch = 4
    maps = [(19, 512, 3), (10, 1024, 6), (5, 512, 6), (3, 256, 6), (2, 256, 6), (1, 128, 6)]
    locs_ref, confs_ref, locs_gpu, confs_gpu = [], [], [], []
    for m, c, a in maps:
        f = r.uniform(0, 6, (batch, m, m, c)).astype(np.float32)
        wl = r.normal(0, 0.01, (a * 4, c, 3, 3)).astype(np.float32)
        wc = r.normal(0, 0.01, (a * 21, c, 3, 3)).astype(np.float32)
        for wt, refs, gpus, last in ((wl, locs_ref, locs_gpu, 4), (wc, confs_ref, confs_gpu, 21)):
            ref = O.conv2d(f, wt, None, 1, 1)
            got = gpu_conv(f, wt, None, 1, 1)
            assert_conv_close(got, ref, O.conv2d_abs(f, wt, None, 1, 1), FP32_RTOL, "head %d" % m)
            refs.append(ref.reshape(batch, -1, last))
            gpus.append(got.reshape(batch, -1, last))
    loc = gpu_concat(locs_gpu, 1)
    conf = gpu_concat(confs_gpu, 1)
    np.testing.assert_array_equal(loc, np.concatenate(locs_gpu, 1))
    np.testing.assert_array_equal(conf, np.concatenate(confs_gpu, 1))
    np.testing.assert_array_equal(O.concat(locs_ref, 1), np.concatenate(locs_ref, 1))
    assert loc.shape == (batch, 1917, 4) and conf.shape == (batch, 1917, 21)
    anchors = ssd_anchors()
    # Features ~U(0,6) over 9*C taps with weights ~N(0,0.01) give logits with a standard
    # deviation near 2, so a good share of the priors passes the 0.3 threshold.  The score
    # filter is compared on identical inputs: the device's own logits and decoded boxes.
    res, boxes = gpu_detect(conf, loc, anchors, 0.3, 300.0, 300.0)
    np.testing.assert_allclose(boxes, O.ssd_decode(loc, anchors), rtol=0, atol=1e-4)
    ora = O.box_info(conf, boxes, 0.3, 300.0, 300.0)
    for b in range(batch):
        assert len(ora[b]["prior"]) > 0
        assert_same_detections(res[b], ora[b], conf[b], 0.3, "C4 image %d" % b)
        np.testing.assert_array_equal(res[b]["prior"], ora[b]["prior"])
        np.testing.assert_array_equal(res[b]["cls"], ora[b]["cls"])


def test_config4_chained_at_batch64():
    """BASELINE config 4 at its full batch of 64, chained: the twelve heads as one grouped call
    -> the two concatenations -> decode + softmax-max + score filter, every stage fed with the
    device's output of the stage before.  The head convolutions are held to a float64 im2col
    product (the scalar oracle would take minutes at this size); concat, decode and the score
    filter to the oracle on the device's own inputs."""
    import ctypes
    import torch
    from util import pack_filter
    r = rng(20240004)
    batch = 64
    keep, heads = [], []
    args = (H.ConvArgs * 12)()
    for mi, (m, c, a) in enumerate(C4_MAPS):
        f = r.uniform(0, 6, (batch, m, m, c)).astype(np.float32)
        fd = torch.from_numpy(f).cuda()
        for hi, last in enumerate((4, 21)):
            o = a * last
            wt = r.normal(0, 0.01, (o, c, 3, 3)).astype(np.float32)
            wd = pack_filter(wt, H.FILTER_OHWI)
            y = torch.full((batch, m, m, o), float("nan"), device="cuda")
            ar = H.conv_args(fd.data_ptr(), wd.data_ptr(), None, y.data_ptr(), batch, m, m, c, o, 3, 1, 1)
            need = H.lib().ogle_hip_conv_workspace_bytes(ctypes.byref(ar))
            if need:
                ws = torch.empty(need, dtype=torch.uint8, device="cuda")
                ar.workspace_dev, ar.workspace_bytes = ws.data_ptr(), need
                keep.append(ws)
            args[mi * 2 + hi] = ar
            keep += [fd, wd]
            heads.append((m, a, last, f, wt, y))
    H.check(H.lib().ogle_hip_conv2d_batch(args, 12, 0))
    torch.cuda.synchronize()
    locs, confs = [], []
    for m, a, last, f, wt, y in heads:
        got = y.cpu().numpy()
        assert_conv_close(got, _conv3x3_f64(f, wt).astype(np.float32), _conv3x3_f64(np.abs(f), np.abs(wt)),
                          FP32_RTOL, "C4 b64 chained head %dx%d x%d" % (m, m, last))
        (locs if last == 4 else confs).append(got.reshape(batch, m * m * a, last))
    loc, conf = gpu_concat(locs, 1), gpu_concat(confs, 1)
    np.testing.assert_array_equal(loc, O.concat(locs, 1))
    np.testing.assert_array_equal(conf, O.concat(confs, 1))
    assert loc.shape == (batch, 1917, 4) and conf.shape == (batch, 1917, 21)
    anchors = ssd_anchors()
    res, boxes = gpu_detect(conf, loc, anchors, 0.3, 300.0, 300.0)
    np.testing.assert_allclose(boxes, O.ssd_decode(loc, anchors), rtol=0, atol=1e-4)
    ora = O.box_info(conf, boxes, 0.3, 300.0, 300.0)
    kept = 0
    for b in range(batch):
        assert_same_detections(res[b], ora[b], conf[b], 0.3, "C4 b64 image %d" % b)
        np.testing.assert_array_equal(res[b]["prior"], ora[b]["prior"])
        np.testing.assert_array_equal(res[b]["cls"], ora[b]["cls"])
        kept += len(ora[b]["prior"])
    assert kept > batch  # the threshold keeps a good share of the priors at these logits


@pytest.mark.parametrize("batch", [1, 64])
def test_detect_kept_sets_bit_exact(batch):
    """Logits scaled so that a few percent of the priors pass the threshold."""
    r = rng(20240014 + batch)
    priors, classes = 1917, 21
    logits = r.normal(0, 0.9, (batch, priors, classes)).astype(np.float32)
    pred = r.normal(0, 1.0, (batch, priors, 4)).astype(np.float32)
    anchors = ssd_anchors()
    res, boxes = gpu_detect(logits, pred, anchors, 0.3, 300.0, 300.0)
    ref_boxes = O.ssd_decode(pred, anchors)
    np.testing.assert_allclose(boxes, ref_boxes, rtol=0, atol=1e-4)
    # identical inputs to the score filter on both sides: the device's own decoded boxes
    ora = O.box_info(logits, boxes, 0.3, 300.0, 300.0)
    kept = 0
    for b in range(batch):
        assert_same_detections(res[b], ora[b], logits[b], 0.3, "image %d" % b)
        np.testing.assert_array_equal(res[b]["prior"], ora[b]["prior"])
        np.testing.assert_array_equal(res[b]["cls"], ora[b]["cls"])
        kept += len(res[b]["prior"])
    frac = kept / (batch * priors)
    assert 0.005 < frac < 0.6, frac
    # with already-decoded boxes as input
    res2, _ = gpu_detect(logits, None, None, 0.3, 300.0, 300.0, boxes_in=boxes)
    for b in range(batch):
        np.testing.assert_array_equal(res2[b]["prior"], ora[b]["prior"])
        np.testing.assert_array_equal(res2[b]["box"], ora[b]["box"])


def test_detect_single_kernel_path_and_optional_outputs():
    """Fewer than 257 priors, or a missing optional output, takes the one-kernel form."""
    import ctypes
    import torch
    r = rng(3300)
    for priors, drop_rect in ((200, False), (700, True)):
        logits = r.normal(0, 0.9, (3, priors, 21)).astype(np.float32)
        pred = r.normal(0, 1.0, (3, priors, 4)).astype(np.float32)
        anchors = np.concatenate([r.uniform(.1, .9, (priors, 2)), r.uniform(.05, .5, (priors, 2))],
                                 1).astype(np.float32)
        if not drop_rect:
            res, boxes = gpu_detect(logits, pred, anchors, 0.3, 100.0, 50.0)
            ora = O.box_info(logits, boxes, 0.3, 100.0, 50.0)
            for b in range(3):
                np.testing.assert_array_equal(res[b]["prior"], ora[b]["prior"])
                np.testing.assert_array_equal(res[b]["rect"], ora[b]["rect"])
            continue
        ld, pd, ad = (torch.from_numpy(a).cuda() for a in (logits, pred, anchors))
        cnt = torch.full((3,), -1, dtype=torch.int32, device="cuda")
        prior = torch.full((3, priors), -1, dtype=torch.int32, device="cuda")
        args = H.DetectArgs(ld.data_ptr(), pd.data_ptr(), ad.data_ptr(), None, 3, priors, 21, 0,
                            (ctypes.c_float * 4)(.1, .1, .2, .2), 0.3, 100.0, 50.0, cnt.data_ptr(),
                            prior.data_ptr(), None, None, None, None)
        H.check(H.lib().ogle_hip_ssd_detect(ctypes.byref(args), torch.cuda.current_stream().cuda_stream))
        torch.cuda.synchronize()
        ora = O.box_info(logits, O.ssd_decode(pred, anchors), 0.3, 100.0, 50.0)
        for b in range(3):
            k = int(cnt[b])
            np.testing.assert_array_equal(prior[b, :k].cpu().numpy(), ora[b]["prior"])


def test_device_exp_matches_host_libm():
    """The device exponential is the correctly rounded expf (binary64 exp, rounded once).  The
    host's libm expf is within 0.502 ulp of the true value, so the two agree except on the few
    inputs where libm is not correctly rounded; there they differ by one ulp."""
    import ctypes
    import torch
    r = rng(77)
    x = np.concatenate([r.uniform(-20, 20, 1 << 20), r.normal(0, 3, 1 << 20),
                        np.linspace(-87, 88, 1 << 18)]).astype(np.float32)
    xd = torch.from_numpy(x).cuda()
    yd = torch.empty_like(xd)
    H.check(H.lib().ogle_hip_expf(xd.data_ptr(), yd.data_ptr(), x.size,
                                  torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    got, ref = yd.cpu().numpy(), O.expf(x)
    mism = np.count_nonzero(got != ref)
    assert mism <= x.size * 2e-3, "device exp differs from libm expf on %d of %d inputs" % (mism, x.size)
    ulp = np.abs(got.view(np.int32).astype(np.int64) - ref.view(np.int32).astype(np.int64))
    assert ulp.max() <= 1
    # against binary64: the device result is the nearest binary32 to exp(x)
    exact = np.exp(x.astype(np.float64))
    ok = np.isfinite(ref) & (ref > 1e-37)
    dev_err = np.abs(got[ok].astype(np.float64) - exact[ok])
    host_err = np.abs(ref[ok].astype(np.float64) - exact[ok])
    assert np.all(dev_err <= host_err * (1 + 1e-12) + 0.0)


def test_decode_matches_oracle():
    r = rng(3100)
    anchors = ssd_anchors()
    pred = r.normal(0, 1.5, (3, 1917, 4)).astype(np.float32)
    got = gpu_decode(pred, anchors)
    np.testing.assert_allclose(got, O.ssd_decode(pred, anchors), rtol=0, atol=1e-4)
    # zero prediction: the anchor in corner form, exactly
    z = gpu_decode(np.zeros((1, 1917, 4), np.float32), anchors)
    exp = np.concatenate([anchors[:, :2] - anchors[:, 2:] * np.float32(0.5),
                          anchors[:, :2] + anchors[:, 2:] * np.float32(0.5)], 1)
    np.testing.assert_array_equal(z[0], exp)
    # per-image anchors (the graph-op form)
    a3 = np.stack([anchors, anchors * np.float32(0.5), anchors * np.float32(0.25)])
    got = gpu_decode(pred, a3)
    for b in range(3):
        np.testing.assert_allclose(got[b:b + 1], O.ssd_decode(pred[b:b + 1], a3[b]), rtol=0, atol=1e-4)


POOL_CASES = [
    (1, 112, 112, 64, 3, 2, 1), (2, 11, 9, 5, 2, 2, 0), (1, 8, 8, 7, 3, 1, 1), (3, 13, 13, 16, 5, 3, 2),
    (1, 4, 4, 4, 2, 2, 2),       # corner windows with no in-image tap
    (4, 112, 112, 64, 3, 2, 1),  # 3x3 stride 2 on a large map: the 2x2-patch kernel
    (3, 75, 61, 32, 3, 2, 0),    # the same with odd output sizes (the last patch row / column is half empty)
    (2, 90, 90, 16, 3, 2, 2),    # and with padding 2: whole windows outside the image
]


@pytest.mark.parametrize("case", POOL_CASES)
def test_pool_matches_oracle(case):
    n, h, w, c, k, s, p = case
    x = rng(4000 + h).normal(0, 1, (n, h, w, c)).astype(np.float32)
    np.testing.assert_array_equal(gpu_pool(x, k, s, p, H.POOL_MAX), O.pool2d(x, k, s, p, O.POOL_MAX))
    np.testing.assert_array_equal(gpu_pool(x, k, s, p, H.POOL_AVG), O.pool2d(x, k, s, p, O.POOL_AVG))


def test_global_average_pool():
    r = rng(4100)
    for (n, hw, c) in ((2, 7, 1024), (1, 3, 10), (3, 10, 130)):
        x = r.normal(0, 1, (n, hw, hw, c)).astype(np.float32)
        got = gpu_pool(x, 0, 0, 0, H.POOL_GLOBAL_AVG)
        ref = O.pool2d(x, 0, 0, 0, O.POOL_GLOBAL_AVG)
        scale = np.abs(x).sum(axis=(1, 2), keepdims=True) / (hw * hw)
        assert np.all(np.abs(got - ref) <= 1e-5 * scale + 1e-12)


@pytest.mark.parametrize("rank", [1, 2, 3, 4])
def test_concat_every_axis(rank):
    r = rng(5000 + rank)
    base = [2, 3, 5, 4][:rank]
    for axis in list(range(rank)) + [-1]:
        for lens in ((1, 4, 2), (8, 4), (3, 1, 2, 5, 7, 1)):
            ins = []
            for ln in lens:
                shp = list(base)
                shp[axis] = ln
                ins.append(r.normal(0, 1, shp).astype(np.float32))
            np.testing.assert_array_equal(gpu_concat(ins, axis), O.concat(ins, axis))


def test_concat_ssd_shapes_batch64():
    r = rng(5100)
    for last in (4, 21):
        ins = [r.normal(0, 1, (64, p, last)).astype(np.float32) for p in (1083, 600, 150, 54, 24, 6)]
        np.testing.assert_array_equal(gpu_concat(ins, 1), np.concatenate(ins, 1))


@pytest.mark.parametrize("seed,stride,topk,spread", [
    (1, 1917, 100, 300), (2, 1917, 100, 40), (3, 257, 16, 60), (4, 64, 100, 30), (5, 1917, 1024, 200),
    (6, 8192, 200, 500), (7, 5, 1, 10),
])
def test_topk_nms_matches_oracle(seed, stride, topk, spread):
    """Device top-k + NMS against the oracle's restatement of GetTopK + NMS (detector.cc:114-148):
    quantised scores force ties (stable order = prior order), rectangles cluster so that many
    overlap, include zero-area and negative-size boxes, and one image is empty, one full."""
    r = rng(9000 + seed)
    batch = 5
    counts = np.array([0, stride, min(stride, 3), stride // 2, min(stride, 131)], np.int32)
    prior = np.zeros((batch, stride), np.int32)
    cls = r.integers(1, 21, (batch, stride)).astype(np.int32)
    score = (r.integers(301, 1000, (batch, stride)) / 1000.0).astype(np.float32)   # many equal scores
    score[3] = r.uniform(0.3, 1.0, stride).astype(np.float32)                      # and one image without ties
    xy = r.integers(-20, spread, (batch, stride, 2))
    wh = r.integers(-3, 80, (batch, stride, 2))
    rect = np.concatenate([xy, wh], -1).astype(np.int32)
    box = r.uniform(0, 300, (batch, stride, 4)).astype(np.float32)
    for b in range(batch):
        prior[b, :counts[b]] = np.sort(r.choice(max(stride, 1) * 3, counts[b], replace=False))
    got = gpu_topk_nms(counts, prior, cls, score, rect, topk, 0.45, box)
    for b in range(batch):
        n = counts[b]
        keep = O.topk_nms(score[b, :n], rect[b, :n], topk, 0.45)
        np.testing.assert_array_equal(got[b]["prior"], prior[b, :n][keep])
        np.testing.assert_array_equal(got[b]["cls"], cls[b, :n][keep])
        np.testing.assert_array_equal(got[b]["score"], score[b, :n][keep])
        np.testing.assert_array_equal(got[b]["rect"], rect[b, :n][keep])
        np.testing.assert_array_equal(got[b]["box"], box[b, :n][keep])


@pytest.mark.parametrize("batch,priors,topk,sigma", [(1, 1917, 100, 0.9), (16, 1917, 100, 0.9),
                                                     (3, 1917, 100, 0.35), (2, 1917, 1024, 2.0),
                                                     (4, 300, 16, 1.0), (2, 70, 200, 1.0)])
def test_detect_lists_in_place_then_topk_nms(batch, priors, topk, sigma):
    """ogle_hip_ssd_detect without kept_count_dev leaves every prior's record at its own slot
    (kept_prior = index or -1, no compaction launch); ogle_hip_ssd_topk_nms without
    kept_count_dev reads such lists.  The final lists must equal, bit for bit, those of the
    compacted path, which other tests hold to the oracle."""
    import ctypes
    import torch
    r = rng(9700 + batch + priors + topk)
    classes = 21
    logits = r.normal(0, sigma, (batch, priors, classes)).astype(np.float32)
    logits[0] = np.round(logits[0] * 4) / 4      # frequent equal scores in image 0
    pred = r.normal(0, 1.0, (batch, priors, 4)).astype(np.float32)
    anchors = ssd_anchors() if priors == 1917 else np.concatenate(
        [r.uniform(.1, .9, (priors, 2)), r.uniform(.05, .5, (priors, 2))], 1).astype(np.float32)
    kept, boxes = gpu_detect(logits, pred, anchors, 0.3, 300.0, 300.0)
    counts = np.array([len(k["prior"]) for k in kept], np.int32)

    def padded(key, shape, dtype):
        out = np.zeros((batch,) + shape, dtype)
        for b in range(batch):
            out[b, :counts[b]] = kept[b][key]
        return out
    ref = gpu_topk_nms(counts, padded("prior", (priors,), np.int32), padded("cls", (priors,), np.int32),
                       padded("score", (priors,), np.float32), padded("rect", (priors, 4), np.int32),
                       topk, 0.45, padded("box", (priors, 4), np.float32))
    i32 = dict(dtype=torch.int32, device="cuda")
    f32 = dict(dtype=torch.float32, device="cuda")
    ld, pd, ad = (torch.from_numpy(a).cuda() for a in (logits, pred, anchors))
    bx = torch.empty((batch, priors, 4), **f32)
    kp = torch.full((batch, priors), -5, **i32)
    kc = torch.full((batch, priors), -5, **i32)
    ks = torch.full((batch, priors), float("nan"), **f32)
    kb = torch.full((batch, priors, 4), float("nan"), **f32)
    kr = torch.full((batch, priors, 4), -5, **i32)
    st = torch.cuda.current_stream().cuda_stream
    da = H.DetectArgs(ld.data_ptr(), pd.data_ptr(), ad.data_ptr(), bx.data_ptr(), batch, priors, classes,
                      0, (ctypes.c_float * 4)(.1, .1, .2, .2), 0.3, 300.0, 300.0, None, kp.data_ptr(),
                      kc.data_ptr(), ks.data_ptr(), kb.data_ptr(), kr.data_ptr())
    H.check(H.lib().ogle_hip_ssd_detect(ctypes.byref(da), st))
    fc = torch.full((batch,), -7, **i32)
    fp = torch.full((batch, topk), -7, **i32)
    fk = torch.full((batch, topk), -7, **i32)
    fs = torch.full((batch, topk), float("nan"), **f32)
    fb = torch.full((batch, topk, 4), float("nan"), **f32)
    fr = torch.full((batch, topk, 4), -7, **i32)
    na = H.NmsArgs(None, kp.data_ptr(), kc.data_ptr(), ks.data_ptr(), kb.data_ptr(), kr.data_ptr(), batch,
                   priors, topk, 0.45, fc.data_ptr(), fp.data_ptr(), fk.data_ptr(), fs.data_ptr(),
                   fb.data_ptr(), fr.data_ptr())
    H.check(H.lib().ogle_hip_ssd_topk_nms(ctypes.byref(na), st))
    torch.cuda.synchronize()
    # the in-place lists: kept priors carry their index, dropped ones -1
    kpn = kp.cpu().numpy()
    for b in range(batch):
        np.testing.assert_array_equal(np.nonzero(kpn[b] >= 0)[0], kept[b]["prior"])
        assert np.all((kpn[b] == -1) | (kpn[b] == np.arange(priors)))
    n = fc.cpu().numpy()
    for b in range(batch):
        k = int(n[b])
        assert k == len(ref[b]["prior"]), (b, k)
        np.testing.assert_array_equal(fp[b, :k].cpu().numpy(), ref[b]["prior"])
        np.testing.assert_array_equal(fk[b, :k].cpu().numpy(), ref[b]["cls"])
        np.testing.assert_array_equal(fs[b, :k].cpu().numpy(), ref[b]["score"])
        np.testing.assert_array_equal(fr[b, :k].cpu().numpy(), ref[b]["rect"])
        np.testing.assert_array_equal(fb[b, :k].cpu().numpy(), ref[b]["box"])
        assert (fp[b, k:] == -7).all()
    # in-place lists need every list
    da.kept_rect_dev = None
    assert H.lib().ogle_hip_ssd_detect(ctypes.byref(da), st) == H.ERR_INVALID_ARG


def test_topk_nms_known_answers_on_device():
    """The hand-built cases of tests/test_oracle.py::test_topk_nms_known_answers on the device,
    with the answers written out (not taken from the oracle): a dropped box still drops a later
    one (detector.cc:127-148), top-k cuts before the suppression, equal scores keep prior order."""
    A, B, C, D = (0, 0, 100, 100), (30, 0, 100, 100), (60, 0, 100, 100), (300, 300, 50, 50)
    cases = [  # rects, scores, topk -> surviving input positions, in sorted order
        ([A, B, C, D], [0.9, 0.8, 0.7, 0.6], 100, [0, 3]),
        ([C, D, A, B], [0.7, 0.6, 0.9, 0.8], 100, [2, 1]),
        ([A, C, D], [0.9, 0.7, 0.6], 100, [0, 1, 2]),
        ([A, B, C, D], [0.9, 0.8, 0.7, 0.6], 2, [0]),
        ([A, B, D], [0.8, 0.8, 0.8], 100, [0, 2]),
        ([B, A, D], [0.8, 0.8, 0.8], 100, [0, 2]),
        ([D, B, A], [0.8, 0.8, 0.8], 2, [0, 1]),
    ]
    stride = 4
    for topk in (100, 2):
        sel = [c for c in cases if c[2] == topk]
        batch = len(sel)
        counts = np.array([len(c[0]) for c in sel], np.int32)
        rect = np.zeros((batch, stride, 4), np.int32)
        score = np.zeros((batch, stride), np.float32)
        prior = np.tile(np.arange(stride, dtype=np.int32) * 10 + 3, (batch, 1))
        cls = np.tile(np.arange(1, stride + 1, dtype=np.int32), (batch, 1))
        for b, (rc, sc, _, _) in enumerate(sel):
            rect[b, :len(rc)] = rc
            score[b, :len(sc)] = sc
        got = gpu_topk_nms(counts, prior, cls, score, rect, topk, 0.45)
        for b, (_, _, _, expect) in enumerate(sel):
            np.testing.assert_array_equal(got[b]["prior"], prior[b][expect])
            np.testing.assert_array_equal(got[b]["cls"], cls[b][expect])
            np.testing.assert_array_equal(got[b]["rect"], rect[b][expect])


def test_topk_nms_rejects_bad_sizes():
    import ctypes
    a = H.NmsArgs()
    a.batch, a.stride, a.topk = 1, 100, 0
    assert H.lib().ogle_hip_ssd_topk_nms(ctypes.byref(a), 0) == H.ERR_UNSUPPORTED
    a.topk = 2000
    assert H.lib().ogle_hip_ssd_topk_nms(ctypes.byref(a), 0) == H.ERR_UNSUPPORTED
    a.topk, a.stride = 10, 10000
    assert H.lib().ogle_hip_ssd_topk_nms(ctypes.byref(a), 0) == H.ERR_UNSUPPORTED
    a.stride = 100
    assert H.lib().ogle_hip_ssd_topk_nms(ctypes.byref(a), 0) == H.ERR_INVALID_ARG   # null pointers


def test_kernels_against_committed_vectors():
    """The HIP kernels on the inputs stored in tests/golden/oracle_vectors.npz against the
    outputs stored beside them (written by the oracle, tests/golden/make_golden.py)."""
    import os
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "oracle_vectors.npz")
    g = dict(np.load(path))
    x = g["dense_x"]
    for name, w, b, kw, ref in (
            ("dense", g["dense_w"], g["dense_b"], dict(stride=2, pad=1, act=H.ACT_RELU), g["dense_y"]),
            ("dw", g["dw_w"], g["dw_b"], dict(stride=1, pad=1, groups=8, act=H.ACT_CLIP, maxv=6.0), g["dw_y"]),
            ("pw", g["pw_w"], g["pw_b"], dict(act=H.ACT_CLIP, minv=-1.0, maxv=0.5, variant=H.VARIANT_PW), g["pw_y"])):
        got = gpu_conv(x, w, b, **kw)
        scale = O.conv2d_abs(x, w, b, kw.get("stride", 1), kw.get("pad", 0), 1, kw.get("groups", 1))
        assert_conv_close(got, ref, scale, FP32_RTOL, name)
    np.testing.assert_array_equal(gpu_pool(x, 3, 2, 1, O.POOL_MAX), g["maxpool_y"])
    np.testing.assert_allclose(gpu_pool(x, 2, 2, 0, O.POOL_AVG), g["avgpool_y"], rtol=1e-6, atol=1e-7)
    np.testing.assert_array_equal(gpu_concat([g["cat_a"], g["cat_b"], g["cat_c"]], 1), g["cat_y"])
    res, boxes = gpu_detect(g["ssd_logits"], g["ssd_pred"], g["ssd_anchors"], 0.3, 320.0, 240.0)
    np.testing.assert_allclose(boxes, g["ssd_boxes"], rtol=1e-5, atol=1e-6)
    for i in range(2):
        ora = {k: g["info%d_%s" % (i, k)] for k in ("prior", "cls", "score", "box", "rect")}
        assert_same_detections(res[i], ora, g["ssd_logits"][i], 0.3, "image %d" % i)
        n = len(ora["prior"])
        final = gpu_topk_nms(np.array([n], np.int32), ora["prior"][None], ora["cls"][None],
                             ora["score"][None], ora["rect"][None], 5, 0.45)
        np.testing.assert_array_equal(final[0]["prior"], ora["prior"][g["info%d_keep" % i]])


def test_fp16_wide_tile_large_pointwise():
    """fp16 storage with at least 512 tiles of 128x256 outputs takes the wide-tile kernel
    (64x128 outputs per wave, 64-byte K slabs); ragged M, and K with a half-filled last slab."""
    import torch
    r = rng(2700)
    n, h, w, c, o = 17, 32, 31, 72, 1024          # M = 16864 (not a multiple of 128), K = 72
    x = r.uniform(0, 2, (n, h, w, c)).astype(np.float16).astype(np.float32)
    wt = r.normal(0, np.sqrt(2 / c), (o, c, 1, 1)).astype(np.float16).astype(np.float32)
    b = r.uniform(-0.1, 0.1, o).astype(np.float32)
    got = gpu_conv(x, wt, b, act=H.ACT_RELU, variant=H.VARIANT_PW, dtype=H.F16)
    a64 = x.reshape(-1, c).astype(np.float64)
    w64 = wt.reshape(o, c).astype(np.float64)
    ref = np.maximum(a64 @ w64.T + b, 0).astype(np.float32)
    scale = np.abs(a64) @ np.abs(w64).T + np.abs(b)
    half_ulp = 0.5 * 2.0 ** (np.floor(np.log2(np.maximum(np.abs(ref.astype(np.float64)), 2.0 ** -14))) - 10)
    assert_conv_close(got.reshape(-1, o), ref, (scale + half_ulp / FP16_RTOL).astype(np.float32), FP16_RTOL,
                      "fp16 wide tile")


ASYNC_F16_CASES = [
    # n, h, w, c, o, bias, act, image stride beyond dense (elements)
    (8, 64, 63, 264, 512, True, H.ACT_CLIP, 0),      # 256x256 tiles; ragged M; K ends inside a stage
    (32, 19, 19, 512, 1000, True, H.ACT_RELU, 0),    # 192x256 tiles; ragged M and N (config 3's M, K)
    (32, 19, 19, 256, 768, False, H.ACT_NONE, 64),   # no bias, images stored with a gap after each
    (36, 19, 19, 2048, 512, True, H.ACT_RELU, 0),    # a long contraction: the stage ring turns 16 times
]


@pytest.mark.parametrize("case", ASYNC_F16_CASES)
def test_fp16_async_pointwise_gemm(case):
    """fp16 storage, pointwise, at least 256 input channels and enough 256-wide tiles: the kernel
    that streams its operands straight into LDS (256x256 / 192x256 tiles, eight waves in two
    alternating groups).  Against a float64 product of the fp16-rounded operands; the first image
    also against the oracle."""
    n, h, w, c, o, with_bias, act, gap = case
    r = rng(2800 + c)
    x = r.uniform(0, 2, (n, h, w, c)).astype(np.float16).astype(np.float32)
    wt = r.normal(0, np.sqrt(2 / c), (o, c, 1, 1)).astype(np.float16).astype(np.float32)
    b = r.uniform(-0.1, 0.1, o).astype(np.float32) if with_bias else None
    stride = h * w * o + gap if gap else 0
    got = gpu_conv(x, wt, b, act=act, maxv=1.5, variant=H.VARIANT_PW, dtype=H.F16, image_stride=stride)
    if gap:   # the gaps keep their NaN fill, the images are dense runs
        got = got.reshape(n, stride)
        assert np.isnan(got[:, h * w * o:]).all()
        got = got[:, :h * w * o]
    a64 = x.reshape(-1, c).astype(np.float64)
    w64 = wt.reshape(o, c).astype(np.float64)
    ref = a64 @ w64.T + (b if with_bias else 0.0)
    if act == H.ACT_RELU:
        ref = np.maximum(ref, 0)
    elif act == H.ACT_CLIP:
        ref = np.clip(ref, 0, 1.5)
    ref = ref.astype(np.float32)
    scale = np.abs(a64) @ np.abs(w64).T + (np.abs(b) if with_bias else 0.0)
    half_ulp = 0.5 * 2.0 ** (np.floor(np.log2(np.maximum(np.abs(ref.astype(np.float64)), 2.0 ** -14))) - 10)
    what = "fp16 async %s" % (case,)
    assert_conv_close(got.reshape(-1, o), ref, (scale + half_ulp / FP16_RTOL).astype(np.float32), FP16_RTOL, what)
    ora = O.conv2d(x[:1], wt, b, act={H.ACT_RELU: O.ACT_RELU, H.ACT_CLIP: O.ACT_CLIP, H.ACT_NONE: O.ACT_NONE}[act],
                   maxv=1.5, variant=O.VARIANT_PW)
    assert_conv_close(got.reshape(n, h, w, o)[:1], ora,
                      (scale + half_ulp / FP16_RTOL)[:h * w].reshape(1, h, w, o).astype(np.float32), FP16_RTOL,
                      what + " vs oracle")


def test_fp16_async_gemm_random_shapes_are_reproducible():
    """Seeded random shapes that the direct-to-LDS kernel takes (ragged M, K and N included): the
    result equals a float64 product of the fp16-rounded operands within the fp16 rule, and five
    launches on the same operands give bit-identical outputs (a stage buffer overwritten before
    every wave has read it, or read before it has landed, would show up as a difference between
    launches long before it showed up against the reference)."""
    import ctypes
    import torch
    from util import dev, pack_filter, stream_ptr
    r = rng(424242)
    taken = 0
    for _ in range(8):
        c = int(r.integers(32, 161)) * 8            # 256 .. 1280 input channels
        o = int(r.choice([512, 768, 1024])) - int(r.integers(0, 8)) * 8   # two to four tile columns
        m_rows = int(r.integers(13000, 30000))      # at least 128 tiles: the kernel's own threshold
        n, hw = 1, m_rows
        x = r.uniform(0, 2, (n, hw, 1, c)).astype(np.float16)
        wt = r.normal(0, np.sqrt(2 / c), (o, c, 1, 1)).astype(np.float16)
        b = r.uniform(-0.1, 0.1, o).astype(np.float32)
        xd = dev(x.astype(np.float32), torch.float16)
        wd = pack_filter(wt.astype(np.float32), H.FILTER_OHWI, H.F16)
        bd = dev(b)
        args = H.conv_args(xd.data_ptr(), wd.data_ptr(), bd.data_ptr(), 0, n, hw, 1, c, o, 1, 1, 0, 1, 1,
                           H.ACT_RELU, 0.0, 0.0, H.VARIANT_PW, H.F16)
        outs = []
        for _rep in range(5):
            y = torch.full((n, hw, 1, o), float("nan"), dtype=torch.float16, device="cuda")
            args.output_dev = y.data_ptr()
            H.check(H.lib().ogle_hip_pwconv_gemm(ctypes.byref(args), stream_ptr()))
            torch.cuda.synchronize()
            outs.append(y.cpu().numpy())
        for other in outs[1:]:
            assert np.array_equal(outs[0].view(np.uint16), other.view(np.uint16)), (c, o, m_rows)
        a64 = x.reshape(-1, c).astype(np.float64)
        w64 = wt.reshape(o, c).astype(np.float64)
        ref = np.maximum(a64 @ w64.T + b, 0).astype(np.float32)
        scale = np.abs(a64) @ np.abs(w64).T + np.abs(b)
        half_ulp = 0.5 * 2.0 ** (np.floor(np.log2(np.maximum(np.abs(ref.astype(np.float64)), 2.0 ** -14))) - 10)
        assert_conv_close(outs[0].astype(np.float32).reshape(-1, o), ref,
                          (scale + half_ulp / FP16_RTOL).astype(np.float32), FP16_RTOL,
                          "fp16 async random (M %d K %d N %d)" % (m_rows, c, o))
        taken += 1
    assert taken == 8


SPLIT_CASES = [
    # n, h, w, c, o1, o2, k, s, p, dtype       (output channels [0,o1) -> y, [o1,o1+o2) -> y2)
    (4, 19, 19, 128, 12, 63, 3, 1, 1, H.F32),      # SSD box + class head, 128x96 tile, element stores
    (2, 10, 10, 256, 24, 126, 3, 1, 1, H.F32),     # 128x160 tile
    (3, 9, 9, 64, 32, 64, 3, 1, 1, H.F32),         # both parts multiples of 4: 16-byte stores
    (2, 7, 7, 96, 40, 24, 1, 1, 0, H.F32),         # pointwise, 64x64 tiles
    (1, 3, 3, 128, 24, 126, 3, 1, 1, H.F32),       # tiny map: the wave-split kernel
    (1, 1, 1, 128, 24, 126, 3, 1, 1, H.F32),       # one pixel
    (2, 9, 9, 64, 16, 48, 3, 1, 1, H.F16),         # fp16 storage
]


@pytest.mark.parametrize("case", SPLIT_CASES)
@pytest.mark.parametrize("workspace", [True, False])
def test_conv_two_destinations(case, workspace):
    """OgleConvArgs.output2_dev: one contraction over the concatenated filters writes each
    part's channels to its own dense tensor; equal to the oracle run on each filter."""
    import ctypes
    import torch
    from util import dev, pack_filter, stream_ptr
    n, h, w, c, o1, o2, k, s, p, dtype = case
    r = rng(2800 + SPLIT_CASES.index(case))
    x = r.uniform(-1, 1, (n, h, w, c)).astype(np.float32)
    wt = r.normal(0, 0.2, (o1 + o2, c, k, k)).astype(np.float32)
    b = r.uniform(-0.1, 0.1, o1 + o2).astype(np.float32)
    tdt = torch.float32
    if dtype == H.F16:
        x, wt = x.astype(np.float16).astype(np.float32), wt.astype(np.float16).astype(np.float32)
        tdt = torch.float16
    xd, bd, wd = dev(x, tdt), dev(b), pack_filter(wt, H.FILTER_OHWI, dtype)
    oh, ow = H.out_size(h, k, s, p), H.out_size(w, k, s, p)
    y1 = torch.full((n, oh, ow, o1), float("nan"), dtype=tdt, device="cuda")
    y2 = torch.full((n, oh, ow, o2), float("nan"), dtype=tdt, device="cuda")
    a = H.conv_args(xd.data_ptr(), wd.data_ptr(), bd.data_ptr(), y1.data_ptr(), n, h, w, c, o1 + o2, k, s, p,
                    act=H.ACT_RELU, dtype=dtype)
    a.output2_dev, a.out_c_split = y2.data_ptr(), o1
    ws = None
    if workspace:
        need = H.lib().ogle_hip_conv_workspace_bytes(ctypes.byref(a))
        if need:
            ws = torch.empty(need, dtype=torch.uint8, device="cuda")
            a.workspace_dev, a.workspace_bytes = ws.data_ptr(), need
    H.check(H.lib().ogle_hip_conv2d(ctypes.byref(a), stream_ptr()))
    torch.cuda.synchronize()
    rtol = FP16_RTOL if dtype == H.F16 else FP32_RTOL
    for part, (lo, hi, y) in enumerate(((0, o1, y1), (o1, o1 + o2, y2))):
        ref = O.conv2d(x, wt[lo:hi], b[lo:hi], s, p, 1, 1, O.ACT_RELU)
        scale = O.conv2d_abs(x, wt[lo:hi], b[lo:hi], s, p, 1, 1)
        if dtype == H.F16:
            scale = scale + 2.0 ** -11 * np.abs(ref) / FP16_RTOL + 1e-3
        assert_conv_close(y.float().cpu().numpy(), ref, scale, rtol, "two destinations part %d %s" % (part, case))


def test_conv_two_destinations_errors():
    import ctypes
    import torch
    from util import stream_ptr
    x = torch.zeros((1, 4, 4, 6), device="cuda")      # C % 4 != 0: no MFMA path
    w = torch.zeros((8 * 6 * 9,), device="cuda")
    y1, y2 = torch.zeros((1, 4, 4, 3), device="cuda"), torch.zeros((1, 4, 4, 5), device="cuda")
    a = H.conv_args(x.data_ptr(), w.data_ptr(), None, y1.data_ptr(), 1, 4, 4, 6, 8, 3, 1, 1)
    a.output2_dev, a.out_c_split = y2.data_ptr(), 3
    assert H.lib().ogle_hip_conv2d(ctypes.byref(a), stream_ptr()) == H.ERR_UNSUPPORTED
    assert "MFMA" in H.last_error()
    for bad in (0, 8, -1):
        a.out_c_split = bad
        assert H.lib().ogle_hip_conv2d(ctypes.byref(a), stream_ptr()) == H.ERR_INVALID_ARG
    torch.cuda.synchronize()


def test_conv_batch_begin_finish_equals_batch():
    """ogle_hip_conv2d_batch_begin + _finish: the same outputs as ogle_hip_conv2d_batch, bit for
    bit, with the reductions of every split-K plan launched once at the end."""
    import ctypes
    import torch
    from util import pack_filter
    r = rng(2900)
    cases = [(4, 19, 19, 128, 12, 3, 1, 1), (4, 10, 10, 256, 126, 3, 1, 1), (2, 7, 7, 64, 96, 1, 1, 0),
             (1, 5, 5, 512, 24, 3, 1, 1), (16, 19, 19, 64, 64, 1, 1, 0)]
    args1, args2 = (H.ConvArgs * len(cases))(), (H.ConvArgs * len(cases))()
    keep, outs = [], []
    for i, (n, h, w, c, o, k, st, p) in enumerate(cases):
        x = torch.from_numpy(r.uniform(-1, 1, (n, h, w, c)).astype(np.float32)).cuda()
        wd = pack_filter(r.normal(0, 0.2, (o, c, k, k)).astype(np.float32), H.FILTER_OHWI)
        b = torch.from_numpy(r.uniform(-.1, .1, o).astype(np.float32)).cuda()
        oh, ow = H.out_size(h, k, st, p), H.out_size(w, k, st, p)
        ya = torch.full((n, oh, ow, o), float("nan"), device="cuda")
        yb = torch.full((n, oh, ow, o), float("nan"), device="cuda")
        a = H.conv_args(x.data_ptr(), wd.data_ptr(), b.data_ptr(), ya.data_ptr(), n, h, w, c, o, k, st, p,
                        1, 1, H.ACT_RELU)
        need = H.lib().ogle_hip_conv_workspace_bytes(ctypes.byref(a))
        wsa = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
        wsb = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
        if need:
            a.workspace_dev, a.workspace_bytes = wsa.data_ptr(), need
        args1[i] = a
        a.output_dev = yb.data_ptr()
        if need:
            a.workspace_dev = wsb.data_ptr()
        args2[i] = a
        keep += [x, wd, b, wsa, wsb]
        outs.append((ya, yb))
    H.check(H.lib().ogle_hip_conv2d_batch(args1, len(cases), 0))
    open_ = (ctypes.c_int32 * len(cases))()
    before = H.lib().ogle_hip_launch_count()
    H.check(H.lib().ogle_hip_conv2d_batch_begin(args2, len(cases), open_, 0))
    assert sum(open_) >= 2                       # the long-K heads leave partial sums
    torch.cuda.synchronize()
    for (ya, yb), pending in zip(outs, open_):
        if not pending:
            assert torch.equal(ya, yb)
    mid = H.lib().ogle_hip_launch_count()
    H.check(H.lib().ogle_hip_conv2d_batch_finish(args2, len(cases), 0))
    assert H.lib().ogle_hip_launch_count() - mid == 1     # one grid for every open reduction
    assert mid > before
    torch.cuda.synchronize()
    for ya, yb in outs:
        assert torch.equal(ya, yb)


def test_kernel_timing_events():
    """ogle_hip_kernel_timing_begin / _end: one device-stamped duration per launched kernel."""
    import ctypes
    import torch
    x = torch.rand(4, 64, 64, 64, device="cuda")
    y = torch.empty_like(x)
    ua = H.UnaryArgs(x.data_ptr(), y.data_ptr(), x.numel(), H.UNARY_CLIP, 0.0, 0.5, H.F32)
    torch.cuda.synchronize()
    assert H.lib().ogle_hip_kernel_timing_begin() == 0
    c0 = H.lib().ogle_hip_launch_count()
    for _ in range(5):
        H.check(H.lib().ogle_hip_unary(ctypes.byref(ua), 0))
    buf = (ctypes.c_float * 8)()
    n = H.lib().ogle_hip_kernel_timing_end(buf, 8)
    assert n == 5 == H.lib().ogle_hip_launch_count() - c0
    assert all(0.5 < buf[i] < 500.0 for i in range(5)), list(buf)
    assert H.lib().ogle_hip_kernel_timing_end(buf, 8) == 0      # nothing recorded while off
    assert torch.equal(y, x.clamp(0.0, 0.5))
