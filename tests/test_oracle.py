"""Pins the CPU oracle against library routines, closed forms and brute force.

The reference holds no stored vectors for this path (its tests draw unseeded
random inputs and compare with in-test CPU functions), so each oracle function
is pinned here by checks an indexing, sign or transposition mistake would fail.
"""
import itertools

import numpy as np
import pytest
import scipy.signal
import torch
import torch.nn.functional as F

import oracle as O


def rng(seed):
    return np.random.Generator(np.random.PCG64(seed))


def torch_conv(x, w, b, stride, pad, dil, groups):
    xt = torch.from_numpy(x).double().permute(0, 3, 1, 2)
    y = F.conv2d(xt, torch.from_numpy(w).double(),
                 None if b is None else torch.from_numpy(b).double(),
                 stride=stride, padding=pad, dilation=dil, groups=groups)
    return y.permute(0, 2, 3, 1).numpy()


CONV_CASES = [
    # n, h, w, c, o, k, s, p, d, g
    (1, 3, 3, 3, 1, 3, 1, 1, 1, 1),
    (2, 7, 5, 4, 6, 3, 1, 1, 1, 1),
    (1, 9, 9, 5, 7, 3, 2, 1, 1, 1),
    (1, 8, 8, 3, 4, 3, 1, 2, 2, 1),     # dilation 2
    (2, 6, 6, 8, 8, 3, 1, 1, 1, 8),     # depthwise
    (1, 6, 7, 8, 12, 3, 2, 1, 1, 4),    # grouped
    (3, 5, 5, 16, 9, 1, 1, 0, 1, 1),    # pointwise
    (1, 10, 10, 6, 4, 5, 1, 2, 1, 1),   # 5x5
    (1, 4, 4, 2, 3, 1, 2, 0, 1, 1),     # 1x1 stride 2
    (1, 1, 1, 20, 5, 3, 1, 1, 1, 1),    # 1x1 image, padded 3x3
]


@pytest.mark.parametrize("case", CONV_CASES)
@pytest.mark.parametrize("use_bias", [False, True])
def test_conv_matches_torch(case, use_bias):
    n, h, w, c, o, k, s, p, d, g = case
    r = rng(hash(case) % 2**31)
    x = r.uniform(-1, 1, (n, h, w, c)).astype(np.float32)
    wt = r.normal(0, 0.5, (o, c // g, k, k)).astype(np.float32)
    b = r.uniform(-0.1, 0.1, o).astype(np.float32) if use_bias else None
    got = O.conv2d(x, wt, b, s, p, d, g)
    ref = torch_conv(x, wt, b, s, p, d, g)
    assert got.shape == ref.shape
    scale = O.conv2d_abs(x, wt, b, s, p, d, g)
    assert np.all(np.abs(got - ref) <= 2e-6 * scale + 1e-12)


def test_conv_brute_force_tiny():
    r = rng(1)
    n, h, w, c, o, k, s, p = 1, 4, 3, 2, 3, 3, 1, 1
    x = r.integers(-3, 4, (n, h, w, c)).astype(np.float32)
    wt = r.integers(-2, 3, (o, c, k, k)).astype(np.float32)
    b = r.integers(-2, 3, o).astype(np.float32)
    ref = np.zeros((n, h, w, o), np.float64)
    for oy, ox, oc in itertools.product(range(h), range(w), range(o)):
        acc = float(b[oc])
        for ky, kx, ci in itertools.product(range(k), range(k), range(c)):
            iy, ix = oy * s - p + ky, ox * s - p + kx
            if 0 <= iy < h and 0 <= ix < w:
                acc += float(x[0, iy, ix, ci]) * float(wt[oc, ci, ky, kx])
        ref[0, oy, ox, oc] = acc
    np.testing.assert_array_equal(O.conv2d(x, wt, b, s, p), ref.astype(np.float32))


def test_conv_all_ones_counts_taps():
    h, w, c, o = 5, 6, 7, 3
    x = np.ones((1, h, w, c), np.float32)
    wt = np.ones((o, c, 3, 3), np.float32)
    y = O.conv2d(x, wt, None, 1, 1)
    ys = np.minimum(np.arange(h) + 2, h) - np.maximum(np.arange(h) - 1, 0)
    xs = np.minimum(np.arange(w) + 2, w) - np.maximum(np.arange(w) - 1, 0)
    expect = (ys[:, None] * xs[None, :] * c).astype(np.float32)
    for oc in range(o):
        np.testing.assert_array_equal(y[0, :, :, oc], expect)


def test_pointwise_is_matmul():
    r = rng(3)
    x = r.uniform(0, 6, (2, 5, 5, 32)).astype(np.float32)
    wt = r.normal(0, 0.25, (48, 32, 1, 1)).astype(np.float32)
    b = r.uniform(-0.1, 0.1, 48).astype(np.float32)
    y = O.conv2d(x, wt, b)
    ref = x.reshape(-1, 32).astype(np.float64) @ wt.reshape(48, 32).astype(np.float64).T + b
    np.testing.assert_allclose(y.reshape(-1, 48), ref, rtol=0, atol=2e-5)


def test_depthwise_is_correlate2d():
    r = rng(4)
    c = 6
    x = r.uniform(0, 6, (1, 9, 8, c)).astype(np.float32)
    wt = r.normal(0, 0.5, (c, 1, 3, 3)).astype(np.float32)
    y = O.conv2d(x, wt, None, 1, 1, 1, c)
    for ch in range(c):
        ref = scipy.signal.correlate2d(x[0, :, :, ch].astype(np.float64),
                                       wt[ch, 0].astype(np.float64), mode="same")
        np.testing.assert_allclose(y[0, :, :, ch], ref, rtol=0, atol=1e-5)


def test_activation_variants():
    x = np.array([-3.0, -0.5, 0.0, 2.0, 7.0], np.float32).reshape(1, 1, 5, 1)
    w = np.ones((1, 1, 1, 1), np.float32)
    flat = lambda a: a.reshape(-1)
    # what the converter emits: min is always 0 (remapper.cc:166-170)
    np.testing.assert_array_equal(flat(O.conv2d(x, w, act=O.ACT_RELU)), [0, 0, 0, 2, 7])
    np.testing.assert_array_equal(flat(O.conv2d(x, w, act=O.ACT_CLIP, minv=0, maxv=6)),
                                  [0, 0, 0, 2, 6])
    # variants: dense clip honours min, pointwise clip ignores it, any4 relu uses min
    np.testing.assert_array_equal(
        flat(O.conv2d(x, w, act=O.ACT_CLIP, minv=-1, maxv=6, variant=O.VARIANT_NHWC4)),
        [-1, -0.5, 0, 2, 6])
    np.testing.assert_array_equal(
        flat(O.conv2d(x, w, act=O.ACT_CLIP, minv=-1, maxv=6, variant=O.VARIANT_PW)),
        [0, 0, 0, 2, 6])
    np.testing.assert_array_equal(
        flat(O.conv2d(x, w, act=O.ACT_RELU, minv=-1, variant=O.VARIANT_ANY4)),
        [-1, -0.5, 0, 2, 7])


def test_out_size_formula():
    assert O.out_size(300, 3, 2, 1) == 150
    assert O.out_size(112, 3, 1, 1) == 112
    assert O.out_size(19, 3, 2, 1) == 10
    assert O.out_size(3, 3, 2, 1) == 2
    assert O.out_size(8, 3, 1, 2, 2) == 8


@pytest.mark.parametrize("k,s,p", [(2, 2, 0), (3, 2, 1), (3, 1, 1), (5, 3, 2)])
def test_pool_matches_torch(k, s, p):
    r = rng(10 + k + s)
    x = r.normal(0, 1, (2, 11, 9, 5)).astype(np.float32)
    xt = torch.from_numpy(x).permute(0, 3, 1, 2)
    ref_max = F.max_pool2d(xt, k, s, p).permute(0, 2, 3, 1).numpy()
    ref_avg = F.avg_pool2d(xt, k, s, p, count_include_pad=True).permute(0, 2, 3, 1).numpy()
    np.testing.assert_array_equal(O.pool2d(x, k, s, p, O.POOL_MAX), ref_max)
    np.testing.assert_allclose(O.pool2d(x, k, s, p, O.POOL_AVG), ref_avg, rtol=0, atol=1e-6)


def test_pool_window_outside_image_is_zero():
    # pad 2 with k 2 s 2: the corner windows hold no in-image tap
    x = -np.ones((1, 4, 4, 1), np.float32)
    y = O.pool2d(x, 2, 2, 2, O.POOL_MAX)
    assert y.shape == (1, 4, 4, 1)
    assert y[0, 0, 0, 0] == 0.0 and y[0, 1, 1, 0] == -1.0


def test_global_average_pool():
    r = rng(12)
    x = r.normal(0, 1, (2, 7, 7, 10)).astype(np.float32)
    y = O.pool2d(x, 0, 0, 0, O.POOL_GLOBAL_AVG)
    assert y.shape == (2, 1, 1, 10)
    np.testing.assert_allclose(y[:, 0, 0, :], x.astype(np.float64).mean(axis=(1, 2)),
                               rtol=0, atol=1e-6)


@pytest.mark.parametrize("rank", [1, 2, 3, 4])
def test_concat_every_axis(rank):
    r = rng(20 + rank)
    base = [2, 3, 5, 4][:rank]
    for axis in list(range(rank)) + [-1]:
        ins = []
        for extra in (1, 4, 2):
            shp = list(base)
            shp[axis] = extra
            ins.append(r.normal(0, 1, shp).astype(np.float32))
        np.testing.assert_array_equal(O.concat(ins, axis), np.concatenate(ins, axis))


def test_concat_shape_mismatch_is_error():
    a = np.zeros((2, 3), np.float32)
    b = np.zeros((3, 3), np.float32)
    with pytest.raises(ValueError):
        O.concat([a, b], 1)


def test_decode_closed_forms():
    r = rng(30)
    anchors = np.concatenate([r.uniform(0.1, 0.9, (50, 2)), r.uniform(0.05, 0.5, (50, 2))],
                             axis=1).astype(np.float32)
    zero = np.zeros((2, 50, 4), np.float32)
    out = O.ssd_decode(zero, anchors)
    expect = np.concatenate([anchors[:, :2] - anchors[:, 2:] * np.float32(0.5),
                             anchors[:, :2] + anchors[:, 2:] * np.float32(0.5)], axis=1)
    np.testing.assert_array_equal(out[0], expect)
    np.testing.assert_array_equal(out[1], expect)
    # general case against a float64 restatement of the published SSD decode
    pred = r.normal(0, 1, (2, 50, 4)).astype(np.float32)
    out = O.ssd_decode(pred, anchors, (0.1, 0.1, 0.2, 0.2))
    p, a = pred.astype(np.float64), anchors.astype(np.float64)[None]
    v = np.array([np.float32(0.1), np.float32(0.1), np.float32(0.2), np.float32(0.2)], np.float64)
    cxy = p[..., :2] * v[:2] * a[..., 2:] + a[..., :2]
    wh = np.exp(p[..., 2:] * v[2:]) * a[..., 2:]
    ref = np.concatenate([cxy - wh / 2, cxy + wh / 2], axis=-1)
    np.testing.assert_allclose(out, ref, rtol=0, atol=1e-6)
    # tw = th = 0 keeps the anchor's size
    pred[..., 2:] = 0
    out = O.ssd_decode(pred, anchors)
    np.testing.assert_allclose(out[..., 2:] - out[..., :2],
                               np.broadcast_to(anchors[None, :, 2:], (2, 50, 2)), atol=1e-6)


def test_box_info_invariants():
    r = rng(40)
    batch, priors, classes = 3, 200, 21
    logits = (r.normal(0, 2.0, (batch, priors, classes))).astype(np.float32)
    boxes = r.uniform(0, 1, (batch, priors, 4)).astype(np.float32)
    res = O.box_info(logits, boxes, 0.3, 300.0, 200.0)
    l64 = logits.astype(np.float64)
    sm = np.exp(l64) / np.exp(l64).sum(-1, keepdims=True)
    fg = sm[..., 1:]
    best = fg.argmax(-1) + 1
    bestp = fg.max(-1)
    for b in range(batch):
        keep = np.nonzero(bestp[b] > 0.3 + 1e-6)[0]
        maybe = np.nonzero(bestp[b] > 0.3 - 1e-6)[0]
        got = res[b]
        assert set(keep) <= set(got["prior"]) <= set(maybe)
        assert np.all(np.diff(got["prior"]) > 0)
        assert np.all(got["cls"] >= 1) and np.all(got["cls"] < classes)
        np.testing.assert_array_equal(got["cls"], best[b][got["prior"]])
        np.testing.assert_allclose(got["score"], bestp[b][got["prior"]], rtol=1e-5)
        assert np.all(got["score"] > np.float32(0.3))
        sb = boxes[b][got["prior"]] * np.array([300, 200, 300, 200], np.float32)
        np.testing.assert_array_equal(got["box"], sb)
        np.testing.assert_array_equal(got["rect"][:, 0], sb[:, 0].astype(np.int32))
        np.testing.assert_array_equal(got["rect"][:, 2], (sb[:, 2] - sb[:, 0]).astype(np.int32))


def test_box_info_background_never_wins_and_threshold_is_strict():
    # background logit huge: the best foreground class is still reported, with p small
    logits = np.zeros((1, 2, 4), np.float32)
    logits[0, 0] = [10, 1, 2, 0]
    logits[0, 1] = [0, 0, 0, 0]          # p = 0.25 for each class
    boxes = np.zeros((1, 2, 4), np.float32)
    res = O.box_info(logits, boxes, 0.25)  # 0.25 > 0.25 is false
    assert len(res[0]["prior"]) == 0
    res = O.box_info(logits, boxes, 0.2)
    np.testing.assert_array_equal(res[0]["prior"], [1])
    np.testing.assert_array_equal(res[0]["cls"], [1])   # first of the tied classes


def test_fold_bn_identity():
    r = rng(50)
    c, o = 16, 24
    x = r.uniform(0, 6, (1, 6, 6, c)).astype(np.float32)
    w = r.normal(0, np.sqrt(2 / (9 * c)), (o, c, 3, 3)).astype(np.float32)
    gamma = r.uniform(0.5, 1.5, o).astype(np.float32)
    beta = r.normal(0, 0.1, o).astype(np.float32)
    mean = r.normal(0, 0.1, o).astype(np.float32)
    var = r.uniform(0.5, 1.5, o).astype(np.float32)
    for bias in (None, r.uniform(-0.1, 0.1, o).astype(np.float32)):
        wf, bf = O.fold_bn(w, bias, gamma, beta, mean, var, 1e-5)
        y = O.conv2d(x, w, bias, 1, 1).astype(np.float64)
        bn = (y - mean) / np.sqrt(var.astype(np.float64) + 1e-5) * gamma + beta
        np.testing.assert_allclose(O.conv2d(x, wf, bf, 1, 1), bn, rtol=0, atol=1e-5)


def test_hwn4c4_layout_formula_and_round_trip():
    r = rng(60)
    for shape in [(5, 3, 3, 3), (8, 8, 1, 1), (1, 1, 3, 3), (13, 6, 5, 5)]:
        w = r.normal(0, 1, shape).astype(np.float32)
        t = O.nchw_to_hwn4c4(w)
        o, i, kh, kw = shape
        o4 = (o + 3) // 4
        assert t.shape == (kh * kw * o4, ((i + 3) // 4) * 4, 4)
        # texel (x=i, y=(ky*kw+kx)*O4+o/4), lane o%4
        oo, ii, ky, kx = o - 1, i - 1, kh - 1, 0
        assert t[(ky * kw + kx) * o4 + oo // 4, ii, oo % 4] == w[oo, ii, ky, kx]
        assert np.count_nonzero(t) <= w.size
        np.testing.assert_array_equal(O.hwn4c4_to_nchw(t, shape), w)


def test_topk_nms_against_python_restatement():
    r = rng(70)
    n = 60
    scores = r.uniform(0.3, 1.0, n).astype(np.float32)
    xy = r.integers(0, 200, (n, 2))
    wh = r.integers(10, 120, (n, 2))
    rects = np.concatenate([xy, wh], axis=1).astype(np.int32)

    def iou(a, b):
        ax0, ay0, ax1, ay1 = a[0], a[1], a[0] + a[2], a[1] + a[3]
        bx0, by0, bx1, by1 = b[0], b[1], b[0] + b[2], b[1] + b[3]
        w = max(0.0, min(ax1, bx1) - max(ax0, bx0))
        h = max(0.0, min(ay1, by1) - max(ay0, by0))
        i = w * h
        u = (ax1 - ax0) * (ay1 - ay0) + (bx1 - bx0) * (by1 - by0) - i
        return 0.0 if u <= 0 else i / u

    for top_k, ties in ((100, False), (25, False), (100, True), (7, True)):
        if ties:  # equal scores keep their input order (the defined choice for std::sort's ties)
            scores = (r.integers(3, 9, n) / 10.0).astype(np.float32)
        order = sorted(range(n), key=lambda i: (-scores[i], i))[:top_k]
        dropped = [False] * len(order)
        for i in range(len(order) - 1):
            for j in range(i + 1, len(order)):
                if np.float32(iou(rects[order[i]], rects[order[j]])) > np.float32(0.45):
                    dropped[j] = True
        expect = [o for o, d in zip(order, dropped) if not d]
        np.testing.assert_array_equal(O.topk_nms(scores, rects, top_k, 0.45), expect)


def test_topk_nms_known_answers():
    """Hand-built cases with the answer worked out on paper (detector.cc:114-148, common.cc:57-77).
    Boxes are (x, y, w, h), 100 x 100 each.  IoU of two such boxes shifted by d along x is
    (100 - d) / (100 + d): 0.538 for d = 30, 0.25 for d = 60."""
    A, B, C, D = (0, 0, 100, 100), (30, 0, 100, 100), (60, 0, 100, 100), (300, 300, 50, 50)
    # The reference's rule: B (dropped by A) still drops C although A and C overlap by 0.25 only;
    # a textbook greedy NMS would keep C.
    rects = np.array([A, B, C, D], np.int32)
    scores = np.array([0.9, 0.8, 0.7, 0.6], np.float32)
    np.testing.assert_array_equal(O.topk_nms(scores, rects, 100, 0.45), [0, 3])
    # same boxes, input order shuffled: the sort by score decides, results are input positions
    perm = [2, 3, 0, 1]                       # input = C, D, A, B
    np.testing.assert_array_equal(O.topk_nms(scores[perm], rects[perm], 100, 0.45), [2, 1])
    # without B the chain is broken and C survives
    keep = [0, 2, 3]
    np.testing.assert_array_equal(O.topk_nms(scores[keep], rects[keep], 100, 0.45), [0, 1, 2])
    # the threshold is strict: IoU(A, B) = 70 / 130 exactly as the host computes it in binary32
    thr = np.float32(np.float32(7000.0) / np.float32(13000.0))
    np.testing.assert_array_equal(O.topk_nms(scores[:2], rects[:2], 100, float(thr)), [0, 1])
    np.testing.assert_array_equal(O.topk_nms(scores[:2], rects[:2], 100, float(np.nextafter(thr, np.float32(0)))), [0])
    # top-k cuts before the suppression: with k = 2 only A and B are looked at, D never appears
    np.testing.assert_array_equal(O.topk_nms(scores, rects, 2, 0.45), [0])
    # equal scores keep their input order (the defined choice for std::sort's ties), so the
    # earlier of two overlapping boxes wins whichever it is
    eq = np.array([0.8, 0.8, 0.8], np.float32)
    np.testing.assert_array_equal(O.topk_nms(eq, np.array([A, B, D], np.int32), 100, 0.45), [0, 2])
    np.testing.assert_array_equal(O.topk_nms(eq, np.array([B, A, D], np.int32), 100, 0.45), [0, 2])
    np.testing.assert_array_equal(O.topk_nms(eq, np.array([D, B, A], np.int32), 2, 0.45), [0, 1])
    # degenerate rectangles: zero area on both sides gives u <= 0 -> IoU 0, nothing is dropped
    z = np.array([(5, 5, 0, 0), (5, 5, 0, 0)], np.int32)
    np.testing.assert_array_equal(O.topk_nms(eq[:2], z, 100, 0.45), [0, 1])
    assert len(O.topk_nms(np.zeros(0, np.float32), np.zeros((0, 4), np.int32), 100, 0.45)) == 0


def test_elementwise_against_numpy():
    r = rng(90)
    a = r.normal(0, 2, (3, 5, 7, 6)).astype(np.float32)
    b = r.normal(0, 2, a.shape).astype(np.float32)
    np.testing.assert_array_equal(O.add(a, b), a + b)
    np.testing.assert_array_equal(O.relu(a), np.maximum(a, 0))
    np.testing.assert_array_equal(O.clip(a, -0.5, 1.25), np.clip(a, -0.5, 1.25))
    # clip.glsl applies max(min_value) first and min(max_value) last: with min > max the result is max
    np.testing.assert_array_equal(O.clip(a, 2.0, 1.0), np.full_like(a, 1.0))


def test_batchnorm_against_float64_and_fold():
    r = rng(91)
    c = 10
    x = r.normal(0, 2, (2, 4, 5, c)).astype(np.float32)
    gamma, beta = r.uniform(0.5, 1.5, c).astype(np.float32), r.normal(0, 0.1, c).astype(np.float32)
    mean, var = r.normal(0, 0.3, c).astype(np.float32), r.uniform(0.5, 1.5, c).astype(np.float32)
    y = O.batchnorm(x, gamma, beta, mean, var, 1e-5)
    ref = (x.astype(np.float64) - mean) / np.sqrt(var.astype(np.float64) + 1e-5) * gamma + beta
    np.testing.assert_allclose(y, ref, rtol=2e-6, atol=2e-6)
    # identity parameters leave x unchanged (sqrt(1 + 0) = 1)
    one, zero = np.ones(c, np.float32), np.zeros(c, np.float32)
    np.testing.assert_array_equal(O.batchnorm(x, one, zero, zero, one, 0.0), x)
    # BN after a convolution equals the convolution with folded parameters (remapper.cc:142-149)
    w = r.normal(0, 0.3, (c, 6, 3, 3)).astype(np.float32)
    b0 = r.normal(0, 0.1, c).astype(np.float32)
    xin = r.normal(0, 1, (1, 6, 6, 6)).astype(np.float32)
    wf, bf = O.fold_bn(w, b0, gamma, beta, mean, var, 1e-5)
    lhs = O.batchnorm(O.conv2d(xin, w, b0, 1, 1), gamma, beta, mean, var, 1e-5)
    np.testing.assert_allclose(lhs, O.conv2d(xin, wf, bf, 1, 1), rtol=1e-4, atol=1e-4)


def test_gemm_against_numpy():
    r = rng(92)
    for m, n, k in ((1, 7, 5), (4, 10, 33), (3, 1, 8)):
        a = r.normal(0, 1, (m, k)).astype(np.float32)
        for trans_b in (True, False):
            b = r.normal(0, 1, (n, k) if trans_b else (k, n)).astype(np.float32)
            bm = b.T if trans_b else b
            for c in (None, r.normal(0, 1, n).astype(np.float32), r.normal(0, 1, (m, n)).astype(np.float32)):
                got = O.gemm(a, b, c, alpha=0.75, beta=-1.5, trans_b=trans_b)
                ref = 0.75 * (a.astype(np.float64) @ bm.astype(np.float64))
                if c is not None:
                    ref = ref - 1.5 * c
                np.testing.assert_allclose(got, ref, rtol=1e-5, atol=1e-5)


def test_oracle_matches_committed_vectors():
    """tests/golden/oracle_vectors.npz was written by tests/golden/make_golden.py; the oracle
    built from today's sources must reproduce every array in it bit for bit."""
    import importlib.util
    import os
    here = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
    spec = importlib.util.spec_from_file_location("make_golden", os.path.join(here, "make_golden.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    now = mod.cases()
    with np.load(os.path.join(here, "oracle_vectors.npz")) as stored:
        assert sorted(stored.files) == sorted(now)
        for k in stored.files:
            np.testing.assert_array_equal(stored[k], now[k], err_msg=k)
