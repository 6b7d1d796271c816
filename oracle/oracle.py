"""ctypes/numpy front end of the CPU oracle (oracle/ogle_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py.  The product package never imports it.

All arrays are float32, C-contiguous; activations are NHWC, filters OIHW, as
the reference's own CPU checkers take them
(ogl_runtime/opengl/nn/kernels/conv2d_test.cc:18-75).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libogle_oracle.so")

ACT_NONE, ACT_CLIP, ACT_RELU = 0, 1, 2
VARIANT_NHWC4, VARIANT_PW, VARIANT_ANY4 = 0, 1, 2
POOL_MAX, POOL_AVG, POOL_GLOBAL_AVG = 0, 1, 2

_lib = None


def build():
    """Compile the oracle with the committed Makefile."""
    subprocess.run(["make", "-C", _HERE, "-B", "libogle_oracle.so"], check=True,
                   stdout=subprocess.DEVNULL)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.oracle_out_size.restype = ctypes.c_int
        _lib.oracle_concat.restype = ctypes.c_int
        _lib.oracle_topk_nms.restype = ctypes.c_int
        _lib.oracle_num_threads.restype = ctypes.c_int
    return _lib


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p) if a is not None else None


def out_size(n, k, stride, pad, dilation=1):
    return lib().oracle_out_size(int(n), int(k), int(stride), int(pad), int(dilation))


def conv2d(x, w, bias=None, stride=1, pad=0, dilation=1, groups=1, act=ACT_NONE,
           minv=0.0, maxv=0.0, variant=VARIANT_NHWC4):
    x, w = _f32(x), _f32(w)
    bias = _f32(bias) if bias is not None else None
    n, h, wd, c = x.shape
    o, cpg, k, k2 = w.shape
    assert k == k2 and cpg * groups == c and o % groups == 0
    oh, ow = out_size(h, k, stride, pad, dilation), out_size(wd, k, stride, pad, dilation)
    y = np.empty((n, oh, ow, o), np.float32)
    lib().oracle_conv2d(_p(x), _p(w), _p(bias), _p(y), n, h, wd, c, o, k, stride, pad,
                        dilation, groups, act, ctypes.c_float(minv), ctypes.c_float(maxv),
                        variant)
    return y


def conv2d_abs(x, w, bias=None, stride=1, pad=0, dilation=1, groups=1):
    """sum |x||w| + |b| per output: the scale fp32 rounding error is relative to."""
    x, w = _f32(x), _f32(w)
    bias = _f32(bias) if bias is not None else None
    n, h, wd, c = x.shape
    o, cpg, k, _ = w.shape
    oh, ow = out_size(h, k, stride, pad, dilation), out_size(wd, k, stride, pad, dilation)
    y = np.empty((n, oh, ow, o), np.float32)
    lib().oracle_conv2d_abs(_p(x), _p(w), _p(bias), _p(y), n, h, wd, c, o, k, stride, pad,
                            dilation, groups)
    return y


def pool2d(x, k, stride, pad, pool_type):
    x = _f32(x)
    n, h, wd, c = x.shape
    if pool_type == POOL_GLOBAL_AVG:
        assert h == wd
        k, stride, pad = h, 1, 0
    oh, ow = out_size(h, k, stride, pad), out_size(wd, k, stride, pad)
    y = np.empty((n, oh, ow, c), np.float32)
    lib().oracle_pool2d(_p(x), _p(y), n, h, wd, c, k, stride, pad, pool_type)
    return y


def concat(inputs, axis):
    inputs = [_f32(a) for a in inputs]
    rank = inputs[0].ndim
    ax = axis + rank if axis < 0 else axis
    shapes = np.array([a.shape for a in inputs], dtype=np.int32).reshape(-1)
    out_shape = list(inputs[0].shape)
    out_shape[ax] = sum(a.shape[ax] for a in inputs)
    out = np.empty(out_shape, np.float32)
    ptrs = (ctypes.c_void_p * len(inputs))(*[a.ctypes.data for a in inputs])
    rc = lib().oracle_concat(ptrs, _p(shapes), len(inputs), rank, axis, _p(out))
    if rc != 0:
        raise ValueError("concat: shapes differ outside the axis")
    return out


def ssd_decode(pred, anchors, variances=(0.1, 0.1, 0.2, 0.2)):
    pred, anchors = _f32(pred), _f32(anchors)
    batch, priors, four = pred.shape
    assert four == 4 and anchors.shape == (priors, 4)
    v = np.array(variances, np.float32)
    out = np.empty_like(pred)
    lib().oracle_ssd_decode(_p(pred), _p(anchors), _p(out), batch, priors, _p(v))
    return out


def box_info(logits, boxes, threshold=0.3, image_w=1.0, image_h=1.0):
    """Returns a list (one entry per image) of dicts with prior, cls, score, box, rect."""
    logits, boxes = _f32(logits), _f32(boxes)
    batch, priors, classes = logits.shape
    assert boxes.shape == (batch, priors, 4)
    cnt = np.zeros(batch, np.int32)
    prior = np.zeros((batch, priors), np.int32)
    cls = np.zeros((batch, priors), np.int32)
    score = np.zeros((batch, priors), np.float32)
    box = np.zeros((batch, priors, 4), np.float32)
    rect = np.zeros((batch, priors, 4), np.int32)
    lib().oracle_box_info(_p(logits), _p(boxes), batch, priors, classes,
                          ctypes.c_float(threshold), ctypes.c_float(image_w),
                          ctypes.c_float(image_h), _p(cnt), _p(prior), _p(cls), _p(score),
                          _p(box), _p(rect))
    res = []
    for b in range(batch):
        k = int(cnt[b])
        res.append(dict(prior=prior[b, :k].copy(), cls=cls[b, :k].copy(),
                        score=score[b, :k].copy(), box=box[b, :k].copy(),
                        rect=rect[b, :k].copy()))
    return res


def expf(x):
    x = _f32(x)
    y = np.empty_like(x)
    lib().oracle_expf_array(_p(x), _p(y), ctypes.c_long(x.size))
    return y


def fold_bn(w, bias, gamma, beta, mean, var, eps=1e-5):
    """Returns (w', b'); bias None means the conv had none (a zero bias is made)."""
    w = _f32(w).copy()
    o = w.shape[0]
    bias = np.zeros(o, np.float32) if bias is None else _f32(bias).copy()
    lib().oracle_fold_bn(_p(w), _p(bias), _p(_f32(gamma)), _p(_f32(beta)), _p(_f32(mean)),
                         _p(_f32(var)), ctypes.c_float(eps), o, int(w.size // o))
    return w, bias


def nchw_to_hwn4c4(w):
    w = _f32(w)
    o, i, kh, kw = w.shape
    o4, i4 = (o + 3) // 4, (i + 3) // 4
    dst = np.empty((kh * kw * o4, i4 * 4, 4), np.float32)
    lib().oracle_nchw_to_hwn4c4(_p(w), _p(dst), o, i, kh, kw)
    return dst


def hwn4c4_to_nchw(t, shape):
    t = _f32(t)
    o, i, kh, kw = shape
    dst = np.empty(shape, np.float32)
    lib().oracle_hwn4c4_to_nchw(_p(t), _p(dst), o, i, kh, kw)
    return dst


def topk_nms(scores, rects, top_k=100, nms_threshold=0.45):
    scores = _f32(scores)
    rects = np.ascontiguousarray(rects, dtype=np.int32)
    order = np.zeros(max(len(scores), 1), np.int32)
    n = lib().oracle_topk_nms(_p(scores), _p(rects), len(scores), top_k,
                              ctypes.c_float(nms_threshold), _p(order))
    return order[:n].copy()


def add(a, b):
    a, b = _f32(a), _f32(b)
    assert a.shape == b.shape
    y = np.empty_like(a)
    lib().oracle_add(_p(a), _p(b), _p(y), ctypes.c_long(a.size))
    return y


def relu(x):
    x = _f32(x)
    y = np.empty_like(x)
    lib().oracle_relu(_p(x), _p(y), ctypes.c_long(x.size))
    return y


def clip(x, minv, maxv):
    x = _f32(x)
    y = np.empty_like(x)
    lib().oracle_clip(_p(x), _p(y), ctypes.c_long(x.size), ctypes.c_float(minv), ctypes.c_float(maxv))
    return y


def batchnorm(x, gamma, beta, mean, var, eps):
    """Parameters index the last dimension of x."""
    x = _f32(x)
    gamma, beta, mean, var = _f32(gamma), _f32(beta), _f32(mean), _f32(var)
    c = x.shape[-1]
    assert gamma.size == beta.size == mean.size == var.size == c
    y = np.empty_like(x)
    lib().oracle_batchnorm(_p(x), _p(gamma), _p(beta), _p(mean), _p(var), _p(y),
                           ctypes.c_long(x.size // c), c, ctypes.c_float(eps))
    return y


def gemm(a, b, c=None, alpha=1.0, beta=1.0, trans_b=True):
    a, b = _f32(a), _f32(b)
    m, k = a.shape
    n = b.shape[0] if trans_b else b.shape[1]
    assert (b.shape[1] if trans_b else b.shape[0]) == k
    c = _f32(c) if c is not None else None
    y = np.empty((m, n), np.float32)
    lib().oracle_gemm(_p(a), _p(b), _p(c), _p(y), m, n, k, int(bool(trans_b)),
                      c.ndim if c is not None else 0, ctypes.c_float(alpha), ctypes.c_float(beta))
    return y


def num_threads():
    return lib().oracle_num_threads()
