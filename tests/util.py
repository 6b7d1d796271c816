"""Helpers shared by the GPU parity tests: seeded inputs, thin wrappers that run
one op through the C ABI on torch-owned device memory, and the tolerance rule."""
import ctypes

import numpy as np

from ogle_amd import hip as H


def rng(seed):
    return np.random.Generator(np.random.PCG64(seed))


def _torch():
    import torch
    return torch


def dev(a, dtype=None):
    torch = _torch()
    t = torch.from_numpy(np.ascontiguousarray(a)).to("cuda")
    if dtype is not None:
        t = t.to(dtype)
    return t


def stream_ptr():
    return _torch().cuda.current_stream().cuda_stream


def pack_filter(w_oihw, layout, dtype=H.F32):
    """OIHW fp32 numpy -> packed device tensor."""
    torch = _torch()
    o, i, kh, kw = w_oihw.shape
    src = dev(w_oihw.astype(np.float32))
    n = H.lib().ogle_hip_packed_filter_elems(layout, o, i, kh, kw)
    assert n == w_oihw.size
    dst = torch.empty(n, dtype=torch.float16 if dtype == H.F16 else torch.float32, device="cuda")
    H.check(H.lib().ogle_hip_pack_filter(src.data_ptr(), dst.data_ptr(), layout, dtype, o, i, kh,
                                         kw, stream_ptr()))
    return dst


def gpu_conv(x, w, b=None, stride=1, pad=0, dilation=1, groups=1, act=H.ACT_NONE, minv=0.0,
             maxv=0.0, variant=H.VARIANT_NHWC4, dtype=H.F32, entry=None, workspace=True,
             image_stride=0, lead=0):
    """x NHWC numpy, w OIHW numpy.  Returns NHWC numpy fp32.  With workspace=True the launch gets
    the scratch buffer ogle_hip_conv_workspace_bytes asks for (enables the split-K plans).
    With image_stride (elements) the output goes into a NaN-filled buffer of `lead` +
    n * image_stride elements, image b at lead + b * image_stride, and the whole buffer is
    returned flat (fp32)."""
    torch = _torch()
    tdt = torch.float16 if dtype == H.F16 else torch.float32
    n, h, wd, c = x.shape
    o, cpg, k, _ = w.shape
    depthwise = groups == c and groups == o and groups != 1
    if entry is None:
        if depthwise:
            entry = "ogle_hip_dwconv2d"
        elif k == 1 and groups == 1 and dilation == 1 and stride == 1 and pad == 0:
            entry = "ogle_hip_pwconv_gemm"
        else:
            entry = "ogle_hip_conv2d"
    layout = H.FILTER_HWC if entry == "ogle_hip_dwconv2d" else H.FILTER_OHWI
    xd = dev(x.astype(np.float32), tdt)
    wdv = pack_filter(w, layout, dtype)
    bd = dev(b.astype(np.float32)) if b is not None else None
    oh, ow = H.out_size(h, k, stride, pad, dilation), H.out_size(wd, k, stride, pad, dilation)
    if image_stride:
        y = torch.full((lead + n * image_stride,), float("nan"), dtype=tdt, device="cuda")
    else:
        y = torch.full((n, oh, ow, o), float("nan"), dtype=tdt, device="cuda")
    args = H.conv_args(xd.data_ptr(), wdv.data_ptr(), bd.data_ptr() if bd is not None else None,
                       y.data_ptr() + lead * y.element_size(), n, h, wd, c, o, k, stride, pad, dilation,
                       groups, act, minv, maxv, variant, dtype)
    args.out_image_stride = image_stride
    ws = None
    if workspace:
        need = H.lib().ogle_hip_conv_workspace_bytes(ctypes.byref(args))
        if need:
            ws = torch.empty(need, dtype=torch.uint8, device="cuda")
            args.workspace_dev, args.workspace_bytes = ws.data_ptr(), need
    H.check(getattr(H.lib(), entry)(ctypes.byref(args), stream_ptr()))
    torch.cuda.synchronize()
    return y.float().cpu().numpy()


def gpu_pool(x, k, stride, pad, pool_type, dtype=H.F32):
    torch = _torch()
    tdt = torch.float16 if dtype == H.F16 else torch.float32
    n, h, wd, c = x.shape
    if pool_type == H.POOL_GLOBAL_AVG:
        k, stride, pad = h, 1, 0
    oh, ow = H.out_size(h, k, stride, pad), H.out_size(wd, k, stride, pad)
    xd = dev(x.astype(np.float32), tdt)
    y = torch.full((n, oh, ow, c), float("nan"), dtype=tdt, device="cuda")
    args = H.PoolArgs(xd.data_ptr(), y.data_ptr(), n, h, wd, c, oh, ow, k, stride, pad, pool_type,
                      dtype)
    H.check(H.lib().ogle_hip_pool2d(ctypes.byref(args), stream_ptr()))
    torch.cuda.synchronize()
    return y.float().cpu().numpy()


def gpu_concat(inputs, axis):
    torch = _torch()
    rank = inputs[0].ndim
    ax = axis + rank if axis < 0 else axis
    shape = list(inputs[0].shape)
    shape[ax] = sum(a.shape[ax] for a in inputs)
    outer = int(np.prod(shape[:ax], dtype=np.int64))
    inner = int(np.prod(shape[ax + 1:], dtype=np.int64))
    devs = [dev(a.astype(np.float32)) for a in inputs]
    out = torch.full(shape, float("nan"), dtype=torch.float32, device="cuda")
    args = H.ConcatArgs()
    for i, (a, d) in enumerate(zip(inputs, devs)):
        args.inputs_dev[i] = d.data_ptr()
        args.axis_len[i] = a.shape[ax]
    args.output_dev = out.data_ptr()
    args.n_inputs = len(inputs)
    args.outer, args.inner, args.dtype = outer, inner, H.F32
    H.check(H.lib().ogle_hip_concat(ctypes.byref(args), stream_ptr()))
    torch.cuda.synchronize()
    return out.cpu().numpy()


def gpu_decode(pred, anchors, variances=(0.1, 0.1, 0.2, 0.2)):
    torch = _torch()
    batch, priors, _ = pred.shape
    pd, ad = dev(pred.astype(np.float32)), dev(anchors.astype(np.float32))
    out = torch.full((batch, priors, 4), float("nan"), dtype=torch.float32, device="cuda")
    stride = 0 if anchors.ndim == 2 else priors * 4
    args = H.DecodeArgs(pd.data_ptr(), ad.data_ptr(), out.data_ptr(), batch, priors, stride,
                        (ctypes.c_float * 4)(*variances))
    H.check(H.lib().ogle_hip_ssd_decode(ctypes.byref(args), stream_ptr()))
    torch.cuda.synchronize()
    return out.cpu().numpy()


def gpu_detect(logits, pred, anchors, threshold=0.3, image_w=1.0, image_h=1.0,
               variances=(0.1, 0.1, 0.2, 0.2), boxes_in=None):
    """Returns (per-image list of dicts as oracle.box_info, decoded boxes numpy)."""
    torch = _torch()
    batch, priors, classes = logits.shape
    ld = dev(logits.astype(np.float32))
    i32 = dict(dtype=torch.int32, device="cuda")
    f32 = dict(dtype=torch.float32, device="cuda")
    cnt = torch.full((batch,), -1, **i32)
    prior = torch.full((batch, priors), -1, **i32)
    cls = torch.full((batch, priors), -1, **i32)
    score = torch.full((batch, priors), float("nan"), **f32)
    box = torch.full((batch, priors, 4), float("nan"), **f32)
    rect = torch.full((batch, priors, 4), -1, **i32)
    if boxes_in is None:
        pd, ad = dev(pred.astype(np.float32)), dev(anchors.astype(np.float32))
        boxes = torch.full((batch, priors, 4), float("nan"), **f32)
        pp, ap = pd.data_ptr(), ad.data_ptr()
    else:
        boxes = dev(boxes_in.astype(np.float32))
        pp, ap = None, None
    args = H.DetectArgs(ld.data_ptr(), pp, ap, boxes.data_ptr(), batch, priors, classes, 0,
                        (ctypes.c_float * 4)(*variances), threshold, image_w, image_h,
                        cnt.data_ptr(), prior.data_ptr(), cls.data_ptr(), score.data_ptr(),
                        box.data_ptr(), rect.data_ptr())
    H.check(H.lib().ogle_hip_ssd_detect(ctypes.byref(args), stream_ptr()))
    torch.cuda.synchronize()
    cnt = cnt.cpu().numpy()
    res = []
    for b in range(batch):
        k = int(cnt[b])
        res.append(dict(prior=prior[b, :k].cpu().numpy(), cls=cls[b, :k].cpu().numpy(),
                        score=score[b, :k].cpu().numpy(), box=box[b, :k].cpu().numpy(),
                        rect=rect[b, :k].cpu().numpy()))
    return res, boxes.cpu().numpy()


def gpu_topk_nms(counts, prior, cls, score, rect, topk, threshold, box=None):
    """Per-image lists (batch, stride[, 4]) as ogle_hip_ssd_detect leaves them -> per-image dict
    of the final lists of ogle_hip_ssd_topk_nms."""
    torch = _torch()
    batch, stride = prior.shape
    i32 = dict(dtype=torch.int32, device="cuda")
    cd, pd, kd = dev(counts.astype(np.int32)), dev(prior.astype(np.int32)), dev(cls.astype(np.int32))
    sd, rd = dev(score.astype(np.float32)), dev(rect.astype(np.int32))
    bd = dev(box.astype(np.float32)) if box is not None else None
    fc = torch.full((batch,), -7, **i32)
    fp = torch.full((batch, topk), -7, **i32)
    fk = torch.full((batch, topk), -7, **i32)
    fs = torch.full((batch, topk), float("nan"), dtype=torch.float32, device="cuda")
    fr = torch.full((batch, topk, 4), -7, **i32)
    fb = torch.full((batch, topk, 4), float("nan"), dtype=torch.float32, device="cuda") if box is not None else None
    a = H.NmsArgs(cd.data_ptr(), pd.data_ptr(), kd.data_ptr(), sd.data_ptr(),
                  bd.data_ptr() if bd is not None else None, rd.data_ptr(), batch, stride, topk,
                  threshold, fc.data_ptr(), fp.data_ptr(), fk.data_ptr(), fs.data_ptr(),
                  fb.data_ptr() if fb is not None else None, fr.data_ptr())
    H.check(H.lib().ogle_hip_ssd_topk_nms(ctypes.byref(a), stream_ptr()))
    torch.cuda.synchronize()
    n = fc.cpu().numpy()
    out = []
    for b in range(batch):
        k = int(n[b])
        d = dict(prior=fp[b, :k].cpu().numpy(), cls=fk[b, :k].cpu().numpy(),
                 score=fs[b, :k].cpu().numpy(), rect=fr[b, :k].cpu().numpy())
        if fb is not None:
            d["box"] = fb[b, :k].cpu().numpy()
        # nothing past the count may have been written
        assert (fp[b, k:] == -7).all() and (fr[b, k:] == -7).all()
        out.append(d)
    return out


# Parity rule for contractions (BASELINE: fp32 max relative error 1e-4, fp16 5e-3).
# Two tests per output tensor:
#  (1) normwise: |got - ref| <= RTOL * (sum|x||w| + |b|) for EVERY output.  This is the bound
#      fp32 summation can be held to: it stays meaningful where cancellation or the activation
#      leaves an output at or near zero, where no relative bound can hold.
#  (2) BASELINE's literal wording on every output that is not dominated by cancellation,
#      |ref| >= REL_FLOOR * (sum|x||w| + |b|): |got - ref| <= REL * |ref|.  With fp16 storage
#      the operands themselves are rounded (2^-11 each), an error proportional to sum|x||w|, not
#      to the output, so the literal bound can only be asked of outputs that keep at least
#      FP16_REL_FLOOR of that magnitude.
FP32_RTOL = 1e-5
FP16_RTOL = 5e-3
FP32_REL = 1e-4
FP16_REL = 5e-3
REL_FLOOR = 1e-2
FP16_REL_FLOOR = 5e-2

# what -> (worst normwise ratio err/scale, worst relative error where test (2) applies):
# the achieved figures, written as parity_achieved.json at the end of a GPU session (conftest.py).
PARITY_LOG = {}


def assert_conv_close(got, ref, scale, rtol, what="", rel=None, min_abs=0.0):
    """Both parity tests above.  `scale` is sum|x||w| + |b| per output (oracle.conv2d_abs, or
    the same contraction of absolute values in float64).  rtol FP32_RTOL or FP16_RTOL selects
    the matching relative bound unless `rel` is given.  Outputs with |ref| < min_abs are left
    to test (1) alone (fp16 storage: below 2^-14 the output format itself has fewer than eleven
    bits, so no relative bound can be asked of them).  Returns the worst err / scale."""
    assert got.shape == ref.shape, (got.shape, ref.shape)
    assert np.all(np.isfinite(got)), "non-finite output " + what
    if rel is None:
        rel = FP32_REL if rtol <= FP32_REL else FP16_REL
    floor = REL_FLOOR if rtol <= FP32_REL else FP16_REL_FLOOR
    g64, r64, s64 = got.astype(np.float64), ref.astype(np.float64), scale.astype(np.float64)
    err = np.abs(g64 - r64)
    norm = float(np.max(err / (s64 + 1e-30))) if err.size else 0.0
    assert norm <= rtol, "%s: error is %.3g of sum|x||w|, allowed %g (max abs err %.3g)" % (
        what, norm, rtol, float(err.max()))
    big = np.abs(r64) >= floor * s64
    big &= np.abs(r64) > 0
    big &= np.abs(r64) >= min_abs
    worst_rel = float(np.max(err[big] / np.abs(r64[big]))) if big.any() else 0.0
    assert worst_rel <= rel, "%s: max relative error %.3g over outputs with |ref| >= %g*scale, " \
        "allowed %g" % (what, worst_rel, floor, rel)
    key = what or "conv"
    old = PARITY_LOG.get(key, (0.0, 0.0, rtol))
    PARITY_LOG[key] = (max(old[0], norm), max(old[1], worst_rel), rtol)
    return norm
