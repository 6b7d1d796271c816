#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X.

Workload (BASELINE configs[4]): MobileNet-v1 SSD 300x300, fp32, random init, BN folded,
21 classes, 1917 priors, followed by the SSD decode + score filter and top-k + NMS (all on
the device).  A step is one pass of
the whole network over one batch of 16 synthetic images that are already resident in HBM.
The graph is a .dlx model loaded into the C++ FBOSession; the pass is replayed as a hipGraph.

Printed JSON (one line): images/s at batch 16 (`value`), p50 latency at batch 1, the roofline
of the dominant kernel family measured with HIP events on the session's stream inside this
process, a per-family table, and the CPU restatement timed on the host cores.

Timing protocol: --warmup untimed steps, then untimed replays until --clock-ramp seconds have
gone by (the clocks of an idle GPU take longer to settle than 20 steps last), then --repeats
timed regions of exactly --steps steps each, every region bracketed by a wait for all streams;
`ms_per_step` / `value` are the median region, the extremes are reported beside them.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

import numpy as np  # noqa: E402

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E
MFMA_F32_PEAK_TFLOPS = 157.3   # dense fp32 MFMA

METRIC = "MobileNet-SSD 300² images/s (b16) + p50 ms (b1); per-kernel % of roofline"


def build_session(batch, seed=20240005, input_seed=None):
    from ogle_amd import models, session
    g, info = models.mobilenet_v1_ssd(batch, seed=seed)
    x = np.random.Generator(np.random.PCG64(seed + 1 if input_seed is None else input_seed)) \
        .uniform(-1, 1, (batch, 300, 300, 3)).astype(np.float32)
    s = session.Session()
    s.load_graph(g)
    s.run({"input": x})   # allocates, uploads weights and the input; inputs stay resident
    s.sync()
    return s, info


TAIL_FAMILY = "concat + detector tail (decode / score filter, top-k + NMS)"


def detector_tail_parts(batch, priors=1917, classes=21, topk=100):
    """Algorithmic bytes of the detector tail per pass, by launch.  Decode + softmax-max + score
    filter: per image the class logits and box predictions in, the decoded boxes and one
    (score, class) pair per prior out, and the anchors once for the batch.  Top-k + NMS: per image
    one 28-byte record per prior in (score, class, prior, rectangle) and at most `topk` 44-byte
    records out.  The concatenations move nothing: the heads write straight into their outputs."""
    per_image = priors * classes * 4 + priors * 16 + priors * 16 + priors * 8   # 161,028 + 30,672 + 30,672 + 15,336
    return {"detector.score_filter": batch * per_image + priors * 16,
            "detector.topk_nms": batch * (priors * 28 + topk * 44)}


def detector_tail_bytes(batch):
    return sum(detector_tail_parts(batch).values())


def family_of(nodes, layers):
    """Kernel family of one entry of the launch plan, from the nodes it was launched for."""
    fams = set()
    for n in nodes:
        l = layers.get(n)
        if l is None:
            fams.add(TAIL_FAMILY)
        elif n.startswith("head") or n.startswith("extra"):
            fams.add("SSD heads + extras chain (dense 3x3 and 1x1, MFMA implicit GEMM)")
        elif l["kind"] == "pw":
            fams.add("pointwise 1x1 backbone (MFMA implicit GEMM)")
        elif l["kind"] == "dw":
            fams.add("depthwise 3x3")
        else:
            fams.add("dense 3x3 stem (direct MFMA)")
    return " + ".join(sorted(fams))


def per_family_roofline(sess, info, batch, passes, pass_us):
    """Kernel time per family from the kernels' own durations: every kernel of `passes` eager
    passes carries a start / stop HIP event pair that the device stamps with the kernel's begin
    and end (ogle_hip_kernel_timing_begin), the same quantity a rocprofv3 kernel trace reports,
    and the launch plan says which node(s) each kernel ran for.  FLOPs / bytes are the layers'
    algorithmic work (2 x multiply-adds; input + weights + bias + output once each)."""
    import re
    layers = {l["name"]: l for l in info["layers"]}
    fams, per_label = {}, {}
    dispatches = 0
    for p in range(passes):
        plan = sess.launch_plan(with_detect=True, durations=True)
        dispatches = sum(len(us) for _, us in plan)
        for label, us in plan:
            nodes = [m[0] for m in re.findall(r"([^#+:]+)#([A-Za-z0-9_]+)#", label)]
            name = family_of(nodes, layers)
            f = fams.setdefault(name, dict(us=0.0, flops=0.0, bytes=0.0, launches=0, layers=0))
            f["us"] += sum(us) / passes
            per_label[label] = per_label.get(label, 0.0) + sum(us) / passes
            if p == 0:
                f["launches"] += len(us)
                if name == TAIL_FAMILY and not f["bytes"]:
                    f["bytes"] = float(detector_tail_bytes(batch))
                if not label.startswith("reduce:"):
                    for n in nodes:
                        if n in layers:
                            f["layers"] += 1
                            f["flops"] += layers[n]["flops_per_image"] * batch
                            f["bytes"] += layers[n]["act_bytes_per_image"] * batch + layers[n]["weight_bytes"]
    # A kernel trace of the replayed pass takes a kernel's begin when its dispatch packet is picked
    # up, i.e. at the previous kernel's end: its durations add up to the pass.  The events here
    # bracket the kernel alone, so the pass's dispatch gaps (replayed pass - sum of kernel
    # durations, shared equally among its dispatches) are added back before rates are formed.
    kernel_sum = sum(f["us"] for f in fams.values())
    gap_us = max(pass_us - kernel_sum, 0.0) / max(dispatches, 1)
    out = []
    for name, f in fams.items():
        bound = "mfma" if "MFMA implicit GEMM" in name else "hbm"
        f["span_us"] = f["us"] + gap_us * f["launches"]
        tflops, gbs = f["flops"] / f["span_us"] / 1e6, f["bytes"] / f["span_us"] / 1e3
        out.append(dict(kernel=name, layers=f["layers"], launches=f["launches"],
                        ms_per_step=round(f["span_us"] / 1e3, 4),
                        avg_launch_us=round(f["span_us"] / max(f["launches"], 1), 2),
                        avg_kernel_only_us=round(f["us"] / max(f["launches"], 1), 2), bound=bound,
                        tflops=round(tflops, 2), gbs=round(gbs, 1),
                        frac=round(gbs / HBM_PEAK_GBS if bound == "hbm" else tflops / MFMA_F32_PEAK_TFLOPS, 4),
                        flops_per_step=f["flops"], bytes_per_step=f["bytes"]))
    out.sort(key=lambda d: -d["ms_per_step"])
    return out, kernel_sum / 1e3, dispatches, gap_us


def calibration_copy(megabytes=256, launches=3):
    """A plain copy of known size through the library's own copy kernel (ogle_hip_convert
    f32 -> f32), so that a counter run of this script also holds the reference reading that the
    FETCH_SIZE / WRITE_SIZE counters are scaled by."""
    import torch
    from ogle_amd import hip as H
    n = megabytes * 1024 * 1024 // 4
    src = torch.ones(n, dtype=torch.float32, device="cuda")
    dst = torch.empty_like(src)
    for _ in range(launches):
        H.check(H.lib().ogle_hip_convert(src.data_ptr(), H.F32, dst.data_ptr(), H.F32, n,
                                         torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    return n * 4


# bench family -> family name in the summaries ogle_amd.profile_layers writes
PROFILE_FAMILY = {"pointwise 1x1 backbone (MFMA implicit GEMM)": "pointwise",
                  "SSD heads + extras chain (dense 3x3 and 1x1, MFMA implicit GEMM)": "heads+extras",
                  "depthwise 3x3": "depthwise", "dense 3x3 stem (direct MFMA)": "stem"}


def read_traffic_summary(kernel_family):
    """HBM bytes per launch of the dominant kernel from the committed counter summary
    (profiles/bench_b16_per_layer_traffic.txt, made by ogle_amd.profile_layers from two
    rocprofv3 --pmc runs of `bench.py --profile-layers ... --eager`)."""
    path = os.path.join(ROOT, "profiles", "bench_b16_per_layer_traffic.txt")
    key = "traffic_bytes_per_launch[%s]=" % PROFILE_FAMILY.get(kernel_family, kernel_family)
    try:
        for line in open(path):
            if line.startswith(key):
                return float(line.split("=", 1)[1])
    except OSError:
        pass
    return None


def kernel_table(iters=50, warm=5, only=None):
    """Each kernel of the path on its own, at the shapes the baseline configurations name,
    called through the C ABI on torch's current stream and timed with events on that stream.
    FLOPs = 2 x multiply-adds; bytes = input + weights + bias + output once each.
    `only`: run just the rows whose name contains this text (for a profiler run of one kernel)."""
    import ctypes
    import torch
    from ogle_amd import hip as H
    L = H.lib()
    st = torch.cuda.current_stream().cuda_stream
    rows = []

    def want(name):
        return only is None or only in name

    def timed(fn):
        for _ in range(warm):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(iters):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / iters * 1e3  # microseconds per call

    def row(name, us, flops, nbytes, bound, peak_tflops=MFMA_F32_PEAK_TFLOPS):
        tf, gb = flops / us / 1e6, nbytes / us / 1e3
        rows.append(dict(kernel=name, us=round(us, 2), tflops=round(tf, 2), gbs=round(gb, 1),
                         bound=bound, peak=HBM_PEAK_GBS if bound == "hbm" else peak_tflops,
                         frac=round(gb / HBM_PEAK_GBS if bound == "hbm" else tf / peak_tflops, 4)))

    def conv_problem(n, h, w, c, o, k, s, p, g=1, dtype=H.F32, act=H.ACT_RELU, maxv=0.0):
        tdt = torch.float16 if dtype == H.F16 else torch.float32
        x = torch.rand(n, h, w, c, device="cuda").to(tdt)
        dw = g == c and g != 1
        src = torch.randn(o, c // g, k, k, device="cuda") * 0.05
        wd = torch.empty(src.numel(), dtype=tdt, device="cuda")
        H.check(L.ogle_hip_pack_filter(src.data_ptr(), wd.data_ptr(),
                                       H.FILTER_HWC if dw else H.FILTER_OHWI, dtype, o, c // g, k, k, st))
        b = torch.rand(o, device="cuda")
        oh, ow = H.out_size(h, k, s, p), H.out_size(w, k, s, p)
        y = torch.empty(n, oh, ow, o, device="cuda", dtype=tdt)
        a = H.conv_args(x.data_ptr(), wd.data_ptr(), b.data_ptr(), y.data_ptr(), n, h, w, c, o, k, s,
                        p, 1, g, act, 0.0, maxv, H.VARIANT_NHWC4, dtype)
        need = L.ogle_hip_conv_workspace_bytes(ctypes.byref(a))
        ws = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
        if need:
            a.workspace_dev, a.workspace_bytes = ws.data_ptr(), need
        esz = 2 if dtype == H.F16 else 4
        flops = 2.0 * n * oh * ow * o * (c // g) * k * k
        nbytes = esz * (x.numel() + wd.numel() + y.numel()) + 4 * o
        return a, flops, nbytes, (x, wd, b, y, ws)

    def conv_row(name, entry, bound, *shape, peak=MFMA_F32_PEAK_TFLOPS, **kw):
        if not want(name):
            return
        a, flops, nbytes, keep = conv_problem(*shape, **kw)
        f = getattr(L, entry)
        row(name, timed(lambda: H.check(f(ctypes.byref(a), st))), flops, nbytes, bound, peak)

    conv_row("dense 3x3 @C1 (1x112x112x32->64)", "ogle_hip_conv2d", "mfma", 1, 112, 112, 32, 64, 3, 1, 1)
    for b in (1, 8):
        conv_row("depthwise 3x3 @C2 b%d (38x38x256)" % b, "ogle_hip_dwconv2d", "hbm",
                 b, 38, 38, 256, 256, 3, 1, 1, g=256, act=H.ACT_CLIP, maxv=6.0)
        conv_row("pointwise @C2 b%d (M=%d K=256 N=512)" % (b, b * 1444), "ogle_hip_pwconv_gemm", "mfma",
                 b, 38, 38, 256, 512, 1, 1, 0, act=H.ACT_CLIP, maxv=6.0)
    # the depthwise layers of the headline pass (C5 at batch 16) with the largest maps
    conv_row("depthwise 3x3 @C5 b16 block1 (150x150x32)", "ogle_hip_dwconv2d", "hbm",
             16, 150, 150, 32, 32, 3, 1, 1, g=32, act=H.ACT_CLIP, maxv=6.0)
    conv_row("depthwise 3x3 s2 @C5 b16 block2 (150x150x64)", "ogle_hip_dwconv2d", "hbm",
             16, 150, 150, 64, 64, 3, 2, 1, g=64, act=H.ACT_CLIP, maxv=6.0)
    conv_row("depthwise 3x3 @C5 b16 block3 (75x75x128)", "ogle_hip_dwconv2d", "hbm",
             16, 75, 75, 128, 128, 3, 1, 1, g=128, act=H.ACT_CLIP, maxv=6.0)
    # pointwise layers of the headline pass (C5 at batch 16)
    conv_row("pointwise @C5 b16 block2 (M=90000 K=64 N=128)", "ogle_hip_pwconv_gemm", "mfma",
             16, 75, 75, 64, 128, 1, 1, 0, act=H.ACT_CLIP, maxv=6.0)
    conv_row("pointwise @C5 b16 block8 (M=5776 K=512 N=512)", "ogle_hip_pwconv_gemm", "mfma",
             16, 19, 19, 512, 512, 1, 1, 0, act=H.ACT_CLIP, maxv=6.0)
    conv_row("pointwise @C5 b16 block13 (M=1600 K=1024 N=1024)", "ogle_hip_pwconv_gemm", "mfma",
             16, 10, 10, 1024, 1024, 1, 1, 0, act=H.ACT_CLIP, maxv=6.0)
    conv_row("pointwise GEMM @C3 fp32 (M=11552 K=512 N=1024)", "ogle_hip_pwconv_gemm", "mfma",
             32, 19, 19, 512, 1024, 1, 1, 0)
    conv_row("pointwise GEMM @C3 fp16 storage, fp32 accumulate", "ogle_hip_pwconv_gemm", "mfma",
             32, 19, 19, 512, 1024, 1, 1, 0, dtype=H.F16, peak=2500.0)

    conv_row("pointwise GEMM fp16 storage, large (M=46208 K=1024 N=1024)", "ogle_hip_pwconv_gemm", "mfma",
             128, 19, 19, 1024, 1024, 1, 1, 0, dtype=H.F16, peak=2500.0)
    if only is not None:
        return rows   # only the convolution rows can be picked one by one

    # yardstick for the two rows above: the vendor library's GEMM (torch.matmul -> hipBLASLt /
    # rocBLAS) on the same shape and types; a comparison figure, not part of the path
    for dt, tag in ((torch.float32, "fp32"), (torch.float16, "fp16")):
        ga = torch.randn(11552, 512, device="cuda", dtype=dt)
        gb = torch.randn(1024, 512, device="cuda", dtype=dt)
        gc = torch.empty(11552, 1024, device="cuda", dtype=dt)
        row("vendor library GEMM on the C3 shape, %s (yardstick)" % tag,
            timed(lambda: torch.matmul(ga, gb.t(), out=gc)), 2.0 * 11552 * 512 * 1024,
            ga.element_size() * (ga.numel() + gb.numel() + gc.numel()), "mfma",
            MFMA_F32_PEAK_TFLOPS if dt == torch.float32 else 2500.0)

    # yardstick for the bandwidth-bound rows: a plain copy too large for the 256 MB last-level
    # cache (1 GiB in, 1 GiB out), i.e. what HBM itself delivers to a streaming kernel here
    big = 1 << 28
    gsrc = torch.ones(big, dtype=torch.float32, device="cuda")
    gdst = torch.empty_like(gsrc)
    row("plain copy 1 GiB -> 1 GiB, library copy kernel (HBM yardstick)",
        timed(lambda: H.check(L.ogle_hip_convert(gsrc.data_ptr(), H.F32, gdst.data_ptr(), H.F32, big, st)),
              ), 0.0, 8.0 * big, "hbm")
    row("plain copy 1 GiB -> 1 GiB, torch copy_ (HBM yardstick)", timed(lambda: gdst.copy_(gsrc)), 0.0,
        8.0 * big, "hbm")
    del gsrc, gdst

    # C4: the twelve SSD head convolutions of 64 images in one grouped call
    maps = [(19, 512, 3), (10, 1024, 6), (5, 512, 6), (3, 256, 6), (2, 256, 6), (1, 128, 6)]
    probs = []
    for m, c, anchors in maps:
        probs.append(conv_problem(64, m, m, c, anchors * 4, 3, 1, 1, act=H.ACT_NONE))
        probs.append(conv_problem(64, m, m, c, anchors * 21, 3, 1, 1, act=H.ACT_NONE))
    arr = (H.ConvArgs * len(probs))(*[q[0] for q in probs])
    row("SSD heads @C4 b64 (12 convs, one grouped call)",
        timed(lambda: H.check(L.ogle_hip_conv2d_batch(arr, len(probs), st))),
        sum(q[1] for q in probs), sum(q[2] for q in probs), "mfma")

    # concat @C4: six maps -> (64, 1917, 4) and (64, 1917, 21)
    for width, label in ((4, "loc"), (21, "conf")):
        lens = [m * m * a for m, _, a in maps]
        ins = [torch.rand(64, n, width, device="cuda") for n in lens]
        out = torch.empty(64, sum(lens), width, device="cuda")
        ca = H.ConcatArgs()
        for i, t in enumerate(ins):
            ca.inputs_dev[i] = t.data_ptr()
            ca.axis_len[i] = lens[i]
        ca.output_dev, ca.n_inputs, ca.outer, ca.inner, ca.dtype = out.data_ptr(), len(ins), 64, width, H.F32
        row("concat @C4 b64 %s (6 inputs)" % label, timed(lambda: H.check(L.ogle_hip_concat(ctypes.byref(ca), st))),
            0.0, 2.0 * out.numel() * 4, "hbm")

    # decode + softmax-max + score filter @C4
    batch, priors, classes = 64, 1917, 21
    logits = torch.randn(batch, priors, classes, device="cuda") * 2
    pred = torch.randn(batch, priors, 4, device="cuda")
    anchors = torch.rand(priors, 4, device="cuda")
    i32 = dict(dtype=torch.int32, device="cuda")
    boxes = torch.empty(batch, priors, 4, device="cuda")
    cnt, kp, kc = torch.zeros(batch, **i32), torch.zeros(batch, priors, **i32), torch.zeros(batch, priors, **i32)
    ks, kb = torch.empty(batch, priors, device="cuda"), torch.empty(batch, priors, 4, device="cuda")
    kr = torch.zeros(batch, priors, 4, **i32)
    da = H.DetectArgs(logits.data_ptr(), pred.data_ptr(), anchors.data_ptr(), boxes.data_ptr(), batch,
                      priors, classes, 0, (ctypes.c_float * 4)(0.1, 0.1, 0.2, 0.2), 0.3, 300.0, 300.0,
                      cnt.data_ptr(), kp.data_ptr(), kc.data_ptr(), ks.data_ptr(), kb.data_ptr(),
                      kr.data_ptr())
    row("SSD decode + score filter @C4 b64", timed(lambda: H.check(L.ogle_hip_ssd_detect(ctypes.byref(da), st))),
        0.0, batch * (161028 + 30672 + 30672 + 15336) + 30672, "hbm")

    # pooling parity shapes
    for name, n, h, c, k, s, p, typ in (("max-pool 3x3 s2 p1 (1x112x112x64)", 1, 112, 64, 3, 2, 1, 0),
                                        ("max-pool 3x3 s2 p1 (16x112x112x64)", 16, 112, 64, 3, 2, 1, 0),
                                        ("avg-pool 2x2 s2 (16x112x112x64)", 16, 112, 64, 2, 2, 0, 1)):
        x = torch.rand(n, h, h, c, device="cuda")
        oh = H.out_size(h, k, s, p)
        y = torch.empty(n, oh, oh, c, device="cuda")
        pa = H.PoolArgs(x.data_ptr(), y.data_ptr(), n, h, h, c, oh, oh, k, s, p, typ, H.F32)
        row(name, timed(lambda: H.check(L.ogle_hip_pool2d(ctypes.byref(pa), st))), 0.0,
            4.0 * (x.numel() + y.numel()), "hbm")
    # elementwise ops of classification graphs, on a 16x75x75x128 activation (36.9 MB)
    shape = (16, 75, 75, 128)
    xe, ye = torch.rand(shape, device="cuda"), torch.rand(shape, device="cuda")
    oe = torch.empty(shape, device="cuda")
    ua = H.UnaryArgs(xe.data_ptr(), oe.data_ptr(), xe.numel(), H.UNARY_CLIP, 0.0, 6.0, H.F32)
    row("clip (16x75x75x128)", timed(lambda: H.check(L.ogle_hip_unary(ctypes.byref(ua), st))), 0.0,
        8.0 * xe.numel(), "hbm")
    ba = H.BinaryArgs(xe.data_ptr(), ye.data_ptr(), oe.data_ptr(), xe.numel(), H.F32)
    row("add (16x75x75x128)", timed(lambda: H.check(L.ogle_hip_add(ctypes.byref(ba), st))), 0.0,
        12.0 * xe.numel(), "hbm")
    prm = [torch.rand(128, device="cuda") + 0.5 for _ in range(4)]
    na = H.BatchNormArgs(xe.data_ptr(), prm[0].data_ptr(), prm[1].data_ptr(), prm[2].data_ptr(),
                         prm[3].data_ptr(), oe.data_ptr(), xe.numel() // 128, 128, 1e-5, H.F32)
    row("batchnorm (16x75x75x128)", timed(lambda: H.check(L.ogle_hip_batchnorm(ctypes.byref(na), st))),
        0.0, 8.0 * xe.numel(), "hbm")
    # classifier head: (16, 1024) x (1000, 1024)^T + bias, the Linear form on the MFMA kernel
    ga_, gb_, gc_ = torch.rand(16, 1024, device="cuda"), torch.randn(1000, 1024, device="cuda") * 0.03, \
        torch.rand(1000, device="cuda")
    gy = torch.empty(16, 1000, device="cuda")
    gg = H.GemmArgs(ga_.data_ptr(), gb_.data_ptr(), gc_.data_ptr(), gy.data_ptr(), 16, 1000, 1024, 1, 1,
                    1.0, 1.0, None, 0)
    need = L.ogle_hip_gemm_workspace_bytes(ctypes.byref(gg))
    gws = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
    if need:
        gg.workspace_dev, gg.workspace_bytes = gws.data_ptr(), need
    row("gemm classifier head (M=16 K=1024 N=1000)", timed(lambda: H.check(L.ogle_hip_gemm(ctypes.byref(gg), st))),
        2.0 * 16 * 1000 * 1024, 4.0 * (16 * 1024 + 1000 * 1024 + 1000 + 16 * 1000), "hbm")
    # what a launch costs when there is nothing to do: the floor under every small row above
    # (calls in a row on one stream, as all rows are timed)
    tiny = H.UnaryArgs(xe.data_ptr(), oe.data_ptr(), 4, H.UNARY_CLIP, 0.0, 6.0, H.F32)
    row("launch floor: clip on 4 elements", timed(lambda: H.check(L.ogle_hip_unary(ctypes.byref(tiny), st))),
        0.0, 32.0, "hbm")
    return rows


def cpu_baseline(seed=20240005, images=2, repeats=1):
    """The oracle (CPU restatement of the reference's arithmetic) on the host cores: every conv
    layer of the network, concat and the decode + score filter, for `images` images."""
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import oracle as O
    from ogle_amd import models
    _, info = models.mobilenet_v1_ssd(images, seed=seed, with_weights=True)
    x = np.random.Generator(np.random.PCG64(seed + 1)).uniform(-1, 1, (images, 300, 300, 3)) \
        .astype(np.float32)

    def one_pass():
        cur, feats, locs, confs = x, [], [], []
        for l in info["layers"]:
            w, b = info["weights"][l["name"]]
            if l["name"].startswith("head"):
                y = O.conv2d(feats[int(l["name"][4])], w, b, 1, 1)
                if l["name"].endswith("loc"):
                    locs.append(y.reshape(images, -1, 4))
                else:
                    confs.append(y.reshape(images, -1, info["num_classes"]))
                continue
            cur = O.conv2d(cur, w, b, l["stride"], l["pad"], 1, l["group"], O.ACT_CLIP, 0.0, 6.0,
                           O.VARIANT_PW if l["kind"] == "pw" else O.VARIANT_NHWC4)
            if l["name"] in ("block11.pw", "block13.pw") or l["name"].endswith(".conv"):
                feats.append(cur)
        loc, conf = O.concat(locs, 1), O.concat(confs, 1)
        boxes = O.ssd_decode(loc, info["anchors"])
        return O.box_info(conf, boxes, 0.3, 300.0, 300.0)

    # the reference's own protocol (nn/main.cc:76-111): 3 warm-up runs, then timed runs, here the
    # median of at least 20 and as many more as fit in about 10 s of CPU work
    for _ in range(3):
        one_pass()
    times = []
    t_all = time.perf_counter()
    while len(times) < max(20, repeats) or (time.perf_counter() - t_all < 10.0 and len(times) < 2000):
        t0 = time.perf_counter()
        one_pass()
        times.append(time.perf_counter() - t0)
    dt = time.perf_counter() - t_all
    med = float(np.median(times))
    return dict(value=round(images / med, 3), unit="images/s", cores=O.num_threads(),
                kind="port", protocol="3 warm-up passes, then the median of %d timed passes" % len(times),
                ms_per_pass=dict(median=round(med * 1e3, 3), min=round(min(times) * 1e3, 3),
                                 max=round(max(times) * 1e3, 3)),
                sample="%d timed pass(es) of the full network + decoder over %d image(s), %.1f s of CPU work; "
                       "C restatement of the shaders' arithmetic, OpenMP over output rows "
                       "(not the reference under Mesa llvmpipe, which cannot be built here)"
                       % (len(times), images, dt))


def profile_layers_run(args):
    """Replays of the pass and nothing after them, plus the plan file that lets
    ogle_amd.profile_layers attribute a kernel trace of this run to layers."""
    import torch
    sess, info = build_session(args.batch)
    plan = sess.launch_plan(with_detect=True)
    copy_bytes = calibration_copy()
    sess.time_compute(args.warmup, args.steps, graph=not args.eager, with_detect=True)
    sess.sync()
    torch.cuda.synchronize()
    me = "python3 bench.py --profile-layers %s --steps %d --warmup %d --batch %d%s" % (
        args.profile_layers, args.steps, args.warmup, args.batch, " --eager" if args.eager else "")
    doc = dict(workload="MobileNet-v1-SSD 300x300 fp32, batch %d, one session, %s, "
                        "network + decode/score filter + top-k/NMS"
                        % (args.batch, "kernel-by-kernel launches" if args.eager else "hipGraph replay"),
               batch=args.batch, replays=args.steps, dispatches_per_pass=sum(k for _, k in plan),
               tail_bytes=detector_tail_parts(args.batch),
               plan=plan, calibration=dict(kernel="convert_kernel<float, float>", kib_per_launch=copy_bytes // 1024),
               layers={l["name"]: dict(kind=l["kind"], flops_per_image=l["flops_per_image"],
                                       act_bytes_per_image=l["act_bytes_per_image"],
                                       weight_bytes=l["weight_bytes"]) for l in info["layers"]},
               commands=["cd /tmp && export TMPDIR=/tmp && cd $GRAFT_REPO_ROOT",
                         "rocprofv3 --kernel-trace --output-format csv -d gpurun_out/layers -o b%d -- %s"
                         % (args.batch, me),
                         "python3 -m ogle_amd.profile_layers gpurun_out/layers/b%d_kernel_trace.csv %s"
                         % (args.batch, args.profile_layers)] if not args.eager else
               ["cd /tmp && export TMPDIR=/tmp && cd $GRAFT_REPO_ROOT",
                "rocprofv3 --pmc FETCH_SIZE --output-format csv -d gpurun_out/layers -o fetch%d -- %s"
                % (args.batch, me),
                "rocprofv3 --pmc WRITE_SIZE --output-format csv -d gpurun_out/layers -o write%d -- %s"
                % (args.batch, me),
                "python3 -m ogle_amd.profile_layers --fetch gpurun_out/layers/fetch%d_counter_collection.csv "
                "--write gpurun_out/layers/write%d_counter_collection.csv %s"
                % (args.batch, args.batch, args.profile_layers)])
    with open(args.profile_layers, "w") as f:
        json.dump(doc, f)
    print(json.dumps(dict(profile_layers=args.profile_layers, dispatches_per_pass=doc["dispatches_per_pass"],
                          replays=args.steps)))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--batch", type=int, default=16)
    ap.add_argument("--repeats", type=int, default=7,
                    help="timed regions of --steps steps each; the median region is reported")
    ap.add_argument("--clock-ramp", type=float, default=0.5,
                    help="seconds of untimed replays of the pass between the warm-up steps and the "
                         "first timed region (lets the clocks settle)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--eager", action="store_true", help="launch kernel by kernel instead of a hipGraph")
    ap.add_argument("--streams", type=int, default=4,
                    help="sessions that replay the pass concurrently, each on its own stream, with the "
                         "steps dealt round-robin (1: one stream; forced to 1 with --eager)")
    ap.add_argument("--skip-kernel-table", action="store_true",
                    help="leave out the per-kernel leg at the single-kernel configurations")
    ap.add_argument("--skip-b1", action="store_true",
                    help="leave out the batch-1 latency leg (keeps a profiler trace to the batch-16 pass)")
    ap.add_argument("--only-kernel", metavar="TEXT",
                    help="run only the convolution rows of the per-kernel table whose name contains TEXT, "
                         "--steps calls each after --warmup, and print them (for a profiler run of one kernel)")
    ap.add_argument("--profile-layers", metavar="PLAN.json",
                    help="only replay the pass --steps times as a hipGraph (after --warmup) and write the "
                         "pass's dispatch sequence to PLAN.json: run under `rocprofv3 --kernel-trace` and "
                         "feed trace + plan to `python -m ogle_amd.profile_layers`")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus %d is not supported (every image is "
              "independent, so more GPUs would each take a slice of the batch)" % args.gpus,
              file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(2)

    if args.profile_layers:
        profile_layers_run(args)
        return
    if args.only_kernel:
        print(json.dumps(dict(kernel_table=kernel_table(iters=args.steps, warm=args.warmup,
                                                        only=args.only_kernel))))
        return
    use_graph = not args.eager
    streams = 1 if args.eager else max(1, min(args.streams, 16))
    # The sessions of the pipelined leg.  The first four sessions of a process take their
    # streams from a pool the runtime created in one go, so they sit on different hardware
    # queues (two sessions that share a queue do not overlap) wherever they are created.
    sess, info = build_session(args.batch)
    pool = [sess] + [build_session(args.batch, input_seed=100 + i)[0] for i in range(1, streams)]
    from ogle_amd import session as _session

    def run_single(k):
        return sess.time_compute(0, k, graph=use_graph, with_detect=True)

    def run_pipelined(k):
        _session.Session.time_pipelined(pool, 0, k, with_detect=True)

    def all_idle():
        for s_ in pool:
            s_.sync()
        torch.cuda.synchronize()

    def timed_regions(run, repeats):
        """`repeats` timed regions of exactly args.steps steps each, every region bracketed by a
        wait for all streams on both sides; wall-clock ms of each region."""
        out = []
        for _ in range(repeats):
            all_idle()
            t0 = time.perf_counter()
            run(args.steps)
            all_idle()
            out.append((time.perf_counter() - t0) * 1e3)
        return out

    def spread(ms_list):
        per = sorted(m / args.steps for m in ms_list)
        return dict(median=round(float(np.median(per)), 4), min=round(per[0], 4), max=round(per[-1], 4),
                    regions=len(per))

    headline_run = run_single if streams == 1 else run_pipelined
    # W untimed warm-up steps, then the clock ramp: the headline's pass is replayed until
    # --clock-ramp seconds have gone by, so that the timed regions see settled clocks whatever
    # the step count (20 steps of 0.6 ms are over before the clocks have moved)
    sess.time_compute(args.warmup, 0, graph=use_graph, with_detect=True)
    if streams > 1:
        _session.Session.time_pipelined(pool, args.warmup, 0, with_detect=True)
    all_idle()
    t_ramp = time.perf_counter()
    ramp_steps = 0
    while time.perf_counter() - t_ramp < args.clock_ramp:
        headline_run(50)
        all_idle()
        ramp_steps += 50
    clock_ramp_s = time.perf_counter() - t_ramp

    # one stream: K passes (network + decode/score filter + top-k/NMS) one after the other,
    # inputs resident, bracketed by syncs; the median of args.repeats such regions
    single_ms = timed_regions(run_single, args.repeats)
    each, total_ms = sess.time_compute(0, args.steps, graph=use_graph, with_detect=True)
    all_idle()
    single_wall_ms = float(np.median(single_ms))
    single = {"images_per_s": round(args.batch * args.steps / (single_wall_ms * 1e-3), 1),
              "ms_per_step": round(single_wall_ms / args.steps, 4),
              "ms_per_step_spread": spread(single_ms),
              "event_ms_per_step": round(total_ms / args.steps, 4)}
    # the same, with the final detections (at most 100 per image) read back to the host inside
    # every step, as the reference's own timing loop does (nn/main.cc:76-111 includes GetOutputs):
    # the step ends when the host holds the boxes, so steps do not overlap
    sess.sync()
    t0 = time.perf_counter()
    kept = 0
    for _ in range(args.steps):
        sess.time_compute(0, 1, graph=use_graph, with_detect=True)
        kept += sum(len(d) for d in sess.detect_results(args.batch))
    rb_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    single["with_detection_readback"] = {
        "images_per_s": round(args.batch / (rb_ms * 1e-3), 1), "ms_per_step": round(rb_ms, 4),
        "detections_per_step": kept / args.steps,
        "note": "one pass, then wait for the stream and copy the final lists to the host (pageable copies, the "
                "lists unpacked into Python objects), then the next pass; driven from Python step by step"}
    if use_graph:
        # the same serial loop inside the runtime: the pass ends with one copy of the final
        # lists to page-locked memory (part of the replayed graph), the host waits for the
        # event behind the pass, reads the lists, and only then launches the next pass
        def run_serial_readback(k):
            return _session.Session.time_pipelined_readback([sess], 0, k)[0]
        _session.Session.time_pipelined_readback([sess], max(args.warmup, 3), max(args.warmup, 3))
        srb = timed_regions(run_serial_readback, args.repeats)
        srb_ms = float(np.median(srb))
        _, seen = _session.Session.time_pipelined_readback([sess], 0, args.steps)
        single["serial_readback"] = {
            "images_per_s": round(args.batch * args.steps / (srb_ms * 1e-3), 1),
            "ms_per_step": round(srb_ms / args.steps, 4), "ms_per_step_spread": spread(srb),
            "detections_per_step": seen / args.steps,
            "note": "one session, one pass at a time, the host holds every pass's final lists before it launches "
                    "the next (nn/main.cc:76-111 times Run + GetOutputs the same way): the lists are copied to "
                    "page-locked memory inside the replayed graph and the host waits for one event per pass"}
    if streams == 1:
        region_ms = single_ms
    else:
        # the timed region of the headline: the same K passes dealt round-robin over `streams`
        # sessions (same graph and weights, own buffers and stream, own resident input), each a
        # hipGraph replay, so that one pass's launch gaps and under-filled kernels are covered by
        # the others' work; bracketed by syncs of every stream; the median of args.repeats regions
        region_ms = timed_regions(run_pipelined, args.repeats)
    wall_ms = float(np.median(region_ms))
    ms_per_step = wall_ms / args.steps
    images_per_s = args.batch * args.steps / (wall_ms * 1e-3)
    # the headline's passes with the host in the loop: every pass ends with one asynchronous copy
    # of its final detection lists (count + at most 100 records of 44 bytes per image) to
    # page-locked memory, recorded inside the captured graph; before a session's next pass is
    # launched the host waits for the event behind its previous pass and reads the lists
    pipelined_readback = None
    if use_graph:
        _session.Session.time_pipelined_readback(pool, args.warmup, 0)
        rb_regions, rb_seen = [], 0
        for _ in range(args.repeats):
            all_idle()
            ms_, seen_ = _session.Session.time_pipelined_readback(pool, 0, args.steps)
            rb_regions.append(ms_)
            rb_seen = seen_
        rb_med = float(np.median(rb_regions))
        pipelined_readback = {
            "images_per_s": round(args.batch * args.steps / (rb_med * 1e-3), 1),
            "ms_per_step": round(rb_med / args.steps, 4), "ms_per_step_spread": spread(rb_regions),
            "detections_per_step": rb_seen / args.steps, "streams": streams,
            "note": "as `value`, and the host reads every pass's final lists: one device-to-host copy "
                    "per pass inside the graph, the host waits for that pass's event only"}

    # the same pass with the host buffer handed over at the boundary each time (pageable
    # host memory -> device copy inside FBOSession::Run, then the pass, eager launches)
    x_host = np.random.Generator(np.random.PCG64(7)).uniform(-1, 1, (args.batch, 300, 300, 3)) \
        .astype(np.float32)
    for _ in range(3):
        sess.run({"input": x_host})
    sess.sync()
    t1 = time.perf_counter()
    upload_steps = 20
    for _ in range(upload_steps):
        sess.run({"input": x_host})
    sess.sync()
    upload_ms = (time.perf_counter() - t1) * 1e3 / upload_steps
    upload = {"images_per_s": round(args.batch / (upload_ms * 1e-3), 1),
              "ms_per_step": round(upload_ms, 4),
              "note": "FBOSession::Run per step: pageable host input -> HBM over PCIe, "
                      "then the pass (no detect leg); not the headline value"}
    if streams > 1:
        # and pipelined: every step copies its batch from page-locked host memory on its
        # session's stream, then replays the pass (with the detector's work)
        from ogle_amd import session as _session
        pinned = [_session.PinnedBuffer((args.batch, 300, 300, 3)) for _ in pool]
        for pb in pinned:
            pb.array[...] = x_host
        _session.Session.time_pipelined(pool, args.warmup, 0, True, "input", pinned)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        _session.Session.time_pipelined(pool, 0, args.steps, True, "input", pinned)
        torch.cuda.synchronize()
        pipe_ms = (time.perf_counter() - t1) * 1e3 / args.steps
        upload["pipelined_pinned"] = {
            "images_per_s": round(args.batch / (pipe_ms * 1e-3), 1), "ms_per_step": round(pipe_ms, 4),
            "note": "%d pipelined sessions, each step: page-locked host input -> HBM on the session's "
                    "stream, then the pass with the detector's device work" % streams}
        for pb in pinned:
            pb.close()

    fams, kernel_sum_ms, dispatches, gap_us = per_family_roofline(
        sess, info, args.batch, passes=10, pass_us=single["event_ms_per_step"] * 1e3)
    dom = fams[0]
    roofline = dict(bound=dom["bound"], kernel=dom["kernel"],
                    achieved=dom["gbs"] if dom["bound"] == "hbm" else dom["tflops"],
                    peak=HBM_PEAK_GBS if dom["bound"] == "hbm" else MFMA_F32_PEAK_TFLOPS,
                    unit="GB/s" if dom["bound"] == "hbm" else "TFLOP/s", frac=dom["frac"],
                    traffic=read_traffic_summary(dom["kernel"]),
                    traffic_source="profiles/bench_b16_per_layer_traffic.txt (two rocprofv3 --pmc runs, "
                                   "FETCH_SIZE and WRITE_SIZE, of this script's --profile-layers leg; read "
                                   "from that committed summary, not measured in this run)",
                    launches_per_step=dom["launches"],
                    avg_launch_us=dom["avg_launch_us"],
                    avg_kernel_only_us=dom["avg_kernel_only_us"],
                    dispatch_gap_us=round(gap_us, 3),
                    measured="avg_kernel_only_us: start / stop HIP events carried by every kernel of 10 eager "
                             "passes, stamped by the device with the kernel's own begin and end, summed over "
                             "the family; avg_launch_us (what frac uses) adds the replayed pass's mean dispatch "
                             "gap (single-stream pass time - sum of kernel durations) / dispatches, because a "
                             "rocprofv3 kernel trace of the replayed pass counts a kernel from the previous "
                             "kernel's end",
                    algorithmic_per_step=dom["flops_per_step"] if dom["bound"] == "mfma" else dom["bytes_per_step"])

    # batch-1 latency: each pass waits for the previous one
    if args.skip_b1:
        lat = lat_eager = np.array([float("nan")])
    else:
        s1, _ = build_session(1)
        lat, _ = s1.time_compute(20, 300, graph=use_graph, with_detect=True, sync_each=True)
        lat_eager, _ = s1.time_compute(5, 100, graph=False, with_detect=True, sync_each=True)

    result = {
        "metric": METRIC, "value": round(images_per_s, 1), "unit": "images/s",
        "single_stream": single, "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
        "ms_per_step_spread": spread(region_ms),
        "value_spread": {"min": round(args.batch * args.steps / (max(region_ms) * 1e-3), 1),
                         "max": round(args.batch * args.steps / (min(region_ms) * 1e-3), 1),
                         "note": "value is the median of %d timed regions of %d steps each"
                                 % (len(region_ms), args.steps)},
        "clock_ramp_s": round(clock_ramp_s, 3), "clock_ramp_steps": ramp_steps,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "MobileNet-v1-SSD 300x300 fp32, random init, BN folded, 21 classes, "
                               "1917 priors + SSD decode/score filter + top-k/NMS on the device "
                               "(BASELINE configs[4])",
                   "batch": args.batch, "launch": "hipGraph" if use_graph else "eager",
                   "streams": streams,
                   "pipelining": ("%d sessions, each replaying the batch-%d pass as a hipGraph on its own "
                                  "stream; the K steps are dealt round-robin" % (streams, args.batch))
                   if streams > 1 else "none: one stream, one pass after the other",
                   "inputs": "resident in HBM", "flops_per_image": 2803531136},
        "p50_ms_b1": round(float(np.percentile(lat, 50)), 4),
        "p50_ms_b1_eager": round(float(np.percentile(lat_eager, 50)), 4),
        "network_tflops": round(2803531136 * args.batch / (ms_per_step * 1e-3) / 1e12, 2),
        "roofline": roofline,
        "kernels": fams,
        "kernel_time_sum_ms_per_step": round(kernel_sum_ms, 4),
        "dispatches_per_step": dispatches,
        "with_host_upload": upload,
        "pipelined_with_readback": pipelined_readback,
    }
    if not args.skip_kernel_table:
        result["kernel_table"] = kernel_table()
    result["calibration_copy_bytes"] = calibration_copy()
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
