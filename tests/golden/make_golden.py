#!/usr/bin/env python3
"""Writes tests/golden/oracle_vectors.npz: small seeded inputs and the outputs the CPU
oracle gives for them, one case per function of the hot path.

The reference stores no golden vectors of its own (its tests compare the GL result with
a CPU loop at run time), so these vectors pin the ORACLE: a later change to
oracle/ogle_oracle.c that alters any result shows up as a diff against this file
(tests/test_oracle.py::test_oracle_matches_committed_vectors), and the GPU tests compare
the HIP kernels with the same arrays.  Regenerate only on purpose:
    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "..", "..", "oracle"))
import oracle as O  # noqa: E402


def cases():
    r = np.random.Generator(np.random.PCG64(20240099))
    f = np.float32
    out = {}
    x = r.uniform(-1, 1, (2, 9, 8, 8)).astype(f)
    w = r.normal(0, 0.3, (12, 8, 3, 3)).astype(f)
    b = r.uniform(-0.1, 0.1, 12).astype(f)
    out.update(dense_x=x, dense_w=w, dense_b=b,
               dense_y=O.conv2d(x, w, b, 2, 1, 1, 1, O.ACT_RELU))
    wd = r.normal(0, 0.4, (8, 1, 3, 3)).astype(f)
    bd = r.uniform(-0.1, 0.1, 8).astype(f)
    out.update(dw_w=wd, dw_b=bd, dw_y=O.conv2d(x, wd, bd, 1, 1, 1, 8, O.ACT_CLIP, 0.0, 6.0))
    wp = r.normal(0, 0.3, (20, 8, 1, 1)).astype(f)
    bp = r.uniform(-0.1, 0.1, 20).astype(f)
    out.update(pw_w=wp, pw_b=bp,
               pw_y=O.conv2d(x, wp, bp, 1, 0, 1, 1, O.ACT_CLIP, -1.0, 0.5, O.VARIANT_PW))
    out.update(maxpool_y=O.pool2d(x, 3, 2, 1, O.POOL_MAX), avgpool_y=O.pool2d(x, 2, 2, 0, O.POOL_AVG))
    parts = [r.normal(0, 1, (2, n, 4)).astype(f) for n in (5, 3, 7)]
    out.update(cat_a=parts[0], cat_b=parts[1], cat_c=parts[2], cat_y=O.concat(parts, 1))
    priors, classes = 40, 6
    anchors = np.concatenate([r.uniform(0.1, 0.9, (priors, 2)), r.uniform(0.05, 0.5, (priors, 2))], 1).astype(f)
    pred = r.normal(0, 1, (2, priors, 4)).astype(f)
    logits = r.normal(0, 2.5, (2, priors, classes)).astype(f)
    boxes = O.ssd_decode(pred, anchors)
    out.update(ssd_anchors=anchors, ssd_pred=pred, ssd_logits=logits, ssd_boxes=boxes)
    info = O.box_info(logits, boxes, 0.3, 320.0, 240.0)
    for i, d in enumerate(info):
        for k in ("prior", "cls", "score", "box", "rect"):
            out["info%d_%s" % (i, k)] = d[k]
        out["info%d_keep" % i] = O.topk_nms(d["score"], d["rect"], 5, 0.45)
    g, bt = r.uniform(0.5, 1.5, 8).astype(f), r.normal(0, 0.1, 8).astype(f)
    mu, var = r.normal(0, 0.2, 8).astype(f), r.uniform(0.5, 1.5, 8).astype(f)
    out.update(bn_g=g, bn_b=bt, bn_m=mu, bn_v=var, bn_y=O.batchnorm(x, g, bt, mu, var, 1e-5))
    wf, bf = O.fold_bn(w, b, *(np.resize(v, 12) for v in (g, bt, mu, var)), 1e-5)
    out.update(fold_w=wf, fold_b=bf)
    a = r.normal(0, 1, (3, 10)).astype(f)
    bm = r.normal(0, 1, (7, 10)).astype(f)
    cm = r.normal(0, 1, 7).astype(f)
    out.update(gemm_a=a, gemm_b=bm, gemm_c=cm, gemm_y=O.gemm(a, bm, cm, 0.5, 2.0, True))
    return out


if __name__ == "__main__":
    np.savez_compressed(os.path.join(HERE, "oracle_vectors.npz"), **cases())
    print("wrote", os.path.join(HERE, "oracle_vectors.npz"))
