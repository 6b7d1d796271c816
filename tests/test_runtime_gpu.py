"""GPU tests of the graph runtime: .dlx graphs are loaded into the C++ FBOSession through
its C ABI, run on the device, read back with GetOutputs and compared with the CPU oracle.

The single-node tests follow the pattern of the reference's kernel tests
(ogl_runtime/opengl/nn/kernels/conv2d_test.cc:141-204, concat_test.cc:51-95): build a one-node
graph, Run, fetch the result AND the constants as the device holds them, compare with the
in-test CPU function (here the oracle)."""
import numpy as np
import pytest

import oracle as O
from ogle_amd import dlx, models, session
from util import FP32_RTOL, assert_conv_close, rng

pytestmark = pytest.mark.gpu


def conv_graph(x_shape, w, b, k, s, p, d=1, g=1, act="", minv=0.0, maxv=0.0):
    n, h, wd, c = x_shape
    gb = dlx.GraphBuilder()
    x = gb.add_input("input", [n, c, h, wd])
    wi = gb.add_filter("conv2d1.weight", w)
    bi = gb.add_const("conv2d1.bias", b) if b is not None else None
    gb.add_conv("output", x, wi, bi, k, s, p, d, g, act, minv, maxv)
    gb.add_output_name("output")
    return gb


CONV_GRAPH_CASES = [
    # n, h, w, c, o, k, s, p, d, g, bias, act
    (1, 3, 3, 3, 1, 3, 1, 1, 1, 1, True, ""),
    (2, 16, 16, 8, 12, 3, 1, 1, 1, 1, False, "Relu"),
    (1, 32, 32, 3, 32, 3, 2, 1, 1, 1, True, "Clip"),     # stem-like
    (2, 9, 9, 16, 16, 3, 1, 1, 1, 16, True, "Clip"),     # depthwise
    (1, 8, 8, 8, 12, 3, 1, 1, 1, 4, True, ""),           # grouped
    (3, 7, 7, 32, 48, 1, 1, 0, 1, 1, True, "Clip"),      # pointwise
    (1, 8, 8, 4, 4, 3, 1, 2, 2, 1, False, ""),           # dilation 2
    (1, 6, 6, 8, 8, 1, 2, 0, 1, 1, True, "Relu"),        # 1x1 stride 2 -> dense variant
]


@pytest.mark.parametrize("case", CONV_GRAPH_CASES)
def test_single_conv_node_graph(case):
    n, h, w, c, o, k, s, p, d, g, use_bias, act = case
    r = rng(7000 + CONV_GRAPH_CASES.index(case))
    x = r.uniform(-1, 1, (n, h, w, c)).astype(np.float32)
    wt = r.normal(0, 0.5, (o, c // g, k, k)).astype(np.float32)
    b = r.uniform(-0.1, 0.1, o).astype(np.float32) if use_bias else None
    sess = session.Session()
    sess.load_graph(conv_graph(x.shape, wt, b, k, s, p, d, g, act, 0.0, 6.0 if act == "Clip" else 0.0))
    sess.run({"input": x})
    got = sess.get_output("output", "NHWC")
    # constants as the device saw them
    np.testing.assert_array_equal(sess.get_output("conv2d1.weight", "NCHW"), wt)
    if use_bias:
        np.testing.assert_array_equal(sess.get_output("conv2d1.bias", "ANY"), b)
    oact = {"": O.ACT_NONE, "Relu": O.ACT_RELU, "Clip": O.ACT_CLIP}[act]
    variant = O.VARIANT_PW if (k == 1 and s == 1 and p == 0 and g == 1) else O.VARIANT_NHWC4
    ref = O.conv2d(x, wt, b, s, p, d, g, oact, 0.0, 6.0, variant)
    assert_conv_close(got, ref, O.conv2d_abs(x, wt, b, s, p, d, g), FP32_RTOL, str(case))
    # NCHW readback is the transpose of the NHWC one
    np.testing.assert_array_equal(sess.get_output("output", "NCHW"), got.transpose(0, 3, 1, 2))
    # a second Run with new data reuses the allocation
    x2 = r.uniform(-1, 1, x.shape).astype(np.float32)
    sess.run({"input": x2})
    ref2 = O.conv2d(x2, wt, b, s, p, d, g, oact, 0.0, 6.0, variant)
    assert_conv_close(sess.get_output("output", "NHWC"), ref2, O.conv2d_abs(x2, wt, b, s, p, d, g), FP32_RTOL, "second run")
    # the input shape is fixed after the first Run
    with pytest.raises(RuntimeError, match="changed shape"):
        sess.run({"input": np.zeros((n, h + 1, w, c), np.float32)})


@pytest.mark.parametrize("shapes,axis", [
    (((2, 3, 5), (2, 3, 5)), 0), (((2, 3, 5), (2, 4, 5)), 1), (((2, 3, 5), (2, 3, 7)), 2),
    (((1, 2, 3, 4), (1, 2, 3, 6)), -1), (((5,), (3,)), 0), (((2, 6), (2, 1)), 1),
    (((3, 2, 4, 4), (1, 2, 4, 4)), 0),
])
def test_concat_of_constants(shapes, axis):
    """concat_test.cc:51-95: both inputs are Const nodes, Run({}) computes at Setup."""
    r = rng(7200)
    a = [r.normal(0, 1, s).astype(np.float32) for s in shapes]
    gb = dlx.GraphBuilder()
    ids = [gb.add_const("const%d" % (i + 1), t) for i, t in enumerate(a)]
    gb.add_concat("output", ids, axis)
    sess = session.Session()
    sess.load_graph(gb)
    sess.run({})
    np.testing.assert_array_equal(sess.get_output("const1", "ANY"), a[0])
    np.testing.assert_array_equal(sess.get_output("output", "ANY"), O.concat(a, axis))


def test_concat_shape_mismatch_is_fatal():
    gb = dlx.GraphBuilder()
    ids = [gb.add_const("a", np.zeros((2, 3), np.float32)), gb.add_const("b", np.zeros((3, 3), np.float32))]
    gb.add_concat("output", ids, 1)
    sess = session.Session()
    sess.load_graph(gb)
    with pytest.raises(RuntimeError, match="Check failed"):
        sess.run({})


@pytest.mark.parametrize("kind,k,s,p", [("MaxPool", 3, 2, 1), ("MaxPool", 2, 2, 0), ("AveragePool", 3, 1, 1),
                                        ("GlobalAveragePool", 0, 0, 0)])
def test_pool_node_graph(kind, k, s, p):
    r = rng(7300)
    x = r.normal(0, 1, (2, 14, 14, 12)).astype(np.float32)
    gb = dlx.GraphBuilder()
    xi = gb.add_input("input", [2, 12, 14, 14])
    gb.add_pool("output", xi, kind, k, s, p)
    sess = session.Session()
    sess.load_graph(gb)
    sess.run({"input": x})
    ptype = {"MaxPool": O.POOL_MAX, "AveragePool": O.POOL_AVG, "GlobalAveragePool": O.POOL_GLOBAL_AVG}[kind]
    ref = O.pool2d(x, k, s, p, ptype)
    got = sess.get_output("output", "NHWC")
    if kind == "GlobalAveragePool":
        np.testing.assert_allclose(got, ref, rtol=0, atol=1e-6)
    else:
        np.testing.assert_array_equal(got, ref)


def test_decoder_node_graph():
    r = rng(7400)
    batch, hh, ww = 2, 5, 6
    pred = r.normal(0, 1, (batch, hh * ww, 4)).astype(np.float32)
    anchors = np.concatenate([r.uniform(.1, .9, (batch, hh, ww, 2)), r.uniform(.05, .5, (batch, hh, ww, 2))],
                             -1).astype(np.float32)
    gb = dlx.GraphBuilder()
    pi = gb.add_const("pred", pred)
    ai = gb.add_const("anchors", anchors)
    gb.add_decoder("boxes", pi, ai)
    sess = session.Session()
    sess.load_graph(gb)
    sess.run({})
    got = sess.get_output("boxes", "ANY")
    for b in range(batch):
        ref = O.ssd_decode(pred[b:b + 1], anchors[b].reshape(-1, 4))
        np.testing.assert_allclose(got[b:b + 1], ref, rtol=0, atol=1e-4)
    # anchors must be (N, H, W, 4) with H*W == priors (decoder.cc:82-85)
    gb = dlx.GraphBuilder()
    gb.add_decoder("boxes", gb.add_const("pred", pred), gb.add_const("anchors", anchors[:, :, :5]))
    sess = session.Session()
    sess.load_graph(gb)
    with pytest.raises(RuntimeError, match="Check failed"):
        sess.run({})


def test_transpose_and_reshape_nodes():
    r = rng(7500)
    x = r.normal(0, 1, (2, 5, 4, 6)).astype(np.float32)   # NHWC
    gb = dlx.GraphBuilder()
    xi = gb.add_input("input", [2, 6, 5, 4])
    # ONNX perm over NCHW axes: [0,2,3,1] is the identity on NHWC storage (a view here)
    t0 = gb.add_transpose("t_identity", xi, [0, 2, 3, 1])
    shp = gb.add_const("shape", np.array([0, -1, 3], np.float32))
    gb.add_reshape("view", t0, shp)
    # ONNX perm [0,1,3,2] over NCHW axes; the output is laid out in the ONNX output axis order
    gb.add_transpose("t_swap", xi, [0, 1, 3, 2])
    sess = session.Session()
    sess.load_graph(gb)
    sess.run({"input": x})
    np.testing.assert_array_equal(sess.get_output("t_identity", "ANY"), x)
    np.testing.assert_array_equal(sess.get_output("view", "ANY"), x.reshape(2, -1, 3))
    # renamed perm: p -> {0,3,1,2}[p], so [0,1,3,2] -> [0,3,2,1]; out[d] = in[perm[d]]
    np.testing.assert_array_equal(sess.get_output("t_swap", "ANY"), x.transpose(0, 3, 2, 1))
    assert sess.tensor_device_ptr("view") == sess.tensor_device_ptr("input")


def test_exported_view_chain_folds_at_setup():
    """PyTorch exports x.permute(0,2,3,1).view(N, -1, K) with the batch size taken from the
    tensor: Shape -> Gather(0) -> Unsqueeze -> Concat([n], [-1], [K]) -> Reshape.  The chain runs
    once while the session is set up (shape.h:19, fbo_session.cc:240-244) and the view aliases
    its input.  Gather's index counts NCHW positions while the shape vector is NHWC
    (gather.glsl:10-18)."""
    r = rng(7600)
    x = r.normal(0, 1, (3, 5, 4, 8)).astype(np.float32)   # NHWC
    gb = dlx.GraphBuilder()
    xi = gb.add_input("input", [3, 8, 5, 4])
    t0 = gb.add_transpose("perm", xi, [0, 2, 3, 1])
    shp = gb.add_shape("shape_of", xi)
    dims = {}
    for name, idx in (("n", 0), ("c", 1), ("h", 2), ("w", 3)):
        ci = gb.add_const("idx_" + name, np.array([idx], np.float32), dims=[])
        gi = gb.add_gather("dim_" + name, shp, ci)
        dims[name] = gb.add_unsqueeze("dim_" + name + "_1", gi, 0)
    minus1 = gb.add_const("minus1", np.array([-1], np.float32))
    four = gb.add_const("four", np.array([4], np.float32))
    target = gb.add_concat("target", [dims["n"], minus1, four], 0)
    gb.add_reshape("view", t0, target)
    alldims = gb.add_concat("nchw", [dims["n"], dims["c"], dims["h"], dims["w"]], 0)
    sess = session.Session()
    sess.load_graph(gb)
    sess.run({"input": x})
    np.testing.assert_array_equal(sess.get_output("shape_of", "ANY"), [3, 5, 4, 8])
    np.testing.assert_array_equal(sess.get_output("nchw", "ANY"), [3, 8, 5, 4])
    np.testing.assert_array_equal(sess.get_output("target", "ANY"), [3, -1, 4])
    np.testing.assert_array_equal(sess.get_output("view", "ANY"), x.reshape(3, -1, 4))
    assert sess.tensor_device_ptr("view") == sess.tensor_device_ptr("input")
    assert sess.tensor_shape("dim_n") == () and sess.tensor_shape("dim_n_1") == (1,)
    # nothing of the chain is left on the per-pass path
    assert sess.issue_order() == ["perm", "view"]


@pytest.mark.parametrize("batch", [1, 8])
def test_config2_block_through_session(batch):
    g, w = models.separable_block(batch)
    x = rng(20240002).uniform(0, 6, (batch, 38, 38, 256)).astype(np.float32)
    sess = session.Session()
    sess.load_graph(g)
    sess.run({"input": x})
    dw = sess.get_output("dw", "NHWC")
    pw = sess.get_output("pw", "NHWC")
    ref1 = O.conv2d(x, w["wd"], w["bd"], 1, 1, 1, 256, O.ACT_CLIP, 0.0, 6.0)
    assert_conv_close(dw, ref1, O.conv2d_abs(x, w["wd"], w["bd"], 1, 1, 1, 256), FP32_RTOL, "dw")
    ref2 = O.conv2d(dw, w["wp"], w["bp"], act=O.ACT_CLIP, maxv=6.0, variant=O.VARIANT_PW)
    assert_conv_close(pw, ref2, O.conv2d_abs(dw, w["wp"], w["bp"]), FP32_RTOL, "pw")


def _run_ssd(batch, seed=20240005):
    g, info = models.mobilenet_v1_ssd(batch, seed=seed, with_weights=True)
    x = rng(seed + 1).uniform(-1, 1, (batch, 300, 300, 3)).astype(np.float32)
    sess = session.Session()
    sess.load_graph(g)
    sess.run({"input": x})
    return sess, info, x


def _check_every_layer(sess, info, x, images):
    """Every conv layer of the network against the oracle applied to the DEVICE's input of that
    layer, for the listed images of the batch, so each of the 47 convolutions is held to the fp32
    tolerance on its own (errors do not compound across the check).  Returns the device's outputs
    (those images only) by layer name and the worst normwise error."""
    images = list(images)
    produced = {"input": x[images]}
    prev = "input"
    feature_of = {}
    worst = 0.0
    for l in info["layers"]:
        name = l["name"]
        src = feature_of[int(name[4])] if name.startswith("head") else prev
        xin = produced[src]
        w, b = info["weights"][name]
        act = O.ACT_CLIP if l["act"] else O.ACT_NONE
        variant = O.VARIANT_PW if l["kind"] == "pw" else O.VARIANT_NHWC4
        ref = O.conv2d(xin, w, b, l["stride"], l["pad"], 1, l["group"], act, 0.0, 6.0, variant)
        got = np.ascontiguousarray(sess.get_output(name, "NHWC")[images])
        worst = max(worst, assert_conv_close(got, ref, O.conv2d_abs(xin, w, b, l["stride"], l["pad"], 1,
                                                                    l["group"]), FP32_RTOL, name))
        produced[name] = got
        if not name.startswith("head"):
            prev = name
            if name in ("block11.pw", "block13.pw"):
                feature_of[0 if name == "block11.pw" else 1] = name
            if name.startswith("extra") and name.endswith(".conv"):
                feature_of[int(name[5]) + 1] = name
    assert 0.0 < worst <= FP32_RTOL
    return produced, worst


def test_mobilenet_ssd_every_layer_matches_oracle():
    """Full MobileNet-v1 SSD 300x300, batch 1: each of the 47 convolutions against the oracle on
    the device's own input of that layer, then the concatenations and the anchors."""
    sess, info, x = _run_ssd(1)
    produced, worst = _check_every_layer(sess, info, x, [0])
    print("47 layers, worst |err| / sum|x||w| = %.3g" % worst)
    loc = sess.get_output("box_preds", "ANY")
    conf = sess.get_output("cls_logits", "ANY")
    assert loc.shape == (1, 1917, 4) and conf.shape == (1, 1917, 21)
    np.testing.assert_array_equal(
        loc, np.concatenate([produced["head%d.loc" % i].reshape(1, -1, 4) for i in range(6)], 1))
    np.testing.assert_array_equal(
        conf, np.concatenate([produced["head%d.conf" % i].reshape(1, -1, 21) for i in range(6)], 1))
    np.testing.assert_array_equal(sess.get_output("anchors", "ANY"), info["anchors"])


def test_mobilenet_ssd_batch16_every_layer_matches_oracle():
    """The headline configuration (batch 16) runs other kernels than batch 1: 64x64 LDS tiles
    instead of the wave-split kernel, the twelve heads as one grid with their K split, outputs
    stored an image stride apart inside the concatenations.  Each of the 47 convolutions is held
    to the oracle on the device's own input of that layer, for the first and the last image of the
    batch (the oracle takes those two images only), and the concatenations to the heads' outputs."""
    sess, info, x = _run_ssd(16)
    images = [0, 15]
    produced, worst = _check_every_layer(sess, info, x, images)
    print("batch 16, 47 layers x 2 images, worst |err| / sum|x||w| = %.3g" % worst)
    loc = sess.get_output("box_preds", "ANY")
    conf = sess.get_output("cls_logits", "ANY")
    assert loc.shape == (16, 1917, 4) and conf.shape == (16, 1917, 21)
    np.testing.assert_array_equal(
        loc[images], np.concatenate([produced["head%d.loc" % i].reshape(2, -1, 4) for i in range(6)], 1))
    np.testing.assert_array_equal(
        conf[images], np.concatenate([produced["head%d.conf" % i].reshape(2, -1, 21) for i in range(6)], 1))
    # and the replayed pass (hipGraph) gives what the eager pass gave
    sess.compute(graph=True)
    np.testing.assert_array_equal(sess.get_output("box_preds", "ANY"), loc)
    np.testing.assert_array_equal(sess.get_output("cls_logits", "ANY"), conf)


def test_concat_inputs_are_produced_in_place_at_batch1():
    """With a single slice before the concat axis (batch 1) the heads write straight into the
    concat outputs: every head output sits at its running offset inside box_preds / cls_logits
    (the class heads at offsets that are only 4-byte aligned: 63 and 126 channels are stored
    element by element), the concat has nothing to copy, and a replay after new input still gives
    the concatenation."""
    sess, info, x = _run_ssd(1)
    for out_name, suffix, last in (("box_preds", "loc", 4), ("cls_logits", "conf", 21)):
        base = sess.tensor_device_ptr(out_name)
        off = 0
        for i in range(6):
            assert sess.tensor_device_ptr("head%d.%s" % (i, suffix)) == base + off, (out_name, i)
            assert sess.tensor_device_ptr("head%d.%s.view" % (i, suffix)) == base + off
            off += int(np.prod(sess.tensor_shape("head%d.%s" % (i, suffix)))) * 4
        assert off == 1917 * last * 4
    x2 = rng(77).uniform(-1, 1, x.shape).astype(np.float32)
    sess.run({"input": x2})
    for out_name, suffix, last in (("box_preds", "loc", 4), ("cls_logits", "conf", 21)):
        parts = [sess.get_output("head%d.%s" % (i, suffix), "NHWC").reshape(1, -1, last) for i in range(6)]
        np.testing.assert_array_equal(sess.get_output(out_name, "ANY"), np.concatenate(parts, 1))
    # the same network at batch 1 and as image 0 of a batch of 2
    sess2, _, xb = _run_ssd(2)
    sess.run({"input": xb[:1]})
    for name in ("box_preds", "cls_logits"):
        a, b = sess.get_output(name, "ANY"), sess2.get_output(name, "ANY")[:1]
        assert np.all(np.abs(a - b) <= 1e-4 * (np.abs(b) + 1.0)), name


def test_concat_inputs_are_produced_in_place_at_batch3():
    """With several slices before the concat axis (batch > 1) the heads write their images
    one output slice apart (OgleConvArgs.out_image_stride), straight into box_preds /
    cls_logits: no Concat launch is left in the pass, a head's tensor is no longer dense on
    the device (no device pointer; reading it back gathers its images), every head still
    matches the oracle on the device's own feature map, the concat outputs are exactly the
    heads side by side, and a replayed hipGraph gives the same."""
    batch = 3
    g, info = models.mobilenet_v1_ssd(batch, seed=20240005, with_weights=True)
    x = rng(79).uniform(-1, 1, (batch, 300, 300, 3)).astype(np.float32)
    sess = session.Session()
    sess.load_graph(g)
    sess.run({"input": x})
    labels = [l for l, _ in sess.launch_plan()]
    assert not any("#Concat#" in l for l in labels), labels
    assert any("head0.loc#Conv#" in l for l in labels)
    feats = ["block11.pw", "block13.pw", "extra1.conv", "extra2.conv", "extra3.conv", "extra4.conv"]
    for out_name, suffix, last in (("box_preds", "loc", 4), ("cls_logits", "conf", 21)):
        assert sess.tensor_device_ptr(out_name) is not None
        parts = []
        for i, feat in enumerate(feats):
            name = "head%d.%s" % (i, suffix)
            assert sess.tensor_device_ptr(name) is None and sess.tensor_device_ptr(name + ".view") is None
            got = sess.get_output(name, "NHWC")
            xin = sess.get_output(feat, "NHWC")
            w, b = info["weights"][name]
            assert_conv_close(got, O.conv2d(xin, w, b, 1, 1), O.conv2d_abs(xin, w, b, 1, 1), FP32_RTOL,
                              "in place " + name)
            np.testing.assert_array_equal(sess.get_output(name + ".view", "ANY"), got.reshape(batch, -1, last))
            # NCHW readback of a tensor whose images lie apart
            np.testing.assert_array_equal(sess.get_output(name, "NCHW"), got.transpose(0, 3, 1, 2))
            parts.append(got.reshape(batch, -1, last))
        whole = sess.get_output(out_name, "ANY")
        assert whole.shape == (batch, 1917, last)
        np.testing.assert_array_equal(whole, np.concatenate(parts, 1))
        sess.compute(graph=True)
        np.testing.assert_array_equal(sess.get_output(out_name, "ANY"), whole)
        sess.compute(graph=False)
        np.testing.assert_array_equal(sess.get_output(out_name, "ANY"), whole)


def test_concat_at_batch2_copies_what_cannot_be_produced_in_place():
    """Batch 2, concat over axis 1: a pooling output cannot be written with its images apart and
    a convolution with a second reader must stay dense, so the concat copies; two convolutions
    read by nothing else are placed.  Same values either way."""
    r = rng(7995)
    x = r.uniform(-1, 1, (2, 6, 6, 16)).astype(np.float32)
    wa = r.normal(0, 0.3, (8, 16, 3, 3)).astype(np.float32)
    wb = r.normal(0, 0.3, (8, 16, 3, 3)).astype(np.float32)
    ra, rb = O.conv2d(x, wa, None, 1, 1), O.conv2d(x, wb, None, 1, 1)
    for kind in ("placed", "pool", "second_reader"):
        gb = dlx.GraphBuilder()
        xi = gb.add_input("input", [2, 16, 6, 6])
        a = gb.add_conv("a", xi, gb.add_filter("a.weight", wa), None, 3, 1, 1)
        b = gb.add_conv("b", xi, gb.add_filter("b.weight", wb), None, 3, 1, 1)
        second = b
        if kind == "pool":
            second = gb.add_pool("b.pool", b, "MaxPool", 1, 1, 0)     # a copy of b made by another kernel
        if kind == "second_reader":
            gb.add_relu("b.relu", b)
        outs = []
        for name, y in (("a", a), ("b", second)):
            t = gb.add_transpose(name + ".permute", y, [0, 2, 3, 1])
            shp = gb.add_const(name + ".shape", np.array([2, -1, 4], np.float32))
            outs.append(gb.add_reshape(name + ".view", t, shp))
        gb.add_concat("cat", outs, 1)
        sess = session.Session()
        sess.load_graph(gb)
        sess.run({"input": x})
        cat = sess.get_output("cat", "ANY")
        ref = np.concatenate([ra.reshape(2, -1, 4), rb.reshape(2, -1, 4)], 1)
        assert cat.shape == ref.shape
        np.testing.assert_allclose(cat, ref, rtol=0, atol=1e-4)
        labels = " ".join(l for l, _ in sess.launch_plan())
        if kind == "placed":
            assert "#Concat#" not in labels and sess.tensor_device_ptr("a") is None
        else:
            assert "cat#Concat#" in labels and sess.tensor_device_ptr("a") is not None
        if kind == "second_reader":
            np.testing.assert_array_equal(sess.get_output("b.relu", "NHWC"), np.maximum(sess.get_output("b", "NHWC"), 0))
        np.testing.assert_array_equal(sess.get_output("a", "NHWC").reshape(2, -1, 4), cat[:, :72])


def test_graph_replay_equals_eager_batch2():
    """The captured hipGraph is replayed several times with eager work and synchronisations in
    between; every replay must reproduce the eager result bit for bit."""
    sess, info, x = _run_ssd(2, seed=77)
    eager_loc = sess.get_output("box_preds", "ANY")
    eager_conf = sess.get_output("cls_logits", "ANY")
    for i in range(3):
        sess.compute(graph=True)
        np.testing.assert_array_equal(sess.get_output("box_preds", "ANY"), eager_loc)
        np.testing.assert_array_equal(sess.get_output("cls_logits", "ANY"), eager_conf)
        sess.compute(graph=False)
        sess.sync()
    # new input through the normal path, then replay: the graph reads the same buffers
    x2 = rng(1234).uniform(-1, 1, x.shape).astype(np.float32)
    sess.run({"input": x2})
    loc2 = sess.get_output("box_preds", "ANY")
    assert not np.array_equal(loc2, eager_loc)
    sess.compute(graph=True)
    np.testing.assert_array_equal(sess.get_output("box_preds", "ANY"), loc2)
    # per-node profile covers every live node once
    prof = sess.profile()
    assert len(prof) == 47 + 24 + 2 and all(ms >= 0 for _, _, ms in prof)
    assert prof[0][0] == "conv0#Conv#"


def test_reordered_issue_equals_file_order():
    """The executor issues the SSD heads early, next to the feature-extractor chain, so that
    they share launches.  The issue order must be a dependency-respecting permutation of the
    file order, and every output must be bit-identical to a strict file-order run (eager and
    replayed as a graph)."""
    # batch 8: below a few images the heads cost less than one launch and nothing is moved
    g, info = models.mobilenet_v1_ssd(8, seed=99, with_weights=True)
    x = rng(100).uniform(-1, 1, (8, 300, 300, 3)).astype(np.float32)
    outs = {}
    orders = {}
    for reorder in (False, True):
        sess = session.Session()
        sess.set_reorder(reorder)
        sess.load_graph(g)
        sess.run({"input": x})
        orders[reorder] = sess.issue_order()
        eager = {n: sess.get_output(n, "ANY") for n in ("box_preds", "cls_logits", "extra4.conv",
                                                        "head0.conf", "head5.loc")}
        sess.compute(graph=True)
        sess.compute(graph=True)
        for n, v in eager.items():
            np.testing.assert_array_equal(sess.get_output(n, "ANY"), v)
        outs[reorder] = eager
    for n in outs[False]:
        np.testing.assert_array_equal(outs[True][n], outs[False][n])
    file_order, issued = orders[False], orders[True]
    assert sorted(file_order) == sorted(issued) and file_order != issued
    pos = {n: i for i, n in enumerate(issued)}
    # heads move ahead of (part of) the extras chain, never ahead of their feature map
    assert pos["head0.conf"] < pos["extra4.conv"]
    for i, feat in enumerate(["block11.pw", "block13.pw", "extra1.conv", "extra2.conv",
                              "extra3.conv", "extra4.conv"]):
        assert pos["head%d.loc" % i] > pos[feat] and pos["head%d.conf" % i] > pos[feat]
    # everything that is not a head keeps its relative order
    rest = [n for n in issued if not n.startswith("head")]
    assert rest == [n for n in file_order if not n.startswith("head")]


@pytest.mark.parametrize("device_nms", [True, False])
def test_detector_matches_oracle_pipeline(device_nms):
    """Detector::Detect: graph -> decode + score filter (device) -> top-k -> NMS (device, or the
    host loop the reference uses), against the oracle's restatement of GenerateBoxInfo / GetTopK /
    NMS fed with the device's own logits and box predictions.  Head weights ~N(0, 0.05) give
    logits wide enough that priors pass."""
    batch = 2
    g, info = models.mobilenet_v1_ssd(batch, seed=31, head_std=0.05)
    x = rng(32).uniform(-1, 1, (batch, 300, 300, 3)).astype(np.float32)
    sess = session.Session()
    sess.set_device_nms(device_nms)
    sess.load_graph(g)
    dets = sess.detect(x, 640, 480, 0.3, 0.45, 100)
    conf = sess.get_output("cls_logits", "ANY")
    loc = sess.get_output("box_preds", "ANY")
    boxes = O.ssd_decode(loc, info["anchors"])
    ora = O.box_info(conf, boxes, 0.3, 640.0, 480.0)
    total = 0
    for b in range(batch):
        keep = O.topk_nms(ora[b]["score"], ora[b]["rect"], 100, 0.45)
        exp_prior = ora[b]["prior"][keep]
        got_prior = np.array([d["prior"] for d in dets[b]], np.int32)
        np.testing.assert_array_equal(got_prior, exp_prior)
        np.testing.assert_array_equal(np.array([d["cls"] for d in dets[b]], np.int32), ora[b]["cls"][keep])
        got_rect = np.array([d["rect"] for d in dets[b]], np.int32).reshape(-1, 4)
        exp_rect = ora[b]["rect"][keep]
        assert np.abs(got_rect - exp_rect).max(initial=0) <= 1   # 1e-4 in coordinates can move a truncation
        total += len(got_prior)
    assert total > 0


@pytest.mark.parametrize("device_nms", [True, False])
def test_detector_inside_graph_equals_eager(device_nms):
    """time_compute(with_detect) records the detector's device work behind the pass in one
    hipGraph; its detections after several replays must equal Detector::Detect run eagerly on
    the same input (time_compute scales boxes to 300x300)."""
    batch = 3
    g, info = models.mobilenet_v1_ssd(batch, seed=41, head_std=0.05)
    x = rng(42).uniform(-1, 1, (batch, 300, 300, 3)).astype(np.float32)
    sess = session.Session()
    sess.set_device_nms(device_nms)
    sess.load_graph(g)
    eager = sess.detect(x, 300, 300, 0.3, 0.45, 100)
    assert sum(len(e) for e in eager) > 0
    for use_graph in (False, True):
        sess.time_compute(1, 3, graph=use_graph, with_detect=True)
        got = sess.detect_results(batch)
        assert got == eager


def test_pipelined_sessions_keep_their_own_results():
    """ogle_rt_time_pipelined deals passes round-robin over several sessions, each replaying its
    hipGraph on its own stream.  Every session must end with exactly what it computes alone:
    outputs bit-identical to its own eager pass, detections equal to Detector::Detect on its own
    input, whatever ran next to it."""
    batch = 2
    sessions, inputs, eager_out, eager_det = [], [], [], []
    for i in range(3):
        g, info = models.mobilenet_v1_ssd(batch, seed=41, head_std=0.05)
        x = rng(500 + i).uniform(-1, 1, (batch, 300, 300, 3)).astype(np.float32)
        s = session.Session()
        s.load_graph(g)
        eager_det.append(s.detect(x, 300, 300, 0.3, 0.45, 100))
        eager_out.append([s.get_output(n, "ANY") for n in ("box_preds", "cls_logits")])
        sessions.append(s)
        inputs.append(x)
    assert eager_det[0] != eager_det[1]          # different inputs, different detections
    total = session.Session.time_pipelined(sessions, 3, 10, with_detect=True)
    assert total > 0
    for i, s in enumerate(sessions):
        for name, ref in zip(("box_preds", "cls_logits"), eager_out[i]):
            np.testing.assert_array_equal(s.get_output(name, "ANY"), ref)
        assert s.detect_results(batch) == eager_det[i]
    # a single session is accepted too, and so is the pass without the detector's work
    assert session.Session.time_pipelined(sessions[:1], 0, 2, with_detect=False) > 0
    np.testing.assert_array_equal(sessions[0].get_output("box_preds", "ANY"), eager_out[0][0])
    # with uploads from page-locked memory: the sessions swap inputs, and their results follow
    pinned = [session.PinnedBuffer((batch, 300, 300, 3)) for _ in sessions]
    order = [1, 2, 0]
    for pb, j in zip(pinned, order):
        pb.array[...] = inputs[j]
    session.Session.time_pipelined(sessions, 1, 5, True, "input", pinned)
    for s, j in zip(sessions, order):
        for name, ref in zip(("box_preds", "cls_logits"), eager_out[j]):
            np.testing.assert_array_equal(s.get_output(name, "ANY"), ref)
        assert s.detect_results(batch) == eager_det[j]
    for pb in pinned:
        pb.close()


def test_pipelined_readback_lists_equal_detect_results():
    """Passes whose final detection lists are copied to page-locked host memory inside the
    captured graph, the host waiting only for the event behind a session's previous pass: the
    lists read that way equal what the synchronous readback of the same session gives and what
    Detector::Detect computes eagerly, for one session alone (every pass waits for the one
    before) and for three sessions with different inputs in flight together, replay after replay
    and after an input change."""
    batch = 3
    g, _ = models.mobilenet_v1_ssd(batch, seed=41, head_std=0.05)
    inputs = [rng(90 + i).uniform(-1, 1, (batch, 300, 300, 3)).astype(np.float32) for i in range(3)]
    sessions, eager = [], []
    for x in inputs:
        s = session.Session()
        s.load_graph(g)
        eager.append(s.detect(x, 300, 300, 0.3, 0.45, 100))
        sessions.append(s)
    assert all(sum(len(e) for e in d) > 0 for d in eager)
    per_pass = [sum(len(e) for e in d) for d in eager]
    # one session: 5 timed passes, every one's lists read by the host
    ms, seen = session.Session.time_pipelined_readback(sessions[:1], 2, 5)
    assert ms > 0 and seen == 5 * per_pass[0]
    assert sessions[0].pipelined_results(batch) == eager[0]
    assert sessions[0].detect_results(batch) == eager[0]
    # three sessions in flight: 7 passes dealt round-robin (3 + 2 + 2)
    ms, seen = session.Session.time_pipelined_readback(sessions, 3, 7)
    assert seen == 3 * per_pass[0] + 2 * per_pass[1] + 2 * per_pass[2]
    for s, e in zip(sessions, eager):
        assert s.pipelined_results(batch) == e
        assert s.detect_results(batch) == e
    # new inputs: the replayed copy follows them
    sessions[0].run({"input": inputs[1]})
    sessions[1].run({"input": inputs[2]})
    session.Session.time_pipelined_readback(sessions[:2], 1, 4)
    assert sessions[0].pipelined_results(batch) == eager[1]
    assert sessions[1].pipelined_results(batch) == eager[2]
    # the host loop of the reference is not what is copied: refused with the host top-k + NMS
    sessions[2].set_device_nms(False)
    with pytest.raises(RuntimeError, match="ogle_rt_set_device_nms"):
        session.Session.time_pipelined_readback(sessions[2:], 1, 1)


def test_batch16_images_match_their_batch1_passes():
    """The headline configuration (batch 16) takes other tile shapes, K splits and issue order than
    batch 1.  Every image is independent through every kernel, so image i of a batch-16 pass must
    equal a batch-1 pass over that image, up to the summation order (1e-4 of the output scale)."""
    sess16, info, x = _run_ssd(16)
    loc16 = sess16.get_output("box_preds", "ANY")
    conf16 = sess16.get_output("cls_logits", "ANY")
    feat16 = sess16.get_output("block13.pw", "NHWC")
    assert loc16.shape == (16, 1917, 4) and conf16.shape == (16, 1917, 21)
    g1, _ = models.mobilenet_v1_ssd(1, seed=20240005)
    sess1 = session.Session()
    sess1.load_graph(g1)
    for i in (0, 7, 15):
        sess1.run({"input": x[i:i + 1]})
        for name, ref in (("box_preds", loc16), ("cls_logits", conf16), ("block13.pw", feat16)):
            got = sess1.get_output(name, "ANY" if name != "block13.pw" else "NHWC")
            scale = float(np.abs(ref[i]).max())
            assert np.abs(got[0] - ref[i]).max() <= 1e-4 * scale, (name, i)


# ---- ANY / ANY4 inputs, activation rules, padded readback, reload -----------------------

ANY_INPUT_CASES = [
    # n, h, w, c, o, k, s, p, g, bias, act, minv, maxv
    (1, 2, 2, 1, 1, 3, 1, 1, 1, False, "", 0.0, 0.0),         # conv2d_test.cc:220-234 as written
    (2, 9, 9, 8, 12, 3, 1, 1, 1, True, "Relu", -0.5, 0.0),    # conv2d_any4: relu is max(min, x)
    (1, 7, 7, 16, 16, 3, 1, 1, 16, True, "Clip", 0.25, 2.0),  # conv2d_dw_any4: clip (min, max)
    (2, 5, 5, 32, 24, 1, 1, 0, 1, True, "Clip", 0.25, 2.0),   # conv2d_pw_any4: min is NOT ignored
    (2, 5, 5, 32, 24, 1, 1, 0, 1, True, "Relu", -0.5, 0.0),
]


@pytest.mark.parametrize("case", ANY_INPUT_CASES)
def test_conv_on_any_input_selects_the_any4_variant(case):
    """An ANY host input becomes an ANY4 device tensor and Conv then takes the *_any4 shader
    (conv2d.cc:44-61), whose fused activation reads min / max differently
    (conv2d_any4.glsl:89-94); the output keeps the input's tag (conv2d.cc:64)."""
    n, h, w, c, o, k, s, p, g, use_bias, act, minv, maxv = case
    r = rng(7700 + ANY_INPUT_CASES.index(case))
    x = r.uniform(-1, 1, (n, h, w, c)).astype(np.float32)
    wt = r.normal(0, 0.5, (o, c // g, k, k)).astype(np.float32)
    b = r.uniform(-0.1, 0.1, o).astype(np.float32) if use_bias else None
    sess = session.Session()
    sess.load_graph(conv_graph(x.shape, wt, b, k, s, p, 1, g, act, minv, maxv))
    sess.run({"input": x}, dformats={"input": "ANY"})
    assert sess.tensor_dformat("input") == "ANY4" and sess.tensor_dformat("output") == "ANY4"
    got = sess.get_output("output", "ANY")
    oact = {"": O.ACT_NONE, "Relu": O.ACT_RELU, "Clip": O.ACT_CLIP}[act]
    ref = O.conv2d(x, wt, b, s, p, 1, g, oact, minv, maxv, O.VARIANT_ANY4)
    assert_conv_close(got, ref, O.conv2d_abs(x, wt, b, s, p, 1, g), FP32_RTOL, str(case))
    if act:
        assert got.min() >= minv and (ref != O.conv2d(x, wt, b, s, p, 1, g, oact, 0.0, maxv,
                                                       O.VARIANT_PW)).any()


def test_grouped_conv_activation_reads_min_like_the_any4_shaders():
    """conv2d_grp.glsl:115-121: Relu is max(min_value, x), Clip is (min, max)."""
    r = rng(7750)
    x = r.uniform(-1, 1, (2, 8, 8, 8)).astype(np.float32)
    wt = r.normal(0, 0.5, (12, 2, 3, 3)).astype(np.float32)
    b = r.uniform(-0.1, 0.1, 12).astype(np.float32)
    for act, oact, minv, maxv in (("Relu", O.ACT_RELU, -0.25, 0.0), ("Clip", O.ACT_CLIP, -0.5, 0.75)):
        sess = session.Session()
        sess.load_graph(conv_graph(x.shape, wt, b, 3, 1, 1, 1, 4, act, minv, maxv))
        sess.run({"input": x})
        ref = O.conv2d(x, wt, b, 1, 1, 1, 4, oact, minv, maxv, O.VARIANT_ANY4)
        got = sess.get_output("output", "NHWC")
        assert_conv_close(got, ref, O.conv2d_abs(x, wt, b, 1, 1, 1, 4), FP32_RTOL, act)
        assert got.min() == np.float32(minv)


def test_get_outputs_in_the_padded_host_layouts():
    """GetOutputs with "NHWC4" / "ANY4" / "HWN4C4" returns the reference's stride-4 layouts
    (tensor_format.cc:272-343, cpu_functor.cc:10-127), padding lanes zero; an input handed
    over in a padded layout is unpadded on upload."""
    r = rng(7800)
    x = r.uniform(-1, 1, (2, 5, 4, 6)).astype(np.float32)
    wt = r.normal(0, 0.5, (7, 6, 3, 3)).astype(np.float32)
    b = r.uniform(-0.1, 0.1, 7).astype(np.float32)
    sess = session.Session()
    sess.load_graph(conv_graph(x.shape, wt, b, 3, 1, 1))
    sess.run({"input": x})
    dense = sess.get_output("output", "NHWC")
    pad = sess.get_output("output", "NHWC4")
    assert pad.shape == (2, 5, 4, 8)
    np.testing.assert_array_equal(pad[..., :7], dense)
    assert (pad[..., 7:] == 0).all()
    np.testing.assert_array_equal(sess.get_output("output", "ANY4"), pad)
    bias4 = sess.get_output("conv2d1.bias", "ANY4")
    assert bias4.shape == (8,) and (bias4[:7] == b).all() and bias4[7] == 0
    np.testing.assert_array_equal(sess.get_output("conv2d1.weight", "HWN4C4").ravel(),
                                  O.nchw_to_hwn4c4(wt).ravel())
    with pytest.raises(RuntimeError, match="HWN4C4"):
        sess.get_output("output", "HWN4C4")
    # upload from the padded layout: same device contents, same result
    xp = np.zeros((2, 5, 4, 8), np.float32)
    xp[..., :6] = x
    sess2 = session.Session()
    sess2.load_graph(conv_graph(x.shape, wt, b, 3, 1, 1))
    sess2.run({"input": xp}, dformats={"input": "NHWC4"}, shapes={"input": x.shape})
    np.testing.assert_array_equal(sess2.get_output("input", "NHWC4"), xp)
    np.testing.assert_array_equal(sess2.get_output("output", "NHWC"), dense)


def test_reload_after_a_captured_pass():
    """LoadGraph on a session that has run and recorded its pass: the recorded hipGraph (whose
    kernel arguments are the old tensors' addresses) must be gone, and the new graph runs and
    records on its own."""
    g1, w1 = models.separable_block(1, size=19, cin=64, cout=128)
    r = rng(7900)
    x1 = r.uniform(0, 6, (1, 19, 19, 64)).astype(np.float32)
    sess = session.Session()
    sess.load_graph(g1)
    sess.run({"input": x1})
    sess.compute(graph=True)
    first = sess.get_output("pw", "NHWC")
    assert sess.graph_captured(0)
    g2, w2 = models.separable_block(2, seed=5, size=10, cin=32, cout=48)
    x2 = r.uniform(0, 6, (2, 10, 10, 32)).astype(np.float32)
    sess.load_graph(g2)
    assert not sess.graph_captured(0) and sess.issue_order() == []
    sess.run({"input": x2})
    dw = O.conv2d(x2, w2["wd"], w2["bd"], 1, 1, 1, 32, O.ACT_CLIP, 0.0, 6.0)
    ref = O.conv2d(dw, w2["wp"], w2["bp"], act=O.ACT_CLIP, maxv=6.0, variant=O.VARIANT_PW)
    got = sess.get_output("pw", "NHWC")
    assert_conv_close(got, ref, O.conv2d_abs(dw, w2["wp"], w2["bp"]), FP32_RTOL, "after reload")
    sess.compute(graph=True)
    assert sess.graph_captured(0)
    np.testing.assert_array_equal(sess.get_output("pw", "NHWC"), got)
    # and back to the first graph: same answer as before
    sess.load_graph(g1)
    sess.run({"input": x1})
    np.testing.assert_array_equal(sess.get_output("pw", "NHWC"), first)


@pytest.mark.parametrize("second_reader", [False, True])
def test_unaligned_head_also_read_by_another_node_keeps_its_own_buffer(second_reader):
    """At batch 1 head outputs are produced inside the concat output; a 63-channel head lands
    at a 4-byte-aligned place, which only a convolution's element-wise stores tolerate.  If the
    head also feeds a Relu node (16-byte vector loads from the tensor start), it must not be
    moved there."""
    r = rng(7990)
    x = r.uniform(-1, 1, (1, 3, 3, 16)).astype(np.float32)
    wa = r.normal(0, 0.3, (63, 16, 3, 3)).astype(np.float32)
    wb = r.normal(0, 0.3, (63, 16, 3, 3)).astype(np.float32)
    gb = dlx.GraphBuilder()
    xi = gb.add_input("input", [1, 16, 3, 3])
    outs = []
    for name, wt in (("a", wa), ("b", wb)):
        y = gb.add_conv(name, xi, gb.add_filter(name + ".weight", wt), None, 3, 1, 1)
        t = gb.add_transpose(name + ".permute", y, [0, 2, 3, 1])
        shp = gb.add_const(name + ".shape", np.array([1, -1, 21], np.float32))
        outs.append(gb.add_reshape(name + ".view", t, shp))
        if name == "b" and second_reader:
            gb.add_relu("b.relu", y)
    gb.add_concat("cat", outs, 1)
    sess = session.Session()
    sess.load_graph(gb)
    sess.run({"input": x})
    ra, rb = O.conv2d(x, wa, None, 1, 1), O.conv2d(x, wb, None, 1, 1)
    cat = sess.get_output("cat", "ANY")
    ref = np.concatenate([ra.reshape(1, -1, 21), rb.reshape(1, -1, 21)], 1)
    np.testing.assert_allclose(cat, ref, rtol=0, atol=1e-4)
    base = sess.tensor_device_ptr("cat")
    if second_reader:
        np.testing.assert_array_equal(sess.get_output("b.relu", "NHWC"),
                                      np.maximum(sess.get_output("b", "NHWC"), 0))
        # head b would start at byte 9*63*4 = 2268 of the concat output, which is not 16-byte
        # aligned, and it has a second reader: nothing is placed, the concat copies
        assert sess.tensor_device_ptr("a") != base
        assert sess.tensor_device_ptr("b") != base + 2268
    else:
        assert sess.tensor_device_ptr("a") == base
        assert sess.tensor_device_ptr("b") == base + 2268


def test_sibling_heads_fused_into_one_launch():
    """With sibling fusion on, the box and class head of a feature map run as one contraction
    with two destinations (OgleConvArgs.output2_dev).  Every head output still matches the
    oracle on the device's own feature map, and agrees with the one-launch-per-node run to
    summation order; the absorbed node no longer launches anything."""
    g, info = models.mobilenet_v1_ssd(4, seed=77, with_weights=True)
    x = rng(78).uniform(-1, 1, (4, 300, 300, 3)).astype(np.float32)
    runs = {}
    for fuse in (False, True):
        sess = session.Session()
        sess.set_fuse_siblings(fuse)
        sess.load_graph(g)
        sess.run({"input": x})
        plan = sess.launch_plan()
        runs[fuse] = ({n: sess.get_output(n, "ANY") for n in
                       ["box_preds", "cls_logits"] + ["head%d.%s" % (i, k) for i in range(6) for k in ("loc", "conf")]},
                      plan, sess)
    labels = " ".join(l for l, _ in runs[True][1])
    assert "head0.loc#Conv#" in labels and "head0.conf#Conv#" not in labels   # absorbed by its sibling
    assert "head0.conf#Conv#" in " ".join(l for l, _ in runs[False][1])
    feats = ["block11.pw", "block13.pw", "extra1.conv", "extra2.conv", "extra3.conv", "extra4.conv"]
    sess = runs[True][2]
    for i, feat in enumerate(feats):
        xin = sess.get_output(feat, "NHWC")
        for kind in ("loc", "conf"):
            name = "head%d.%s" % (i, kind)
            w, b = info["weights"][name]
            ref = O.conv2d(xin, w, b, 1, 1)
            got = runs[True][0][name].reshape(ref.shape)
            assert_conv_close(got, ref, O.conv2d_abs(xin, w, b, 1, 1), FP32_RTOL, "fused " + name)
    for n in ("box_preds", "cls_logits"):
        a, b = runs[True][0][n], runs[False][0][n]
        assert np.abs(a - b).max() <= 2e-5 * np.abs(b).max(), n
    sess.compute(graph=True)
    np.testing.assert_array_equal(sess.get_output("cls_logits", "ANY"), runs[True][0]["cls_logits"])


def test_launch_plan_names_every_dispatch_and_times_it():
    """The launch plan of a pass: every call into the kernel library with its node label(s) and
    the device-stamped duration of each kernel it became.  Positive durations, one entry per
    node that launches something, and the same sequence on every pass."""
    g, _ = models.separable_block(2, size=19, cin=64, cout=128)
    x = rng(8100).uniform(0, 6, (2, 19, 19, 64)).astype(np.float32)
    sess = session.Session()
    sess.load_graph(g)
    sess.run({"input": x})
    want = sess.get_output("pw", "NHWC")
    plan = sess.launch_plan(durations=True)
    assert [l for l, _ in plan] == ["dw#Conv#", "pw#Conv#"]
    assert all(len(us) >= 1 and all(0.5 < u < 1000.0 for u in us) for _, us in plan)
    assert [l for l, k in sess.launch_plan()] == ["dw#Conv#", "pw#Conv#"]
    np.testing.assert_array_equal(sess.get_output("pw", "NHWC"), want)


def test_convolution_only_forces_out_what_it_conflicts_with():
    """Deferred convolutions never depend on each other, so one that needs a deferred result
    launches only the convolutions it conflicts with and joins the rest: a -> c with b
    independent of both goes out as [a], then [b + c] in one grid; a launch of any other kind
    (the pool) takes the whole queue.  Outputs equal the oracle's, eager and replayed."""
    r = rng(8200)
    gb = dlx.GraphBuilder()
    x = gb.add_input("input", [2, 16, 12, 12])
    ws = {}
    for name, cin, cout, k in (("a", 16, 32, 3), ("b", 16, 24, 1), ("c", 32, 16, 1)):
        ws[name] = (r.normal(0, 0.2, (cout, cin, k, k)).astype(np.float32),
                    r.normal(0, 0.1, cout).astype(np.float32))
    def conv(name, src, k, pad):
        w, b = ws[name]
        return gb.add_conv(name, src, gb.add_filter(name + ".w", w), gb.add_const(name + ".b", b),
                           kernel=k, pad=pad, activation_type="Relu")
    a = conv("a", x, 3, 1)
    b = conv("b", x, 1, 0)
    c = conv("c", a, 1, 0)
    gb.add_pool("pool", b, "MaxPool", 2, 2, 0)
    xin = r.uniform(-1, 1, (2, 12, 12, 16)).astype(np.float32)
    sess = session.Session()
    sess.load_graph(gb)
    sess.run({"input": xin})
    plan = [l for l, _ in sess.launch_plan()]
    assert plan == ["a#Conv#", "b#Conv#+c#Conv#", "pool#MaxPool#"], plan
    ra = O.conv2d(xin, *ws["a"], 1, 1, 1, 1, O.ACT_RELU)
    rb = O.conv2d(xin, *ws["b"], 1, 0, 1, 1, O.ACT_RELU)
    da = sess.get_output("a", "NHWC")
    assert_conv_close(da, ra, O.conv2d_abs(xin, *ws["a"], 1, 1), FP32_RTOL, "a")
    assert_conv_close(sess.get_output("b", "NHWC"), rb, O.conv2d_abs(xin, *ws["b"], 1, 0), FP32_RTOL, "b")
    assert_conv_close(sess.get_output("c", "NHWC"), O.conv2d(da, *ws["c"], 1, 0, 1, 1, O.ACT_RELU),
                      O.conv2d_abs(da, *ws["c"], 1, 0), FP32_RTOL, "c")
    np.testing.assert_array_equal(sess.get_output("pool", "NHWC"),
                                  O.pool2d(sess.get_output("b", "NHWC"), 2, 2, 0, O.POOL_MAX))
    eager = {n: sess.get_output(n, "NHWC") for n in ("a", "b", "c", "pool")}
    sess.compute(graph=True)
    sess.compute(graph=True)
    for n, v in eager.items():
        np.testing.assert_array_equal(sess.get_output(n, "NHWC"), v)


def test_sessions_take_their_streams_from_one_pool():
    """The first four sessions alive on the device get streams that were created together (so
    they sit on different hardware queues whatever streams the application creates in between);
    a closed session's stream goes to the next session; further sessions get streams of their
    own.  Outputs do not depend on which stream a session got."""
    import gc
    import torch
    gc.collect()   # sessions of earlier tests give their streams back
    g, info = models.mobilenet_v1_ssd(1, seed=5)
    x = rng(7).uniform(-1, 1, (1, 300, 300, 3)).astype(np.float32)
    made, other = [], []
    for _ in range(4):
        s = session.Session()
        s.load_graph(g)
        made.append(s)
        other.append(torch.cuda.Stream())   # an unrelated stream between two sessions
    streams = [int(s.stream or 0) for s in made]
    assert all(streams) and len(set(streams)) == 4
    fifth = session.Session()
    fifth.load_graph(g)
    assert int(fifth.stream) not in streams
    made[1].run({"input": x})
    ref = made[1].get_output("cls_logits", "ANY")
    made[1].close()
    again = session.Session()
    again.load_graph(g)
    assert int(again.stream) == streams[1]
    again.run({"input": x})
    np.testing.assert_array_equal(again.get_output("cls_logits", "ANY"), ref)
    fifth.run({"input": x})
    np.testing.assert_array_equal(fifth.get_output("cls_logits", "ANY"), ref)
