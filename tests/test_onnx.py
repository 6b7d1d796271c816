"""The ONNX front end (ogle_amd/onnx.py; reference converter/converter/onnx/onnx_converter.cc:19-196
and onnx/ops/*.cc): structure of the converted model on the CPU, and ONNX -> .dlx -> device
against the oracle on the GPU.  The ONNX bytes come from the protobuf runtime (onnx_schema.py),
not from the hand-written codec under test."""
import struct

import numpy as np
import pytest

import oracle as O
from ogle_amd import dlx, onnx
from onnx_schema import INT32, Writer
from test_remapper import bn_params
from util import rng

WRITERS = {"proto2": Writer(False), "proto3": Writer(True)}


def separable_block(w, r, batch=2, size=10, c=8, c_out=16, raw=False):
    """x -> depthwise 3x3 -> BN -> Clip(0,6) -> pointwise 1x1 (bias) -> BN -> Relu, the MobileNet
    block as torch.onnx exports it in training-free mode before constant folding."""
    wd = r.normal(0, 0.4, (c, 1, 3, 3)).astype(np.float32)
    wp = r.normal(0, 0.3, (c_out, c, 1, 1)).astype(np.float32)
    bp = r.normal(0, 0.1, c_out).astype(np.float32)
    p1, p2 = bn_params(r, c), bn_params(r, c_out)
    inits = [w.tensor("dw.w", wd, raw), w.tensor("pw.w", wp, raw), w.tensor("pw.b", bp, raw)]
    for tag, p in (("bn1", p1), ("bn2", p2)):
        inits += [w.tensor("%s.%s" % (tag, t), v, raw) for t, v in zip("gbmv", p)]
    nodes = [
        w.node("Conv", ["input", "dw.w"], ["dw"], kernel_shape=[3, 3], strides=[1, 1], pads=[1, 1, 1, 1],
               dilations=[1, 1], group=c),
        w.node("BatchNormalization", ["dw", "bn1.g", "bn1.b", "bn1.m", "bn1.v"], ["dw.bn"], epsilon=1e-5,
               momentum=0.9),
        w.node("Clip", ["dw.bn"], ["dw.act"], min=0.0, max=6.0),
        w.node("Conv", ["dw.act", "pw.w", "pw.b"], ["pw"], kernel_shape=[1, 1], strides=[1, 1],
               pads=[0, 0, 0, 0], dilations=[1, 1], group=1),
        w.node("BatchNormalization", ["pw", "bn2.g", "bn2.b", "bn2.m", "bn2.v"], ["pw.bn"], epsilon=1e-5,
               momentum=0.9),
        w.node("Relu", ["pw.bn"], ["out"]),
    ]
    blob = w.model(nodes, [w.value_info("input", [batch, c, size, size])],
                   [w.value_info("out", [batch, c_out, size, size])], inits)
    return blob, dict(wd=wd, wp=wp, bp=bp, p1=p1, p2=p2)


def residual_onnx(w, r, batch=2, size=12, c=16):
    """The residual graph of test_remapper.py, as ONNX:
    x -> conv3x3 -> BN -> Clip(0,6) -> conv3x3 (bias) -> BN -> Add(x) -> Relu -> conv1x1 (bias) -> BN"""
    weights, nodes, inits = {}, [], []

    def conv_bn(name, src, k, pad, with_bias):
        wt = r.normal(0, np.sqrt(2.0 / (k * k * c)), (c, c, k, k)).astype(np.float32)
        b = r.normal(0, 0.1, c).astype(np.float32) if with_bias else None
        p = bn_params(r, c)
        inits.append(w.tensor(name + ".w", wt))
        ins = [src, name + ".w"]
        if with_bias:
            inits.append(w.tensor(name + ".b", b))
            ins.append(name + ".b")
        nodes.append(w.node("Conv", ins, [name], kernel_shape=[k, k], strides=[1, 1], pads=[pad] * 4,
                            dilations=[1, 1], group=1))
        names = ["%s.bn.%s" % (name, t) for t in "gbmv"]
        inits.extend(w.tensor(n, v) for n, v in zip(names, p))
        nodes.append(w.node("BatchNormalization", [name] + names, [name + ".bn"], epsilon=1e-5))
        weights[name] = (wt, b, p)
        return name + ".bn"

    t = conv_bn("c1", "input", 3, 1, False)
    nodes.append(w.node("Clip", [t], ["c1.act"], min=0.0, max=6.0))
    t = conv_bn("c2", "c1.act", 3, 1, True)
    nodes.append(w.node("Add", [t, "input"], ["sum"]))
    nodes.append(w.node("Relu", ["sum"], ["sum.act"]))
    conv_bn("c3", "sum.act", 1, 0, True)
    blob = w.model(nodes, [w.value_info("input", [batch, c, size, size])],
                   [w.value_info("c3.bn", [batch, c, size, size])], inits)
    return blob, weights


def const_of(model, name):
    node = {n["name"]: n for n in model["graph"]["nodes"]}[name]
    assert node["type"] == "Const"
    value = [v for f, _, v in dlx._fields(node["attr"][dlx.ATTR_CONST]) if f == 1][0]
    return dlx.decode_tensor(value)


@pytest.mark.parametrize("syntax", ["proto2", "proto3"])
@pytest.mark.parametrize("raw", [False, True])
def test_separable_block_structure(syntax, raw):
    w = WRITERS[syntax]
    blob, p = separable_block(w, rng(31000), raw=raw)
    out = onnx.convert(blob)
    m = dlx.decode_model(out)
    assert (m["producer_name"], m["version"]) == ("ONNX", "0.1")
    g = m["graph"]
    assert g["input_names"] == ["input"] and g["output_names"] == ["out"]
    # Input first, then each node's new constants just in front of it, node named after its output
    assert [(n["name"], n["type"]) for n in g["nodes"]] == [
        ("input", "Input"), ("dw.w", "Const"), ("dw", "Conv"),
        ("bn1.g", "Const"), ("bn1.b", "Const"), ("bn1.m", "Const"), ("bn1.v", "Const"),
        ("dw.bn", "BatchNormalization"), ("dw.act", "Clip"),
        ("pw.w", "Const"), ("pw.b", "Const"), ("pw", "Conv"),
        ("bn2.g", "Const"), ("bn2.b", "Const"), ("bn2.m", "Const"), ("bn2.v", "Const"),
        ("pw.bn", "BatchNormalization"), ("out", "Relu")]
    # tensor indices follow first appearance, and a node's outputs are named by tensor_names
    assert g["tensor_names"] == [n["name"] for n in g["nodes"]]
    for i, n in enumerate(g["nodes"]):
        assert n["output_index"] == [i]
    by = {n["name"]: n for n in g["nodes"]}
    assert by["dw"]["input_index"] == [0, 1] and by["pw"]["input_index"] == [8, 9, 10]
    assert by["dw.bn"]["input_index"] == [2, 3, 4, 5, 6]
    assert dlx._ints(2, [v for f, _, v in dlx._fields(by["input"]["attr"][dlx.ATTR_INPUT]) if f == 3][0]) == \
        [2, 8, 10, 10]
    a = dlx.decode_conv2d_attr(by["dw"]["attr"][dlx.ATTR_CONV2D])
    assert (a["kernel_shape"], a["strides"], a["pads"], a["dilations"], a["group"]) == \
        ([3, 3], [1, 1], [1, 1, 1, 1], [1, 1], 8)
    assert a["activation_type"] == ""
    clip = dict((f, struct.unpack("<f", v)[0]) for f, _, v in dlx._fields(by["dw.act"]["attr"][dlx.ATTR_CLIP]))
    assert clip == {2: 6.0}                       # min 0.0 is the proto3 default: not written
    bn = dict((f, struct.unpack("<f", v)[0]) for f, _, v in dlx._fields(by["dw.bn"]["attr"][dlx.ATTR_BATCHNORM]))
    assert bn == {1: np.float32(0.9), 2: np.float32(1e-5)}
    assert dlx.ATTR_RELU in by["out"]["attr"] and by["out"]["attr"][dlx.ATTR_RELU] == b""
    # constants: values in file order (OIHW), tags per using op
    t = const_of(m, "dw.w")
    assert (t["data_format"], t["target_data_format"], t["dims"]) == (dlx.ANY, dlx.HWN4C4, [8, 1, 3, 3])
    np.testing.assert_array_equal(t["float_data"], p["wd"].reshape(-1))
    t = const_of(m, "pw.b")
    assert (t["data_format"], t["target_data_format"], t["dims"]) == (dlx.ANY, dlx.ANY4, [16])
    np.testing.assert_array_equal(t["float_data"], p["bp"])
    t = const_of(m, "bn2.v")
    assert (t["data_format"], t["target_data_format"]) == (dlx.ANY, dlx.ANY4)
    np.testing.assert_array_equal(t["float_data"], p["p2"][3])


def test_same_bytes_whatever_the_packing():
    a, _ = separable_block(WRITERS["proto2"], rng(31001))
    b, _ = separable_block(WRITERS["proto3"], rng(31001), raw=True)
    assert a != b and onnx.convert(a) == onnx.convert(b)


def test_convert_and_fold_gives_two_convolutions():
    blob, _ = separable_block(WRITERS["proto2"], rng(31002))
    out, n_bn, n_act = onnx.convert_and_fold(blob)
    assert (n_bn, n_act) == (2, 2)
    nodes = dlx.decode_model(out)["graph"]["nodes"]
    assert [n["type"] for n in nodes if n["type"] not in ("Const", "Input")] == ["Conv", "Conv"]
    acts = [dlx.decode_conv2d_attr(n["attr"][dlx.ATTR_CONV2D])["activation_type"] for n in nodes
            if n["type"] == "Conv"]
    assert acts == ["Clip", "Relu"]


def test_int64_constants_shared_initializers_and_optional_inputs():
    w = WRITERS["proto2"]
    shape = w.tensor("shape_value", np.array([2, -1], np.int64))
    nodes = [
        w.node("Constant", [], ["shape"], value=shape),
        w.node("Constant", [], ["shape_raw"], value=w.tensor("v", np.array([2, -1], np.int64), raw=True)),
        w.node("Reshape", ["x", "shape"], ["flat"]),
        w.node("Concat", ["flat", "extra"], ["cat"], axis=1),
        w.node("Concat", ["cat", "extra", ""], ["cat2"], axis=-1),
        w.node("Transpose", ["cat2"], ["t"], perm=[1, 0]),
    ]
    extra = w.tensor("extra", np.arange(6, dtype=np.float32).reshape(2, 3))
    unused = w.tensor("unused", np.zeros(3, np.float32))
    blob = w.model(nodes, [w.value_info("x", ["N", 3, 2, 2])], [w.value_info("t", [])], [extra, unused])
    m = dlx.decode_model(onnx.convert(blob))
    g = m["graph"]
    names = [n["name"] for n in g["nodes"]]
    assert names == ["x", "shape", "shape_raw", "flat", "extra", "cat", "cat2", "t"]     # unused: dropped
    by = {n["name"]: n for n in g["nodes"]}
    assert by["shape"]["type"] == "Constant"
    for name in ("shape", "shape_raw"):
        value = [v for f, _, v in dlx._fields(by[name]["attr"][dlx.ATTR_CONST]) if f == 1][0]
        t = dlx.decode_tensor(value)
        assert t["dims"] == [2] and list(t["float_data"]) == [2.0, -1.0]
        assert (t["data_format"], t["target_data_format"]) == (dlx.ANY, dlx.ANY4)
    # a symbolic dimension reads as 0
    assert dlx._ints(2, [v for f, _, v in dlx._fields(by["x"]["attr"][dlx.ATTR_INPUT]) if f == 3][0]) == \
        [0, 3, 2, 2]
    # the initializer is made a Const once, by its first user; the empty operand is skipped
    assert by["cat"]["input_index"] == [3, 4] and by["cat2"]["input_index"] == [5, 4]
    axis = [dlx._signed(v) for f, _, v in dlx._fields(by["cat2"]["attr"][dlx.ATTR_CONCAT]) if f == 1]
    assert axis == [-1]
    assert dlx._ints(2, [v for f, _, v in dlx._fields(by["t"]["attr"][dlx.ATTR_TRANSPOSE]) if f == 1][0]) == [1, 0]


def test_errors():
    w = WRITERS["proto2"]
    x = [w.value_info("x", [1, 4, 4, 4])]
    with pytest.raises(onnx.ConvertError, match="Cannot find Type: Softmax"):
        onnx.convert(w.model([w.node("Softmax", ["x"], ["y"])], x, []))
    # a Reshape whose shape is an initializer: the reference's converter refuses it
    with pytest.raises(onnx.ConvertError, match="reshape"):
        onnx.convert(w.model([w.node("Reshape", ["x", "s"], ["y"])], x, [],
                             [w.tensor("s", np.array([1, -1], np.int64))]))
    with pytest.raises(onnx.ConvertError, match="group and dilations"):
        onnx.convert(w.model([w.node("Conv", ["x", "f"], ["y"], kernel_shape=[1, 1])], x, [],
                             [w.tensor("f", np.zeros((4, 4, 1, 1), np.float32))]))
    with pytest.raises(onnx.ConvertError, match="4 dims"):
        onnx.convert(w.model([w.node("Conv", ["x", "f"], ["y"], dilations=[1, 1], group=1)], x, [],
                             [w.tensor("f", np.zeros((4, 4), np.float32))]))
    with pytest.raises(onnx.ConvertError, match="unsupported data type"):
        onnx.convert(w.model([w.node("Concat", ["x", "f"], ["y"], axis=1)], x, [],
                             [w.tensor("f", np.zeros(4), data_type=INT32)]))
    with pytest.raises(onnx.ConvertError, match="Cannot find the input tensor 'nowhere'"):
        onnx.convert(w.model([w.node("Relu", ["nowhere"], ["y"])], x, []))
    with pytest.raises(onnx.ConvertError, match="no graph"):
        onnx.convert(b"")


def test_initializer_with_a_zero_dimension_is_an_empty_tensor():
    """A tensor whose dims hold a zero has no data fields at all; it converts to an empty
    constant (MakeTensorFromProto copies `count` = 0 values) instead of being refused."""
    w = WRITERS["proto2"]
    x = [w.value_info("x", [1, 4, 4, 4])]
    model = onnx.convert(w.model([w.node("Concat", ["x", "e"], ["y"], axis=1)], x, [],
                                 [w.tensor("e", np.zeros((0, 4), np.float32))]))
    nodes = {n["name"]: n for n in dlx.decode_model(model)["graph"]["nodes"]}
    (field, _, payload), = list(dlx._fields(nodes["e"]["attr"][dlx.ATTR_CONST]))
    t = dlx.decode_tensor(payload)
    assert t["dims"] == [0, 4] and len(t["float_data"]) == 0


@pytest.mark.gpu
@pytest.mark.parametrize("fold", [False, True])
def test_separable_block_onnx_to_device(fold):
    from ogle_amd import session
    from util import FP32_RTOL, assert_conv_close
    r = rng(31010)
    batch, size, c, c_out = 2, 10, 8, 16
    blob, p = separable_block(WRITERS["proto2"], r, batch, size, c, c_out)
    x = r.uniform(-1, 1, (batch, size, size, c)).astype(np.float32)
    model = onnx.convert_and_fold(blob)[0] if fold else onnx.convert(blob)
    sess = session.Session()
    sess.load_graph(model)
    sess.run({"input": x})
    got = sess.get_output("out", "NHWC")
    if fold:
        wd, bd = O.fold_bn(p["wd"], None, *p["p1"], 1e-5)
        wp, bp = O.fold_bn(p["wp"], p["bp"], *p["p2"], 1e-5)
        mid_ref = O.conv2d(x, wd, bd, 1, 1, 1, c, O.ACT_CLIP, 0.0, 6.0)
        mid = sess.get_output("dw.act", "NHWC")
        assert_conv_close(mid, mid_ref, O.conv2d_abs(x, wd, bd, 1, 1, 1, c), FP32_RTOL, "onnx dw")
        ref = O.conv2d(mid, wp, bp, 1, 0, 1, 1, O.ACT_RELU)
        assert_conv_close(got, ref, O.conv2d_abs(mid, wp, bp, 1, 0), FP32_RTOL, "onnx pw")
        assert len(sess.issue_order()) == 2
    else:
        dw = sess.get_output("dw", "NHWC")
        assert_conv_close(dw, O.conv2d(x, p["wd"], None, 1, 1, 1, c), O.conv2d_abs(x, p["wd"], None, 1, 1, 1, c),
                          FP32_RTOL, "onnx dw unfused")
        act = O.clip(O.batchnorm(dw, *p["p1"], 1e-5), 0.0, 6.0)
        np.testing.assert_array_equal(sess.get_output("dw.act", "NHWC"), act)
        pw = sess.get_output("pw", "NHWC")
        assert_conv_close(pw, O.conv2d(act, p["wp"], p["bp"], 1, 0), O.conv2d_abs(act, p["wp"], p["bp"], 1, 0),
                          FP32_RTOL, "onnx pw unfused")
        np.testing.assert_array_equal(got, O.relu(O.batchnorm(pw, *p["p2"], 1e-5)))


@pytest.mark.gpu
def test_residual_graph_onnx_to_device():
    from ogle_amd import session
    from util import FP32_RTOL, assert_conv_close
    r = rng(31011)
    batch, size, c = 2, 12, 16
    blob, weights = residual_onnx(WRITERS["proto3"], r, batch, size, c)
    x = r.uniform(-1, 1, (batch, size, size, c)).astype(np.float32)
    w1, b1, p1 = weights["c1"]
    w2, b2, p2 = weights["c2"]
    w3, b3, p3 = weights["c3"]
    t = O.clip(O.batchnorm(O.conv2d(x, w1, b1, 1, 1), *p1, 1e-5), 0.0, 6.0)
    t2 = O.batchnorm(O.conv2d(t, w2, b2, 1, 1), *p2, 1e-5)
    s = O.relu(O.add(t2, x))
    ref = O.batchnorm(O.conv2d(s, w3, b3, 1, 0), *p3, 1e-5)

    unfused = session.Session()
    unfused.load_graph(onnx.convert(blob))
    unfused.run({"input": x})
    got_u = unfused.get_output("c3.bn", "NHWC")
    np.testing.assert_allclose(got_u, ref, rtol=2e-4, atol=2e-4)
    assert len(unfused.issue_order()) == 9

    folded_bytes, n_bn, n_act = onnx.convert_and_fold(blob)
    assert (n_bn, n_act) == (3, 1)
    folded = session.Session()
    folded.load_graph(folded_bytes)
    folded.run({"input": x})
    np.testing.assert_allclose(folded.get_output("c3.bn", "NHWC"), got_u, rtol=2e-4, atol=2e-4)
    wf, bf = O.fold_bn(w1, b1, *p1, 1e-5)
    ref1 = O.conv2d(x, wf, bf, 1, 1, 1, 1, O.ACT_CLIP, 0.0, 6.0)
    assert_conv_close(folded.get_output("c1.act", "NHWC"), ref1, O.conv2d_abs(x, wf, bf, 1, 1), FP32_RTOL,
                      "onnx c1")
    assert len(folded.issue_order()) == 5


@pytest.mark.gpu
def test_classifier_tail_onnx_to_device():
    """GlobalAveragePool -> Flatten -> Gemm (transB = 1, the Linear form) from ONNX: the converters
    of the ops that close a MobileNet classifier, end to end."""
    from ogle_amd import session
    w = WRITERS["proto2"]
    r = rng(31020)
    batch, c, classes = 3, 256, 40
    wt = r.normal(0, 0.05, (classes, c)).astype(np.float32)
    b = r.normal(0, 0.1, classes).astype(np.float32)
    nodes = [w.node("GlobalAveragePool", ["input"], ["pool"]),
             w.node("Flatten", ["pool"], ["flat"], axis=1),
             w.node("Gemm", ["flat", "fc.w", "fc.b"], ["logits"], alpha=1.0, beta=1.0, transB=1)]
    blob = w.model(nodes, [w.value_info("input", [batch, c, 7, 7])], [w.value_info("logits", [batch, classes])],
                   [w.tensor("fc.w", wt), w.tensor("fc.b", b, raw=True)])
    model = onnx.convert(blob)
    by = {n["name"]: n for n in dlx.decode_model(model)["graph"]["nodes"]}
    assert [by[n]["type"] for n in ("pool", "flat", "fc.w", "fc.b", "logits")] == \
        ["GlobalAveragePool", "Flatten", "Const", "Const", "Gemm"]
    gemm = dict((f, v) for f, _, v in dlx._fields(by["logits"]["attr"][dlx.ATTR_GEMM]))
    assert struct.unpack("<f", gemm[1])[0] == 1.0 and struct.unpack("<f", gemm[2])[0] == 1.0 and gemm[3] == 1
    x = r.uniform(0, 6, (batch, 7, 7, c)).astype(np.float32)
    sess = session.Session()
    sess.load_graph(model)
    sess.run({"input": x})
    pooled = sess.get_output("flat", "ANY")
    np.testing.assert_allclose(pooled, O.pool2d(x, 7, 1, 0, O.POOL_GLOBAL_AVG).reshape(batch, c), rtol=1e-6, atol=1e-6)
    ref = O.gemm(pooled, wt, b, 1.0, 1.0, True)
    scale = np.abs(pooled).astype(np.float64) @ np.abs(wt).astype(np.float64).T + np.abs(b)
    got = sess.get_output("logits", "ANY")
    assert got.shape == (batch, classes)
    assert np.all(np.abs(got - ref) <= 1e-5 * scale)


def ssd_onnx(w, info, batch, image=300):
    """MobileNet-v1-SSD as an exporter writes it before constant folding: every backbone and
    extra layer Conv -> BatchNormalization -> Clip(0, 6), every head Conv -> Transpose(0,2,3,1)
    -> Reshape (shape from a Constant node) and the two Concat nodes over axis 1, with the
    weights of models.mobilenet_v1_ssd(with_weights=True) before their folding."""
    nodes, inits = [], []
    taps = {"block11.pw": 0, "block13.pw": 1, "extra1.conv": 2, "extra2.conv": 3, "extra3.conv": 4,
            "extra4.conv": 5}
    maps, cur = {}, "input"
    locs, confs = [], []
    for l in info["layers"]:
        name, un = l["name"], info["unfolded"][l["name"]]
        head = name.startswith("head")
        src = maps[int(name[4:name.index(".")])] if head else cur
        inits.append(w.tensor(name + ".w", un[0], raw=True))
        nodes.append(w.node("Conv", [src, name + ".w"], [name if head else name + ".conv"],
                            kernel_shape=[l["k"]] * 2, strides=[l["stride"]] * 2, pads=[l["pad"]] * 4,
                            dilations=[1, 1], group=l["group"]))
        if head:
            last = 4 if name.endswith(".loc") else info["num_classes"]
            nodes.append(w.node("Transpose", [name], [name + ".permute"], perm=[0, 2, 3, 1]))
            nodes.append(w.node("Constant", [], [name + ".shape"],
                                value=w.tensor("", np.array([batch, -1, last], np.int64))))
            nodes.append(w.node("Reshape", [name + ".permute", name + ".shape"], [name + ".view"]))
            (locs if last == 4 else confs).append(name + ".view")
            continue
        inits += [w.tensor("%s.%s" % (name, t), v) for t, v in zip("gbmv", un[1:])]
        nodes.append(w.node("BatchNormalization", [name + ".conv"] + ["%s.%s" % (name, t) for t in "gbmv"],
                            [name + ".bn"], epsilon=1e-5, momentum=0.9))
        nodes.append(w.node("Clip", [name + ".bn"], [name], min=0.0, max=6.0))
        cur = name
        if name in taps:
            maps[taps[name]] = name
    nodes.append(w.node("Concat", locs, ["box_preds"], axis=1))
    nodes.append(w.node("Concat", confs, ["cls_logits"], axis=1))
    nodes.append(w.node("Constant", [], ["anchors"], value=w.tensor("", info["anchors"], raw=True)))
    outs = [w.value_info("cls_logits", [batch, info["priors"], info["num_classes"]]),
            w.value_info("box_preds", [batch, info["priors"], 4]),
            w.value_info("anchors", [info["priors"], 4])]
    return w.model(nodes, [w.value_info("input", [batch, 3, image, image])], outs, inits)


def test_whole_detector_converts_and_folds():
    """47 convolutions, 35 of them with BatchNormalization and Clip behind them: after conversion
    and the remapper, what is left is the graph models.mobilenet_v1_ssd builds directly, with the
    same folded weights."""
    from ogle_amd import models
    g, info = models.mobilenet_v1_ssd(1, with_weights=True)
    blob = ssd_onnx(WRITERS["proto3"], info, 1)
    plain = dlx.decode_model(onnx.convert(blob))["graph"]["nodes"]
    kinds = [n["type"] for n in plain]
    assert kinds.count("Conv") == 47 and kinds.count("BatchNormalization") == 35 and kinds.count("Clip") == 35
    folded, n_bn, n_act = onnx.convert_and_fold(blob)
    assert (n_bn, n_act) == (35, 35)
    model = dlx.decode_model(folded)
    nodes, names = model["graph"]["nodes"], model["graph"]["tensor_names"]
    kinds = [n["type"] for n in nodes]
    assert kinds.count("Conv") == 47 and "BatchNormalization" not in kinds and "Clip" not in kinds
    assert kinds.count("Concat") == 2 and kinds.count("Reshape") == 12 and kinds.count("Transpose") == 12
    direct = {n["name"]: n for n in dlx.decode_model(g.serialize())["graph"]["nodes"]}
    by = {n["name"]: n for n in nodes}
    for name in ("conv0", "block7.dw", "block13.pw", "extra2.conv"):
        conv = by[name]
        wf, bf = info["weights"][name]
        got_w = const_of(model, names[conv["input_index"][1]])
        got_b = const_of(model, names[conv["input_index"][2]])
        assert got_w["dims"] == list(wf.shape)
        np.testing.assert_allclose(got_w["float_data"].reshape(wf.shape), wf, rtol=2e-6, atol=1e-7)
        np.testing.assert_allclose(got_b["float_data"], bf, rtol=2e-6, atol=1e-7)
        assert dlx.decode_conv2d_attr(conv["attr"][dlx.ATTR_CONV2D]) == \
            dlx.decode_conv2d_attr(direct[name]["attr"][dlx.ATTR_CONV2D])


@pytest.mark.gpu
def test_whole_detector_onnx_to_device():
    """The detector's ONNX form, converted and folded, gives the outputs of the directly built
    graph on the device (both run the same kernels; the folded weights may differ in the last
    bit, so outputs agree to a small multiple of the fp32 unit against their scale)."""
    from ogle_amd import models, session
    batch = 2
    g, info = models.mobilenet_v1_ssd(batch, with_weights=True)
    folded = onnx.convert_and_fold(ssd_onnx(WRITERS["proto2"], info, batch))[0]
    x = rng(31030).uniform(-1, 1, (batch, 300, 300, 3)).astype(np.float32)
    outs = {}
    for tag, blob in (("direct", g.serialize()), ("onnx", folded)):
        sess = session.Session()
        sess.load_graph(blob)
        sess.run({"input": x})
        outs[tag] = {n: sess.get_output(n, "ANY") for n in ("cls_logits", "box_preds", "anchors")}
    np.testing.assert_array_equal(outs["onnx"]["anchors"], outs["direct"]["anchors"])
    for name in ("cls_logits", "box_preds"):
        a, b = outs["onnx"][name], outs["direct"][name]
        assert a.shape == b.shape
        assert np.abs(a - b).max() <= 1e-4 * np.abs(b).max(), name
