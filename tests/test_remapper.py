"""The BN / activation folding pass (ogle_amd/remapper.py, reference remapper.cc:36-176):
graph surgery on the CPU, and unfused vs folded graphs through the runtime on the GPU."""
import numpy as np
import pytest

import oracle as O
from ogle_amd import dlx, remapper
from util import rng


def bn_params(r, c):
    return (r.uniform(0.5, 1.5, c).astype(np.float32), r.normal(0, 0.1, c).astype(np.float32),
            r.normal(0, 0.1, c).astype(np.float32), r.uniform(0.5, 1.5, c).astype(np.float32))


def residual_graph(r, batch=2, size=12, c=16):
    """x -> conv3x3 -> BN -> Clip(0,6) -> conv3x3 (bias) -> BN -> Add(x) -> Relu -> conv1x1 -> BN"""
    gb = dlx.GraphBuilder()
    weights = {}
    x = gb.add_input("input", [batch, c, size, size])

    def conv_bn(name, src, k, pad, with_bias):
        w = r.normal(0, np.sqrt(2.0 / (k * k * c)), (c, c, k, k)).astype(np.float32)
        b = r.normal(0, 0.1, c).astype(np.float32) if with_bias else None
        wi = gb.add_filter(name + ".w", w)
        bi = gb.add_const(name + ".b", b) if with_bias else None
        ci = gb.add_conv(name, src, wi, bi, kernel=k, pad=pad)
        p = bn_params(r, c)
        ids = [gb.add_const("%s.bn.%s" % (name, t), v) for t, v in zip("gbmv", p)]
        weights[name] = (w, b, p)
        return gb.add_batchnorm(name + ".bn", ci, *ids, epsilon=1e-5)

    t = conv_bn("c1", x, 3, 1, False)
    t = gb.add_clip("c1.act", t, 0.0, 6.0)
    t = conv_bn("c2", t, 3, 1, True)
    t = gb.add_add("sum", t, x)
    t = gb.add_relu("sum.act", t)
    t = conv_bn("c3", t, 1, 0, True)
    gb.add_output_name("c3.bn")
    return gb, weights


def test_remap_structure_and_folded_values():
    r = rng(30000)
    gb, weights = residual_graph(r)
    before = dlx.decode_model(gb.serialize())
    out, n_bn, n_act = remapper.remap(gb.serialize())
    assert (n_bn, n_act) == (3, 1)
    after = dlx.decode_model(out)
    types = [n["type"] for n in after["graph"]["nodes"]]
    assert "BatchNormalization" not in types and "Clip" not in types
    assert types.count("Conv") == 3 and types.count("Add") == 1 and types.count("Relu") == 1
    by_name = {n["name"]: n for n in after["graph"]["nodes"]}
    # fused nodes carry the name and the output tensor of the pattern's last node
    assert by_name["c1.act"]["type"] == "Conv" and by_name["c2.bn"]["type"] == "Conv"
    # ... under the name that tensor had (tensors are renumbered in emission order)
    old = {n["name"]: n for n in before["graph"]["nodes"]}
    names_before, names_after = before["graph"]["tensor_names"], after["graph"]["tensor_names"]
    assert names_after[by_name["c1.act"]["output_index"][0]] == names_before[old["c1.act"]["output_index"][0]]
    assert [names_after[n["output_index"][0]] for n in after["graph"]["nodes"]] == names_after
    a1 = dlx.decode_conv2d_attr(by_name["c1.act"]["attr"][dlx.ATTR_CONV2D])
    assert (a1["activation_type"], a1["min"], a1["max"]) == ("Clip", 0.0, 6.0)
    assert dlx.decode_conv2d_attr(by_name["c2.bn"]["attr"][dlx.ATTR_CONV2D])["activation_type"] == ""
    # c1 had no bias: a Const was made, as its third input.  Its id follows every node of the
    # file, so Graph::ToGraphDef (graph.cc:12-54) writes all other constants first, then the made
    # bias, then the convolutions, which could not start before it; the folded BatchNormalization
    # parameters (no consumer left) are gone, and the tensor list is dense again
    assert len(by_name["c1.act"]["input_index"]) == 3 and "c1:2" in by_name
    order = [n["name"] for n in after["graph"]["nodes"]]
    assert order == ["input", "c1.w", "c2.w", "c2.b", "c3.w", "c3.b", "c1:2",
                     "c1.act", "c2.bn", "sum", "sum.act", "c3.bn"]
    assert len(names_after) == len(order)
    assert after["graph"]["output_names"] == ["c3.bn"] and after["graph"]["input_names"] == ["input"]
    # folded numbers are those of the reference's formula (the oracle restates it)
    for conv, fused in (("c1", "c1.act"), ("c2", "c2.bn"), ("c3", "c3.bn")):
        w, b, (g, bt, mu, var) = weights[conv]
        wf, bf = O.fold_bn(w, b, g, bt, mu, var, 1e-5)
        node = by_name[fused]
        tensors = {n["output_index"][0]: n for n in after["graph"]["nodes"] if n["type"] == "Const"}
        got_w = remapper._const_tensor(tensors[node["input_index"][1]])["float_data"].reshape(w.shape)
        got_b = remapper._const_tensor(tensors[node["input_index"][2]])["float_data"]
        np.testing.assert_allclose(got_w, wf, rtol=1e-6, atol=1e-7)
        np.testing.assert_allclose(got_b, bf, rtol=1e-6, atol=1e-7)


def test_remap_sorts_an_out_of_order_graph():
    """A file whose nodes are not in topological order (a consumer written before its producer):
    the graph constructor orders them (graph_constructor.cc:144-190, smallest file position
    among the ready nodes first), so the result is executable in file order and equals the
    result for the sorted file, node for node."""
    r = rng(30002)
    gb, _ = residual_graph(r)
    model = dlx.decode_model(gb.serialize())
    nodes = model["graph"]["nodes"]
    pos = {n["name"]: i for i, n in enumerate(nodes)}
    # move the first convolution behind its batchnorm and the Add in front of everything
    shuffled = list(nodes)
    shuffled.insert(0, shuffled.pop(pos["sum"]))
    c1 = next(i for i, n in enumerate(shuffled) if n["name"] == "c1")
    shuffled.insert(c1 + 6, shuffled.pop(c1))
    assert [n["name"] for n in shuffled] != [n["name"] for n in nodes]
    model["graph"]["nodes"] = shuffled
    out_shuffled, n_bn, n_act = remapper.remap(remapper.encode_model(model))
    out_sorted, _, _ = remapper.remap(gb.serialize())
    assert (n_bn, n_act) == (3, 1)
    a, b = dlx.decode_model(out_shuffled)["graph"], dlx.decode_model(out_sorted)["graph"]
    seen = set()
    for n in a["nodes"]:                       # every input is produced by an earlier node
        assert all(t in seen for t in n["input_index"]), n["name"]
        seen.update(n["output_index"])
    assert sorted(n["name"] for n in a["nodes"]) == sorted(n["name"] for n in b["nodes"])
    bn = {n["name"]: n for n in b["nodes"]}
    for n in a["nodes"]:
        assert n["type"] == bn[n["name"]]["type"] and n["attr"] == bn[n["name"]]["attr"]
        assert [a["tensor_names"][t] for t in n["input_index"]] == \
            [b["tensor_names"][t] for t in bn[n["name"]]["input_index"]]
    # a reference to a tensor nobody produces is fatal, as in the reference
    model["graph"]["nodes"] = [n for n in shuffled if n["name"] != "c2.w"]
    with pytest.raises(ValueError, match="Unknown input node 'c2.w'"):
        remapper.remap(remapper.encode_model(model))


def test_remap_leaves_shared_or_activated_patterns_alone():
    r = rng(30001)
    gb = dlx.GraphBuilder()
    x = gb.add_input("input", [1, 4, 6, 6])
    w = gb.add_filter("w", r.normal(0, 0.3, (4, 4, 3, 3)).astype(np.float32))
    c = gb.add_conv("conv", x, w, None, kernel=3, pad=1)
    ids = [gb.add_const("p" + t, v) for t, v in zip("gbmv", bn_params(r, 4))]
    bn = gb.add_batchnorm("bn", c, *ids)
    gb.add_add("sum", bn, c)            # the conv output has a second consumer
    out, n_bn, n_act = remapper.remap(gb.serialize())
    assert (n_bn, n_act) == (0, 0)
    assert [n["type"] for n in dlx.decode_model(out)["graph"]["nodes"]].count("BatchNormalization") == 1


@pytest.mark.gpu
def test_unfused_and_folded_graphs_on_the_device():
    from ogle_amd import session
    from util import FP32_RTOL, assert_conv_close
    r = rng(30002)
    batch, size, c = 2, 12, 16
    gb, weights = residual_graph(r, batch, size, c)
    x = r.uniform(-1, 1, (batch, size, size, c)).astype(np.float32)
    # oracle, op by op
    w1, b1, p1 = weights["c1"]
    w2, b2, p2 = weights["c2"]
    w3, b3, p3 = weights["c3"]
    t = O.clip(O.batchnorm(O.conv2d(x, w1, b1, 1, 1), *p1, 1e-5), 0.0, 6.0)
    t2 = O.batchnorm(O.conv2d(t, w2, b2, 1, 1), *p2, 1e-5)
    s = O.relu(O.add(t2, x))
    ref = O.batchnorm(O.conv2d(s, w3, b3, 1, 0), *p3, 1e-5)

    unfused = session.Session()
    unfused.load_graph(gb)
    unfused.run({"input": x})
    got_u = unfused.get_output("c3.bn", "NHWC")
    # every elementwise stage is exact given its input; check them on the device's own inputs
    d_c1 = unfused.get_output("c1", "NHWC")
    np.testing.assert_array_equal(unfused.get_output("c1.bn", "NHWC"), O.batchnorm(d_c1, *p1, 1e-5))
    np.testing.assert_array_equal(unfused.get_output("c1.act", "NHWC"),
                                  O.clip(unfused.get_output("c1.bn", "NHWC"), 0.0, 6.0))
    np.testing.assert_array_equal(unfused.get_output("sum", "NHWC"),
                                  O.add(unfused.get_output("c2.bn", "NHWC"), x))
    np.testing.assert_array_equal(unfused.get_output("sum.act", "NHWC"),
                                  O.relu(unfused.get_output("sum", "NHWC")))
    np.testing.assert_allclose(got_u, ref, rtol=2e-4, atol=2e-4)

    folded_bytes, n_bn, n_act = remapper.remap(gb.serialize())
    assert (n_bn, n_act) == (3, 1)
    folded = session.Session()
    folded.load_graph(folded_bytes)
    folded.run({"input": x})
    got_f = folded.get_output("c3.bn", "NHWC")
    np.testing.assert_allclose(got_f, got_u, rtol=2e-4, atol=2e-4)
    # the folded first stage against the oracle with the oracle's folded parameters
    wf, bf = O.fold_bn(w1, b1, *p1, 1e-5)
    ref1 = O.conv2d(x, wf, bf, 1, 1, 1, 1, O.ACT_CLIP, 0.0, 6.0)
    assert_conv_close(folded.get_output("c1.act", "NHWC"), ref1, O.conv2d_abs(x, wf, bf, 1, 1), FP32_RTOL, "c1")
    assert len(folded.issue_order()) == 5 and len(unfused.issue_order()) == 9


@pytest.mark.gpu
@pytest.mark.parametrize("batch", [1, 16])
def test_classifier_tail_on_the_device(batch):
    """GlobalAveragePool -> Flatten -> Gemm (Linear form), the end of a MobileNet classifier."""
    from ogle_amd import session
    r = rng(30003 + batch)
    c, classes = 1024, 1000
    x = r.uniform(0, 6, (batch, 7, 7, c)).astype(np.float32)
    w = r.normal(0, 0.03, (classes, c)).astype(np.float32)
    b = r.normal(0, 0.1, classes).astype(np.float32)
    gb = dlx.GraphBuilder()
    xi = gb.add_input("input", [batch, c, 7, 7])
    p = gb.add_pool("pool", xi, "GlobalAveragePool")
    f = gb.add_flatten("flat", p, 1)
    wi = gb.add_const("fc.w", w)
    bi = gb.add_const("fc.b", b)
    gb.add_gemm("logits", f, wi, bi, 1.0, 1.0, True)
    sess = session.Session()
    sess.load_graph(gb)
    sess.run({"input": x})
    pooled = O.pool2d(x, 7, 1, 0, O.POOL_GLOBAL_AVG)
    np.testing.assert_allclose(sess.get_output("pool", "NHWC"), pooled, rtol=1e-6, atol=1e-6)
    assert sess.tensor_shape("flat") == (batch, c)
    assert sess.tensor_device_ptr("flat") == sess.tensor_device_ptr("pool")
    dev_pooled = sess.get_output("flat", "ANY")
    ref = O.gemm(dev_pooled, w, b, 1.0, 1.0, True)
    scale = np.abs(dev_pooled).astype(np.float64) @ np.abs(w).astype(np.float64).T + np.abs(b)
    got = sess.get_output("logits", "ANY")
    assert got.shape == (batch, classes)
    assert np.all(np.abs(got - ref) <= 1e-4 * scale)
    # replayed as a graph: same numbers
    sess.compute(graph=True)
    np.testing.assert_array_equal(sess.get_output("logits", "ANY"), got)
