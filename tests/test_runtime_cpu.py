"""CPU-only checks of the graph runtime: the .dlx codec against google.protobuf, the C ABI's
exported symbols, and the fatal conditions the reference aborts on, which surface as errors
(fbo_session.cc:66-67 missing model, :113-115 unknown op; conv2d.cc:71-86 attribute rules).
No device work is done."""
import os
import re

import numpy as np
import pytest

from ogle_amd import dlx, models, session

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _pb_classes():
    """The dlxnet schema (ogl_runtime/opengl/core/dlxnet.proto) rebuilt as a descriptor for the
    protobuf runtime: an independent implementation of the wire format."""
    from google.protobuf import descriptor_pb2, descriptor_pool, message_factory
    F = descriptor_pb2.FieldDescriptorProto
    fd = descriptor_pb2.FileDescriptorProto(name="dlxnet_test.proto", package="dlxt", syntax="proto3")

    def msg(name, fields):
        m = fd.message_type.add(name=name)
        for fname, num, typ, label, tname in fields:
            f = m.field.add(name=fname, number=num, type=typ, label=label)
            if tname:
                f.type_name = ".dlxt." + tname
        return m

    OPT, REP = F.LABEL_OPTIONAL, F.LABEL_REPEATED
    msg("TensorProto", [("data_format", 1, F.TYPE_INT32, OPT, None), ("data_type", 2, F.TYPE_INT32, OPT, None),
                        ("dims", 3, F.TYPE_INT32, REP, None), ("float_data", 4, F.TYPE_FLOAT, REP, None),
                        ("target_data_format", 8, F.TYPE_INT32, OPT, None)])
    msg("Conv2dAttribute", [("kernel_shape", 1, F.TYPE_INT64, REP, None), ("strides", 2, F.TYPE_INT64, REP, None),
                            ("pads", 3, F.TYPE_INT64, REP, None), ("dilations", 4, F.TYPE_INT64, REP, None),
                            ("group", 5, F.TYPE_INT64, OPT, None), ("activation_type", 6, F.TYPE_STRING, OPT, None),
                            ("min", 7, F.TYPE_FLOAT, OPT, None), ("max", 8, F.TYPE_FLOAT, OPT, None)])
    msg("ConstAttribute", [("value", 1, F.TYPE_MESSAGE, OPT, "TensorProto")])
    msg("MaxPoolAttribute", [("kernel_shape", 1, F.TYPE_INT64, REP, None), ("strides", 2, F.TYPE_INT64, REP, None),
                             ("pads", 3, F.TYPE_INT64, REP, None)])
    msg("InputAttribute", [("dims", 3, F.TYPE_INT32, REP, None)])
    msg("TransposeAttribute", [("perm", 1, F.TYPE_INT32, REP, None)])
    msg("ConcatAttribute", [("axis", 1, F.TYPE_INT32, OPT, None)])
    msg("ReshapeAttribute", [("axis", 1, F.TYPE_INT32, OPT, None)])
    msg("Attribute", [("conv2d_attr", 1, F.TYPE_MESSAGE, OPT, "Conv2dAttribute"),
                      ("const_attr", 2, F.TYPE_MESSAGE, OPT, "ConstAttribute"),
                      ("maxpool_attr", 5, F.TYPE_MESSAGE, OPT, "MaxPoolAttribute"),
                      ("input_attr", 10, F.TYPE_MESSAGE, OPT, "InputAttribute"),
                      ("transpose_attr", 12, F.TYPE_MESSAGE, OPT, "TransposeAttribute"),
                      ("concat_attr", 16, F.TYPE_MESSAGE, OPT, "ConcatAttribute"),
                      ("reshape_attr", 17, F.TYPE_MESSAGE, OPT, "ReshapeAttribute")])
    msg("NodeProto", [("input_index", 1, F.TYPE_INT64, REP, None), ("output_index", 2, F.TYPE_INT64, REP, None),
                      ("attr", 3, F.TYPE_MESSAGE, OPT, "Attribute"), ("doc_string", 4, F.TYPE_STRING, OPT, None),
                      ("name", 5, F.TYPE_STRING, OPT, None), ("type", 6, F.TYPE_STRING, OPT, None)])
    msg("GraphProto", [("node", 1, F.TYPE_MESSAGE, REP, "NodeProto"), ("name", 2, F.TYPE_STRING, OPT, None),
                       ("tensor_names", 3, F.TYPE_STRING, REP, None), ("output_names", 4, F.TYPE_STRING, REP, None),
                       ("input_names", 5, F.TYPE_STRING, REP, None)])
    msg("ModelProto", [("graph", 1, F.TYPE_MESSAGE, OPT, "GraphProto"), ("version", 2, F.TYPE_STRING, OPT, None),
                       ("producer_name", 3, F.TYPE_STRING, OPT, None), ("doc_string", 4, F.TYPE_STRING, OPT, None)])
    pool = descriptor_pool.DescriptorPool()
    pool.Add(fd)
    return message_factory.GetMessageClass(pool.FindMessageTypeByName("dlxt.ModelProto"))


def _small_graph():
    r = np.random.Generator(np.random.PCG64(5))
    g = dlx.GraphBuilder()
    x = g.add_input("input", [1, 3, 8, 8])
    w = g.add_filter("w", r.normal(0, 1, (4, 3, 3, 3)).astype(np.float32))
    b = g.add_const("b", r.normal(0, 1, 4).astype(np.float32))
    y = g.add_conv("conv", x, w, b, 3, 2, 1, 1, 1, "Clip", 0.0, 6.0)
    p = g.add_pool("pool", y, "MaxPool", 2, 2, 0)
    t = g.add_transpose("perm", p, [0, 2, 3, 1])
    s = g.add_const("shape", np.array([1, -1, 4], np.float32))
    v = g.add_reshape("view", t, s)
    g.add_concat("cat", [v, v], -1)
    g.add_output_name("cat")
    return g


def _check_against_protobuf(raw):
    Model = _pb_classes()
    m = Model()
    m.ParseFromString(raw)
    assert m.producer_name == "ONNX"
    nodes = {n.name: n for n in m.graph.node}
    assert list(m.graph.tensor_names) == ["input", "w", "b", "conv", "pool", "perm", "shape", "view", "cat"]
    assert list(m.graph.input_names) == ["input"] and list(m.graph.output_names) == ["cat"]
    c = nodes["conv"]
    assert c.type == "Conv" and list(c.input_index) == [0, 1, 2] and list(c.output_index) == [3]
    a = c.attr.conv2d_attr
    assert list(a.kernel_shape) == [3, 3] and list(a.strides) == [2, 2] and list(a.pads) == [1] * 4
    assert a.group == 1 and a.activation_type == "Clip" and a.min == 0.0 and a.max == 6.0
    wv = nodes["w"].attr.const_attr.value
    assert list(wv.dims) == [4, 3, 3, 3] and wv.data_format == dlx.ANY and wv.target_data_format == dlx.HWN4C4
    assert len(wv.float_data) == 108
    assert list(nodes["perm"].attr.transpose_attr.perm) == [0, 2, 3, 1]
    assert nodes["cat"].attr.concat_attr.axis == -1
    assert list(nodes["shape"].attr.const_attr.value.float_data) == [1.0, -1.0, 4.0]
    assert list(nodes["input"].attr.input_attr.dims) == [1, 3, 8, 8]
    assert list(nodes["pool"].attr.maxpool_attr.kernel_shape) == [2, 2]
    return m


def test_python_writer_matches_protobuf_runtime():
    raw = _small_graph().serialize()
    m = _check_against_protobuf(raw)
    # and protobuf's own serialization is read back identically by the python decoder
    d = dlx.decode_model(m.SerializeToString())
    assert [n["name"] for n in d["graph"]["nodes"]] == [n.name for n in m.graph.node]
    attr = dlx.decode_conv2d_attr(d["graph"]["nodes"][3]["attr"][dlx.ATTR_CONV2D])
    assert attr["strides"] == [2, 2] and attr["activation_type"] == "Clip" and attr["max"] == 6.0


def test_cpp_codec_round_trip_matches_protobuf_runtime():
    raw = _small_graph().serialize()
    again = session.reserialize(raw)
    _check_against_protobuf(again)           # C++ parse + serialize keeps every field
    const_attr = dlx.decode_model(again)["graph"]["nodes"][1]["attr"][dlx.ATTR_CONST]
    (field, _, payload), = list(dlx._fields(const_attr))
    assert field == 1
    w0 = dlx.decode_tensor(payload)
    text = session.model_debug_string(raw)
    assert 'type: Conv' in text and 'activation_type: Clip' in text and 'producer_name: ONNX' in text
    assert w0["dims"] == [4, 3, 3, 3]
    # unpacked repeated scalars (what a proto2-style writer emits) parse too
    Model = _pb_classes()
    m = Model()
    m.ParseFromString(raw)
    assert session.reserialize(m.SerializeToString()) == again


def test_runtime_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "ogle_runtime.h")).read()
    declared = set(re.findall(r"\b(ogle_rt_[a-z0-9_]+)\s*\(", header))
    assert declared == set(session.SYMBOLS)
    lib = session.lib()
    for name in declared:
        assert getattr(lib, name) is not None


def test_host_elements_and_input_size_check():
    """Sizes of the host layouts (tensor_format.cc:251-343) and the check Session.run makes with
    them: a dense array handed over under a padded tag would be read past its end."""
    assert session.host_elements((2, 5, 7, 3), "NHWC") == 210
    assert session.host_elements((2, 5, 7, 3), "NCHW") == 210
    assert session.host_elements((2, 5, 7, 3), "NHWC4") == 2 * 5 * 7 * 4
    assert session.host_elements((2, 5, 7, 8), "NHWC4") == 2 * 5 * 7 * 8
    assert session.host_elements((6, 1917, 21), "ANY4") == 6 * 1917 * 24
    assert session.host_elements((5,), "ANY4") == 8
    assert session.host_elements((5,), "ANY") == 5
    # OIHW (13, 6, 3, 3): 9 * ceil(13/4) rows of 4 * ceil(6/4) texels of 4 lanes
    assert session.host_elements((13, 6, 3, 3), "HWN4C4") == 9 * 4 * 8 * 4
    with pytest.raises(RuntimeError, match="unsupported dformat"):
        session.host_elements((1, 2), "NC4HW4")
    with pytest.raises(RuntimeError, match="rank-4"):
        session.host_elements((3, 3), "NHWC4")
    s = session.Session()
    s.load_graph(_small_graph())
    x = np.zeros((1, 8, 8, 3), np.float32)
    with pytest.raises(ValueError, match=r"layout NHWC4 .* takes 256 floats, the array holds 192"):
        s.run({"input": x}, dformats={"input": "NHWC4"})
    with pytest.raises(ValueError, match="takes 192 floats, the array holds 256"):
        s.run({"input": np.zeros((1, 8, 8, 4), np.float32)}, shapes={"input": (1, 8, 8, 3)})


def test_registered_op_types():
    names = session.registered_kernels()
    for op in ["Conv", "MaxPool", "AveragePool", "GlobalAveragePool", "Concat", "Decoder", "Const",
               "Constant", "Transpose", "Reshape", "Shape", "Gather", "Unsqueeze", "Add", "Relu", "Clip",
               "BatchNormalization", "Gemm", "Flatten"]:
        assert op in names


def test_load_errors_surface_instead_of_aborting(tmp_path):
    s = session.Session()
    with pytest.raises(RuntimeError, match="cannot open file"):
        s.load_graph(str(tmp_path / "missing.dlx"))
    with pytest.raises(RuntimeError, match="not a .dlx model"):
        s.load_graph(b"\x0a\x05hello")
    g = dlx.GraphBuilder()
    g.add_node("x", "Bogus", [])
    with pytest.raises(RuntimeError, match="unsupported kernel name Bogus"):
        s.load_graph(g)
    # a valid graph loads from bytes and from a file, and creates one kernel per non-Input node
    g = _small_graph()
    s.load_graph(g)
    assert s.num_kernels == len(g.nodes) - 1
    path = tmp_path / "m.dlx"
    g.save(str(path))
    s.load_graph(str(path))
    assert s.num_kernels == len(g.nodes) - 1
    with pytest.raises(RuntimeError, match="tensor_name: nope Cannot Find"):
        s.run({"nope": np.zeros((1, 8, 8, 3), np.float32)})


@pytest.mark.parametrize("bad", ["pads", "strides", "kernel"])
def test_conv_attribute_rules(bad):
    """conv2d.cc:71-86: four equal pads, two equal strides, a square kernel."""
    attr = dict(kernel=[3, 3], strides=[1, 1], pads=[1, 1, 1, 1])
    if bad == "pads":
        attr["pads"] = [1, 1, 0, 1]
    elif bad == "strides":
        attr["strides"] = [1, 2]
    else:
        attr["kernel"] = [3, 1]
    payload = (dlx._packed_ints(1, attr["kernel"]) + dlx._packed_ints(2, attr["strides"]) +
               dlx._packed_ints(3, attr["pads"]))
    g = dlx.GraphBuilder()
    x = g.add_input("input", [1, 3, 8, 8])
    w = g.add_filter("w", np.zeros((4, 3, 3, 3), np.float32))
    g.add_node("conv", "Conv", [x, w], dlx.ATTR_CONV2D, payload)
    s = session.Session()
    with pytest.raises(RuntimeError, match="Check failed"):
        s.load_graph(g)


def test_mobilenet_ssd_graph_shape_and_flops():
    g, info = models.mobilenet_v1_ssd(1)
    assert info["priors"] == 1917
    convs = [l for l in info["layers"]]
    assert len(convs) == 1 + 26 + 8 + 12
    # BASELINE: 2,803,531,136 FLOPs per image
    assert sum(l["flops_per_image"] for l in convs) == 2803531136
    s = session.Session()
    s.load_graph(g)
    assert s.num_kernels == len(g.nodes) - 1


def test_fold_batchnorm_is_the_bn_of_the_conv():
    r = np.random.Generator(np.random.PCG64(9))
    o, c = 6, 5
    w = r.normal(0, 1, (o, c, 3, 3)).astype(np.float32)
    gamma, beta = r.uniform(.5, 1.5, o).astype(np.float32), r.normal(0, .1, o).astype(np.float32)
    mean, var = r.normal(0, .1, o).astype(np.float32), r.uniform(.5, 1.5, o).astype(np.float32)
    wf, bf = models.fold_batchnorm(w, None, gamma, beta, mean, var)
    import oracle as O
    wo, bo = O.fold_bn(w, None, gamma, beta, mean, var, 1e-5)
    np.testing.assert_allclose(wf, wo, rtol=2e-7, atol=0)
    np.testing.assert_allclose(bf, bo, rtol=0, atol=1e-7)


# ---- dependency rule of the deferred-convolution queue (no device) --------------------

def _fake_conv(inp, out, n=1, h=4, w=4, c=8, o=16, k=1, ws=0, ws_bytes=0, filt=0x10000, bias=0x20000):
    from ogle_amd import hip as H
    a = H.conv_args(inp, filt, bias, out, n, h, w, c, o, k)
    a.workspace_dev, a.workspace_bytes = (ws or None), ws_bytes
    return a


def test_hazard_rule_is_interval_overlap():
    """Two deferred convolutions write slices at non-zero offsets inside one larger buffer
    (what placing concat inputs in the concat output produces).  Readers and writers are
    given as byte ranges; the rule must see every overlap, wherever the range starts."""
    big = 0x1000000                      # the enclosing buffer (a concat output), 4 KiB
    out_bytes = 4 * 4 * 16 * 4           # 1 KiB per convolution output
    pend = [_fake_conv(0x5000000, big + 1024), _fake_conv(0x6000000, big + 2048, ws=0x7000000, ws_bytes=512)]
    C = session.hazard_conflicts
    # a reader of the whole enclosing buffer starts BEFORE both pending outputs
    assert C(pend, [(big, 4096)], [])
    # a reader that straddles the start of a pending output
    assert C(pend, [(big + 512, 600)], [])
    # the in-place concat slice itself, and a range that ends exactly where an output begins
    assert C(pend, [(big + 2048, out_bytes)], [])
    assert not C(pend, [(big, 1024)], [])
    assert not C(pend, [(big + 3072, 1024)], [])
    # reading what a pending convolution only reads is no hazard; writing it is
    assert not C(pend, [(0x5000000, 512)], [])
    assert C(pend, [], [(0x5000000 + 500, 8)])
    assert C(pend, [], [(0x10000 + 4, 4)])          # inside a pending filter
    assert C(pend, [], [(0x20000, 4)])              # a pending bias
    # workspace of a pending convolution: reads and writes both conflict
    assert C(pend, [(0x7000000 + 100, 4)], [])
    assert C(pend, [], [(0x7000000 + 511, 1)])
    assert not C(pend, [], [(0x7000000 + 512, 64)])
    # write-after-write into the enclosing buffer
    assert C(pend, [], [(big, 4096)])
    # empty ranges and null pointers never conflict; nothing pending never conflicts
    assert not C(pend, [(big + 1024, 0), (0, 100)], [(0, 8)])
    assert not C([], [(big, 4096)], [(big, 4096)])


def test_hazard_rule_with_images_written_apart():
    """Convolutions that write their images into interleaved places of one tensor (heads
    produced inside a concat's output at batch > 1): image b of head i lies at base + b * stride
    + offset_i.  Heads whose places differ do not conflict although their hulls overlap; a
    reader of the enclosing tensor, of one image's slice, or a head on the same place does."""
    base, n = 0x1000000, 4
    img = 4 * 4 * 16 * 4                 # one image of a 4x4x16 head, 1 KiB
    stride = 3 * img + 256               # three heads and a gap per output slice

    def head(slot, inp=0x5000000, **kw):
        a = _fake_conv(inp, base + slot * img, n=n, **kw)
        a.out_image_stride = stride // 4
        return a
    C, CC = session.hazard_conflicts, session.conv_hazard_conflicts
    pend = [head(0), head(1)]
    assert not CC(pend, head(2))                          # its own place in every slice
    assert CC(pend, head(1))                              # the same place: write after write
    half = head(0)
    half.output_dev = base + img // 2                     # straddles heads 0 and 1
    assert CC(pend, half)
    later = head(0)
    later.output_dev = base + n * stride                  # the next tensor: past the last image
    assert not CC(pend, later)
    assert CC(pend, head(2, inp=base + stride))           # reads what head 0 writes (image 1)
    gap = head(2)
    gap.input_dev = base + 3 * img                        # an input that fits in the 256-byte gap
    gap.in_h, gap.in_w, gap.in_c, gap.n = 1, 1, 8, 1
    assert not CC(pend, gap)
    dense = _fake_conv(0x5000000, base, n=n)              # dense writer over the same hull
    assert CC(pend, dense)
    # plain ranges against the strided writes
    assert C(pend, [(base, n * stride)], [])              # the enclosing tensor (a detector read)
    assert C(pend, [(base + 2 * stride + img, 4)], [])    # image 2 of head 1
    assert not C(pend, [(base + 2 * img, img + 256)], []) # head 2's place and the gap in slice 0
    assert not C(pend, [], [(base + stride + 2 * img, img)])
    assert C(pend, [], [(base + 3 * stride + img - 4, 8)])
    # one image: the stride means nothing
    one = _fake_conv(0x5000000, base, n=1)
    one.out_image_stride = stride // 4
    assert C([one], [(base + img - 4, 4)], []) and not C([one], [(base + img, 4)], [])


def test_reloading_a_graph_resets_the_session():
    """LoadGraph on a session that already holds a graph starts from scratch: kernel count
    follows the new graph and no recorded pass survives (checked on the device as well)."""
    g1, _ = models.separable_block(1, size=8, cin=8, cout=16)
    sess = session.Session()
    sess.load_graph(g1)
    n1 = sess.num_kernels
    gb = dlx.GraphBuilder()
    x = gb.add_input("input", [1, 4, 6, 6])
    gb.add_pool("output", x, "MaxPool", 2, 2, 0)
    sess.load_graph(gb)
    assert sess.num_kernels == 1 and n1 > 1
    assert not sess.graph_captured(0) and not sess.graph_captured(1)
    assert sess.issue_order() == []
    sess.load_graph(g1)
    assert sess.num_kernels == n1
