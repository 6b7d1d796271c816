"""ONNX -> .dlx: the front end of the reference's converter.

Restates converter/converter/onnx/onnx_converter.cc:19-196 (graph walk), onnx/onnx_utils.cc:
50-108 (MakeTensorFromProto) and the op converters of converter/converter/onnx/ops/*.cc on the
serialized protobufs, with the wire codec of dlx.py (no protobuf runtime):

  * every graph input becomes an "Input" node whose input_attr.dims are the declared dims
    (onnx_converter.cc:43-69); a graph input that is also an initializer therefore stays an
    input, as in the reference (its lookup finds the name already taken, :101-105);
  * the first time a node uses an initializer, a "Const" node is emitted just before it
    (:101-127); the using op decides the layout tags of the constant (SetTensorInfo):
    Conv filter ANY -> HWN4C4 (rank 4), Conv bias ANY -> ANY4 (rank 1), conv2d.cc:12-27;
    BatchNormalization parameters and Gemm operands ANY -> ANY4; Concat the default ANY -> ANY4.
    Ops whose converter refuses constants (Transpose, Reshape, Clip, MaxPool, Flatten, Gather,
    Unsqueeze, Shape, Add, GlobalAveragePool: LOG(FATAL) in their SetTensorInfo) raise here too:
    exporters hand those operands over as "Constant" nodes, which are converted;
  * FLOAT and INT64 tensors only, from the typed field or raw_data, INT64 values stored as
    floats (onnx_utils.cc:95-103); anything else is an error;
  * a node is named after its first output, keeps its op_type as the node type, and gets the
    attribute message of its converter; tensor indices are assigned in order of first
    appearance: inputs, then per node its new constants, then its outputs (:129-150);
  * graph outputs and inputs are copied to output_names / input_names (:183-191);
    producer_name "ONNX", version "0.1", doc_string "ignored" (:12-16).

The reference emits the Input nodes in the iteration order of an unordered_map (:52-69), which
the C++ standard leaves open; here they come in the order the graph declares them, which is
also the order of their tensor indices.

`convert` returns the serialized .dlx model; `convert_and_fold` also runs the Conv +
BatchNormalization (+ Relu / Clip) folding pass (remapper.remap), which is what the reference's
Converter does between Run and Save (converter.cpp:33-40).
"""
import struct

import numpy as np

from . import dlx

# onnx.proto TensorProto.DataType
FLOAT, INT64 = 1, 7


class ConvertError(ValueError):
    pass


# ------------------------------------------------------------------ onnx decode --
def _decode_tensor(buf):
    """onnx.TensorProto (onnx.proto:320-459) -> dict(name, dims, data_type, values float32)."""
    dims, data_type, name, raw = [], 0, "", None
    floats, int64s = None, []
    for field, wt, v in dlx._fields(buf):
        if field == 1:
            dims += dlx._ints(wt, v)
        elif field == 2:
            data_type = v
        elif field == 4:      # float_data, packed or not
            part = np.frombuffer(v, "<f4")
            floats = part.copy() if floats is None else np.concatenate([floats, part])
        elif field == 7:      # int64_data
            int64s += dlx._ints(wt, v)
        elif field == 8:
            name = v.decode()
        elif field == 9:
            raw = v
    count = int(np.prod(dims, dtype=np.int64)) if dims else 1
    if data_type == FLOAT:
        values = floats if floats is not None and floats.size else \
            (np.frombuffer(raw, "<f4") if raw is not None else None)
    elif data_type == INT64:
        values = np.array(int64s, np.float32) if int64s else \
            (np.frombuffer(raw, "<i8").astype(np.float32) if raw is not None else None)
    else:
        raise ConvertError("unsupported data type when converting tensor %d ('%s')" % (data_type, name))
    if count == 0:   # a zero-sized dimension: an empty tensor, as the reference emits it
        values = np.zeros(0, np.float32)
    if values is None or values.size < count:
        raise ConvertError("tensor '%s' holds %d values, its dims %s need %d" % (
            name, 0 if values is None else values.size, dims, count))
    return dict(name=name, dims=dims, data_type=data_type, values=np.asarray(values[:count], np.float32))


def _decode_attribute(buf):
    a = dict(name="", f=0.0, i=0, floats=[], ints=[], t=None, s=b"")
    for field, wt, v in dlx._fields(buf):
        if field == 1:
            a["name"] = v.decode()
        elif field == 2:
            a["f"] = struct.unpack("<f", v)[0]
        elif field == 3:
            a["i"] = dlx._signed(v)
        elif field == 4:
            a["s"] = v
        elif field == 5:
            a["t"] = v
        elif field == 7:
            a["floats"] += list(np.frombuffer(v, "<f4")) if wt == 2 else [struct.unpack("<f", v)[0]]
        elif field == 8:
            a["ints"] += dlx._ints(wt, v)
    return a


def _decode_node(buf):
    n = dict(input=[], output=[], name="", op_type="", attrs={})
    for field, wt, v in dlx._fields(buf):
        if field == 1:
            n["input"].append(v.decode())
        elif field == 2:
            n["output"].append(v.decode())
        elif field == 3:
            n["name"] = v.decode()
        elif field == 4:
            n["op_type"] = v.decode()
        elif field == 5:
            a = _decode_attribute(v)
            n["attrs"][a["name"]] = a
    return n


def _decode_value_info(buf):
    """ValueInfoProto -> (name, dims); a symbolic dimension (dim_param) reads as 0, which is
    what dim_value() returns for it in the reference."""
    name, dims = "", []
    for field, wt, v in dlx._fields(buf):
        if field == 1:
            name = v.decode()
        elif field == 2:                                  # TypeProto
            for f2, _, v2 in dlx._fields(v):
                if f2 != 1:                               # tensor_type
                    continue
                for f3, _, v3 in dlx._fields(v2):
                    if f3 != 2:                           # shape
                        continue
                    for f4, _, v4 in dlx._fields(v3):
                        if f4 != 1:                       # dim
                            continue
                        value = 0
                        for f5, wt5, v5 in dlx._fields(v4):
                            if f5 == 1 and wt5 == 0:
                                value = dlx._signed(v5)
                        dims.append(value)
    return name, dims


def decode_model(buf):
    """onnx.ModelProto bytes -> dict(nodes, initializers {name: tensor}, inputs [(name, dims)],
    outputs [name])."""
    graph = None
    for field, wt, v in dlx._fields(buf):
        if field == 7:
            graph = v
    if graph is None:
        raise ConvertError("load onnx model failed: no graph")
    g = dict(nodes=[], initializers={}, inputs=[], outputs=[])
    for field, wt, v in dlx._fields(graph):
        if field == 1:
            g["nodes"].append(_decode_node(v))
        elif field == 5:
            t = _decode_tensor(v)
            g["initializers"][t["name"]] = t
        elif field == 11:
            g["inputs"].append(_decode_value_info(v))
        elif field == 12:
            g["outputs"].append(_decode_value_info(v)[0])
    return g


# ----------------------------------------------------------------- op converters --
def _no_constants(op):
    def info(tensor, index):
        raise ConvertError("Cannot set tensor info for %s: its converter takes no constant "
                           "operand (export it as a Constant node)" % op)
    return info


def _default_info(tensor, index):
    tensor["data_format"], tensor["target_data_format"] = dlx.ANY, dlx.ANY4


def _conv_info(tensor, index):                              # onnx/ops/conv2d.cc:12-27
    if index == 1:
        if len(tensor["dims"]) != 4:
            raise ConvertError("Conv filter must have 4 dims, has %d" % len(tensor["dims"]))
        tensor["data_format"], tensor["target_data_format"] = dlx.ANY, dlx.HWN4C4
    elif index == 2:
        if len(tensor["dims"]) != 1:
            raise ConvertError("Conv bias must have 1 dim, has %d" % len(tensor["dims"]))
        tensor["data_format"], tensor["target_data_format"] = dlx.ANY, dlx.ANY4
    else:
        raise ConvertError("Conv: a constant cannot be operand %d" % index)


def _rank1_info(tensor, index):                             # onnx/ops/batchnorm.cc:11-16
    if len(tensor["dims"]) != 1:
        raise ConvertError("BatchNormalization parameters must have 1 dim")
    _default_info(tensor, index)


def _gemm_info(tensor, index):                              # onnx/ops/gemm.cc:7-13
    if index not in (1, 2):
        raise ConvertError("Gemm: a constant cannot be operand %d" % index)
    _default_info(tensor, index)


def _conv_attr(node):                                       # onnx/ops/conv2d.cc:30-66
    a = node["attrs"]
    out = b""
    if "kernel_shape" in a:
        out += dlx._packed_ints(1, a["kernel_shape"]["ints"])
    if "strides" in a:
        out += dlx._packed_ints(2, a["strides"]["ints"])
    if "pads" in a:
        out += dlx._packed_ints(3, a["pads"]["ints"])
    group = a["group"]["i"] if "group" in a else 0
    dil = a["dilations"]["ints"] if "dilations" in a else []
    if group <= 0 or len(dil) == 0 or any(d <= 0 for d in dil):
        raise ConvertError("Conv '%s': group and dilations must be present and positive" % node["output"][0])
    return dlx.ATTR_CONV2D, out + dlx._packed_ints(4, dil) + dlx._int(5, group)


def _pool_attr(node):                                       # onnx/ops/maxpool.cc:14-35
    a = node["attrs"]
    out = b""
    for field, key in ((1, "kernel_shape"), (2, "strides"), (3, "pads")):
        if key in a:
            out += dlx._packed_ints(field, a[key]["ints"])
    return dlx.ATTR_MAXPOOL, out


def _f(a, key, field):
    return dlx._float(field, a[key]["f"]) if key in a else b""


def _i(a, key, field):
    return dlx._int(field, a[key]["i"]) if key in a else b""


def _const_attr(node):                                      # onnx/ops/const.cc:15-31
    if "value" not in node["attrs"] or node["attrs"]["value"]["t"] is None:
        raise ConvertError("Constant '%s' has no tensor value" % node["output"][0])
    t = _decode_tensor(node["attrs"]["value"]["t"])
    _default_info(t, 0)
    return dlx.ATTR_CONST, dlx._sub(1, _encode_const(t))


# op_type -> (SetTensorInfo, attribute builder); the registry of converter/.../onnx/ops
CONVERTERS = {
    "Conv": (_conv_info, _conv_attr),
    "BatchNormalization": (_rank1_info, lambda n: (dlx.ATTR_BATCHNORM, _f(n["attrs"], "momentum", 1) +
                                                   _f(n["attrs"], "epsilon", 2))),
    "Relu": (lambda t, i: None, lambda n: (dlx.ATTR_RELU, _f(n["attrs"], "alpha", 1))),
    "Clip": (_no_constants("clip"), lambda n: (dlx.ATTR_CLIP, _f(n["attrs"], "min", 1) + _f(n["attrs"], "max", 2))),
    "Add": (_no_constants("binary"), lambda n: (dlx.ATTR_BINARY, b"")),
    "MaxPool": (_no_constants("maxpool"), _pool_attr),
    "GlobalAveragePool": (_no_constants("avepool"), lambda n: (dlx.ATTR_AVEPOOL, b"")),
    "Concat": (_default_info, lambda n: (dlx.ATTR_CONCAT, _i(n["attrs"], "axis", 1))),
    "Transpose": (_no_constants("transpose"),
                  lambda n: (dlx.ATTR_TRANSPOSE, dlx._packed_ints(1, n["attrs"]["perm"]["ints"])
                             if "perm" in n["attrs"] else b"")),
    "Reshape": (_no_constants("reshape"), lambda n: (dlx.ATTR_RESHAPE, b"")),
    "Flatten": (_no_constants("flatten"), lambda n: (dlx.ATTR_FLATTEN, _i(n["attrs"], "axis", 1))),
    "Gemm": (_gemm_info, lambda n: (dlx.ATTR_GEMM, _f(n["attrs"], "alpha", 1) + _f(n["attrs"], "beta", 2) +
                                    _i(n["attrs"], "transB", 3))),
    "Shape": (_no_constants("shape"), lambda n: (dlx.ATTR_SHAPE, b"")),
    "Gather": (_no_constants("gather"), lambda n: (dlx.ATTR_GATHER, _i(n["attrs"], "axis", 1))),
    "Unsqueeze": (_no_constants("unsqueeze"),
                  lambda n: (dlx.ATTR_UNSQUEEZE, dlx._packed_ints(1, n["attrs"]["axes"]["ints"])
                             if "axes" in n["attrs"] else b"")),
    "Constant": (_default_info, _const_attr),
}


def _encode_const(t):
    # data_type stays FLOAT32 (dlxnet.proto:32-43, value 0, not written), as MakeTensorFromProto sets it
    return dlx.encode_tensor(t["values"], t["dims"], t["data_format"], t["target_data_format"])


def convert(onnx_bytes):
    """Serialized onnx.ModelProto -> serialized dlxnet.ModelProto (.dlx)."""
    g = decode_model(onnx_bytes)
    names = {}                      # tensor name -> index, in order of first appearance
    nodes = []                      # encoded dlxnet.NodeProto payloads, in emission order

    def index_of(name):
        names.setdefault(name, len(names))
        return names[name]

    for name, dims in g["inputs"]:
        if name in names:
            continue
        idx = index_of(name)
        nodes.append(dlx.encode_node(name, "Input", [], [idx], dlx.ATTR_INPUT, dlx._packed_ints(3, dims)))
    pending = []                    # (position in `nodes`, onnx node): indices are filled in afterwards
    for node in g["nodes"]:
        conv = CONVERTERS.get(node["op_type"])
        if conv is None:
            raise ConvertError("Cannot find Type: %s" % node["op_type"])
        if not node["output"]:
            raise ConvertError("node '%s' has no output" % node["name"])
        set_info, build_attr = conv
        for j, inp in enumerate(node["input"]):
            if inp in names or inp not in g["initializers"]:
                continue
            t = dict(g["initializers"][inp])
            set_info(t, j)
            idx = index_of(inp)
            nodes.append(dlx.encode_node(inp, "Const", [], [idx], dlx.ATTR_CONST, dlx._sub(1, _encode_const(t))))
        field, payload = build_attr(node)
        pending.append((len(nodes), node, field, payload))
        nodes.append(None)
        for out in node["output"]:
            index_of(out)
    for pos, node, field, payload in pending:
        inputs = []
        for inp in node["input"]:
            if inp == "":
                continue            # an omitted optional operand (onnx_converter.cc:163-165)
            if inp not in names:
                raise ConvertError("Cannot find the input tensor '%s' of node '%s'" % (inp, node["output"][0]))
            inputs.append(names[inp])
        nodes[pos] = dlx.encode_node(node["output"][0], node["op_type"], inputs,
                                     [names[o] for o in node["output"]], field, payload)
    ordered = sorted(names, key=names.get)
    graph = b"".join(dlx._bytes(1, n) for n in nodes)
    graph += b"".join(dlx._bytes(3, n.encode()) for n in ordered)
    graph += b"".join(dlx._bytes(4, n.encode()) for n in g["outputs"])
    graph += b"".join(dlx._bytes(5, n.encode()) for n, _ in g["inputs"])
    return dlx._sub(1, graph) + dlx._string(2, "0.1") + dlx._string(3, "ONNX") + dlx._string(4, "ignored")


def convert_and_fold(onnx_bytes):
    """convert, then the Conv + BatchNormalization (+ Relu / Clip) folding pass.
    Returns (dlx bytes, folded batchnorms, folded activations)."""
    from . import remapper
    return remapper.remap(convert(onnx_bytes))


def main(argv=None):
    """`python -m ogle_amd.onnx model.onnx [demo.dlx]`: the reference's ./Converter
    (converter/converter/converter.cpp:9-47)."""
    import sys
    argv = sys.argv[1:] if argv is None else argv
    if not argv:
        print("usage: python -m ogle_amd.onnx model.onnx [demo.dlx]", file=sys.stderr)
        return 2
    dst = argv[1] if len(argv) > 1 else "demo.dlx"
    with open(argv[0], "rb") as f:
        out, n_bn, n_act = convert_and_fold(f.read())
    with open(dst, "wb") as f:
        f.write(out)
    print("%s -> %s: folded %d BatchNormalization and %d activation nodes" % (argv[0], dst, n_bn, n_act))
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
