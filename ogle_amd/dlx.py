"""Reader / writer of the .dlx model format and a small graph builder.

.dlx is a protobuf-binary `dlxnet.ModelProto`
(ogl_runtime/opengl/core/dlxnet.proto:5-215).  No protobuf runtime is needed: the
subset of the wire format the schema uses (varint, 32-bit, length-delimited, packed
repeated scalars) is encoded and decoded here.

`GraphBuilder` plays the role of the reference's Scope + nn_ops helpers
(ogl_runtime/opengl/core/scope.cc, opengl/nn/apis/nn_ops.h:39-64): it emits nodes in
topological order, one output per node, the output tensor named after the node and
indexed by emission order, which are the invariants the converter establishes
(converter/converter/graph/graph.cc:233-331) and the executor relies on.
"""
import struct

import numpy as np

# TensorProto.DataFormat (dlxnet.proto:7-30)
NCHW, NHWC, NHWC4, HWN4C4, ANY, ANY4 = 0, 1, 3, 4, 5, 6
DFORMAT_NAMES = {NCHW: "NCHW", NHWC: "NHWC", NHWC4: "NHWC4", HWN4C4: "HWN4C4", ANY: "ANY",
                 ANY4: "ANY4"}


# ------------------------------------------------------------------ wire encode --
def _varint(v):
    v &= (1 << 64) - 1
    out = bytearray()
    while v >= 0x80:
        out.append((v & 0x7F) | 0x80)
        v >>= 7
    out.append(v)
    return bytes(out)


def _tag(field, wt):
    return _varint((field << 3) | wt)


def _int(field, v):
    return b"" if v == 0 else _tag(field, 0) + _varint(int(v))


def _float(field, v):
    bits = struct.pack("<f", float(v))
    return b"" if bits == b"\0\0\0\0" else _tag(field, 5) + bits


def _bytes(field, b):
    return _tag(field, 2) + _varint(len(b)) + b


def _string(field, s):
    return b"" if not s else _bytes(field, s.encode())


def _packed_ints(field, values):
    if len(values) == 0:
        return b""
    return _bytes(field, b"".join(_varint(int(v)) for v in values))


def _packed_floats(field, values):
    a = np.ascontiguousarray(values, dtype="<f4").reshape(-1)
    if a.size == 0:
        return b""
    return _bytes(field, a.tobytes())


def _sub(field, payload):
    """Sub-message; written even when empty so that presence survives."""
    return _bytes(field, payload)


def encode_tensor(values, dims, data_format=ANY, target_data_format=ANY4):
    return (_int(1, data_format) + _packed_ints(3, dims) + _packed_floats(4, values) +
            _int(8, target_data_format))


def encode_conv2d_attr(kernel, stride, pad, dilation=1, group=1, activation_type="", minv=0.0,
                       maxv=0.0):
    return (_packed_ints(1, [kernel, kernel]) + _packed_ints(2, [stride, stride]) +
            _packed_ints(3, [pad] * 4) + _packed_ints(4, [dilation, dilation]) + _int(5, group) +
            _string(6, activation_type) + _float(7, minv) + _float(8, maxv))


def encode_pool_attr(kernel, stride, pad):
    return _packed_ints(1, [kernel, kernel]) + _packed_ints(2, [stride, stride]) + \
        _packed_ints(3, [pad] * 4)


# Attribute field numbers (dlxnet.proto:165-187)
ATTR_CONV2D, ATTR_CONST, ATTR_MAXPOOL, ATTR_AVEPOOL, ATTR_INPUT = 1, 2, 5, 6, 10
ATTR_TRANSPOSE, ATTR_CONCAT, ATTR_RESHAPE = 12, 16, 17
ATTR_SHAPE, ATTR_GATHER, ATTR_UNSQUEEZE = 13, 14, 15
ATTR_BATCHNORM, ATTR_RELU, ATTR_FLATTEN, ATTR_BINARY, ATTR_GEMM, ATTR_CLIP = 3, 4, 7, 8, 9, 11


def encode_node(name, type_, inputs, outputs, attr_field=None, attr_payload=b""):
    attr = b"" if attr_field is None else _sub(attr_field, attr_payload)
    return (_packed_ints(1, inputs) + _packed_ints(2, outputs) + _sub(3, attr) + _string(5, name) +
            _string(6, type_))


class GraphBuilder:
    """Builds a ModelProto node by node; every add_* returns the new tensor's index."""

    def __init__(self, producer_name="ONNX", name="graph"):
        self.producer_name = producer_name
        self.name = name
        self.nodes = []
        self.tensor_names = []
        self.input_names = []
        self.output_names = []

    def _emit(self, name, type_, inputs, attr_field=None, attr_payload=b""):
        if name in self.tensor_names:
            raise ValueError("duplicate node name %r" % name)
        index = len(self.tensor_names)
        self.tensor_names.append(name)
        self.nodes.append(encode_node(name, type_, list(inputs), [index], attr_field, attr_payload))
        return index

    def add_input(self, name, dims):
        self.input_names.append(name)
        return self._emit(name, "Input", [], ATTR_INPUT, _packed_ints(3, dims))

    def add_const(self, name, values, dims=None, data_format=ANY, target_data_format=ANY4):
        values = np.asarray(values, dtype=np.float32)
        dims = list(values.shape) if dims is None else list(dims)
        return self._emit(name, "Const", [], ATTR_CONST,
                          _sub(1, encode_tensor(values, dims, data_format, target_data_format)))

    def add_filter(self, name, w_oihw):
        """Conv filter constant: OIHW values, ANY in the file, HWN4C4 on the device
        (converter/converter/onnx/ops/conv2d.cc:12-27)."""
        return self.add_const(name, w_oihw, data_format=ANY, target_data_format=HWN4C4)

    def add_conv(self, name, x, w, b=None, kernel=1, stride=1, pad=0, dilation=1, group=1,
                 activation_type="", minv=0.0, maxv=0.0):
        inputs = [x, w] + ([b] if b is not None else [])
        return self._emit(name, "Conv", inputs, ATTR_CONV2D,
                          encode_conv2d_attr(kernel, stride, pad, dilation, group, activation_type,
                                             minv, maxv))

    def add_pool(self, name, x, kind="MaxPool", kernel=2, stride=2, pad=0):
        assert kind in ("MaxPool", "AveragePool", "GlobalAveragePool")
        # AveragePool also reads maxpool_attr (pool.cc:32)
        payload = b"" if kind == "GlobalAveragePool" else encode_pool_attr(kernel, stride, pad)
        return self._emit(name, kind, [x], ATTR_MAXPOOL, payload)

    def add_concat(self, name, inputs, axis):
        return self._emit(name, "Concat", inputs, ATTR_CONCAT, _int(1, axis))

    def add_transpose(self, name, x, perm):
        return self._emit(name, "Transpose", [x], ATTR_TRANSPOSE, _packed_ints(1, perm))

    def add_reshape(self, name, x, shape_tensor):
        return self._emit(name, "Reshape", [x, shape_tensor], ATTR_RESHAPE, b"")

    def add_add(self, name, a, b):
        return self._emit(name, "Add", [a, b], ATTR_BINARY, b"")

    def add_relu(self, name, x):
        return self._emit(name, "Relu", [x], ATTR_RELU, b"")

    def add_clip(self, name, x, minv, maxv):
        return self._emit(name, "Clip", [x], ATTR_CLIP, _float(1, minv) + _float(2, maxv))

    def add_batchnorm(self, name, x, gamma, beta, mean, var, epsilon=1e-5, momentum=0.9):
        return self._emit(name, "BatchNormalization", [x, gamma, beta, mean, var], ATTR_BATCHNORM,
                          _float(1, momentum) + _float(2, epsilon))

    def add_gemm(self, name, a, b, c=None, alpha=1.0, beta=1.0, trans_b=True):
        ins = [a, b] + ([c] if c is not None else [])
        return self._emit(name, "Gemm", ins, ATTR_GEMM,
                          _float(1, alpha) + _float(2, beta) + _int(3, int(bool(trans_b))))

    def add_flatten(self, name, x, axis=1):
        return self._emit(name, "Flatten", [x], ATTR_FLATTEN, _int(1, axis))

    def add_shape(self, name, x):
        return self._emit(name, "Shape", [x], ATTR_SHAPE, b"")

    def add_gather(self, name, data, index, axis=0):
        return self._emit(name, "Gather", [data, index], ATTR_GATHER, _int(1, axis))

    def add_unsqueeze(self, name, x, axis):
        return self._emit(name, "Unsqueeze", [x], ATTR_UNSQUEEZE, _packed_ints(1, [axis]))

    def add_decoder(self, name, prediction, anchors):
        return self._emit(name, "Decoder", [prediction, anchors])

    def add_node(self, name, type_, inputs, attr_field=None, attr_payload=b""):
        return self._emit(name, type_, inputs, attr_field, attr_payload)

    def add_output_name(self, name):
        self.output_names.append(name)

    def serialize(self):
        graph = b"".join(_bytes(1, n) for n in self.nodes) + _string(2, self.name)
        graph += b"".join(_bytes(3, n.encode()) for n in self.tensor_names)
        graph += b"".join(_bytes(4, n.encode()) for n in self.output_names)
        graph += b"".join(_bytes(5, n.encode()) for n in self.input_names)
        return _sub(1, graph) + _string(2, "1") + _string(3, self.producer_name)

    def save(self, path):
        with open(path, "wb") as f:
            f.write(self.serialize())


# ------------------------------------------------------------------ wire decode --
def _read_varint(buf, pos):
    v, shift = 0, 0
    while True:
        b = buf[pos]
        pos += 1
        v |= (b & 0x7F) << shift
        if not b & 0x80:
            return v, pos
        shift += 7


def _fields(buf):
    """Yields (field, wire_type, value) with value an int, or bytes for wire types 2/5."""
    pos, n = 0, len(buf)
    while pos < n:
        t, pos = _read_varint(buf, pos)
        field, wt = t >> 3, t & 7
        if wt == 0:
            v, pos = _read_varint(buf, pos)
        elif wt == 2:
            ln, pos = _read_varint(buf, pos)
            v = bytes(buf[pos:pos + ln])
            pos += ln
        elif wt == 5:
            v = bytes(buf[pos:pos + 4])
            pos += 4
        elif wt == 1:
            v = bytes(buf[pos:pos + 8])
            pos += 8
        else:
            raise ValueError("unsupported wire type %d" % wt)
        yield field, wt, v


def _signed(v, bits=64):
    return v - (1 << bits) if v >= 1 << (bits - 1) else v


def _ints(wt, v):
    if wt == 0:
        return [_signed(v)]
    out, pos = [], 0
    while pos < len(v):
        x, pos = _read_varint(v, pos)
        out.append(_signed(x))
    return out


def decode_tensor(buf):
    t = dict(data_format=NCHW, target_data_format=NCHW, dims=[], float_data=np.zeros(0, np.float32))
    for field, wt, v in _fields(buf):
        if field == 1:
            t["data_format"] = v
        elif field == 8:
            t["target_data_format"] = v
        elif field == 3:
            t["dims"] += _ints(wt, v)
        elif field == 4:
            t["float_data"] = np.frombuffer(v, "<f4").copy()
    return t


def decode_model(buf):
    """Parses a serialized ModelProto into plain dicts (enough for inspection and tests)."""
    model = dict(producer_name="", version="", graph=None)
    for field, wt, v in _fields(buf):
        if field == 3:
            model["producer_name"] = v.decode()
        elif field == 2:
            model["version"] = v.decode()
        elif field == 1:
            g = dict(name="", nodes=[], tensor_names=[], input_names=[], output_names=[])
            for f2, wt2, v2 in _fields(v):
                if f2 == 2:
                    g["name"] = v2.decode()
                elif f2 == 3:
                    g["tensor_names"].append(v2.decode())
                elif f2 == 4:
                    g["output_names"].append(v2.decode())
                elif f2 == 5:
                    g["input_names"].append(v2.decode())
                elif f2 == 1:
                    node = dict(name="", type="", input_index=[], output_index=[], attr={})
                    for f3, wt3, v3 in _fields(v2):
                        if f3 == 5:
                            node["name"] = v3.decode()
                        elif f3 == 6:
                            node["type"] = v3.decode()
                        elif f3 == 1:
                            node["input_index"] += _ints(wt3, v3)
                        elif f3 == 2:
                            node["output_index"] += _ints(wt3, v3)
                        elif f3 == 3:
                            for f4, _, v4 in _fields(v3):
                                node["attr"][f4] = v4
                    g["nodes"].append(node)
            model["graph"] = g
    return model


def decode_conv2d_attr(buf):
    a = dict(kernel_shape=[], strides=[], pads=[], dilations=[], group=0, activation_type="",
             min=0.0, max=0.0)
    for field, wt, v in _fields(buf):
        if field == 1:
            a["kernel_shape"] += _ints(wt, v)
        elif field == 2:
            a["strides"] += _ints(wt, v)
        elif field == 3:
            a["pads"] += _ints(wt, v)
        elif field == 4:
            a["dilations"] += _ints(wt, v)
        elif field == 5:
            a["group"] = v
        elif field == 6:
            a["activation_type"] = v.decode()
        elif field == 7:
            a["min"] = struct.unpack("<f", v)[0]
        elif field == 8:
            a["max"] = struct.unpack("<f", v)[0]
    return a
