"""An independent ONNX writer for the tests: message classes made by the protobuf runtime from
a descriptor of the subset of onnx.proto the converter reads (field numbers and types as
published in onnx.proto and as vendored by the reference, converter/converter/onnx/onnx.proto).
The front end under test decodes the wire format by hand; these bytes come from Google's
encoder, so a wrong field number, wire type or packing rule on either side shows up."""
import numpy as np
from google.protobuf import descriptor_pb2, descriptor_pool, message_factory

F = descriptor_pb2.FieldDescriptorProto
_SCALAR = {"int64": F.TYPE_INT64, "int32": F.TYPE_INT32, "float": F.TYPE_FLOAT, "string": F.TYPE_STRING,
           "bytes": F.TYPE_BYTES, "double": F.TYPE_DOUBLE, "uint64": F.TYPE_UINT64}

# message -> [(name, number, type, repeated)]
_SCHEMA = {
    "TensorShapeProto.Dimension": [("dim_value", 1, "int64", False), ("dim_param", 2, "string", False)],
    "TensorShapeProto": [("dim", 1, "TensorShapeProto.Dimension", True)],
    "TypeProto.Tensor": [("elem_type", 1, "int32", False), ("shape", 2, "TensorShapeProto", False)],
    "TypeProto": [("tensor_type", 1, "TypeProto.Tensor", False)],
    "ValueInfoProto": [("name", 1, "string", False), ("type", 2, "TypeProto", False),
                       ("doc_string", 3, "string", False)],
    "TensorProto": [("dims", 1, "int64", True), ("data_type", 2, "int32", False),
                    ("float_data", 4, "float", True), ("int32_data", 5, "int32", True),
                    ("string_data", 6, "bytes", True), ("int64_data", 7, "int64", True),
                    ("name", 8, "string", False), ("raw_data", 9, "bytes", False),
                    ("double_data", 10, "double", True), ("uint64_data", 11, "uint64", True),
                    ("doc_string", 12, "string", False)],
    "AttributeProto": [("name", 1, "string", False), ("f", 2, "float", False), ("i", 3, "int64", False),
                       ("s", 4, "bytes", False), ("t", 5, "TensorProto", False),
                       ("floats", 7, "float", True), ("ints", 8, "int64", True),
                       ("strings", 9, "bytes", True), ("doc_string", 13, "string", False),
                       ("type", 20, "int32", False)],
    "NodeProto": [("input", 1, "string", True), ("output", 2, "string", True), ("name", 3, "string", False),
                  ("op_type", 4, "string", False), ("attribute", 5, "AttributeProto", True),
                  ("doc_string", 6, "string", False), ("domain", 7, "string", False)],
    "GraphProto": [("node", 1, "NodeProto", True), ("name", 2, "string", False),
                   ("initializer", 5, "TensorProto", True), ("doc_string", 10, "string", False),
                   ("input", 11, "ValueInfoProto", True), ("output", 12, "ValueInfoProto", True),
                   ("value_info", 13, "ValueInfoProto", True)],
    "OperatorSetIdProto": [("domain", 1, "string", False), ("version", 2, "int64", False)],
    "ModelProto": [("ir_version", 1, "int64", False), ("producer_name", 2, "string", False),
                   ("producer_version", 3, "string", False), ("domain", 4, "string", False),
                   ("model_version", 5, "int64", False), ("doc_string", 6, "string", False),
                   ("graph", 7, "GraphProto", False), ("opset_import", 8, "OperatorSetIdProto", True)],
}


# the fields onnx.proto marks [packed = true]; under proto2 the other repeated scalars (dims, ints,
# floats) go out one tag per element, under proto3 (the reference's copy) all of them are packed
_PACKED = {"float_data", "int32_data", "int64_data", "double_data", "uint64_data"}


def _build(pack_all):
    package = "onnxtest3" if pack_all else "onnxtest2"
    fd = descriptor_pb2.FileDescriptorProto(name=package + ".proto", package=package, syntax="proto2")
    made = {}
    for full in sorted(_SCHEMA, key=lambda n: n.count(".")):   # parents before nested
        parts = full.split(".")
        holder = fd.message_type if len(parts) == 1 else made[".".join(parts[:-1])].nested_type
        msg = holder.add(name=parts[-1])
        made[full] = msg
    for full, fields in _SCHEMA.items():
        for name, number, type_, repeated in fields:
            f = made[full].field.add(name=name, number=number,
                                     label=F.LABEL_REPEATED if repeated else F.LABEL_OPTIONAL)
            if type_ in _SCALAR:
                f.type = _SCALAR[type_]
                if repeated and type_ not in ("string", "bytes"):
                    f.options.packed = pack_all or name in _PACKED
            else:
                f.type = F.TYPE_MESSAGE
                f.type_name = "." + package + "." + type_
    pool = descriptor_pool.DescriptorPool()
    pool.Add(fd)
    return {full: message_factory.GetMessageClass(pool.FindMessageTypeByName(package + "." + full))
            for full in _SCHEMA}


FLOAT, INT64, INT32 = 1, 7, 6
ATTR_FLOAT, ATTR_INT, ATTR_TENSOR, ATTR_FLOATS, ATTR_INTS = 1, 2, 4, 6, 7


class Writer:
    """ONNX messages under one packing rule: Writer(False) writes like proto2 onnx (what exporters
    ship), Writer(True) like the reference's proto3 copy of the schema."""

    def __init__(self, pack_all):
        self.M = _build(pack_all)

    def tensor(self, name, array, raw=False, data_type=None):
        a = np.asarray(array)
        t = self.M["TensorProto"](name=name, dims=list(a.shape))
        if data_type is not None:
            t.data_type = data_type
            return t
        if a.dtype.kind == "f":
            t.data_type = FLOAT
            if raw:
                t.raw_data = a.astype("<f4").tobytes()
            else:
                t.float_data.extend(float(v) for v in a.astype(np.float32).reshape(-1))
        else:
            t.data_type = INT64
            if raw:
                t.raw_data = a.astype("<i8").tobytes()
            else:
                t.int64_data.extend(int(v) for v in a.reshape(-1))
        return t

    def value_info(self, name, dims):
        v = self.M["ValueInfoProto"](name=name)
        v.type.tensor_type.elem_type = FLOAT
        for d in dims:
            dim = v.type.tensor_type.shape.dim.add()
            if isinstance(d, str):
                dim.dim_param = d
            else:
                dim.dim_value = d
        return v

    def node(self, op_type, inputs, outputs, name="", **attrs):
        n = self.M["NodeProto"](op_type=op_type, input=list(inputs), output=list(outputs), name=name)
        for key, value in attrs.items():
            a = n.attribute.add(name=key)
            if isinstance(value, float):
                a.f, a.type = value, ATTR_FLOAT
            elif isinstance(value, int):
                a.i, a.type = value, ATTR_INT
            elif isinstance(value, (list, tuple)):
                a.ints.extend(value)
                a.type = ATTR_INTS
            else:
                a.t.CopyFrom(value)
                a.type = ATTR_TENSOR
        return n

    def model(self, nodes, inputs, outputs, initializers=()):
        m = self.M["ModelProto"](ir_version=4, producer_name="tests")
        m.opset_import.add(version=9)
        m.graph.name = "g"
        m.graph.node.extend(nodes)
        m.graph.input.extend(inputs)
        m.graph.output.extend(outputs)
        m.graph.initializer.extend(initializers)
        return m.SerializeToString()
