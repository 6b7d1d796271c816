// Wire codec of the .dlx schema (ogl_runtime/opengl/core/dlxnet.proto:5-215).
#include "opengl/core/dlxnet.h"

#include <cstdio>

namespace dlxnet {
namespace wire {

uint64_t Reader::Varint() {
  uint64_t v = 0;
  for (int shift = 0; shift < 64; shift += 7) {
    if (p_ >= end_) {
      ok_ = false;
      return 0;
    }
    const uint8_t b = *p_++;
    v |= static_cast<uint64_t>(b & 0x7f) << shift;
    if (!(b & 0x80)) return v;
  }
  ok_ = false;
  return 0;
}

uint32_t Reader::Fixed32() {
  if (remaining() < 4) {
    ok_ = false;
    p_ = end_;
    return 0;
  }
  uint32_t v;
  std::memcpy(&v, p_, 4);
  p_ += 4;
  return v;
}

uint64_t Reader::Fixed64() {
  if (remaining() < 8) {
    ok_ = false;
    p_ = end_;
    return 0;
  }
  uint64_t v;
  std::memcpy(&v, p_, 8);
  p_ += 8;
  return v;
}

Reader Reader::Sub() {
  const uint64_t n = Varint();
  if (!ok_ || n > remaining()) {
    ok_ = false;
    p_ = end_;
    return Reader(end_, 0);
  }
  Reader s(p_, static_cast<size_t>(n));
  p_ += n;
  return s;
}

std::string Reader::Bytes() {
  Reader s = Sub();
  return std::string(reinterpret_cast<const char*>(s.data()), s.remaining());
}

bool Reader::Skip(int wire_type) {
  switch (wire_type) {
    case 0: Varint(); break;
    case 1: Fixed64(); break;
    case 2: Sub(); break;
    case 5: Fixed32(); break;
    default: ok_ = false;
  }
  return ok_;
}

bool Reader::Tag(int* field, int* wire_type) {
  if (done()) return false;
  const uint64_t t = Varint();
  if (!ok_) return false;
  *field = static_cast<int>(t >> 3);
  *wire_type = static_cast<int>(t & 7);
  if (*field == 0) ok_ = false;
  return ok_;
}

void Writer::Varint(uint64_t v) {
  while (v >= 0x80) {
    out.push_back(static_cast<char>((v & 0x7f) | 0x80));
    v >>= 7;
  }
  out.push_back(static_cast<char>(v));
}

void Writer::Fixed32(uint32_t v) {
  char b[4];
  std::memcpy(b, &v, 4);
  out.append(b, 4);
}

void Writer::Bytes(int field, const std::string& s) {
  Tag(field, 2);
  Varint(s.size());
  out.append(s);
}

void Writer::Float(int field, float v) {
  uint32_t bits;
  std::memcpy(&bits, &v, 4);
  if (bits == 0) return;  // proto3 omits +0.0
  Tag(field, 5);
  Fixed32(bits);
}

void Writer::PackedFloats(int field, const std::vector<float>& v) {
  if (v.empty()) return;
  Tag(field, 2);
  Varint(v.size() * 4);
  out.append(reinterpret_cast<const char*>(v.data()), v.size() * 4);
}

void ReadFloats(Reader& r, int wire_type, std::vector<float>* dst) {
  if (wire_type == 2) {
    Reader s = r.Sub();
    const size_t n = s.remaining() / 4;
    const size_t old = dst->size();
    dst->resize(old + n);
    std::memcpy(dst->data() + old, s.data(), n * 4);
  } else {
    const uint32_t bits = r.Fixed32();
    float f;
    std::memcpy(&f, &bits, 4);
    dst->push_back(f);
  }
}

}  // namespace wire

namespace {

float AsFloat(uint32_t bits) {
  float f;
  std::memcpy(&f, &bits, 4);
  return f;
}

void Indent(std::string* out, int n) { out->append(static_cast<size_t>(n) * 2, ' '); }

void PrintKV(std::string* out, int indent, const char* key, const std::string& value) {
  Indent(out, indent);
  out->append(key).append(": ").append(value).append("\n");
}

template <typename T>
void PrintInts(std::string* out, int indent, const char* key, const std::vector<T>& v) {
  for (T x : v) PrintKV(out, indent, key, std::to_string(x));
}

void PrintFloat(std::string* out, int indent, const char* key, float v) {
  char buf[48];
  std::snprintf(buf, sizeof(buf), "%g", v);
  PrintKV(out, indent, key, buf);
}

void PrintSub(std::string* out, int indent, const char* key, const Message& m) {
  Indent(out, indent);
  out->append(key).append(" {\n");
  m.Print(out, indent + 1);
  Indent(out, indent);
  out->append("}\n");
}

template <typename M>
void WriteSub(wire::Writer& w, int field, const M& m) {
  w.Bytes(field, m.SerializeAsString());
}

}  // namespace

const char* DataFormatName(TensorProto::DataFormat f) {
  switch (f) {
    case TensorProto::NCHW: return "NCHW";
    case TensorProto::NHWC: return "NHWC";
    case TensorProto::NHWC4: return "NHWC4";
    case TensorProto::HWN4C4: return "HWN4C4";
    case TensorProto::ANY: return "ANY";
    case TensorProto::ANY4: return "ANY4";
  }
  return "?";
}

// Each ParseFrom walks the tags once; unknown fields are skipped.
#define DLX_PARSE_BEGIN(Type)                 \
  bool Type::ParseFrom(wire::Reader& r) {     \
    int field, wt;                            \
    while (r.Tag(&field, &wt)) {              \
      switch (field) {
#define DLX_PARSE_END      \
  default: r.Skip(wt);     \
    }                      \
    }                      \
    return r.ok();         \
    }

// ---- TensorProto
DLX_PARSE_BEGIN(TensorProto)
  case 1: data_format_ = static_cast<DataFormat>(r.Varint()); break;
  case 8: target_data_format_ = static_cast<DataFormat>(r.Varint()); break;
  case 2: data_type_ = static_cast<DataType>(r.Varint()); break;
  case 3: wire::ReadInts(r, wt, &dims_); break;
  case 4: wire::ReadFloats(r, wt, &float_data_); break;
  case 5: wire::ReadInts(r, wt, &int32_data_); break;
  case 6: string_data_.push_back(r.Bytes()); break;
  case 7: wire::ReadInts(r, wt, &int64_data_); break;
DLX_PARSE_END
void TensorProto::SerializeTo(wire::Writer& w) const {
  w.Int(1, data_format_);
  w.Int(2, data_type_);
  w.PackedInts(3, dims_);
  w.PackedFloats(4, float_data_);
  w.PackedInts(5, int32_data_);
  for (const auto& s : string_data_) w.Bytes(6, s);
  w.PackedInts(7, int64_data_);
  w.Int(8, target_data_format_);
}
void TensorProto::Print(std::string* out, int indent) const {
  PrintKV(out, indent, "data_format", DataFormatName(data_format_));
  PrintKV(out, indent, "target_data_format", DataFormatName(target_data_format_));
  PrintInts(out, indent, "dims", dims_);
  PrintKV(out, indent, "float_data", "<" + std::to_string(float_data_.size()) + " values>");
}

// ---- Conv2dAttribute
DLX_PARSE_BEGIN(Conv2dAttribute)
  case 1: wire::ReadInts(r, wt, &kernel_shape_); break;
  case 2: wire::ReadInts(r, wt, &strides_); break;
  case 3: wire::ReadInts(r, wt, &pads_); break;
  case 4: wire::ReadInts(r, wt, &dilations_); break;
  case 5: group_ = static_cast<int64_t>(r.Varint()); break;
  case 6: activation_type_ = r.Bytes(); break;
  case 7: min_ = AsFloat(r.Fixed32()); break;
  case 8: max_ = AsFloat(r.Fixed32()); break;
DLX_PARSE_END
void Conv2dAttribute::SerializeTo(wire::Writer& w) const {
  w.PackedInts(1, kernel_shape_);
  w.PackedInts(2, strides_);
  w.PackedInts(3, pads_);
  w.PackedInts(4, dilations_);
  w.Int(5, group_);
  w.String(6, activation_type_);
  w.Float(7, min_);
  w.Float(8, max_);
}
void Conv2dAttribute::Print(std::string* out, int indent) const {
  PrintInts(out, indent, "kernel_shape", kernel_shape_);
  PrintInts(out, indent, "strides", strides_);
  PrintInts(out, indent, "pads", pads_);
  PrintInts(out, indent, "dilations", dilations_);
  PrintKV(out, indent, "group", std::to_string(group_));
  if (!activation_type_.empty()) PrintKV(out, indent, "activation_type", activation_type_);
  PrintFloat(out, indent, "min", min_);
  PrintFloat(out, indent, "max", max_);
}

// ---- ConstAttribute
DLX_PARSE_BEGIN(ConstAttribute)
  case 1: { wire::Reader s = r.Sub(); if (!mutable_value()->ParseFrom(s)) return false; break; }
DLX_PARSE_END
void ConstAttribute::SerializeTo(wire::Writer& w) const {
  if (has_value()) WriteSub(w, 1, value());
}
void ConstAttribute::Print(std::string* out, int indent) const {
  if (has_value()) PrintSub(out, indent, "value", value());
}

// ---- BatchNormAttribute
DLX_PARSE_BEGIN(BatchNormAttribute)
  case 1: momentum_ = AsFloat(r.Fixed32()); break;
  case 2: epsilon_ = AsFloat(r.Fixed32()); break;
DLX_PARSE_END
void BatchNormAttribute::SerializeTo(wire::Writer& w) const {
  w.Float(1, momentum_);
  w.Float(2, epsilon_);
}
void BatchNormAttribute::Print(std::string* out, int indent) const {
  PrintFloat(out, indent, "momentum", momentum_);
  PrintFloat(out, indent, "epsilon", epsilon_);
}

// ---- ReluAttribute
DLX_PARSE_BEGIN(ReluAttribute)
  case 1: slope_ = AsFloat(r.Fixed32()); break;
DLX_PARSE_END
void ReluAttribute::SerializeTo(wire::Writer& w) const { w.Float(1, slope_); }
void ReluAttribute::Print(std::string* out, int indent) const {
  PrintFloat(out, indent, "slope", slope_);
}

// ---- MaxPoolAttribute / AvePoolAttribute
DLX_PARSE_BEGIN(MaxPoolAttribute)
  case 1: wire::ReadInts(r, wt, &kernel_shape_); break;
  case 2: wire::ReadInts(r, wt, &strides_); break;
  case 3: wire::ReadInts(r, wt, &pads_); break;
DLX_PARSE_END
void MaxPoolAttribute::SerializeTo(wire::Writer& w) const {
  w.PackedInts(1, kernel_shape_);
  w.PackedInts(2, strides_);
  w.PackedInts(3, pads_);
}
void MaxPoolAttribute::Print(std::string* out, int indent) const {
  PrintInts(out, indent, "kernel_shape", kernel_shape_);
  PrintInts(out, indent, "strides", strides_);
  PrintInts(out, indent, "pads", pads_);
}

// ---- BinaryAttribute
DLX_PARSE_BEGIN(BinaryAttribute)
  case 1: binary_op_type_ = r.Bytes(); break;
DLX_PARSE_END
void BinaryAttribute::SerializeTo(wire::Writer& w) const { w.String(1, binary_op_type_); }
void BinaryAttribute::Print(std::string* out, int indent) const {
  PrintKV(out, indent, "binary_op_type", binary_op_type_);
}

// ---- AxisAttribute (Flatten / Concat / Reshape / Gather)
DLX_PARSE_BEGIN(AxisAttribute)
  case 1: axis_ = static_cast<int32_t>(r.Varint()); break;
DLX_PARSE_END
void AxisAttribute::SerializeTo(wire::Writer& w) const { w.Int(1, axis_); }
void AxisAttribute::Print(std::string* out, int indent) const {
  PrintKV(out, indent, "axis", std::to_string(axis_));
}

// ---- ClipAttribute
DLX_PARSE_BEGIN(ClipAttribute)
  case 1: min_ = AsFloat(r.Fixed32()); break;
  case 2: max_ = AsFloat(r.Fixed32()); break;
DLX_PARSE_END
void ClipAttribute::SerializeTo(wire::Writer& w) const {
  w.Float(1, min_);
  w.Float(2, max_);
}
void ClipAttribute::Print(std::string* out, int indent) const {
  PrintFloat(out, indent, "min", min_);
  PrintFloat(out, indent, "max", max_);
}

// ---- TransposeAttribute
DLX_PARSE_BEGIN(TransposeAttribute)
  case 1: wire::ReadInts(r, wt, &perm_); break;
DLX_PARSE_END
void TransposeAttribute::SerializeTo(wire::Writer& w) const { w.PackedInts(1, perm_); }
void TransposeAttribute::Print(std::string* out, int indent) const {
  PrintInts(out, indent, "perm", perm_);
}

// ---- ShapeAttribute
DLX_PARSE_BEGIN(ShapeAttribute)
DLX_PARSE_END
void ShapeAttribute::SerializeTo(wire::Writer&) const {}
void ShapeAttribute::Print(std::string*, int) const {}

// ---- GemmAttribute
DLX_PARSE_BEGIN(GemmAttribute)
  case 1: alpha_ = AsFloat(r.Fixed32()); break;
  case 2: beta_ = AsFloat(r.Fixed32()); break;
  case 3: transB_ = static_cast<int32_t>(r.Varint()); break;
DLX_PARSE_END
void GemmAttribute::SerializeTo(wire::Writer& w) const {
  w.Float(1, alpha_);
  w.Float(2, beta_);
  w.Int(3, transB_);
}
void GemmAttribute::Print(std::string* out, int indent) const {
  PrintFloat(out, indent, "alpha", alpha_);
  PrintFloat(out, indent, "beta", beta_);
  PrintKV(out, indent, "transB", std::to_string(transB_));
}

// ---- InputAttribute
DLX_PARSE_BEGIN(InputAttribute)
  case 3: wire::ReadInts(r, wt, &dims_); break;
DLX_PARSE_END
void InputAttribute::SerializeTo(wire::Writer& w) const { w.PackedInts(3, dims_); }
void InputAttribute::Print(std::string* out, int indent) const {
  PrintInts(out, indent, "dims", dims_);
}

// ---- UnsqueezeAttribute
DLX_PARSE_BEGIN(UnsqueezeAttribute)
  case 1: wire::ReadInts(r, wt, &axes_); break;
DLX_PARSE_END
void UnsqueezeAttribute::SerializeTo(wire::Writer& w) const { w.PackedInts(1, axes_); }
void UnsqueezeAttribute::Print(std::string* out, int indent) const {
  PrintInts(out, indent, "axes", axes_);
}

// ---- Attribute
#define DLX_SUB_CASE(num, name)                                    \
  case num: {                                                      \
    wire::Reader s = r.Sub();                                      \
    if (!mutable_##name()->ParseFrom(s)) return false;             \
    break;                                                         \
  }
DLX_PARSE_BEGIN(Attribute)
  DLX_SUB_CASE(1, conv2d_attr)
  DLX_SUB_CASE(2, const_attr)
  DLX_SUB_CASE(3, batchnorm_attr)
  DLX_SUB_CASE(4, relu_attr)
  DLX_SUB_CASE(5, maxpool_attr)
  DLX_SUB_CASE(6, avepool_attr)
  DLX_SUB_CASE(7, flatten_attr)
  DLX_SUB_CASE(8, binary_attr)
  DLX_SUB_CASE(9, gemm_attr)
  DLX_SUB_CASE(10, input_attr)
  DLX_SUB_CASE(11, clip_attr)
  DLX_SUB_CASE(12, transpose_attr)
  DLX_SUB_CASE(13, shape_attr)
  DLX_SUB_CASE(14, gather_attr)
  DLX_SUB_CASE(15, unsqueeze_attr)
  DLX_SUB_CASE(16, concat_attr)
  DLX_SUB_CASE(17, reshape_attr)
DLX_PARSE_END
#define DLX_SUB_EACH(X)                                                                       \
  X(1, conv2d_attr) X(2, const_attr) X(3, batchnorm_attr) X(4, relu_attr) X(5, maxpool_attr)  \
  X(6, avepool_attr) X(7, flatten_attr) X(8, binary_attr) X(9, gemm_attr) X(10, input_attr)   \
  X(11, clip_attr) X(12, transpose_attr) X(13, shape_attr) X(14, gather_attr)                 \
  X(15, unsqueeze_attr) X(16, concat_attr) X(17, reshape_attr)
void Attribute::SerializeTo(wire::Writer& w) const {
#define X(num, name) \
  if (has_##name()) WriteSub(w, num, name());
  DLX_SUB_EACH(X)
#undef X
}
void Attribute::Print(std::string* out, int indent) const {
#define X(num, name) \
  if (has_##name()) PrintSub(out, indent, #name, name());
  DLX_SUB_EACH(X)
#undef X
}

// ---- NodeProto
DLX_PARSE_BEGIN(NodeProto)
  case 5: name_ = r.Bytes(); break;
  case 6: type_ = r.Bytes(); break;
  case 1: wire::ReadInts(r, wt, &input_index_); break;
  case 2: wire::ReadInts(r, wt, &output_index_); break;
  DLX_SUB_CASE(3, attr)
  case 4: doc_string_ = r.Bytes(); break;
DLX_PARSE_END
void NodeProto::SerializeTo(wire::Writer& w) const {
  w.PackedInts(1, input_index_);
  w.PackedInts(2, output_index_);
  if (has_attr()) WriteSub(w, 3, attr());
  w.String(4, doc_string_);
  w.String(5, name_);
  w.String(6, type_);
}
void NodeProto::Print(std::string* out, int indent) const {
  PrintKV(out, indent, "name", name_);
  PrintKV(out, indent, "type", type_);
  PrintInts(out, indent, "input_index", input_index_);
  PrintInts(out, indent, "output_index", output_index_);
  if (has_attr()) PrintSub(out, indent, "attr", attr());
}

// ---- GraphProto
DLX_PARSE_BEGIN(GraphProto)
  case 2: name_ = r.Bytes(); break;
  case 5: input_names_.push_back(r.Bytes()); break;
  case 3: tensor_names_.push_back(r.Bytes()); break;
  case 4: output_names_.push_back(r.Bytes()); break;
  case 1: { wire::Reader s = r.Sub(); if (!add_node()->ParseFrom(s)) return false; break; }
DLX_PARSE_END
void GraphProto::SerializeTo(wire::Writer& w) const {
  for (const auto& n : node_) WriteSub(w, 1, n);
  w.String(2, name_);
  for (const auto& s : tensor_names_) w.Bytes(3, s);
  for (const auto& s : output_names_) w.Bytes(4, s);
  for (const auto& s : input_names_) w.Bytes(5, s);
}
void GraphProto::Print(std::string* out, int indent) const {
  PrintKV(out, indent, "name", name_);
  for (const auto& s : input_names_) PrintKV(out, indent, "input_names", s);
  for (const auto& s : output_names_) PrintKV(out, indent, "output_names", s);
  for (const auto& n : node_) PrintSub(out, indent, "node", n);
}

// ---- ModelProto
DLX_PARSE_BEGIN(ModelProto)
  case 3: producer_name_ = r.Bytes(); break;
  DLX_SUB_CASE(1, graph)
  case 2: version_ = r.Bytes(); break;
  case 4: doc_string_ = r.Bytes(); break;
DLX_PARSE_END
void ModelProto::SerializeTo(wire::Writer& w) const {
  if (has_graph()) WriteSub(w, 1, graph());
  w.String(2, version_);
  w.String(3, producer_name_);
  w.String(4, doc_string_);
}
void ModelProto::Print(std::string* out, int indent) const {
  PrintKV(out, indent, "producer_name", producer_name_);
  PrintKV(out, indent, "version", version_);
  if (has_graph()) PrintSub(out, indent, "graph", graph());
}

}  // namespace dlxnet
