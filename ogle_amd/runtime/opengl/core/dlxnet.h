// The .dlx model schema as plain C++ classes with a built-in protobuf wire codec.
//
// The schema is ogl_runtime/opengl/core/dlxnet.proto:5-215 (proto3, package
// dlxnet): field numbers, types and names below follow it one to one, and the
// accessors have the shape protoc would generate (name(), name_size(), name(i),
// set_name(), add_name(), mutable_name(), has_name()), so code written against
// the generated dlxnet.pb.h compiles against this header.  No libprotobuf is
// needed: Parse/Serialize implement the subset of the wire format the schema
// uses (varint, 32-bit, length-delimited, packed and unpacked repeated scalars).
#ifndef OPENGL_CORE_DLXNET_H_
#define OPENGL_CORE_DLXNET_H_

#include <cstdint>
#include <cstring>
#include <memory>
#include <string>
#include <vector>

namespace dlxnet {

namespace wire {

// Reader over a byte range.  ok() turns false on any malformed input.
class Reader {
 public:
  Reader(const uint8_t* p, size_t n) : p_(p), end_(p + n) {}
  bool ok() const { return ok_; }
  bool done() const { return p_ >= end_ || !ok_; }
  uint64_t Varint();
  uint32_t Fixed32();
  uint64_t Fixed64();
  Reader Sub();  // length-delimited payload
  std::string Bytes();
  bool Skip(int wire_type);
  bool Tag(int* field, int* wire_type);
  size_t remaining() const { return static_cast<size_t>(end_ - p_); }
  const uint8_t* data() const { return p_; }

 private:
  const uint8_t* p_;
  const uint8_t* end_;
  bool ok_ = true;
};

class Writer {
 public:
  void Varint(uint64_t v);
  void Tag(int field, int wire_type) { Varint((static_cast<uint64_t>(field) << 3) | wire_type); }
  void Fixed32(uint32_t v);
  void Bytes(int field, const std::string& s);
  void Int(int field, int64_t v) {  // proto3: default values are not written
    if (v != 0) {
      Tag(field, 0);
      Varint(static_cast<uint64_t>(v));
    }
  }
  void Float(int field, float v);
  void String(int field, const std::string& s) {
    if (!s.empty()) Bytes(field, s);
  }
  template <typename T>
  void PackedInts(int field, const std::vector<T>& v) {
    if (v.empty()) return;
    Writer w;
    for (T x : v) w.Varint(static_cast<uint64_t>(static_cast<int64_t>(x)));
    Bytes(field, w.out);
  }
  void PackedFloats(int field, const std::vector<float>& v);
  std::string out;
};

template <typename T>
void ReadInts(Reader& r, int wire_type, std::vector<T>* dst) {
  if (wire_type == 2) {
    Reader s = r.Sub();
    while (!s.done()) dst->push_back(static_cast<T>(s.Varint()));
  } else {
    dst->push_back(static_cast<T>(r.Varint()));
  }
}
void ReadFloats(Reader& r, int wire_type, std::vector<float>* dst);

}  // namespace wire

// Owning pointer whose copy is a deep copy, so that messages have value semantics.
template <typename T>
class ClonePtr {
 public:
  ClonePtr() {}
  ClonePtr(const ClonePtr& o) : p_(o.p_ ? new T(*o.p_) : nullptr) {}
  ClonePtr& operator=(const ClonePtr& o) {
    if (this != &o) p_.reset(o.p_ ? new T(*o.p_) : nullptr);
    return *this;
  }
  ClonePtr(ClonePtr&&) = default;
  ClonePtr& operator=(ClonePtr&&) = default;
  T* get() const { return p_.get(); }
  void reset(T* p = nullptr) { p_.reset(p); }
  explicit operator bool() const { return p_ != nullptr; }
  T& operator*() const { return *p_; }

 private:
  std::unique_ptr<T> p_;
};

// Common base: binary parse / serialize plus a text dump.
class Message {
 public:
  virtual ~Message() {}
  virtual bool ParseFrom(wire::Reader& r) = 0;
  virtual void SerializeTo(wire::Writer& w) const = 0;
  virtual void Print(std::string* out, int indent) const = 0;
  bool ParseFromArray(const void* data, size_t size) {
    wire::Reader r(static_cast<const uint8_t*>(data), size);
    return ParseFrom(r) && r.ok();
  }
  bool ParseFromString(const std::string& s) { return ParseFromArray(s.data(), s.size()); }
  std::string SerializeAsString() const {
    wire::Writer w;
    SerializeTo(w);
    return w.out;
  }
  bool SerializeToString(std::string* out) const {
    *out = SerializeAsString();
    return true;
  }
  std::string DebugString() const {
    std::string s;
    Print(&s, 0);
    return s;
  }
};

#define DLX_SCALAR(type, name)                 \
 public:                                       \
  type name() const { return name##_; }        \
  void set_##name(type v) { name##_ = v; }     \
                                               \
 private:                                      \
  type name##_ = type();

#define DLX_STRING(name)                                   \
 public:                                                   \
  const std::string& name() const { return name##_; }      \
  void set_##name(const std::string& v) { name##_ = v; }   \
  std::string* mutable_##name() { return &name##_; }       \
                                                           \
 private:                                                  \
  std::string name##_;

#define DLX_REPEATED(type, name)                                   \
 public:                                                           \
  int name##_size() const { return static_cast<int>(name##_.size()); } \
  const type& name(int i) const { return name##_[i]; }             \
  void set_##name(int i, const type& v) { name##_[i] = v; }        \
  void add_##name(const type& v) { name##_.push_back(v); }         \
  const std::vector<type>& name() const { return name##_; }        \
  std::vector<type>* mutable_##name() { return &name##_; }         \
  void clear_##name() { name##_.clear(); }                         \
                                                                   \
 private:                                                          \
  std::vector<type> name##_;

// Sub-message field: absent until mutable_name() is called; name() of an absent
// field returns a default instance, as generated code does.
#define DLX_MESSAGE(type, name)                                        \
 public:                                                               \
  bool has_##name() const { return static_cast<bool>(name##_); }               \
  const type& name() const { return name##_ ? *name##_ : type::Default(); } \
  type* mutable_##name() {                                             \
    if (!name##_) name##_.reset(new type);                             \
    return name##_.get();                                              \
  }                                                                    \
  void clear_##name() { name##_.reset(); }                             \
                                                                       \
 private:                                                              \
  ClonePtr<type> name##_;

#define DLX_COMMON(Type)                                   \
 public:                                                   \
  static const Type& Default() {                           \
    static const Type instance;                            \
    return instance;                                       \
  }                                                        \
  bool ParseFrom(wire::Reader& r) override;                \
  void SerializeTo(wire::Writer& w) const override;        \
  void Print(std::string* out, int indent) const override; \
  void CopyFrom(const Type& other) { *this = other; }

class TensorProto : public Message {
  DLX_COMMON(TensorProto)
 public:
  enum DataFormat { NCHW = 0, NHWC = 1, NHWC4 = 3, HWN4C4 = 4, ANY = 5, ANY4 = 6 };
  enum DataType { FLOAT32 = 0, FLOAT16 = 1, INT32 = 2, INT8 = 3 };
  DLX_SCALAR(DataFormat, data_format)          // = 1
  DLX_SCALAR(DataFormat, target_data_format)   // = 8
  DLX_SCALAR(DataType, data_type)              // = 2
  DLX_REPEATED(int32_t, dims)                  // = 3
  DLX_REPEATED(float, float_data)              // = 4 packed
  DLX_REPEATED(int32_t, int32_data)            // = 5 packed
  DLX_REPEATED(std::string, string_data)       // = 6
  DLX_REPEATED(int64_t, int64_data)            // = 7 packed
};

class Conv2dAttribute : public Message {
  DLX_COMMON(Conv2dAttribute)
  DLX_REPEATED(int64_t, kernel_shape)  // = 1
  DLX_REPEATED(int64_t, strides)       // = 2
  DLX_REPEATED(int64_t, pads)          // = 3
  DLX_REPEATED(int64_t, dilations)     // = 4
  DLX_SCALAR(int64_t, group)           // = 5
  DLX_STRING(activation_type)          // = 6
  DLX_SCALAR(float, min)               // = 7
  DLX_SCALAR(float, max)               // = 8
};

class ConstAttribute : public Message {
  DLX_COMMON(ConstAttribute)
  DLX_MESSAGE(TensorProto, value)  // = 1
};

class BatchNormAttribute : public Message {
  DLX_COMMON(BatchNormAttribute)
  DLX_SCALAR(float, momentum)  // = 1
  DLX_SCALAR(float, epsilon)   // = 2
};

class ReluAttribute : public Message {
  DLX_COMMON(ReluAttribute)
  DLX_SCALAR(float, slope)  // = 1
};

// MaxPoolAttribute and AvePoolAttribute share one layout (dlxnet.proto:98-103,121-125).
class MaxPoolAttribute : public Message {
  DLX_COMMON(MaxPoolAttribute)
  DLX_REPEATED(int64_t, kernel_shape)  // = 1
  DLX_REPEATED(int64_t, strides)       // = 2
  DLX_REPEATED(int64_t, pads)          // = 3
};
typedef MaxPoolAttribute AvePoolAttribute;

class BinaryAttribute : public Message {
  DLX_COMMON(BinaryAttribute)
  DLX_STRING(binary_op_type)  // = 1
};

// One int32 "axis" at field 1: Flatten, Concat, Reshape, Gather attributes.
class AxisAttribute : public Message {
  DLX_COMMON(AxisAttribute)
  DLX_SCALAR(int32_t, axis)  // = 1
};
typedef AxisAttribute FlattenAttribute;
typedef AxisAttribute ConcatAttribute;
typedef AxisAttribute ReshapeAttribute;
typedef AxisAttribute GatherAttribute;

class ClipAttribute : public Message {
  DLX_COMMON(ClipAttribute)
  DLX_SCALAR(float, min)  // = 1
  DLX_SCALAR(float, max)  // = 2
};

class TransposeAttribute : public Message {
  DLX_COMMON(TransposeAttribute)
  DLX_REPEATED(int32_t, perm)  // = 1
};

class ShapeAttribute : public Message {
  DLX_COMMON(ShapeAttribute)
};

class GemmAttribute : public Message {
  DLX_COMMON(GemmAttribute)
  DLX_SCALAR(float, alpha)     // = 1
  DLX_SCALAR(float, beta)      // = 2
  DLX_SCALAR(int32_t, transB)  // = 3
};

class InputAttribute : public Message {
  DLX_COMMON(InputAttribute)
  DLX_REPEATED(int32_t, dims)  // = 3
};

class UnsqueezeAttribute : public Message {
  DLX_COMMON(UnsqueezeAttribute)
  DLX_REPEATED(int32_t, axes)  // = 1
};

class Attribute : public Message {
  DLX_COMMON(Attribute)
  DLX_MESSAGE(Conv2dAttribute, conv2d_attr)        // = 1
  DLX_MESSAGE(ConstAttribute, const_attr)          // = 2
  DLX_MESSAGE(BatchNormAttribute, batchnorm_attr)  // = 3
  DLX_MESSAGE(ReluAttribute, relu_attr)            // = 4
  DLX_MESSAGE(MaxPoolAttribute, maxpool_attr)      // = 5
  DLX_MESSAGE(AvePoolAttribute, avepool_attr)      // = 6
  DLX_MESSAGE(FlattenAttribute, flatten_attr)      // = 7
  DLX_MESSAGE(BinaryAttribute, binary_attr)        // = 8
  DLX_MESSAGE(GemmAttribute, gemm_attr)            // = 9
  DLX_MESSAGE(InputAttribute, input_attr)          // = 10
  DLX_MESSAGE(ClipAttribute, clip_attr)            // = 11
  DLX_MESSAGE(TransposeAttribute, transpose_attr)  // = 12
  DLX_MESSAGE(ShapeAttribute, shape_attr)          // = 13
  DLX_MESSAGE(GatherAttribute, gather_attr)        // = 14
  DLX_MESSAGE(UnsqueezeAttribute, unsqueeze_attr)  // = 15
  DLX_MESSAGE(ConcatAttribute, concat_attr)        // = 16
  DLX_MESSAGE(ReshapeAttribute, reshape_attr)      // = 17
};

class NodeProto : public Message {
  DLX_COMMON(NodeProto)
  DLX_STRING(name)                      // = 5
  DLX_STRING(type)                      // = 6
  DLX_REPEATED(int64_t, input_index)    // = 1
  DLX_REPEATED(int64_t, output_index)   // = 2
  DLX_MESSAGE(Attribute, attr)          // = 3
  DLX_STRING(doc_string)                // = 4
};

class GraphProto : public Message {
  DLX_COMMON(GraphProto)
  DLX_STRING(name)                        // = 2
  DLX_REPEATED(std::string, input_names)  // = 5
  DLX_REPEATED(std::string, tensor_names) // = 3
  DLX_REPEATED(std::string, output_names) // = 4
 public:
  int node_size() const { return static_cast<int>(node_.size()); }
  const NodeProto& node(int i) const { return node_[i]; }
  NodeProto* mutable_node(int i) { return &node_[i]; }
  NodeProto* add_node() {
    node_.emplace_back();
    return &node_.back();
  }
  const std::vector<NodeProto>& node() const { return node_; }  // = 1

 private:
  std::vector<NodeProto> node_;
};

class ModelProto : public Message {
  DLX_COMMON(ModelProto)
  DLX_STRING(producer_name)      // = 3
  DLX_MESSAGE(GraphProto, graph) // = 1
  DLX_STRING(version)            // = 2
  DLX_STRING(doc_string)         // = 4
};

const char* DataFormatName(TensorProto::DataFormat f);

}  // namespace dlxnet

#endif  // OPENGL_CORE_DLXNET_H_
