#include "opengl/core/tensor.h"

#include <hip/hip_runtime_api.h>

#include <cstdlib>
#include <sstream>

namespace opengl {

namespace {
size_t ElementSize(Tensor::DataType dtype) {
  switch (dtype) {
    case Tensor::DT_INT: return sizeof(int32_t);
    case Tensor::DT_FLOAT: return sizeof(float);
    case Tensor::DT_DOUBLE: return sizeof(double);
    default: LOG(FATAL) << "invalid tensor dtype " << dtype;
  }
  return 0;
}
}  // namespace

size_t Tensor::num_elements() const {
  size_t n = 1;
  for (int d : shape_) n *= static_cast<size_t>(d);
  return n;
}

Tensor::Tensor(DataType dtype, IntList shape, MemoryType mem_type, DataFormat dformat)
    : dtype_(dtype), mem_type_(mem_type), shape_(std::move(shape)), dformat_(dformat) {
  for (int d : shape_) CHECK_GE(d, 0) << "negative dimension in tensor shape";
  if (shape_.size() != 4) {
    // Only general tensors may have a rank other than 4 (tensor.h:247-252 of the reference).
    CHECK(dformat_ == dlxnet::TensorProto::ANY || dformat_ == dlxnet::TensorProto::ANY4)
        << "a rank-" << shape_.size() << " tensor must be ANY or ANY4, got " << FormatToStr(dformat_);
  }
  requested_size_ = num_elements() * ElementSize(dtype_);
  allocated_size_ = requested_size_;
  // Host tensors with a stride-4 tag hold the reference's padded layout (what
  // GetOutputs hands back for "NHWC4" / "ANY4" / "HWN4C4"); device tensors are dense.
  if (mem_type_ == HOST_MEMORY) allocated_size_ = HostElements(shape_, dformat_) * ElementSize(dtype_);
  const size_t bytes = allocated_size_ > 0 ? allocated_size_ : 16;
  if (mem_type_ == HOST_MEMORY) {
    host_ = std::malloc(bytes);
    CHECK(host_ != nullptr) << "host allocation of " << bytes << " bytes failed";
  } else {
    DeviceBuffer* buf = new DeviceBuffer;
    const hipError_t e = hipMalloc(&buf->ptr, bytes);
    if (e != hipSuccess) {
      delete buf;
      LOG(FATAL) << "hipMalloc(" << bytes << ") failed: " << hipGetErrorString(e);
    }
    buf->bytes = bytes;
    device_ = buf;
  }
}

Tensor::Tensor(const dlxnet::TensorProto& proto)
    : Tensor(DT_FLOAT, IntList(proto.dims().begin(), proto.dims().end()), HOST_MEMORY,
             proto.data_format()) {
  float* dst = host<float>();
  const size_t n = num_elements();
  if (proto.float_data_size() > 0) {
    CHECK_EQ(static_cast<size_t>(proto.float_data_size()), n) << "constant size mismatch";
    std::memcpy(dst, proto.float_data().data(), n * sizeof(float));
  } else if (proto.int32_data_size() > 0) {
    CHECK_EQ(static_cast<size_t>(proto.int32_data_size()), n);
    for (size_t i = 0; i < n; ++i) dst[i] = static_cast<float>(proto.int32_data(i));
  } else if (proto.int64_data_size() > 0) {
    CHECK_EQ(static_cast<size_t>(proto.int64_data_size()), n);
    for (size_t i = 0; i < n; ++i) dst[i] = static_cast<float>(proto.int64_data(i));
  } else {
    CHECK_EQ(n, 0u) << "constant without data";
  }
  initialized_ = true;
}

Tensor::Tensor(const Tensor* other, IntList shape, DataFormat dformat)
    : dtype_(other->dtype()), mem_type_(other->mem_type()), shape_(std::move(shape)),
      dformat_(dformat) {
  CHECK(other->mem_type() != HOST_MEMORY) << "only device tensors can be aliased";
  CHECK_EQ(num_elements(), other->num_elements()) << "a view keeps the element count";
  DeviceBuffer* buf = new DeviceBuffer(*other->device<DeviceBuffer>());
  buf->owned = false;
  device_ = buf;
  requested_size_ = other->RequestedSize();
  allocated_size_ = other->AllocatedSize();
}

void Tensor::Rebind(void* ptr, size_t outer_count, size_t outer_stride) {
  CHECK(mem_type_ != HOST_MEMORY && device_ != nullptr) << "only device tensors can be rebound";
  DeviceBuffer* buf = device<DeviceBuffer>();
  if (buf->owned && buf->ptr != nullptr) (void)hipFree(buf->ptr);
  buf->ptr = ptr;
  buf->owned = false;
  const bool apart = outer_count > 1 && outer_stride * outer_count != num_elements() * sizeof(float);
  buf->outer_count = apart ? outer_count : 1;
  buf->outer_stride = apart ? outer_stride : 0;
}

Tensor::~Tensor() {
  if (host_ != nullptr) std::free(host_);
  if (device_ != nullptr) {
    DeviceBuffer* buf = device<DeviceBuffer>();
    if (buf->owned && buf->ptr != nullptr) (void)hipFree(buf->ptr);
    delete buf;
  }
}

Tensor* Tensor::Empty(DataType dtype, IntList shape, DataFormat dformat) {
  return new Tensor(dtype, shape, HOST_MEMORY, dformat);
}

Tensor* Tensor::Random(DataType dtype, IntList shape, DataFormat dformat) {
  Tensor* t = Empty(dtype, shape, dformat);
  CHECK_EQ(dtype, DT_FLOAT);
  CHECK_EQ(t->AllocatedSize(), t->RequestedSize()) << "Random fills dense host tensors only";
  float* p = t->host<float>();
  // Uniform in [0, 1) from libc random(), as tensor.cc:105-114 of the reference.
  for (size_t i = 0; i < t->num_elements(); ++i)
    p[i] = static_cast<float>(random()) / static_cast<float>(RAND_MAX);
  t->initialized_ = true;
  return t;
}

Tensor* Tensor::Ones(DataType dtype, IntList shape, DataFormat dformat) {
  Tensor* t = Empty(dtype, shape, dformat);
  CHECK_EQ(dtype, DT_FLOAT);
  CHECK_EQ(t->AllocatedSize(), t->RequestedSize()) << "Ones fills dense host tensors only";
  float* p = t->host<float>();
  for (size_t i = 0; i < t->num_elements(); ++i) p[i] = 1.0f;
  t->initialized_ = true;
  return t;
}

Tensor* Tensor::Zeros(DataType dtype, IntList shape, DataFormat dformat) {
  Tensor* t = Empty(dtype, shape, dformat);
  std::memset(t->host(), 0, t->AllocatedSize());
  t->initialized_ = true;
  return t;
}

namespace {
void CheckImage(const Tensor* t) {
  CHECK(t->dformat() != dlxnet::TensorProto::ANY && t->dformat() != dlxnet::TensorProto::ANY4)
      << "image accessor on a general tensor";
}
bool ChannelLast(DataFormat f) {
  return f == dlxnet::TensorProto::NHWC || f == dlxnet::TensorProto::NHWC4;
}
}  // namespace

int Tensor::channel() const {
  CheckImage(this);
  const int r = dims_size();
  if (ChannelLast(dformat_)) return shape_[r - 1];
  return r >= 3 ? shape_[r - 3] : 1;
}
int Tensor::width() const {
  CheckImage(this);
  const int r = dims_size();
  if (ChannelLast(dformat_)) return r >= 2 ? shape_[r - 2] : 1;
  return shape_[r - 1];
}
int Tensor::height() const {
  CheckImage(this);
  const int r = dims_size();
  if (ChannelLast(dformat_)) return r >= 3 ? shape_[r - 3] : 1;
  return r >= 2 ? shape_[r - 2] : 1;
}
int Tensor::num() const {
  CheckImage(this);
  const int r = dims_size();
  return r >= 4 ? shape_[r - 4] : 1;
}

std::string Tensor::ShortDebugString() const {
  std::ostringstream ss;
  ss << "Tensor(" << FormatToStr(dformat_) << ", [";
  for (size_t i = 0; i < shape_.size(); ++i) ss << (i ? ", " : "") << shape_[i];
  ss << "], " << (mem_type_ == HOST_MEMORY ? "host" : "device") << ")";
  return ss.str();
}

std::string Tensor::DebugString() const {
  std::ostringstream ss;
  ss << ShortDebugString();
  if (is_host() && dtype_ == DT_FLOAT) {
    ss << " values:";
    const size_t n = num_elements() < 16 ? num_elements() : 16;
    for (size_t i = 0; i < n; ++i) ss << " " << host<float>()[i];
    if (n < num_elements()) ss << " ...";
  }
  return ss.str();
}

size_t HostElements(const IntList& shape, DataFormat dformat) {
  size_t n = 1;
  for (int d : shape) n *= static_cast<size_t>(d);
  const auto up4 = [](size_t v) { return (v + 3) / 4 * 4; };
  switch (dformat) {
    case dlxnet::TensorProto::ANY4: {
      if (shape.empty() || shape.back() == 0) return n;
      const size_t last = static_cast<size_t>(shape.back());
      return n / last * up4(last);
    }
    case dlxnet::TensorProto::NHWC4:
      CHECK_EQ(shape.size(), 4u) << "NHWC4 needs a rank-4 shape";
      return static_cast<size_t>(shape[0]) * shape[1] * shape[2] * up4(shape[3]);
    case dlxnet::TensorProto::HWN4C4:
      CHECK_EQ(shape.size(), 4u) << "HWN4C4 needs an OIHW shape";
      return static_cast<size_t>(shape[2]) * shape[3] * ((shape[0] + 3) / 4) * up4(shape[1]) * 4;
    default:
      return n;
  }
}

DataFormat StrToFormat(const std::string& s) {
  if (s == "NHWC") return dlxnet::TensorProto::NHWC;
  if (s == "NCHW") return dlxnet::TensorProto::NCHW;
  if (s == "ANY") return dlxnet::TensorProto::ANY;
  if (s == "NHWC4") return dlxnet::TensorProto::NHWC4;
  if (s == "HWN4C4") return dlxnet::TensorProto::HWN4C4;
  if (s == "ANY4") return dlxnet::TensorProto::ANY4;
  LOG(FATAL) << "unsupported dformat string: " << s;
  return dlxnet::TensorProto::ANY;
}

std::string FormatToStr(DataFormat f) { return dlxnet::DataFormatName(f); }

DataFormat FormatToStride4(DataFormat f) {
  switch (f) {
    case dlxnet::TensorProto::NHWC:
    case dlxnet::TensorProto::NHWC4: return dlxnet::TensorProto::NHWC4;
    case dlxnet::TensorProto::ANY:
    case dlxnet::TensorProto::ANY4: return dlxnet::TensorProto::ANY4;
    case dlxnet::TensorProto::NCHW:
    case dlxnet::TensorProto::HWN4C4: return dlxnet::TensorProto::HWN4C4;
  }
  LOG(FATAL) << "unsupported dformat: " << f;
  return f;
}

}  // namespace opengl
