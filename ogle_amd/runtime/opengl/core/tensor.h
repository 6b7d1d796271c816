// Host / device tensor of the runtime.
//
// Keeps the reference's logical model (ogl_runtime/opengl/core/tensor.h:72-280):
// shape() is always the logical shape (NHWC activations, OIHW filters), dformat()
// tags the layout family, a tensor lives either on the host or on the device.
// What changes is the device side: instead of an RGBA32F texture whose width is
// padded to 4 channels, a device tensor is a DeviceBuffer: a linear, dense,
// row-major HBM allocation in logical-shape order.  The stride-4 tags NHWC4 /
// ANY4 / HWN4C4 are kept as tags only (kernels and the executor select on them as
// the reference does); they imply no padding here.
#ifndef OPENGL_CORE_TENSOR_H_
#define OPENGL_CORE_TENSOR_H_

#include <string>

#include "opengl/core/types.h"
#include "opengl/utils/logging.h"

namespace opengl {

// Linear device allocation; replaces Texture (ogl_runtime/opengl/core/texture.h:10-31).
struct DeviceBuffer {
  void* ptr = nullptr;
  size_t bytes = 0;
  bool owned = true;  // false for a view that aliases another tensor's buffer
  // Dense unless outer_count > 1: then the tensor's elements are outer_count equal runs
  // (one per index of the first dimension) whose starts lie outer_stride bytes apart,
  // i.e. the tensor sits inside a larger one (a convolution output produced in its place
  // inside a concatenation's output).
  size_t outer_count = 1;
  size_t outer_stride = 0;
};

class Tensor {
 public:
  enum DataType { DT_INT = 0, DT_FLOAT = 1, DT_DOUBLE = 2, DT_INVALID };
  enum MemoryType { HOST_MEMORY = 0, DEVICE_TEXTURE, DEVICE_BUFFER };

  // Allocates an uninitialised tensor on the host or the device.
  Tensor(DataType dtype, IntList shape, MemoryType mem_type = HOST_MEMORY,
         DataFormat dformat = dlxnet::TensorProto::NHWC);
  // Host tensor holding a copy of `data` (num_elements values).
  template <typename T>
  Tensor(DataType dtype, IntList shape, const T* data,
         DataFormat dformat = dlxnet::TensorProto::NHWC)
      : Tensor(dtype, shape, HOST_MEMORY, dformat) {
    std::memcpy(host_, data, allocated_size_);  // `data` is in `dformat`'s host layout
    initialized_ = true;
  }
  // Host tensor from a model constant (float_data, int32_data or int64_data are all
  // stored as floats, as the converter does; tensor.cc:41-90 of the reference).
  explicit Tensor(const dlxnet::TensorProto& proto);
  // Device tensor that aliases `other`'s buffer under a new shape / tag.
  Tensor(const Tensor* other, IntList shape, DataFormat dformat);
  ~Tensor();
  Tensor(const Tensor&) = delete;
  Tensor& operator=(const Tensor&) = delete;

  static Tensor* Random(DataType dtype, IntList shape,
                        DataFormat dformat = dlxnet::TensorProto::NHWC);
  static Tensor* Empty(DataType dtype, IntList shape,
                       DataFormat dformat = dlxnet::TensorProto::NHWC);
  static Tensor* Ones(DataType dtype, IntList shape,
                      DataFormat dformat = dlxnet::TensorProto::NHWC);
  static Tensor* Zeros(DataType dtype, IntList shape,
                       DataFormat dformat = dlxnet::TensorProto::NHWC);

  void* device() const { return device_; }
  void* host() const { return host_; }
  template <typename T>
  T* device() const { return reinterpret_cast<T*>(device_); }
  template <typename T>
  T* host() const { return reinterpret_cast<T*>(host_); }
  // Raw device address of the first element.
  void* device_ptr() const { return device_ ? device<DeviceBuffer>()->ptr : nullptr; }
  // True when this tensor's device memory is its own allocation (not a view).
  bool owns_device_buffer() const { return device_ != nullptr && device<DeviceBuffer>()->owned; }
  // Makes this device tensor a view of memory owned elsewhere, starting at `ptr`
  // (its own allocation, if any, is released).  The contents are not moved.  With
  // outer_count > 1 the view is that many equal runs, outer_stride bytes apart.
  void Rebind(void* ptr, size_t outer_count = 1, size_t outer_stride = 0);
  // 0 for a dense tensor, else the distance between the runs (see DeviceBuffer).
  size_t outer_stride_bytes() const {
    return device_ && device<DeviceBuffer>()->outer_count > 1 ? device<DeviceBuffer>()->outer_stride : 0;
  }
  size_t outer_count() const { return device_ ? device<DeviceBuffer>()->outer_count : 1; }

  const IntList& shape() const { return shape_; }
  size_t num_elements() const;
  DataType dtype() const { return dtype_; }
  MemoryType mem_type() const { return mem_type_; }
  int dims_size() const { return static_cast<int>(shape_.size()); }
  DataFormat dformat() const { return dformat_; }
  void set_dformat(DataFormat f) { dformat_ = f; }
  bool is_host() const { return host_ != nullptr; }
  bool Initialized() const { return initialized_; }
  void set_initialized(bool v) { initialized_ = v; }
  int last_stride() const { return shape_.empty() ? 1 : shape_.back(); }
  uint64 AllocatedSize() const { return allocated_size_; }
  uint64 AllocatedElements() const { return allocated_size_ / sizeof(float); }
  uint64 RequestedSize() const { return requested_size_; }

  // Image accessors (tensor.h:171-229 of the reference).
  int num() const;
  int height() const;
  int width() const;
  int channel() const;

  std::string DebugString() const;
  std::string ShortDebugString() const;

 private:
  void* device_ = nullptr;  // DeviceBuffer*
  void* host_ = nullptr;
  bool initialized_ = false;
  uint64 allocated_size_ = 0;
  uint64 requested_size_ = 0;
  DataType dtype_;
  MemoryType mem_type_;
  IntList shape_;
  DataFormat dformat_;
};

// Elements (floats) a HOST tensor of this shape and tag occupies.  Dense for NHWC, NCHW
// and ANY; for the stride-4 tags the reference's padded texture layouts
// (ogl_runtime/opengl/core/tensor_format.cc:251-298): NHWC4 pads the channels of every
// pixel to a multiple of 4, ANY4 the last dimension, HWN4C4 (OIHW filters) is
// kh*kw*ceil(O/4) rows of ceil(I/4)*4 texels of 4 output channels.  The reference
// further rounds sizes above GL_MAX_TEXTURE_SIZE*4 elements up to whole texture rows;
// there is no texture here, so that rounding is not applied.
size_t HostElements(const IntList& shape, DataFormat dformat);

// "NHWC", "NCHW", "ANY", "NHWC4", "HWN4C4", "ANY4" <-> DataFormat
// (ogl_runtime/opengl/core/tensor_format.cc:136-152).
DataFormat StrToFormat(const std::string& s);
std::string FormatToStr(DataFormat f);
// NHWC -> NHWC4, ANY -> ANY4, NCHW -> HWN4C4 (tensor_format.cc FormatToStride4).
DataFormat FormatToStride4(DataFormat f);

}  // namespace opengl

#endif  // OPENGL_CORE_TENSOR_H_
