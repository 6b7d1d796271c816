#include "opengl/nn/kernels/const.h"

#include "opengl/core/context.h"
#include "opengl/core/kernel_registry.h"

namespace opengl {

void ConstKernel::SetupAttr(const dlxnet::Attribute& attr) {
  const dlxnet::TensorProto& value = attr.const_attr().value();
  CHECK(!tensor_) << "constant set twice";
  tensor_.reset(new Tensor(value));
  output_tensor_dformats_.emplace_back(value.target_data_format());
}

// Only general tensors (ANY4) and filters (HWN4C4) are valid targets (const.cc:39-58).
// The device copy keeps the file's element order; for a filter that is OIHW, which
// the convolution repacks once for the kernel variant it selected.
void ConstKernel::InferOutputShape(TensorShapeList& inputs, TensorShapeList& outputs) {
  CHECK(inputs.empty()) << "Input should be empty in ConstKernel";
  CHECK_EQ(output_tensor_dformats_.size(), 1u);
  const DataFormat dformat = output_tensor_dformats_[0];
  if (dformat != dlxnet::TensorProto::ANY4 && dformat != dlxnet::TensorProto::HWN4C4)
    LOG(FATAL) << "unsupported dformat " << FormatToStr(dformat) << " in Const Kernel";
  if (dformat == dlxnet::TensorProto::HWN4C4) CHECK_EQ(tensor_->shape().size(), 4u);
  outputs.clear();
  outputs.emplace_back(tensor_->shape());
}

void ConstKernel::Compute(TensorList& inputs, TensorList& outputs) {
  CHECK(inputs.empty()) << "Input should be empty in ConstKernel";
  context_->CopyCPUTensorToDevice(tensor_.get(), outputs[0]);
}

REGISTER_KERNEL_WITH_NAME(ConstKernel, "Const");
REGISTER_KERNEL_WITH_NAME(ConstKernel, "Constant");

}  // namespace opengl
