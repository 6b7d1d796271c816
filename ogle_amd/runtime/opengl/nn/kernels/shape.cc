#include "opengl/nn/kernels/shape.h"

#include "opengl/core/context.h"
#include "opengl/core/kernel_registry.h"

namespace opengl {

// ---- Shape -----------------------------------------------------------------

void ShapeKernel::InferOutputShape(TensorShapeList& input_shapes, TensorShapeList& output_shapes) {
  output_tensor_dformats_.emplace_back(dlxnet::TensorProto::ANY4);
  output_shapes.clear();
  output_shapes.resize(1);
  CHECK_EQ(input_shapes.size(), 1u);
  const int rank = static_cast<int>(input_shapes[0].size());
  output_shapes[0] = {rank};
  values_.reset(new Tensor(Tensor::DT_FLOAT, output_shapes[0], Tensor::HOST_MEMORY,
                           dlxnet::TensorProto::ANY));
  for (int i = 0; i < rank; ++i) values_->host<float>()[i] = static_cast<float>(input_shapes[0][i]);
}

void ShapeKernel::Compute(TensorList& inputs, TensorList& outputs) {
  CHECK_EQ(inputs.size(), 1u);
  CHECK(values_ != nullptr) << "InferOutputShape first";
  context_->CopyCPUTensorToDevice(values_.get(), outputs[0]);
}

// ---- Gather ----------------------------------------------------------------

void GatherKernel::SetupAttr(const dlxnet::Attribute& attr) { axis_ = attr.gather_attr().axis(); }

void GatherKernel::InferOutputShape(TensorShapeList& input_shapes, TensorShapeList& output_shapes) {
  output_tensor_dformats_.emplace_back(dlxnet::TensorProto::ANY4);
  output_shapes.clear();
  output_shapes.resize(1);
  CHECK_EQ(input_shapes.size(), 2u);
  output_shapes[0] = input_shapes[1];  // a scalar index gives a scalar
}

void GatherKernel::Compute(TensorList& inputs, TensorList& outputs) {
  CHECK_EQ(inputs.size(), 2u);
  const Tensor* data = inputs[0];
  const Tensor* index = inputs[1];
  CHECK_EQ(index->num_elements(), 1u) << "Gather: only a single index is supported";
  CHECK(data->num_elements() >= 1 && data->num_elements() <= 4)
      << "Gather: the input must be a shape vector of at most 4 entries";
  Tensor data_host(Tensor::DT_FLOAT, data->shape(), Tensor::HOST_MEMORY, dlxnet::TensorProto::ANY);
  Tensor index_host(Tensor::DT_FLOAT, index->shape(), Tensor::HOST_MEMORY, dlxnet::TensorProto::ANY);
  context_->CopyDeviceTensorToCPU(data, &data_host);
  context_->CopyDeviceTensorToCPU(index, &index_host);
  // the four lanes of the first texel, missing entries reading as zero
  float lanes[4] = {0.f, 0.f, 0.f, 0.f};
  for (size_t i = 0; i < data->num_elements(); ++i) lanes[i] = data_host.host<float>()[i];
  const int selected = static_cast<int>(index_host.host<float>()[0]);
  // NCHW position -> NHWC lane; anything else falls through to lane z as the shader does
  const float value = selected == 0 ? lanes[0] : selected == 1 ? lanes[3] : selected == 2 ? lanes[1]
                                                                                          : lanes[2];
  Tensor out_host(Tensor::DT_FLOAT, outputs[0]->shape(), Tensor::HOST_MEMORY,
                  dlxnet::TensorProto::ANY);
  CHECK_EQ(out_host.num_elements(), 1u);
  out_host.host<float>()[0] = value;
  context_->CopyCPUTensorToDevice(&out_host, outputs[0]);
}

// ---- Unsqueeze -------------------------------------------------------------

void UnsqueezeKernel::SetupAttr(const dlxnet::Attribute& attr) {
  for (auto a : attr.unsqueeze_attr().axes()) axes_.push_back(static_cast<int>(a));
  CHECK_EQ(axes_.size(), 1u) << "Unsqueeze: one axis, as torch.unsqueeze";
}

void UnsqueezeKernel::InferOutputShape(TensorShapeList& input_shapes, TensorShapeList& output_shapes) {
  output_tensor_dformats_.emplace_back(dlxnet::TensorProto::ANY4);
  output_shapes.clear();
  output_shapes.resize(1);
  CHECK_EQ(input_shapes.size(), 1u);
  output_shapes[0] = input_shapes[0];
  CHECK(axes_[0] >= 0 && axes_[0] <= static_cast<int>(input_shapes[0].size()))
      << "Unsqueeze: axis " << axes_[0] << " out of range";
  output_shapes[0].insert(output_shapes[0].begin() + axes_[0], 1);
}

REGISTER_KERNEL_WITH_NAME(ShapeKernel, "Shape");
REGISTER_KERNEL_WITH_NAME(GatherKernel, "Gather");
REGISTER_KERNEL_WITH_NAME(UnsqueezeKernel, "Unsqueeze");

}  // namespace opengl
