#include "opengl/nn/kernels/reshape.h"

#include <memory>

#include "opengl/core/context.h"
#include "opengl/core/fbo_session.h"
#include "opengl/core/kernel_registry.h"
#include "opengl/core/tensor.h"

namespace opengl {

void ReshapeKernel::SetupAttr(const dlxnet::Attribute&) {}

void ReshapeKernel::SelectKernel(const TensorList& inputs) {
  if (inputs[0]->dformat() == dlxnet::TensorProto::ANY4) {
    kernel_fname_ = "reshape_any4";
  } else {
    CHECK_EQ(inputs[0]->dformat(), dlxnet::TensorProto::NHWC4);
    kernel_fname_ = "reshape";
  }
  output_tensor_dformats_.emplace_back(dlxnet::TensorProto::ANY4);
}

// The target shape is the VALUE of the second input, read back from the device;
// 0 copies the input's dimension, one -1 takes what is left (reshape.cc:53-90).
void ReshapeKernel::InferOutputShape(const TensorList& inputs, TensorShapeList& output_shapes) {
  output_shapes.clear();
  output_shapes.resize(1);
  CHECK_EQ(inputs.size(), 2u);
  const Tensor* shape_tensor = inputs[1];
  IntList& output_shape = output_shapes[0];
  std::unique_ptr<Tensor> host(new Tensor(Tensor::DT_FLOAT, shape_tensor->shape(),
                                          Tensor::HOST_MEMORY, dlxnet::TensorProto::ANY));
  session_->context()->CopyDeviceTensorToCPU(shape_tensor, host.get());
  for (size_t i = 0; i < host->num_elements(); ++i)
    output_shape.push_back(static_cast<int>(host->host<float>()[i]));

  const IntList& input_shape = inputs[0]->shape();
  const long num_elements = static_cast<long>(inputs[0]->num_elements());
  long known = 1;
  for (size_t i = 0; i < output_shape.size(); ++i) {
    if (output_shape[i] == 0) {
      CHECK_LT(i, input_shape.size()) << "reshape: 0 refers to a missing input dimension";
      output_shape[i] = input_shape[i];
    }
    if (output_shape[i] != -1) known *= output_shape[i];
  }
  bool inferred = false;
  for (int& d : output_shape) {
    if (d != -1) continue;
    CHECK(!inferred) << "reshape: more than one -1";
    CHECK_GT(known, 0);
    d = static_cast<int>(num_elements / known);
    inferred = true;
  }
  long total = 1;
  for (int d : output_shape) total *= d;
  CHECK_EQ(total, num_elements) << "reshape: element count changes";
  CHECK_EQ(target_shape_.size(), 0u);
  target_shape_ = output_shape;
}

void ReshapeKernel::Compute(TensorList&, TensorList&) {}

REGISTER_KERNEL_WITH_NAME(ReshapeKernel, "Reshape");

}  // namespace opengl
