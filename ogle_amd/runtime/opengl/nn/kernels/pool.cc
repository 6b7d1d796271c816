#include "opengl/nn/kernels/pool.h"

#include "ogle_hip.h"
#include "opengl/core/context.h"
#include "opengl/core/kernel_registry.h"
#include "opengl/core/program.h"
#include "opengl/core/tensor.h"

namespace opengl {

template <PoolType pool_type>
void PoolKernel<pool_type>::SelectKernel(const TensorList& inputs) {
  // The reference names a shader *file path* here, which its program loader cannot
  // compile (pool.cc:18-20); the registry stems are used instead.
  kernel_fname_ = inputs[0]->dformat() == dlxnet::TensorProto::ANY4 ? "pool_any4" : "pool";
  output_tensor_dformats_.emplace_back(inputs[0]->dformat());
}

// pool.cc:27-51: AveragePool also reads maxpool_attr; GlobalAveragePool has no attrs.
template <PoolType pool_type>
void PoolKernel<pool_type>::SetupAttr(const dlxnet::Attribute& attr) {
  if (pool_type_ == GlobalAveragePool) return;
  const dlxnet::MaxPoolAttribute& p = attr.maxpool_attr();
  CHECK_EQ(p.pads_size(), 4);
  for (auto pad : p.pads()) CHECK_EQ(p.pads(0), pad);
  padding_ = static_cast<int>(p.pads(0));
  CHECK_EQ(p.strides_size(), 2);
  CHECK_EQ(p.strides(0), p.strides(1));
  stride_ = static_cast<int>(p.strides(0));
  CHECK_EQ(p.kernel_shape_size(), 2);
  CHECK_EQ(p.kernel_shape(0), p.kernel_shape(1));
  kernel_size_ = static_cast<int>(p.kernel_shape(0));
}

template <PoolType pool_type>
void PoolKernel<pool_type>::InferOutputShape(TensorShapeList& input_shapes,
                                             TensorShapeList& output_shapes) {
  CHECK_EQ(input_shapes.size(), 1u);
  output_shapes.clear();
  output_shapes.resize(1);
  const IntList& image_shape = input_shapes[0];
  CHECK_EQ(image_shape.size(), 4u);
  if (pool_type_ == GlobalAveragePool) {
    // The window is the whole (square) image (pool.cc:84-91).
    CHECK_EQ(image_shape[1], image_shape[2]);
    stride_ = 1;
    kernel_size_ = image_shape[1];
    padding_ = 0;
    output_shapes[0] = {image_shape[0], 1, 1, image_shape[3]};
  } else {
    const int output_height = (image_shape[1] - kernel_size_ + 2 * padding_) / stride_ + 1;
    const int output_width = (image_shape[2] - kernel_size_ + 2 * padding_) / stride_ + 1;
    output_shapes[0] = {image_shape[0], output_height, output_width, image_shape[3]};
  }
}

template <PoolType pool_type>
void PoolKernel<pool_type>::Compute(TensorList& inputs, TensorList& outputs) {
  program_->Activate();
  const IntList& in = inputs[0]->shape();
  const IntList& out = outputs[0]->shape();
  OglePoolArgs a{};
  a.input_dev = inputs[0]->device_ptr();
  a.output_dev = outputs[0]->device_ptr();
  a.n = in[0]; a.in_h = in[1]; a.in_w = in[2]; a.c = in[3];
  a.out_h = out[1]; a.out_w = out[2];
  a.kernel_size = kernel_size_; a.stride = stride_; a.padding = padding_;
  a.pool_type = pool_type_;
  a.dtype = OGLE_F32;
  program_->RunPool(a);
}

template class PoolKernel<MaxPool>;
template class PoolKernel<AveragePool>;
template class PoolKernel<GlobalAveragePool>;

REGISTER_KERNEL_WITH_NAME(PoolKernel<MaxPool>, "MaxPool");
REGISTER_KERNEL_WITH_NAME(PoolKernel<AveragePool>, "AveragePool");
REGISTER_KERNEL_WITH_NAME(PoolKernel<GlobalAveragePool>, "GlobalAveragePool");

}  // namespace opengl
