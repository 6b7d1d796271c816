#include "opengl/nn/kernels/decoder.h"

#include "ogle_hip.h"
#include "opengl/core/context.h"
#include "opengl/core/kernel_registry.h"
#include "opengl/core/program.h"
#include "opengl/core/tensor.h"

namespace opengl {

DecoderKernel::DecoderKernel(Context* context)
    : Kernel(context), score_threshold_(0.3f), nms_threshold_(0.45f),
      variances_({0.1f, 0.1f, 0.2f, 0.2f}) {}  // decoder.cc:13-18

void DecoderKernel::SetupAttr(const dlxnet::Attribute&) {}

void DecoderKernel::SelectKernel(const TensorList& inputs) {
  CHECK_EQ(inputs.size(), 2u);
  CHECK_EQ(inputs[0]->dformat(), dlxnet::TensorProto::ANY4);
  kernel_fname_ = "decoder";
  output_tensor_dformats_.emplace_back(dlxnet::TensorProto::ANY4);
}

void DecoderKernel::InferOutputShape(const TensorList& input_tensors, TensorShapeList& output_shapes) {
  CHECK_GE(input_tensors.size(), 2u);
  const Tensor* prediction = input_tensors[0];
  const Tensor* anchors = input_tensors[1];
  CHECK_EQ(prediction->shape().size(), 3u);
  CHECK_EQ(prediction->shape()[2], 4);
  const int num_batches = prediction->shape()[0];
  const int num_samples = prediction->shape()[1];
  // Anchors come as (N, H, W, 4) with H*W == priors (decoder.cc:76-85).
  const IntList& as = anchors->shape();
  CHECK_EQ(as.size(), 4u);
  CHECK_EQ(as[0], num_batches);
  CHECK_EQ(as[1] * as[2], num_samples);
  CHECK_EQ(as[3], 4);
  output_shapes.clear();
  output_shapes.resize(1);
  output_shapes[0] = {num_batches, num_samples, 4};
}

void DecoderKernel::Compute(TensorList& inputs, TensorList& outputs) {
  program_->Activate();
  OgleDecodeArgs a{};
  a.prediction_dev = static_cast<const float*>(inputs[0]->device_ptr());
  a.anchors_dev = static_cast<const float*>(inputs[1]->device_ptr());
  a.boxes_dev = static_cast<float*>(outputs[0]->device_ptr());
  a.batch = inputs[0]->shape()[0];
  a.priors = inputs[0]->shape()[1];
  a.anchors_batch_stride = static_cast<int64_t>(a.priors) * 4;
  for (int i = 0; i < 4; ++i) a.variances[i] = variances_[i];
  program_->RunDecode(a);
}

REGISTER_KERNEL_WITH_NAME(DecoderKernel, "Decoder");

}  // namespace opengl
