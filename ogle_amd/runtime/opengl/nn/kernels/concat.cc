#include "opengl/nn/kernels/concat.h"

#include "ogle_hip.h"
#include "opengl/core/context.h"
#include "opengl/core/fbo_session.h"
#include "opengl/core/kernel_registry.h"
#include "opengl/core/program.h"
#include "opengl/core/tensor.h"

namespace opengl {

void ConcatKernel::SetupAttr(const dlxnet::Attribute& attr) { axis_ = attr.concat_attr().axis(); }

void ConcatKernel::SelectKernel(const TensorList& inputs) {
  // Only general (ANY4) tensors are concatenated (concat.cc:33).
  CHECK_EQ(inputs[0]->dformat(), dlxnet::TensorProto::ANY4);
  kernel_fname_ = "concat_multi";
  output_tensor_dformats_.emplace_back(dlxnet::TensorProto::ANY4);
}

void ConcatKernel::InferOutputShape(const TensorList& input_tensors, TensorShapeList& output_shapes) {
  CHECK_GE(input_tensors.size(), 2u);
  CHECK_LE(input_tensors.size(), static_cast<size_t>(OGLE_CONCAT_MAX_INPUTS));
  const int rank = static_cast<int>(input_tensors[0]->shape().size());
  if (axis_ == -1) axis_ = rank - 1;  // concat.cc:105-107
  CHECK(axis_ >= 0 && axis_ < rank) << "concat axis " << axis_ << " outside rank " << rank;
  output_shapes.clear();
  output_shapes.resize(1);
  output_shapes[0] = input_tensors[0]->shape();
  output_shapes[0][axis_] = 0;
  for (const Tensor* t : input_tensors) {
    const IntList& s = t->shape();
    CHECK_EQ(output_shapes[0].size(), s.size());
    for (int i = 0; i < rank; ++i) {
      if (i != axis_) {
        CHECK_EQ(s[i], output_shapes[0][i]);  // concat.cc:116-121
      } else {
        output_shapes[0][i] += s[i];
      }
    }
  }
}

// The output is outer (product of the dimensions before the axis) slices, each the
// inputs' slices back to back.
Kernel::Placement ConcatKernel::InputPlacementInOutput() const {
  Placement pl;
  if (input_tensors_.empty() || output_tensors_.empty()) return pl;
  const IntList& out = output_tensors_[0]->shape();
  size_t outer = 1, inner = sizeof(float);
  for (int d = 0; d < axis_; ++d) outer *= out[d];
  for (size_t d = axis_ + 1; d < out.size(); ++d) inner *= out[d];
  if (outer == 0) return pl;
  size_t at = 0;
  for (const Tensor* t : input_tensors_) {
    pl.offsets.push_back(at);
    at += static_cast<size_t>(t->shape()[axis_]) * inner;
  }
  pl.outer_count = outer;
  pl.outer_stride = outer > 1 ? at : 0;
  return pl;
}

void ConcatKernel::Compute(TensorList& inputs, TensorList& outputs) {
  if (inputs_in_place()) return;  // every producer wrote straight into the output
  program_->Activate();
  const IntList& out = outputs[0]->shape();
  OgleConcatArgs a{};
  a.n_inputs = static_cast<int32_t>(inputs.size());
  a.outer = 1;
  a.inner = 1;
  for (int d = 0; d < axis_; ++d) a.outer *= out[d];
  for (size_t d = axis_ + 1; d < out.size(); ++d) a.inner *= out[d];
  for (size_t i = 0; i < inputs.size(); ++i) {
    a.inputs_dev[i] = inputs[i]->device_ptr();
    a.axis_len[i] = inputs[i]->shape()[axis_];
  }
  a.output_dev = outputs[0]->device_ptr();
  a.dtype = OGLE_F32;
  program_->RunConcat(a);  // one launch for all inputs (the reference draws once per input)
}

REGISTER_KERNEL_WITH_NAME(ConcatKernel, "Concat");

}  // namespace opengl
