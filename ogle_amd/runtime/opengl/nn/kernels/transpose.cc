#include "opengl/nn/kernels/transpose.h"

#include "ogle_hip.h"
#include "opengl/core/context.h"
#include "opengl/core/fbo_session.h"
#include "opengl/core/kernel_registry.h"
#include "opengl/core/program.h"
#include "opengl/core/tensor.h"

namespace opengl {

void TransposeKernel::SetupAttr(const dlxnet::Attribute& attr) {
  for (auto item : attr.transpose_attr().perm()) perm_.push_back(item);
}

void TransposeKernel::SelectKernel(const TensorList& inputs) {
  if (inputs[0]->dformat() == dlxnet::TensorProto::ANY4) {
    kernel_fname_ = "transpose_any4";
  } else {
    CHECK_EQ(inputs[0]->dformat(), dlxnet::TensorProto::NHWC4);
    kernel_fname_ = "transpose";
  }
  output_tensor_dformats_.emplace_back(dlxnet::TensorProto::ANY4);
  // An ONNX graph states the permutation over NCHW axes; an image tensor is held as
  // NHWC, so each axis is renamed through {0,3,1,2} (transpose.cc:44-54).
  if (session_->IsONNX() && inputs[0]->dformat() == dlxnet::TensorProto::NHWC4) {
    CHECK_EQ(perm_.size(), 4u);
    const int mapping[4] = {0, 3, 1, 2};
    for (int& p : perm_) {
      CHECK(p >= 0 && p < 4) << "transpose perm out of range";
      p = mapping[p];
    }
  }
  CHECK_LE(perm_.size(), 4u);
  CHECK_LE(inputs[0]->shape().size(), 4u);
  // With dense row-major buffers a permutation that keeps the order of all
  // non-unit dimensions leaves every element where it is.
  const IntList& shape = inputs[0]->shape();
  moves_no_data_ = true;
  int last = -1;
  for (size_t d = 0; d < perm_.size(); ++d) {
    CHECK(perm_[d] >= 0 && perm_[d] < static_cast<int>(shape.size())) << "transpose perm out of range";
    if (shape[perm_[d]] == 1) continue;
    if (perm_[d] < last) moves_no_data_ = false;
    last = perm_[d];
  }
}

int TransposeKernel::OutputAliasesInput(int) const { return moves_no_data_ ? 0 : -1; }

void TransposeKernel::InferOutputShape(TensorShapeList& input_shapes, TensorShapeList& output_shapes) {
  CHECK_EQ(input_shapes.size(), 1u);
  output_shapes.clear();
  output_shapes.resize(1);
  const IntList& in = input_shapes[0];
  IntList& out = output_shapes[0];
  for (int p : perm_) out.push_back(in[p]);
  for (size_t i = perm_.size(); i < in.size(); ++i) out.push_back(in[i]);  // transpose.cc:101-103
}

void TransposeKernel::Compute(TensorList& inputs, TensorList& outputs) {
  if (moves_no_data_) return;  // the output is a view of the input
  program_->Activate();
  const IntList& in = inputs[0]->shape();
  const int rank = static_cast<int>(in.size());
  const int lead = 4 - rank;
  OgleTransposeArgs a{};
  a.input_dev = inputs[0]->device_ptr();
  a.output_dev = outputs[0]->device_ptr();
  for (int d = 0; d < 4; ++d) {
    a.in_shape[d] = d < lead ? 1 : in[d - lead];
    a.perm[d] = d;
  }
  for (size_t d = 0; d < perm_.size(); ++d) a.perm[lead + d] = perm_[d] + lead;
  a.dtype = OGLE_F32;
  program_->RunTranspose(a);
}

REGISTER_KERNEL_WITH_NAME(TransposeKernel, "Transpose");

}  // namespace opengl
