#include "opengl/nn/kernels/eltwise.h"

#include "ogle_hip.h"
#include "opengl/core/context.h"
#include "opengl/core/fbo_session.h"
#include "opengl/core/kernel_registry.h"
#include "opengl/core/program.h"
#include "opengl/core/tensor.h"

namespace opengl {

namespace {
void SameShapeOutput(TensorShapeList& input_shapes, TensorShapeList& output_shapes) {
  CHECK_GE(input_shapes.size(), 1u);
  output_shapes.clear();
  output_shapes.push_back(input_shapes[0]);
}
}  // namespace

// ---- Add -------------------------------------------------------------------

void BinaryKernel::SelectKernel(const TensorList& inputs) {
  kernel_fname_ = "binary";
  output_tensor_dformats_.emplace_back(inputs[0]->dformat());
}

void BinaryKernel::InferOutputShape(TensorShapeList& input_shapes, TensorShapeList& output_shapes) {
  CHECK_EQ(input_shapes.size(), 2u);
  // the shader adds texel by texel: the shapes have to agree (binary.cc leaves the
  // check as a comment)
  CHECK(input_shapes[0] == input_shapes[1]) << "Add: inputs of different shapes";
  SameShapeOutput(input_shapes, output_shapes);
}

void BinaryKernel::Compute(TensorList& inputs, TensorList& outputs) {
  program_->Activate();
  OgleBinaryArgs a{};
  a.a_dev = inputs[0]->device_ptr();
  a.b_dev = inputs[1]->device_ptr();
  a.output_dev = outputs[0]->device_ptr();
  a.count = static_cast<int64_t>(outputs[0]->num_elements());
  a.dtype = OGLE_F32;
  program_->RunAdd(a);
}

// ---- Relu / Clip -----------------------------------------------------------

void ReluKernel::SelectKernel(const TensorList& inputs) {
  kernel_fname_ = "relu";
  // relu.cc:17 tags the output NHWC4 whatever comes in; the tag of the input is kept
  // here, which is the same thing for the image tensors the op is used on
  output_tensor_dformats_.emplace_back(inputs[0]->dformat());
}

void ReluKernel::InferOutputShape(TensorShapeList& input_shapes, TensorShapeList& output_shapes) {
  CHECK_EQ(input_shapes.size(), 1u);
  SameShapeOutput(input_shapes, output_shapes);
}

void ReluKernel::Compute(TensorList& inputs, TensorList& outputs) {
  program_->Activate();
  OgleUnaryArgs a{};
  a.input_dev = inputs[0]->device_ptr();
  a.output_dev = outputs[0]->device_ptr();
  a.count = static_cast<int64_t>(outputs[0]->num_elements());
  a.op = OGLE_UNARY_RELU;
  a.dtype = OGLE_F32;
  program_->RunUnary(a);
}

void ClipKernel::SetupAttr(const dlxnet::Attribute& attr) {
  min_ = attr.clip_attr().min();
  max_ = attr.clip_attr().max();
}

void ClipKernel::SelectKernel(const TensorList& inputs) {
  kernel_fname_ = "clip";
  output_tensor_dformats_.emplace_back(inputs[0]->dformat());
}

void ClipKernel::InferOutputShape(TensorShapeList& input_shapes, TensorShapeList& output_shapes) {
  CHECK_EQ(input_shapes.size(), 1u);
  SameShapeOutput(input_shapes, output_shapes);
}

void ClipKernel::Compute(TensorList& inputs, TensorList& outputs) {
  program_->Activate();
  OgleUnaryArgs a{};
  a.input_dev = inputs[0]->device_ptr();
  a.output_dev = outputs[0]->device_ptr();
  a.count = static_cast<int64_t>(outputs[0]->num_elements());
  a.op = OGLE_UNARY_CLIP;
  a.min_value = min_;
  a.max_value = max_;
  a.dtype = OGLE_F32;
  program_->RunUnary(a);
}

// ---- BatchNormalization ----------------------------------------------------

void BatchNormKernel::SetupAttr(const dlxnet::Attribute& attr) {
  momentum_ = attr.batchnorm_attr().momentum();
  eps_ = attr.batchnorm_attr().epsilon();
}

void BatchNormKernel::SelectKernel(const TensorList& inputs) {
  kernel_fname_ = inputs[0]->dformat() == dlxnet::TensorProto::ANY4 ? "batchnorm_any4" : "batchnorm";
  output_tensor_dformats_.emplace_back(inputs[0]->dformat());
}

void BatchNormKernel::InferOutputShape(TensorShapeList& input_shapes, TensorShapeList& output_shapes) {
  CHECK_EQ(input_shapes.size(), 5u);
  CHECK_GE(input_shapes[0].size(), 1u);
  const size_t channels = static_cast<size_t>(input_shapes[0].back());
  for (int i = 1; i < 5; ++i) {
    size_t n = 1;
    for (int d : input_shapes[i]) n *= static_cast<size_t>(d);
    CHECK_EQ(n, channels) << "BatchNormalization: parameter " << i << " length";
  }
  SameShapeOutput(input_shapes, output_shapes);
}

void BatchNormKernel::Compute(TensorList& inputs, TensorList& outputs) {
  program_->Activate();
  OgleBatchNormArgs a{};
  a.input_dev = inputs[0]->device_ptr();
  a.gamma_dev = static_cast<const float*>(inputs[1]->device_ptr());
  a.beta_dev = static_cast<const float*>(inputs[2]->device_ptr());
  a.mean_dev = static_cast<const float*>(inputs[3]->device_ptr());
  a.var_dev = static_cast<const float*>(inputs[4]->device_ptr());
  a.output_dev = outputs[0]->device_ptr();
  a.channels = inputs[0]->shape().back();
  a.outer = static_cast<int64_t>(inputs[0]->num_elements() / static_cast<size_t>(a.channels));
  a.epsilon = eps_;
  a.dtype = OGLE_F32;
  program_->RunBatchNorm(a);
}

// ---- Gemm ------------------------------------------------------------------

void GemmKernel::SetupAttr(const dlxnet::Attribute& attr) {
  alpha_ = attr.gemm_attr().alpha();
  beta_ = attr.gemm_attr().beta();
  trans_b_ = attr.gemm_attr().transB();
  output_tensor_dformats_.emplace_back(dlxnet::TensorProto::ANY4);
}

// gemm.cc:62-98.
void GemmKernel::InferOutputShape(TensorShapeList& input_shapes, TensorShapeList& output_shapes) {
  CHECK_GE(input_shapes.size(), 2u);
  output_shapes.clear();
  output_shapes.resize(1);
  CHECK_EQ(input_shapes[0].size(), 2u);
  CHECK_EQ(input_shapes[1].size(), 2u);
  if (trans_b_) {
    CHECK_EQ(input_shapes[1][1], input_shapes[0][1]);
    output_shapes[0] = {input_shapes[0][0], input_shapes[1][0]};
  } else {
    CHECK_EQ(input_shapes[1][0], input_shapes[0][1]);
    output_shapes[0] = {input_shapes[0][0], input_shapes[1][1]};
  }
  if (input_shapes.size() > 2) {
    if (input_shapes[2].size() == 2) {
      CHECK_EQ(output_shapes[0][0], input_shapes[2][0]);
      CHECK_EQ(output_shapes[0][1], input_shapes[2][1]);
    } else {
      CHECK_EQ(input_shapes[2].size(), 1u);
      CHECK_EQ(output_shapes[0][1], input_shapes[2][0]);  // broadcast over the rows
    }
  }
}

void GemmKernel::Fill(const TensorList& inputs, const TensorList& outputs, OgleGemmArgs* a) const {
  a->m = outputs[0]->shape()[0];
  a->n = outputs[0]->shape()[1];
  a->k = inputs[0]->shape()[1];
  a->trans_b = trans_b_;
  a->c_rank = inputs.size() > 2 ? static_cast<int>(inputs[2]->shape().size()) : 0;
  a->alpha = alpha_;
  a->beta = beta_;
}

size_t GemmKernel::ScratchBytes() const {
  if (input_tensors_.empty() || output_tensors_.empty()) return 0;
  OgleGemmArgs a{};
  Fill(input_tensors_, output_tensors_, &a);
  // only the addend's presence matters to the plan, not its address
  a.c_dev = input_tensors_.size() > 2 ? reinterpret_cast<const float*>(16) : nullptr;
  return ogle_hip_gemm_workspace_bytes(&a);
}

void GemmKernel::Compute(TensorList& inputs, TensorList& outputs) {
  program_->Activate();
  CHECK_EQ(inputs[0]->dformat(), dlxnet::TensorProto::ANY4);
  CHECK_EQ(inputs[1]->dformat(), dlxnet::TensorProto::ANY4);
  OgleGemmArgs a{};
  Fill(inputs, outputs, &a);
  a.a_dev = static_cast<const float*>(inputs[0]->device_ptr());
  a.b_dev = static_cast<const float*>(inputs[1]->device_ptr());
  a.c_dev = inputs.size() > 2 ? static_cast<const float*>(inputs[2]->device_ptr()) : nullptr;
  a.y_dev = static_cast<float*>(outputs[0]->device_ptr());
  const size_t need = ogle_hip_gemm_workspace_bytes(&a);
  if (need > 0) {
    context_->Flush();  // the bump allocator hands out slices per deferred batch
    a.workspace_dev = context_->Workspace(need);
    a.workspace_bytes = need;
  }
  program_->RunGemm(a);
}

// ---- Flatten ---------------------------------------------------------------

void FlattenKernel::SetupAttr(const dlxnet::Attribute& attr) { axis_ = attr.flatten_attr().axis(); }

void FlattenKernel::SelectKernel(const TensorList& inputs) {
  kernel_fname_ = "reshape";
  if (session_->IsONNX() && inputs[0]->dformat() == dlxnet::TensorProto::NHWC4) {
    // The exporter's axis counts NCHW positions.  flatten.cc:15-21 sends it through
    // {0,3,1,2}, which for the usual axis 1 keeps N, H, W apart and hands Gemm a rank-4
    // tensor it rejects (gemm.cc:72).  Axis 1 means "everything but the batch": on the
    // stored NHWC tensor that is H, W and C merged, from position 1 on.  The elements
    // keep their stored order, which is the exporter's order when H = W = 1 (after
    // global pooling).
    CHECK_EQ(axis_, 1) << "Flatten of an image tensor: only axis 1 is supported";
  }
}

// flatten.cc:62-83.
void FlattenKernel::InferOutputShape(TensorShapeList& input_shapes, TensorShapeList& output_shapes) {
  output_tensor_dformats_.emplace_back(dlxnet::TensorProto::ANY4);
  CHECK_EQ(input_shapes.size(), 1u);
  output_shapes.clear();
  output_shapes.resize(1);
  CHECK_EQ(input_shapes[0].size(), 4u);
  CHECK(axis_ >= 0 && axis_ <= 4) << "Flatten: axis " << axis_;
  int merged = 1;
  for (size_t i = axis_; i < input_shapes[0].size(); ++i) merged *= input_shapes[0][i];
  for (int i = 0; i < axis_; ++i) output_shapes[0].push_back(input_shapes[0][i]);
  output_shapes[0].push_back(merged);
}

REGISTER_KERNEL_WITH_NAME(BinaryKernel, "Add");
REGISTER_KERNEL_WITH_NAME(ReluKernel, "Relu");
REGISTER_KERNEL_WITH_NAME(ClipKernel, "Clip");
REGISTER_KERNEL_WITH_NAME(BatchNormKernel, "BatchNormalization");
REGISTER_KERNEL_WITH_NAME(GemmKernel, "Gemm");
REGISTER_KERNEL_WITH_NAME(FlattenKernel, "Flatten");

}  // namespace opengl
