// "Add", "Relu", "Clip", "BatchNormalization", "Gemm", "Flatten": the ops of
// classification graphs (residual adds, standalone activations and batch norm, the
// final linear layer).  Host side of
// ogl_runtime/opengl/nn/kernels/{binary,relu,clip,batchnorm,gemm,flatten}.{h,cc}.
#ifndef OPENGL_NN_KERNELS_ELTWISE_H_
#define OPENGL_NN_KERNELS_ELTWISE_H_
#include "ogle_hip.h"
#include "opengl/core/kernel.h"

namespace opengl {

// binary.cc: y = a + b, both inputs of one shape; the output keeps input 0's tag.
class BinaryKernel : public Kernel {
 public:
  explicit BinaryKernel(Context* context) : Kernel(context) {}
  void Compute(TensorList& inputs, TensorList& outputs) override;
  void InferOutputShape(TensorShapeList& inputs, TensorShapeList& outputs) override;
  void SetupAttr(const dlxnet::Attribute&) override {}
  void SelectKernel(const TensorList& inputs) override;
};

// relu.cc: max(0, x).
class ReluKernel : public Kernel {
 public:
  explicit ReluKernel(Context* context) : Kernel(context) {}
  void Compute(TensorList& inputs, TensorList& outputs) override;
  void InferOutputShape(TensorShapeList& inputs, TensorShapeList& outputs) override;
  void SetupAttr(const dlxnet::Attribute&) override {}
  void SelectKernel(const TensorList& inputs) override;
};

// clip.cc: min(max, max(min, x)) with min / max from clip_attr.
class ClipKernel : public Kernel {
 public:
  explicit ClipKernel(Context* context) : Kernel(context) {}
  void Compute(TensorList& inputs, TensorList& outputs) override;
  void InferOutputShape(TensorShapeList& inputs, TensorShapeList& outputs) override;
  void SetupAttr(const dlxnet::Attribute& attr) override;
  void SelectKernel(const TensorList& inputs) override;

 private:
  float min_ = 0.f, max_ = 0.f;
};

// batchnorm.cc: inputs x, gamma, beta, mean, var; parameters per channel (last
// dimension of x).
class BatchNormKernel : public Kernel {
 public:
  explicit BatchNormKernel(Context* context) : Kernel(context) {}
  void Compute(TensorList& inputs, TensorList& outputs) override;
  void InferOutputShape(TensorShapeList& inputs, TensorShapeList& outputs) override;
  void SetupAttr(const dlxnet::Attribute& attr) override;
  void SelectKernel(const TensorList& inputs) override;

 private:
  float momentum_ = 0.f, eps_ = 0.f;
};

// gemm.cc: Y = alpha * A * B' + beta * C on rank-2 ANY4 tensors.
class GemmKernel : public Kernel {
 public:
  explicit GemmKernel(Context* context) : Kernel(context) { kernel_fname_ = "gemm"; }
  void Compute(TensorList& inputs, TensorList& outputs) override;
  void InferOutputShape(TensorShapeList& inputs, TensorShapeList& outputs) override;
  void SetupAttr(const dlxnet::Attribute& attr) override;
  size_t ScratchBytes() const override;

 private:
  void Fill(const TensorList& inputs, const TensorList& outputs, OgleGemmArgs* a) const;
  float alpha_ = 1.f, beta_ = 1.f;
  int trans_b_ = 0;
};

// flatten.cc: dimensions from `axis` on are merged; the elements keep their stored
// order, so the output is a view.  For an ONNX graph and an image input only axis 1
// (everything but the batch) is taken.
class FlattenKernel : public Kernel {
 public:
  explicit FlattenKernel(Context* context) : Kernel(context) {}
  void Compute(TensorList&, TensorList&) override {}
  void InferOutputShape(TensorShapeList& inputs, TensorShapeList& outputs) override;
  void SetupAttr(const dlxnet::Attribute& attr) override;
  void SelectKernel(const TensorList& inputs) override;
  int OutputAliasesInput(int) const override { return 0; }

 private:
  int axis_ = 1;
};

}  // namespace opengl
#endif  // OPENGL_NN_KERNELS_ELTWISE_H_
