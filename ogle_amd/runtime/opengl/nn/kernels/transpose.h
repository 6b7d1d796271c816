// "Transpose": dimension permutation.  Host side of
// ogl_runtime/opengl/nn/kernels/transpose.{h,cc}.
#ifndef OPENGL_NN_KERNELS_TRANSPOSE_H_
#define OPENGL_NN_KERNELS_TRANSPOSE_H_
#include "opengl/core/kernel.h"

namespace opengl {

class TransposeKernel : public Kernel {
 public:
  explicit TransposeKernel(Context* context) : Kernel(context) {}
  void Compute(TensorList& inputs, TensorList& outputs) override;
  void InferOutputShape(TensorShapeList& inputs, TensorShapeList& outputs) override;
  void SetupAttr(const dlxnet::Attribute& attr) override;
  void SelectKernel(const TensorList& inputs) override;
  int OutputAliasesInput(int i) const override;

 private:
  IntList perm_;
  bool moves_no_data_ = false;
};

}  // namespace opengl
#endif  // OPENGL_NN_KERNELS_TRANSPOSE_H_
