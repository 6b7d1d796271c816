// "Reshape": new shape over the same row-major elements.  Host side of
// ogl_runtime/opengl/nn/kernels/reshape.{h,cc}.
#ifndef OPENGL_NN_KERNELS_RESHAPE_H_
#define OPENGL_NN_KERNELS_RESHAPE_H_
#include "opengl/core/kernel.h"

namespace opengl {

class ReshapeKernel : public Kernel {
 public:
  explicit ReshapeKernel(Context* context) : Kernel(context) {}
  void Compute(TensorList& inputs, TensorList& outputs) override;
  void InferOutputShape(const TensorList& inputs, TensorShapeList& outputs) override;
  void InferOutputShape(TensorShapeList&, TensorShapeList&) override {}
  void SetupAttr(const dlxnet::Attribute& attr) override;
  void SelectKernel(const TensorList& inputs) override;
  // Dense row-major storage makes a reshape a view: no kernel runs.
  int OutputAliasesInput(int) const override { return 0; }

 private:
  IntList target_shape_;
};

}  // namespace opengl
#endif  // OPENGL_NN_KERNELS_RESHAPE_H_
