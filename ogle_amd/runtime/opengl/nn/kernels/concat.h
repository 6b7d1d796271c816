// "Concat": N-input concatenation along one axis.  Host side of
// ogl_runtime/opengl/nn/kernels/concat.{h,cc}.
#ifndef OPENGL_NN_KERNELS_CONCAT_H_
#define OPENGL_NN_KERNELS_CONCAT_H_
#include "opengl/core/kernel.h"

namespace opengl {

class ConcatKernel : public Kernel {
 public:
  explicit ConcatKernel(Context* context) : Kernel(context) {}
  void Compute(TensorList& inputs, TensorList& outputs) override;
  void InferOutputShape(const TensorList& inputs, TensorShapeList& outputs) override;
  void InferOutputShape(TensorShapeList&, TensorShapeList&) override {}
  void SetupAttr(const dlxnet::Attribute& attr) override;
  void SelectKernel(const TensorList& inputs) override;
  Placement InputPlacementInOutput() const override;

 private:
  int axis_ = 0;
};

}  // namespace opengl
#endif  // OPENGL_NN_KERNELS_CONCAT_H_
