// "Const" / "Constant": uploads a model constant.  Host side of
// ogl_runtime/opengl/nn/kernels/const.{h,cc}.
#ifndef OPENGL_NN_KERNELS_CONST_H_
#define OPENGL_NN_KERNELS_CONST_H_
#include <memory>

#include "opengl/core/kernel.h"
#include "opengl/core/tensor.h"

namespace opengl {

class ConstKernel : public Kernel {
 public:
  explicit ConstKernel(Context* context) : Kernel(context) {}
  void Compute(TensorList& inputs, TensorList& outputs) override;
  void InferOutputShape(TensorShapeList& inputs, TensorShapeList& outputs) override;
  void SetupAttr(const dlxnet::Attribute& attr) override;
  // Host copy of the constant (Reshape reads its target shape from here).
  const Tensor* host_tensor() const { return tensor_.get(); }

 private:
  std::unique_ptr<Tensor> tensor_;
};

}  // namespace opengl
#endif  // OPENGL_NN_KERNELS_CONST_H_
