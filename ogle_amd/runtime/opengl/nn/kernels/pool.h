// "MaxPool", "AveragePool", "GlobalAveragePool".  Host side of
// ogl_runtime/opengl/nn/kernels/pool.{h,cc}.
#ifndef OPENGL_NN_KERNELS_POOL_H_
#define OPENGL_NN_KERNELS_POOL_H_
#include "opengl/core/kernel.h"

namespace opengl {

enum PoolType { MaxPool = 0, AveragePool = 1, GlobalAveragePool = 2 };

template <PoolType pool_type>
class PoolKernel : public Kernel {
 public:
  explicit PoolKernel(Context* context) : Kernel(context) {}
  void Compute(TensorList& inputs, TensorList& outputs) override;
  void InferOutputShape(TensorShapeList& inputs, TensorShapeList& outputs) override;
  void SetupAttr(const dlxnet::Attribute& attr) override;
  void SelectKernel(const TensorList& inputs) override;

 private:
  int padding_ = 0;
  int stride_ = 1;
  int kernel_size_ = 1;
  PoolType pool_type_ = pool_type;
};

}  // namespace opengl
#endif  // OPENGL_NN_KERNELS_POOL_H_
