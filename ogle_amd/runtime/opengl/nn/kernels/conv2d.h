// "Conv": dense, depthwise, pointwise and grouped 2-D convolution with optional
// bias and fused Relu / Clip.  Host side of ogl_runtime/opengl/nn/kernels/conv2d.{h,cc}.
#ifndef OPENGL_NN_KERNELS_CONV2D_H_
#define OPENGL_NN_KERNELS_CONV2D_H_
#include <memory>
#include <string>

#include "ogle_hip.h"
#include "opengl/core/kernel.h"
#include "opengl/core/tensor.h"

namespace opengl {

class Conv2DKernel : public Kernel {
 public:
  explicit Conv2DKernel(Context* context);
  ~Conv2DKernel() override;
  void Compute(TensorList& inputs, TensorList& outputs) override;
  void InferOutputShape(TensorShapeList& inputs, TensorShapeList& outputs) override;
  void SetupAttr(const dlxnet::Attribute& attr) override;
  void SelectKernel(const TensorList& inputs) override;
  bool Deferrable() const override { return variant_ != kDepthwise && !absorbed(); }
  bool TryAbsorb(Kernel* other) override;
  double WorkEstimate() const override;
  size_t ScratchBytes() const override;
  bool CanWriteOuterSlicesApart(size_t count) const override;

 private:
  enum Variant { kDense, kDepthwise, kPointwise, kGrouped };
  void PackFilter(const Tensor* filter);
  // Geometry, activation and dtype of the launch (no device pointers).
  void FillGeometry(const Tensor* image, const Tensor* output, OgleConvArgs* a) const;

  int padding_ = 0;
  int stride_ = 1;
  int kernel_size_ = 1;
  int group_size_ = 1;
  int dilation_ = 1;
  std::string activation_type_;
  float min_ = 0.f;
  float max_ = 0.f;
  Variant variant_ = kDense;
  int act_variant_ = OGLE_VARIANT_NHWC4;
  // The filter in the layout the chosen HIP kernel reads, made once from the OIHW
  // constant the first time the node computes.
  std::unique_ptr<Tensor> packed_filter_;
  const void* packed_from_ = nullptr;
  // Sibling fusion: this node also computes sibling_'s output.  The packed filter then
  // holds both filters (this node's output channels first), fused_bias_ both biases.
  Conv2DKernel* sibling_ = nullptr;
  std::unique_ptr<Tensor> fused_bias_;
  mutable long workspace_need_ = -1;  // bytes of scratch the launch plan wants; -1 until asked
};

}  // namespace opengl
#endif  // OPENGL_NN_KERNELS_CONV2D_H_
