// "Shape", "Gather", "Unsqueeze": the ops a PyTorch export puts in front of a
// Reshape (view(N, -1, K) becomes Shape -> Gather -> Unsqueeze -> Concat -> Reshape).
// Host side of ogl_runtime/opengl/nn/kernels/{shape,gather,unsqueeze}.{h,cc}.  They
// work on vectors of a few numbers and run once, while the session is set up
// (ShapeKernel::ForceReady, fbo_session.cc:254-267, then the ready_ flags), so they
// compute on the host and upload; none of them is on the per-pass path.
#ifndef OPENGL_NN_KERNELS_SHAPE_H_
#define OPENGL_NN_KERNELS_SHAPE_H_
#include <memory>
#include <vector>

#include "opengl/core/kernel.h"
#include "opengl/core/tensor.h"

namespace opengl {

// Output: the input's logical shape as floats, rank-1 (shape.cc:29-45).  For an
// image tensor that is the NHWC order the runtime keeps, not the exporter's NCHW.
class ShapeKernel : public Kernel {
 public:
  explicit ShapeKernel(Context* context) : Kernel(context) {}
  void Compute(TensorList& inputs, TensorList& outputs) override;
  void InferOutputShape(TensorShapeList& inputs, TensorShapeList& outputs) override;
  void SetupAttr(const dlxnet::Attribute&) override {}
  // Needs only the input's shape, so it runs during Setup although its input is an
  // activation (shape.h:19 of the reference).
  bool ForceReady() const override { return true; }

 private:
  std::unique_ptr<Tensor> values_;  // host copy of the shape vector
};

// Picks one entry of a 4-entry shape vector.  The index is a scalar that counts in
// the exporter's NCHW order while the vector is NHWC: 0 -> n, 1 -> c, 2 -> h, 3 -> w
// (gather.glsl:10-18).  The output has the index's shape (gather.cc:47-55).
class GatherKernel : public Kernel {
 public:
  explicit GatherKernel(Context* context) : Kernel(context) {}
  void Compute(TensorList& inputs, TensorList& outputs) override;
  void InferOutputShape(TensorShapeList& inputs, TensorShapeList& outputs) override;
  void SetupAttr(const dlxnet::Attribute& attr) override;

 private:
  int axis_ = 0;
};

// Inserts one dimension of size 1 (unsqueeze.cc:16-26,44-56); the elements do not
// move, so the output is a view of the input.
class UnsqueezeKernel : public Kernel {
 public:
  explicit UnsqueezeKernel(Context* context) : Kernel(context) {}
  void Compute(TensorList&, TensorList&) override {}
  void InferOutputShape(TensorShapeList& inputs, TensorShapeList& outputs) override;
  void SetupAttr(const dlxnet::Attribute& attr) override;
  int OutputAliasesInput(int) const override { return 0; }

 private:
  std::vector<int> axes_;
};

}  // namespace opengl
#endif  // OPENGL_NN_KERNELS_SHAPE_H_
