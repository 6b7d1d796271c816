// "Decoder": SSD box decode as a graph op.  Host side of
// ogl_runtime/opengl/nn/kernels/decoder.{h,cc}.
#ifndef OPENGL_NN_KERNELS_DECODER_H_
#define OPENGL_NN_KERNELS_DECODER_H_
#include <vector>

#include "opengl/core/kernel.h"

namespace opengl {

class DecoderKernel : public Kernel {
 public:
  explicit DecoderKernel(Context* context);
  void Compute(TensorList& inputs, TensorList& outputs) override;
  void InferOutputShape(const TensorList& inputs, TensorShapeList& outputs) override;
  void InferOutputShape(TensorShapeList&, TensorShapeList&) override {}
  void SetupAttr(const dlxnet::Attribute& attr) override;
  void SelectKernel(const TensorList& inputs) override;

 private:
  float score_threshold_;  // kept for parity with the reference's fields; the score
  float nms_threshold_;    // filter and NMS run in the Detector, not in this op
 public:
  float score_threshold() const { return score_threshold_; }
  float nms_threshold() const { return nms_threshold_; }

 private:
  std::vector<float> variances_;
};

}  // namespace opengl
#endif  // OPENGL_NN_KERNELS_DECODER_H_
