#include "opengl/nn/kernels/conv2d.h"

#include "opengl/core/context.h"
#include "opengl/core/kernel_registry.h"
#include "opengl/core/program.h"

namespace opengl {

Conv2DKernel::Conv2DKernel(Context* context) : Kernel(context) {}
Conv2DKernel::~Conv2DKernel() {}

// Attribute rules of conv2d.cc:67-111: four equal pads, two equal strides, a square
// kernel; group 0 means 1; one or two equal dilations, default 1.
void Conv2DKernel::SetupAttr(const dlxnet::Attribute& attr) {
  const dlxnet::Conv2dAttribute& p = attr.conv2d_attr();
  CHECK_EQ(p.pads_size(), 4);
  for (auto pad : p.pads()) CHECK_EQ(p.pads(0), pad);
  padding_ = static_cast<int>(p.pads(0));
  CHECK_EQ(p.strides_size(), 2);
  CHECK_EQ(p.strides(0), p.strides(1));
  stride_ = static_cast<int>(p.strides(0));
  CHECK_EQ(p.kernel_shape_size(), 2);
  CHECK_EQ(p.kernel_shape(0), p.kernel_shape(1));
  kernel_size_ = static_cast<int>(p.kernel_shape(0));
  group_size_ = p.group() == 0 ? 1 : static_cast<int>(p.group());
  if (p.dilations_size() == 2) {
    CHECK_EQ(p.dilations(0), p.dilations(1));
    dilation_ = static_cast<int>(p.dilations(0));
  } else if (p.dilations_size() == 1) {
    dilation_ = static_cast<int>(p.dilations(0));
  } else {
    dilation_ = 1;
  }
  activation_type_ = p.activation_type();
  min_ = p.min();
  max_ = p.max();
}

// Variant choice of conv2d.cc:19-65.  The names are the shader stems the registry
// is keyed by; the *_any4 stems select the same HIP kernels with the any4 reading
// of min/max for the fused activation.
void Conv2DKernel::SelectKernel(const TensorList& inputs) {
  const bool any4 = inputs[0]->dformat() == dlxnet::TensorProto::ANY4;
  const bool pointwise = kernel_size_ == 1 && group_size_ == 1 && dilation_ == 1 && stride_ == 1 &&
                         padding_ == 0;
  if (pointwise) {
    variant_ = kPointwise;
    kernel_fname_ = any4 ? "conv2d_pw_any4" : "conv2d_pw";
  } else if (group_size_ != 1) {
    const int in_c = inputs[0]->shape()[3];
    if (any4) {
      CHECK_EQ(group_size_, in_c);
      variant_ = kDepthwise;
      kernel_fname_ = "conv2d_dw_any4";
    } else if (group_size_ == in_c && group_size_ == inputs[1]->shape()[0]) {
      variant_ = kDepthwise;
      kernel_fname_ = "conv2d_dw";
    } else {
      variant_ = kGrouped;
      kernel_fname_ = "conv2d_grp";
    }
  } else {
    variant_ = kDense;
    kernel_fname_ = any4 ? "conv2d_any4" : "conv2d";
  }
  // How the fused activation reads min / max differs per shader: conv2d_pw.glsl:85 clamps
  // to (0, max); the *_any4 shaders and conv2d_grp.glsl:115-121 use max(min, x) for Relu
  // and (min, max) for Clip; conv2d.glsl / conv2d_dw.glsl use max(0, x) and (min, max).
  if (any4 || variant_ == kGrouped) act_variant_ = OGLE_VARIANT_ANY4;
  else act_variant_ = variant_ == kPointwise ? OGLE_VARIANT_PW : OGLE_VARIANT_NHWC4;

  if (input_tensor_indexes_.size() == 3) build_options_ += "#define USE_BIAS\n";
  if (activation_type_ == "Clip") {
    build_options_ += "#define USE_CLIP\n";
  } else if (activation_type_ == "Relu") {
    build_options_ += "#define USE_RELU\n";
  }
  output_tensor_dformats_.emplace_back(inputs[0]->dformat());
}

void Conv2DKernel::InferOutputShape(TensorShapeList& input_shapes, TensorShapeList& output_shapes) {
  CHECK(input_shapes.size() == 3 || input_shapes.size() == 2);
  output_shapes.clear();
  output_shapes.resize(1);
  const IntList& image_shape = input_shapes[0];   // (n, h, w, c)
  const IntList& filter_shape = input_shapes[1];  // (n_out, n_in / group, k, k)
  CHECK_EQ(image_shape.size(), 4u);
  CHECK_EQ(filter_shape.size(), 4u);
  CHECK_EQ(filter_shape[2], kernel_size_);
  CHECK_EQ(filter_shape[3], kernel_size_);
  CHECK_EQ(filter_shape[1] * group_size_, image_shape[3]);
  if (input_shapes.size() == 3) {
    size_t bias_elems = 1;
    for (int d : input_shapes[2]) bias_elems *= static_cast<size_t>(d);
    CHECK_EQ(bias_elems, static_cast<size_t>(filter_shape[0])) << "bias length";
  }
  const int kernel_size = kernel_size_ * dilation_ - dilation_ + 1;
  const int output_height = (image_shape[1] - kernel_size + 2 * padding_) / stride_ + 1;
  const int output_width = (image_shape[2] - kernel_size + 2 * padding_) / stride_ + 1;
  output_shapes[0] = {image_shape[0], output_height, output_width, filter_shape[0]};
}

void Conv2DKernel::PackFilter(const Tensor* filter) {
  context_->Flush();
  const IntList& fs = filter->shape();
  const int layout = variant_ == kDepthwise ? OGLE_FILTER_HWC : OGLE_FILTER_OHWI;
  if (variant_ == kDepthwise) CHECK_EQ(fs[1], 1) << "depthwise filters have one input channel";
  IntList packed_shape = fs;
  const Tensor* filter2 = sibling_ != nullptr ? sibling_->input_tensors_[1] : nullptr;
  if (filter2 != nullptr) packed_shape[0] += filter2->shape()[0];  // OHWI: output channels are rows
  packed_filter_.reset(new Tensor(Tensor::DT_FLOAT, packed_shape, Tensor::DEVICE_BUFFER, filter->dformat()));
  int32_t st =
      ogle_hip_pack_filter(static_cast<const float*>(filter->device_ptr()), packed_filter_->device_ptr(),
                           layout, OGLE_F32, fs[0], fs[1], fs[2], fs[3], context_->stream());
  if (st == OGLE_OK && filter2 != nullptr) {
    const IntList& f2 = filter2->shape();
    float* second = static_cast<float*>(packed_filter_->device_ptr()) + filter->num_elements();
    st = ogle_hip_pack_filter(static_cast<const float*>(filter2->device_ptr()), second, layout, OGLE_F32,
                              f2[0], f2[1], f2[2], f2[3], context_->stream());
  }
  if (st != OGLE_OK) LOG(FATAL) << "ogle_hip_pack_filter: " << ogle_hip_last_error();
  if (sibling_ != nullptr && input_tensors_.size() > 2) {
    // both bias vectors back to back, this node's first
    const Tensor* b1 = input_tensors_[2];
    const Tensor* b2 = sibling_->input_tensors_[2];
    fused_bias_.reset(new Tensor(Tensor::DT_FLOAT, {static_cast<int>(b1->num_elements() + b2->num_elements())},
                                 Tensor::DEVICE_BUFFER, dlxnet::TensorProto::ANY4));
    const int32_t c1 = ogle_hip_convert(b1->device_ptr(), OGLE_F32, fused_bias_->device_ptr(), OGLE_F32,
                                        static_cast<int64_t>(b1->num_elements()), context_->stream());
    const int32_t c2 = ogle_hip_convert(b2->device_ptr(), OGLE_F32,
                                        static_cast<float*>(fused_bias_->device_ptr()) + b1->num_elements(),
                                        OGLE_F32, static_cast<int64_t>(b2->num_elements()), context_->stream());
    if (c1 != OGLE_OK || c2 != OGLE_OK) LOG(FATAL) << "ogle_hip_convert: " << ogle_hip_last_error();
  }
  packed_from_ = filter->device_ptr();
}

// Two Conv nodes can share one launch when they read the same tensor with the same
// geometry and fused activation, neither is depthwise or grouped, both or neither have a
// bias, and their filters are separate constants.  The fused contraction has
// out_c = O1 + O2 output channels and writes each node's channels to its own tensor
// (OgleConvArgs.output2_dev).  It is only taken when the library would run it on the MFMA
// path with all channels in one tile column (out_c <= 160): that is where fetching the
// input once pays.
bool Conv2DKernel::TryAbsorb(Kernel* other_kernel) {
  Conv2DKernel* other = dynamic_cast<Conv2DKernel*>(other_kernel);
  if (other == nullptr || other == this || sibling_ != nullptr || absorbed() || other->absorbed() ||
      other->sibling_ != nullptr)
    return false;
  if (variant_ != kDense && variant_ != kPointwise) return false;
  if (other->variant_ != variant_ || other->act_variant_ != act_variant_) return false;
  if (input_tensors_.empty() || other->input_tensors_.empty() || output_tensors_.empty() ||
      other->output_tensors_.empty())
    return false;
  if (input_tensor_indexes_[0] != other->input_tensor_indexes_[0]) return false;
  if (input_tensors_.size() != other->input_tensors_.size()) return false;
  if (kernel_size_ != other->kernel_size_ || stride_ != other->stride_ || padding_ != other->padding_ ||
      dilation_ != other->dilation_ || group_size_ != 1 || other->group_size_ != 1 ||
      activation_type_ != other->activation_type_ || min_ != other->min_ || max_ != other->max_)
    return false;
  if (input_tensors_[1] == other->input_tensors_[1]) return false;
  const IntList& f1 = input_tensors_[1]->shape();
  const IntList& f2 = other->input_tensors_[1]->shape();
  if (f1[1] != f2[1] || f1[2] != f2[2] || f1[3] != f2[3]) return false;
  const int in_c = input_tensors_[0]->shape()[3];
  const long k_total = static_cast<long>(kernel_size_) * kernel_size_ * in_c;
  const int out_c = f1[0] + f2[0];
  if (in_c % 4 != 0 || k_total < 512 || out_c <= 64 || out_c > 160 || (out_c > 96 && out_c <= 128))
    return false;
  sibling_ = other;
  other->absorbed_by_ = this;
  packed_filter_.reset();
  packed_from_ = nullptr;
  workspace_need_ = -1;
  return true;
}

void Conv2DKernel::FillGeometry(const Tensor* image, const Tensor* output, OgleConvArgs* a) const {
  const IntList& in = image->shape();
  const IntList& out = output->shape();
  a->n = in[0]; a->in_h = in[1]; a->in_w = in[2]; a->in_c = in[3];
  a->out_h = out[1]; a->out_w = out[2]; a->out_c = out[3];
  if (sibling_ != nullptr) {
    a->out_c_split = out[3];
    a->out_c = out[3] + sibling_->output_tensors_[0]->shape()[3];
  }
  a->kernel_size = kernel_size_; a->stride = stride_; a->padding = padding_;
  a->dilation = dilation_; a->group = group_size_;
  // "act" uniform: 1 clip, otherwise 2 for any non-empty activation (conv2d.cc:137-147).
  a->act = activation_type_.empty() ? OGLE_ACT_NONE
                                    : (activation_type_ == "Clip" ? OGLE_ACT_CLIP : OGLE_ACT_RELU);
  a->min_value = min_;
  a->max_value = max_;
  a->act_variant = act_variant_;
  a->dtype = OGLE_F32;
}

size_t Conv2DKernel::ScratchBytes() const {
  if (workspace_need_ < 0) {
    CHECK(!input_tensors_.empty() && !output_tensors_.empty()) << "tensors are not bound yet";
    OgleConvArgs a{};
    FillGeometry(input_tensors_[0], output_tensors_[0], &a);
    if (sibling_ != nullptr) a.output2_dev = sibling_->output_tensors_[0]->device_ptr();
    workspace_need_ = absorbed() ? 0 : static_cast<long>(ogle_hip_conv_workspace_bytes(&a));
  }
  return static_cast<size_t>(workspace_need_);
}

// One run per image (OgleConvArgs.out_image_stride): only the kernels the library says
// take it, and not a pair of fused siblings (two destinations).
bool Conv2DKernel::CanWriteOuterSlicesApart(size_t count) const {
  if (input_tensors_.empty() || output_tensors_.empty() || sibling_ != nullptr || absorbed()) return false;
  if (variant_ == kDepthwise) return false;
  const IntList& out = output_tensors_[0]->shape();
  if (out.size() != 4 || static_cast<size_t>(out[0]) != count) return false;
  OgleConvArgs a{};
  FillGeometry(input_tensors_[0], output_tensors_[0], &a);
  return ogle_hip_conv_takes_image_stride(&a) == 1;
}

double Conv2DKernel::WorkEstimate() const {
  if (input_tensors_.empty() || output_tensors_.empty() || absorbed()) return 0.0;
  const IntList& in = input_tensors_[0]->shape();
  const IntList& out = output_tensors_[0]->shape();
  const double m = static_cast<double>(out[0]) * out[1] * out[2];
  const int out_c = out[3] + (sibling_ != nullptr ? sibling_->output_tensors_[0]->shape()[3] : 0);
  const double n = 32.0 * ((out_c + 31) / 32);  // the MFMA tiles are at least 32 channels wide
  return m * n * kernel_size_ * kernel_size_ * (in[3] / group_size_);
}

void Conv2DKernel::Compute(TensorList& inputs, TensorList& outputs) {
  if (absorbed()) return;  // the sibling's launch fills this node's output
  program_->Activate();
  const Tensor* image = inputs[0];
  const Tensor* filter = inputs[1];
  if (!packed_filter_ || packed_from_ != filter->device_ptr()) PackFilter(filter);

  OgleConvArgs a{};
  FillGeometry(image, outputs[0], &a);
  a.input_dev = image->device_ptr();
  a.filter_dev = packed_filter_->device_ptr();
  a.bias_dev = inputs.size() > 2 ? static_cast<const float*>(inputs[2]->device_ptr()) : nullptr;
  a.output_dev = outputs[0]->device_ptr();
  a.out_image_stride = static_cast<int64_t>(outputs[0]->outer_stride_bytes() / sizeof(float));
  if (sibling_ != nullptr) {
    a.output2_dev = sibling_->output_tensors_[0]->device_ptr();
    if (fused_bias_) a.bias_dev = static_cast<const float*>(fused_bias_->device_ptr());
  }
  if (variant_ != kDepthwise) context_->BeforeConv(a);
  if (workspace_need_ < 0) workspace_need_ = static_cast<long>(ogle_hip_conv_workspace_bytes(&a));
  if (workspace_need_ > 0) {
    a.workspace_dev = context_->Workspace(static_cast<size_t>(workspace_need_));
    a.workspace_bytes = static_cast<size_t>(workspace_need_);
  }
  switch (variant_) {
    case kPointwise: program_->RunPointwise(a); break;
    case kDepthwise: program_->RunDepthwise(a); break;
    default: program_->RunConv2d(a); break;
  }
}

REGISTER_KERNEL_WITH_NAME(Conv2DKernel, "Conv");

}  // namespace opengl
