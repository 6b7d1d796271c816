#include "opengl/core/context.h"

#include <hip/hip_runtime_api.h>

#include <vector>

namespace opengl {

#define OGLE_HIP_CALL(expr)                                                       \
  do {                                                                            \
    const hipError_t e__ = (expr);                                                \
    if (e__ != hipSuccess) LOG(FATAL) << #expr << ": " << hipGetErrorString(e__); \
  } while (0)

Context::Context() {}

void* Context::stream() {
  if (stream_ == nullptr) {
    hipStream_t s = nullptr;
    OGLE_HIP_CALL(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
    stream_ = s;
  }
  return stream_;
}

void Context::ReserveWorkspace(size_t bytes) {
  if (bytes <= workspace_bytes_) return;
  Finish();  // launches deferred work; earlier launches may still be using the old buffer
  if (workspace_ != nullptr) (void)hipFree(workspace_);
  workspace_ = nullptr;
  workspace_bytes_ = 0;
  const size_t rounded = (bytes + (1u << 20) - 1) & ~((size_t(1) << 20) - 1);
  OGLE_HIP_CALL(hipMalloc(&workspace_, rounded));
  workspace_bytes_ = rounded;
}

void* Context::Workspace(size_t bytes) {
  const size_t need = (bytes + 255) & ~size_t(255);
  if (workspace_used_ + need > workspace_bytes_) {
    // Out of room: grow to twice what the batch would have needed unbroken, so
    // that the next pass keeps it in one piece.
    const size_t want = 2 * (workspace_used_ + need);
    Flush();
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    (void)hipStreamIsCapturing(static_cast<hipStream_t>(stream()), &capturing);
    if (capturing == hipStreamCaptureStatusNone) {
      ReserveWorkspace(want);
    } else {
      CHECK(need <= workspace_bytes_)
          << "convolution workspace too small and the stream is being captured; "
             "run one pass outside the capture or call ReserveWorkspace first";
    }
  }
  void* p = static_cast<char*>(workspace_) + workspace_used_;
  workspace_used_ += need;
  return p;
}

namespace {
size_t ElemBytes(const OgleConvArgs& a) { return a.dtype == OGLE_F16 ? 2 : 4; }
bool Inside(const void* p, const void* base, size_t bytes) {
  const char* q = static_cast<const char*>(p);
  const char* b = static_cast<const char*>(base);
  return q >= b && q < b + bytes;
}
}  // namespace

bool Context::TouchesPending(const void* p, bool written_only) const {
  if (p == nullptr) return false;
  for (const OgleConvArgs& c : pending_) {
    const size_t esz = ElemBytes(c);
    if (Inside(p, c.output_dev, static_cast<size_t>(c.n) * c.out_h * c.out_w * c.out_c * esz))
      return true;
    if (written_only) continue;
    if (Inside(p, c.input_dev, static_cast<size_t>(c.n) * c.in_h * c.in_w * c.in_c * esz)) return true;
    if (p == c.filter_dev || p == c.bias_dev) return true;
  }
  return false;
}

void Context::BeforeConv(const void* input, const void* filter, const void* bias,
                         const void* output) {
  // reads of something a deferred convolution writes; a write into anything one touches
  if (pending_.size() >= 16 || TouchesPending(input, true) || TouchesPending(filter, true) ||
      TouchesPending(bias, true) || TouchesPending(output, false))
    Flush();
}

void Context::BeforeLaunch(const void* const* reads, int n_reads, const void* const* writes,
                           int n_writes) {
  if (pending_.empty()) return;
  bool flush = false;
  for (int i = 0; i < n_reads && !flush; ++i) flush = TouchesPending(reads[i], true);
  for (int i = 0; i < n_writes && !flush; ++i) flush = TouchesPending(writes[i], false);
  if (flush) Flush();
}

void Context::EnqueueConv(const OgleConvArgs& args) {
  pending_.push_back(args);
  if (!batching_) Flush();
}

void Context::Flush() {
  if (pending_.empty()) {
    workspace_used_ = 0;
    return;
  }
  std::vector<OgleConvArgs> batch;
  batch.swap(pending_);
  workspace_used_ = 0;
  const int32_t st = ogle_hip_conv2d_batch(batch.data(), static_cast<int32_t>(batch.size()), stream());
  if (st != OGLE_OK)
    LOG(FATAL) << "ogle_hip_conv2d_batch: " << ogle_hip_status_string(st) << ": "
               << ogle_hip_last_error();
}

Context::~Context() {
  if (workspace_ != nullptr) (void)hipFree(workspace_);
  if (stream_ != nullptr) (void)hipStreamDestroy(static_cast<hipStream_t>(stream_));
}

Program* Context::CreateProgram(const std::string& kernel_fname, const std::string& build_options) {
  if (kernel_fname.empty()) return nullptr;  // ops without device code (Const)
  const std::string key = kernel_fname + "\n" + build_options;
  auto it = programs_.find(key);
  if (it != programs_.end()) return it->second.get();
  int32_t handle = 0;
  const int32_t st = ogle_hip_registry_lookup(kernel_fname.c_str(), build_options.c_str(), &handle);
  if (st != OGLE_OK) LOG(FATAL) << "CreateProgram: " << ogle_hip_last_error();
  Program* p = new Program(kernel_fname, build_options, handle, this);
  programs_[key].reset(p);
  return p;
}

namespace {
// NCHW <-> NHWC on the host, rank 4 only.
void Permute4(const float* src, float* dst, const IntList& nhwc, bool to_nhwc = false) {
  const int n = nhwc[0], h = nhwc[1], w = nhwc[2], c = nhwc[3];
  for (int b = 0; b < n; ++b)
    for (int y = 0; y < h; ++y)
      for (int x = 0; x < w; ++x)
        for (int ch = 0; ch < c; ++ch) {
          const size_t i_nhwc = ((static_cast<size_t>(b) * h + y) * w + x) * c + ch;
          const size_t i_nchw = ((static_cast<size_t>(b) * c + ch) * h + y) * w + x;
          if (to_nhwc) dst[i_nhwc] = src[i_nchw];
          else dst[i_nchw] = src[i_nhwc];
        }
}
bool IsImageTag(DataFormat f) {
  return f == dlxnet::TensorProto::NHWC4 || f == dlxnet::TensorProto::NHWC;
}
}  // namespace

void Context::CopyCPUTensorToDevice(const Tensor* cpu, Tensor* dev) {
  CHECK(cpu->is_host()) << "source must be a host tensor";
  CHECK(dev->mem_type() != Tensor::HOST_MEMORY) << "destination must be a device tensor";
  CHECK_EQ(cpu->num_elements(), dev->num_elements());
  const size_t bytes = cpu->num_elements() * sizeof(float);
  if (bytes == 0) return;
  Flush();
  hipStream_t s = static_cast<hipStream_t>(stream());
  // The host tensor's element order is the device's: NHWC images, ANY tensors and
  // filters in the file's OIHW order are all dense row-major over shape().
  OGLE_HIP_CALL(hipMemcpyAsync(dev->device_ptr(), cpu->host(), bytes, hipMemcpyHostToDevice, s));
  OGLE_HIP_CALL(hipStreamSynchronize(s));
  dev->set_initialized(true);
}

void Context::CopyDeviceTensorToCPU(const Tensor* dev, Tensor* cpu) {
  CHECK(cpu->is_host()) << "destination must be a host tensor";
  CHECK(dev->mem_type() != Tensor::HOST_MEMORY) << "source must be a device tensor";
  CHECK_EQ(cpu->num_elements(), dev->num_elements());
  const size_t bytes = dev->num_elements() * sizeof(float);
  Flush();
  hipStream_t s = static_cast<hipStream_t>(stream());
  if (bytes == 0) {
    OGLE_HIP_CALL(hipStreamSynchronize(s));
    return;
  }
  if (cpu->dformat() == dlxnet::TensorProto::NCHW && IsImageTag(dev->dformat())) {
    CHECK_EQ(dev->dims_size(), 4);
    std::vector<float> tmp(dev->num_elements());
    OGLE_HIP_CALL(hipMemcpyAsync(tmp.data(), dev->device_ptr(), bytes, hipMemcpyDeviceToHost, s));
    OGLE_HIP_CALL(hipStreamSynchronize(s));
    Permute4(tmp.data(), cpu->host<float>(), dev->shape(), false);
  } else {
    OGLE_HIP_CALL(hipMemcpyAsync(cpu->host(), dev->device_ptr(), bytes, hipMemcpyDeviceToHost, s));
    OGLE_HIP_CALL(hipStreamSynchronize(s));
  }
  cpu->set_initialized(true);
}

void Context::Finish() {
  Flush();
  OGLE_HIP_CALL(hipStreamSynchronize(static_cast<hipStream_t>(stream())));
}

Context* GetContext() {
  static Context* context = new Context;
  return context;
}

// ---- Program ---------------------------------------------------------------

void Program::Check(int32_t status, const char* what) const {
  if (status != OGLE_OK)
    LOG(FATAL) << what << " (" << name_ << "): " << ogle_hip_status_string(status) << ": "
               << ogle_hip_last_error();
}
void Program::RunConv2d(const OgleConvArgs& a) const { context_->EnqueueConv(a); }
void Program::RunDepthwise(const OgleConvArgs& a) const {
  const void* reads[] = {a.input_dev, a.filter_dev, a.bias_dev};
  const void* writes[] = {a.output_dev};
  context_->BeforeLaunch(reads, 3, writes, 1);
  Check(ogle_hip_dwconv2d(&a, context_->stream()), "ogle_hip_dwconv2d");
}
void Program::RunPointwise(const OgleConvArgs& a) const {
  // the pointwise attribute rules (conv2d.cc:37) were checked by SelectKernel
  context_->EnqueueConv(a);
}
void Program::RunPool(const OglePoolArgs& a) const {
  const void* reads[] = {a.input_dev};
  const void* writes[] = {a.output_dev};
  context_->BeforeLaunch(reads, 1, writes, 1);
  Check(ogle_hip_pool2d(&a, context_->stream()), "ogle_hip_pool2d");
}
void Program::RunConcat(const OgleConcatArgs& a) const {
  const void* writes[] = {a.output_dev};
  context_->BeforeLaunch(a.inputs_dev, a.n_inputs, writes, 1);
  Check(ogle_hip_concat(&a, context_->stream()), "ogle_hip_concat");
}
void Program::RunDecode(const OgleDecodeArgs& a) const {
  const void* reads[] = {a.prediction_dev, a.anchors_dev};
  const void* writes[] = {a.boxes_dev};
  context_->BeforeLaunch(reads, 2, writes, 1);
  Check(ogle_hip_ssd_decode(&a, context_->stream()), "ogle_hip_ssd_decode");
}
void Program::RunTranspose(const OgleTransposeArgs& a) const {
  const void* reads[] = {a.input_dev};
  const void* writes[] = {a.output_dev};
  context_->BeforeLaunch(reads, 1, writes, 1);
  Check(ogle_hip_transpose(&a, context_->stream()), "ogle_hip_transpose");
}

void Program::RunUnary(const OgleUnaryArgs& a) const {
  const void* reads[] = {a.input_dev};
  const void* writes[] = {a.output_dev};
  context_->BeforeLaunch(reads, 1, writes, 1);
  Check(ogle_hip_unary(&a, context_->stream()), "ogle_hip_unary");
}
void Program::RunAdd(const OgleBinaryArgs& a) const {
  const void* reads[] = {a.a_dev, a.b_dev};
  const void* writes[] = {a.output_dev};
  context_->BeforeLaunch(reads, 2, writes, 1);
  Check(ogle_hip_add(&a, context_->stream()), "ogle_hip_add");
}
void Program::RunBatchNorm(const OgleBatchNormArgs& a) const {
  const void* reads[] = {a.input_dev, a.gamma_dev, a.beta_dev, a.mean_dev, a.var_dev};
  const void* writes[] = {a.output_dev};
  context_->BeforeLaunch(reads, 5, writes, 1);
  Check(ogle_hip_batchnorm(&a, context_->stream()), "ogle_hip_batchnorm");
}
void Program::RunGemm(const OgleGemmArgs& a) const {
  const void* reads[] = {a.a_dev, a.b_dev, a.c_dev};
  const void* writes[] = {a.y_dev};
  context_->BeforeLaunch(reads, 3, writes, 1);
  Check(ogle_hip_gemm(&a, context_->stream()), "ogle_hip_gemm");
}

}  // namespace opengl
