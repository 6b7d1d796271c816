#include "opengl/core/context.h"

#include <hip/hip_runtime_api.h>

#include <dlfcn.h>

#include <cstdlib>
#include <cstring>
#include <deque>
#include <map>
#include <mutex>
#include <vector>

namespace opengl {

#define OGLE_HIP_CALL(expr)                                                       \
  do {                                                                            \
    const hipError_t e__ = (expr);                                                \
    if (e__ != hipSuccess) LOG(FATAL) << #expr << ": " << hipGetErrorString(e__); \
  } while (0)

Context::Context() {}

namespace {
// The HIP runtime spreads streams over its few hardware queues as they are created, and work on
// two streams that share a queue does not overlap.  Streams made one at a time, with the
// application creating streams of its own in between, can therefore end up on one queue (four
// sessions created three unrelated streams apart replay their passes at 24 k images/s instead of
// 29.5 k).  So the first kPooledStreams streams that contexts ask for on a device are created
// together, in one go, and handed out in that order; a context hands its stream back when it is
// destroyed.  Contexts beyond the pool get a stream of their own.
constexpr int kPooledStreams = 4;
struct StreamPool {
  std::mutex mu;
  std::map<int, std::deque<hipStream_t>> idle;   // per device, in creation order
  std::map<int, bool> created;
};
StreamPool& Pool() {
  static StreamPool* pool = new StreamPool;   // never destroyed: streams outlive static teardown
  return *pool;
}
}  // namespace

void* Context::stream() {
  if (stream_ == nullptr) {
    int device = 0;
    OGLE_HIP_CALL(hipGetDevice(&device));
    StreamPool& pool = Pool();
    std::lock_guard<std::mutex> lock(pool.mu);
    if (!pool.created[device]) {
      for (int i = 0; i < kPooledStreams; ++i) {
        hipStream_t s = nullptr;
        OGLE_HIP_CALL(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
        pool.idle[device].push_back(s);
      }
      pool.created[device] = true;
    }
    std::deque<hipStream_t>& idle = pool.idle[device];
    if (!idle.empty()) {
      stream_ = idle.front();
      idle.pop_front();
      stream_pooled_ = true;
    } else {
      hipStream_t s = nullptr;
      OGLE_HIP_CALL(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
      stream_ = s;
      stream_pooled_ = false;
    }
    stream_device_ = device;
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
// True if the two ranges share a byte.  Two strided ranges of the same stride are compared
// by where their runs lie inside one period (exact when both cover the same slices, on the
// safe side otherwise), any other strided pair run by run.
bool Overlap(const MemRange& a, const MemRange& b) {
  if (a.ptr == nullptr || b.ptr == nullptr || a.bytes == 0 || b.bytes == 0) return false;
  const uintptr_t a0 = reinterpret_cast<uintptr_t>(a.ptr), b0 = reinterpret_cast<uintptr_t>(b.ptr);
  const uintptr_t a1 = a0 + (a.count - 1) * a.stride + a.bytes;
  const uintptr_t b1 = b0 + (b.count - 1) * b.stride + b.bytes;
  if (!(a0 < b1 && b0 < a1)) return false;
  if (a.count <= 1 && b.count <= 1) return true;
  if (a.count > 1 && b.count > 1) {
    if (a.stride != b.stride || a.bytes > a.stride || b.bytes > b.stride) return true;
    const size_t d = b0 >= a0 ? (b0 - a0) % a.stride : (a.stride - (a0 - b0) % a.stride) % a.stride;
    return d < a.bytes || d + b.bytes > a.stride;
  }
  const MemRange& many = a.count > 1 ? a : b;
  const MemRange& one = a.count > 1 ? b : a;
  const uintptr_t m0 = reinterpret_cast<uintptr_t>(many.ptr), o0 = reinterpret_cast<uintptr_t>(one.ptr);
  for (size_t i = 0; i < many.count; ++i) {
    const uintptr_t r0 = m0 + i * many.stride;
    if (r0 < o0 + one.bytes && o0 < r0 + many.bytes) return true;
  }
  return false;
}
}  // namespace

void Context::ConvRanges(const OgleConvArgs& c, MemRange reads[3], MemRange writes[3]) {
  const size_t esz = ElemBytes(c);
  const int group = c.group > 0 ? c.group : 1;
  reads[0] = {c.input_dev, static_cast<size_t>(c.n) * c.in_h * c.in_w * c.in_c * esz};
  reads[1] = {c.filter_dev, static_cast<size_t>(c.out_c) * c.kernel_size * c.kernel_size *
                                (c.in_c / group) * esz};
  reads[2] = {c.bias_dev, c.bias_dev != nullptr ? static_cast<size_t>(c.out_c) * sizeof(float) : 0};
  const size_t pixels = static_cast<size_t>(c.n) * c.out_h * c.out_w;
  const int first = c.output2_dev != nullptr ? c.out_c_split : c.out_c;
  writes[0] = {c.output_dev, pixels * first * esz};
  const size_t image = static_cast<size_t>(c.out_h) * c.out_w * first * esz;
  if (c.out_image_stride != 0 && c.n > 1 && static_cast<size_t>(c.out_image_stride) * esz != image)
    writes[0] = {c.output_dev, image, static_cast<size_t>(c.out_image_stride) * esz,
                 static_cast<size_t>(c.n)};
  writes[1] = {c.workspace_dev, c.workspace_dev != nullptr ? c.workspace_bytes : 0};
  writes[2] = {c.output2_dev, c.output2_dev != nullptr ? pixels * (c.out_c - first) * esz : 0};
}

bool Context::Conflicts(const OgleConvArgs* pending, int n_pending, const MemRange* reads,
                        int n_reads, const MemRange* writes, int n_writes) {
  for (int p = 0; p < n_pending; ++p) {
    MemRange pr[3], pw[3];
    ConvRanges(pending[p], pr, pw);
    // read after write
    for (int i = 0; i < n_reads; ++i)
      for (const MemRange& w : pw)
        if (Overlap(reads[i], w)) return true;
    // write after read, write after write
    for (int i = 0; i < n_writes; ++i) {
      for (const MemRange& w : pw)
        if (Overlap(writes[i], w)) return true;
      for (const MemRange& r : pr)
        if (Overlap(writes[i], r)) return true;
    }
  }
  return false;
}

// A convolution that needs a deferred one's result (or overwrites what it reads) only
// forces out the deferred ones it conflicts with: it is deferred itself, and the others
// may still share its grid.  Any other kind of launch goes to the stream at once and
// takes everything deferred with it (BeforeLaunch).
void Context::BeforeConv(const OgleConvArgs& args) {
  if (pending_.empty() && unreduced_.empty()) return;
  MemRange reads[3], writes[3];
  ConvRanges(args, reads, writes);
  if (pending_.size() >= 16)
    LaunchPending();
  else
    LaunchPendingThatConflict(reads, 3, writes, 3);
  FinishReductions(reads, 3, writes, 3, false);
}

void Context::BeforeLaunch(const MemRange* reads, int n_reads, const MemRange* writes,
                           int n_writes) {
  if (pending_.empty() && unreduced_.empty()) return;
  if (Conflicts(pending_.data(), static_cast<int>(pending_.size()), reads, n_reads, writes, n_writes))
    LaunchPending();
  FinishReductions(reads, n_reads, writes, n_writes, false);
}

// A convolution whose contraction is on the stream but whose reduction is not: what it
// still reads is its bias and its partial sums, what it still writes its output(s).
// Its input and filter are free again (later work on the stream is ordered after the
// contraction).
void Context::FinishReductions(const MemRange* reads, int n_reads, const MemRange* writes,
                               int n_writes, bool all) {
  if (unreduced_.empty()) return;
  // One reduction that is needed takes every open one with it: they share the grid, and the
  // others' results are wanted soon after (the box concat asks for six head reductions, the
  // class concat for the other six a launch later).
  bool any = all;
  for (size_t i = 0; i < unreduced_.size() && !any; ++i) {
    OgleConvArgs c = unreduced_[i];
    c.input_dev = nullptr;   // no longer read
    c.filter_dev = nullptr;
    any = Conflicts(&c, 1, reads, n_reads, writes, n_writes);
  }
  if (!any) return;
  std::vector<OgleConvArgs> now;
  std::vector<std::string> now_labels;
  now.swap(unreduced_);
  now_labels.swap(unreduced_labels_);
  if (!current_label_.empty()) LogLaunches(current_label_, node_count_before_);
  const int64_t before = ogle_hip_launch_count();
  const int32_t st = ogle_hip_conv2d_batch_finish(now.data(), static_cast<int32_t>(now.size()), stream());
  if (st != OGLE_OK)
    LOG(FATAL) << "ogle_hip_conv2d_batch_finish: " << ogle_hip_status_string(st) << ": "
               << ogle_hip_last_error();
  if (log_launches_) {
    std::string joined = "reduce:";
    for (size_t i = 0; i < now_labels.size(); ++i) joined += (i ? "+" : "") + now_labels[i];
    LogLaunches(joined, before);
  } else {
    node_count_before_ = ogle_hip_launch_count();
  }
  if (pending_.empty() && unreduced_.empty()) workspace_used_ = 0;
}

void Context::EnqueueConv(const OgleConvArgs& args) {
  pending_.push_back(args);
  pending_labels_.push_back(current_label_);
  if (!batching_) Flush();
}

namespace {
// roctx, looked up at run time so that the runtime has no link-time dependency on a
// profiler library; absent library or OGLE_ROCTX unset: no ranges.
struct Roctx {
  int (*push)(const char*) = nullptr;
  int (*pop)() = nullptr;
  Roctx() {
    const char* env = std::getenv("OGLE_ROCTX");
    if (env == nullptr || env[0] == '\0' || env[0] == '0') return;
    void* lib = dlopen("librocprofiler-sdk-roctx.so", RTLD_NOW | RTLD_GLOBAL);
    if (lib == nullptr) lib = dlopen("libroctx64.so", RTLD_NOW | RTLD_GLOBAL);
    if (lib == nullptr) return;
    push = reinterpret_cast<int (*)(const char*)>(dlsym(lib, "roctxRangePushA"));
    pop = reinterpret_cast<int (*)()>(dlsym(lib, "roctxRangePop"));
    if (push == nullptr || pop == nullptr) push = nullptr;
  }
};
Roctx& roctx() {
  static Roctx r;
  return r;
}
}  // namespace

void Context::BeginNode(const std::string& label) {
  current_label_ = label;
  node_count_before_ = ogle_hip_launch_count();
  if (roctx().push != nullptr) roctx().push(label.c_str());
}

void Context::EndNode() {
  // what the node launched directly (deferred convolutions are logged at Flush, and a
  // Flush inside the node has already moved the mark past its launches)
  LogLaunches(current_label_, node_count_before_);
  current_label_.clear();
  if (roctx().push != nullptr) roctx().pop();
}

void Context::LogLaunches(const std::string& label, int64_t count_before) {
  const int64_t now = ogle_hip_launch_count();
  if (log_launches_ && now > count_before)
    launch_log_.push_back({label, static_cast<int>(now - count_before)});
  node_count_before_ = now;
}

void Context::LaunchPending() {
  if (pending_.empty()) {
    pending_labels_.clear();
    if (unreduced_.empty()) workspace_used_ = 0;
    return;
  }
  std::vector<OgleConvArgs> batch;
  batch.swap(pending_);
  std::vector<std::string> labels;
  labels.swap(pending_labels_);
  LaunchBatch(batch, labels);
}

void Context::LaunchPendingThatConflict(const MemRange* reads, int n_reads, const MemRange* writes,
                                        int n_writes) {
  std::vector<OgleConvArgs> batch, keep;
  std::vector<std::string> labels, keep_labels;
  for (size_t i = 0; i < pending_.size(); ++i) {
    const bool hit = Conflicts(&pending_[i], 1, reads, n_reads, writes, n_writes);
    (hit ? batch : keep).push_back(pending_[i]);
    (hit ? labels : keep_labels).push_back(pending_labels_[i]);
  }
  if (batch.empty()) return;
  pending_.swap(keep);
  pending_labels_.swap(keep_labels);
  LaunchBatch(batch, labels);
}

void Context::LaunchBatch(std::vector<OgleConvArgs>& batch, std::vector<std::string>& labels) {
  // launches the running node made itself before this point belong to that node
  if (!current_label_.empty()) LogLaunches(current_label_, node_count_before_);
  const int64_t before = ogle_hip_launch_count();
  std::vector<int32_t> open(batch.size(), 0);
  const int32_t st = ogle_hip_conv2d_batch_begin(batch.data(), static_cast<int32_t>(batch.size()),
                                                 open.data(), stream());
  if (log_launches_) {
    std::string joined;
    for (const std::string& l : labels) joined += (joined.empty() ? "" : "+") + l;
    LogLaunches(joined, before);
  } else {
    node_count_before_ = ogle_hip_launch_count();
  }
  if (st != OGLE_OK)
    LOG(FATAL) << "ogle_hip_conv2d_batch_begin: " << ogle_hip_status_string(st) << ": "
               << ogle_hip_last_error();
  for (size_t i = 0; i < batch.size(); ++i)
    if (open[i]) {
      unreduced_.push_back(batch[i]);
      unreduced_labels_.push_back(labels[i]);
    }
  if (pending_.empty() && unreduced_.empty()) workspace_used_ = 0;
}

void Context::Flush() {
  LaunchPending();
  FinishReductions(nullptr, 0, nullptr, 0, true);
}

Context::~Context() {
  if (workspace_ != nullptr) (void)hipFree(workspace_);
  if (stream_ != nullptr) {
    hipStream_t s = static_cast<hipStream_t>(stream_);
    if (stream_pooled_) {
      (void)hipStreamSynchronize(s);   // the next owner starts on an idle stream
      StreamPool& pool = Pool();
      std::lock_guard<std::mutex> lock(pool.mu);
      pool.idle[stream_device_].push_front(s);
    } else {
      (void)hipStreamDestroy(s);
    }
  }
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
bool IsPaddedTag(DataFormat f) {
  return f == dlxnet::TensorProto::NHWC4 || f == dlxnet::TensorProto::ANY4 ||
         f == dlxnet::TensorProto::HWN4C4;
}

// Dense row-major `dense` (logical shape order) <-> the reference's padded host layout
// for tag `f` (ogl_runtime/opengl/core/tensor_format.cc:272-343,
// core/cpu_functor.cc:10-127): NHWC4 and ANY4 pad the last dimension to a multiple
// of 4 (for NHWC4 that is the texel row (w*C4 + c/4, n*H + h), lane c%4, read row by
// row); HWN4C4 places OIHW element (o, i, ky, kx) at texel x = i,
// y = (ky*kw + kx)*ceil(O/4) + o/4, lane o%4, rows ceil(I/4)*4 texels wide.
void PaddedIndexWalk(const IntList& shape, DataFormat f, float* dense, float* padded, bool to_padded) {
  size_t n = 1;
  for (int d : shape) n *= static_cast<size_t>(d);
  if (f == dlxnet::TensorProto::HWN4C4) {
    CHECK_EQ(shape.size(), 4u);
    const size_t O = shape[0], I = shape[1], kh = shape[2], kw = shape[3];
    const size_t o4 = (O + 3) / 4, width = (I + 3) / 4 * 4;
    for (size_t o = 0; o < O; ++o)
      for (size_t i = 0; i < I; ++i)
        for (size_t t = 0; t < kh * kw; ++t) {
          const size_t di = ((t * o4 + o / 4) * width + i) * 4 + o % 4;
          const size_t si = (o * I + i) * kh * kw + t;
          if (to_padded) padded[di] = dense[si];
          else dense[si] = padded[di];
        }
    return;
  }
  if (shape.empty() || shape.back() == 0) return;
  const size_t last = static_cast<size_t>(shape.back()), last4 = (last + 3) / 4 * 4;
  for (size_t i = 0; i < n; ++i) {
    const size_t di = i / last * last4 + i % last;
    if (to_padded) padded[di] = dense[i];
    else dense[i] = padded[di];
  }
}
}  // namespace

void Context::CopyCPUTensorToDevice(const Tensor* cpu, Tensor* dev) {
  CHECK(cpu->is_host()) << "source must be a host tensor";
  CHECK(dev->mem_type() != Tensor::HOST_MEMORY) << "destination must be a device tensor";
  CHECK_EQ(cpu->num_elements(), dev->num_elements());
  CHECK_EQ(dev->outer_stride_bytes(), 0u) << "upload into a tensor that lies inside another one";
  const size_t bytes = cpu->num_elements() * sizeof(float);
  if (bytes == 0) return;
  Flush();
  hipStream_t s = static_cast<hipStream_t>(stream());
  if (IsPaddedTag(cpu->dformat()) && cpu->AllocatedSize() != bytes) {
    // a host tensor in one of the reference's padded layouts: strip the padding
    std::vector<float> dense(cpu->num_elements());
    PaddedIndexWalk(cpu->shape(), cpu->dformat(), dense.data(), cpu->host<float>(), false);
    OGLE_HIP_CALL(hipMemcpyAsync(dev->device_ptr(), dense.data(), bytes, hipMemcpyHostToDevice, s));
    OGLE_HIP_CALL(hipStreamSynchronize(s));
    dev->set_initialized(true);
    return;
  }
  // The host tensor's element order is the device's: NHWC images, ANY tensors and
  // filters in the file's OIHW order are all dense row-major over shape().
  OGLE_HIP_CALL(hipMemcpyAsync(dev->device_ptr(), cpu->host(), bytes, hipMemcpyHostToDevice, s));
  OGLE_HIP_CALL(hipStreamSynchronize(s));
  dev->set_initialized(true);
}

namespace {
// Device -> host copy of a tensor's elements in dense order, whether or not its runs lie
// apart on the device.
void ReadDense(const Tensor* dev, void* dst, hipStream_t s) {
  const size_t bytes = dev->num_elements() * sizeof(float);
  const size_t stride = dev->outer_stride_bytes();
  if (stride == 0) {
    OGLE_HIP_CALL(hipMemcpyAsync(dst, dev->device_ptr(), bytes, hipMemcpyDeviceToHost, s));
    return;
  }
  const size_t run = bytes / dev->outer_count();
  OGLE_HIP_CALL(hipMemcpy2DAsync(dst, run, dev->device_ptr(), stride, run, dev->outer_count(),
                                 hipMemcpyDeviceToHost, s));
}
}  // namespace

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
  if (IsPaddedTag(cpu->dformat())) {
    // "NHWC4" / "ANY4" / "HWN4C4": the caller gets the reference's padded layout,
    // padding lanes zero (the texture upload shaders write zeros there,
    // any_to_nhwc4.glsl:44-52).  HWN4C4 is only meaningful for an OIHW filter, NHWC4
    // for a rank-4 tensor; HostElements checked the rank when `cpu` was made.
    if (cpu->dformat() == dlxnet::TensorProto::HWN4C4)
      CHECK(dev->dformat() == dlxnet::TensorProto::HWN4C4)
          << "HWN4C4 readback of a tensor that is not a filter (" << FormatToStr(dev->dformat()) << ")";
    std::vector<float> dense(dev->num_elements());
    ReadDense(dev, dense.data(), s);
    OGLE_HIP_CALL(hipStreamSynchronize(s));
    std::memset(cpu->host(), 0, cpu->AllocatedSize());
    PaddedIndexWalk(dev->shape(), cpu->dformat(), dense.data(), cpu->host<float>(), true);
  } else if (cpu->dformat() == dlxnet::TensorProto::NCHW && IsImageTag(dev->dformat())) {
    CHECK_EQ(dev->dims_size(), 4);
    std::vector<float> tmp(dev->num_elements());
    ReadDense(dev, tmp.data(), s);
    OGLE_HIP_CALL(hipStreamSynchronize(s));
    Permute4(tmp.data(), cpu->host<float>(), dev->shape(), false);
  } else {
    ReadDense(dev, cpu->host(), s);
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
  MemRange reads[3], writes[3];
  Context::ConvRanges(a, reads, writes);
  context_->BeforeLaunch(reads, 3, writes, 3);
  Check(ogle_hip_dwconv2d(&a, context_->stream()), "ogle_hip_dwconv2d");
}
void Program::RunPointwise(const OgleConvArgs& a) const {
  // the pointwise attribute rules (conv2d.cc:37) were checked by SelectKernel
  context_->EnqueueConv(a);
}
namespace {
size_t DtypeBytes(int32_t dtype) { return dtype == OGLE_F16 ? 2 : 4; }
}  // namespace
void Program::RunPool(const OglePoolArgs& a) const {
  const size_t esz = DtypeBytes(a.dtype);
  const MemRange reads[] = {{a.input_dev, static_cast<size_t>(a.n) * a.in_h * a.in_w * a.c * esz}};
  const MemRange writes[] = {{a.output_dev, static_cast<size_t>(a.n) * a.out_h * a.out_w * a.c * esz}};
  context_->BeforeLaunch(reads, 1, writes, 1);
  Check(ogle_hip_pool2d(&a, context_->stream()), "ogle_hip_pool2d");
}
void Program::RunConcat(const OgleConcatArgs& a) const {
  const size_t esz = DtypeBytes(a.dtype);
  MemRange reads[OGLE_CONCAT_MAX_INPUTS];
  int64_t total = 0;
  for (int i = 0; i < a.n_inputs; ++i) {
    reads[i] = {a.inputs_dev[i], static_cast<size_t>(a.outer * a.axis_len[i] * a.inner) * esz};
    total += a.axis_len[i];
  }
  const MemRange writes[] = {{a.output_dev, static_cast<size_t>(a.outer * total * a.inner) * esz}};
  context_->BeforeLaunch(reads, a.n_inputs, writes, 1);
  Check(ogle_hip_concat(&a, context_->stream()), "ogle_hip_concat");
}
void Program::RunDecode(const OgleDecodeArgs& a) const {
  const size_t boxes = static_cast<size_t>(a.batch) * a.priors * 4 * sizeof(float);
  const size_t anchors = a.anchors_batch_stride != 0 ? boxes : static_cast<size_t>(a.priors) * 4 * sizeof(float);
  const MemRange reads[] = {{a.prediction_dev, boxes}, {a.anchors_dev, anchors}};
  const MemRange writes[] = {{a.boxes_dev, boxes}};
  context_->BeforeLaunch(reads, 2, writes, 1);
  Check(ogle_hip_ssd_decode(&a, context_->stream()), "ogle_hip_ssd_decode");
}
void Program::RunTranspose(const OgleTransposeArgs& a) const {
  size_t bytes = DtypeBytes(a.dtype);
  for (int d = 0; d < 4; ++d) bytes *= static_cast<size_t>(a.in_shape[d]);
  const MemRange reads[] = {{a.input_dev, bytes}};
  const MemRange writes[] = {{a.output_dev, bytes}};
  context_->BeforeLaunch(reads, 1, writes, 1);
  Check(ogle_hip_transpose(&a, context_->stream()), "ogle_hip_transpose");
}

void Program::RunUnary(const OgleUnaryArgs& a) const {
  const size_t bytes = static_cast<size_t>(a.count) * DtypeBytes(a.dtype);
  const MemRange reads[] = {{a.input_dev, bytes}};
  const MemRange writes[] = {{a.output_dev, bytes}};
  context_->BeforeLaunch(reads, 1, writes, 1);
  Check(ogle_hip_unary(&a, context_->stream()), "ogle_hip_unary");
}
void Program::RunAdd(const OgleBinaryArgs& a) const {
  const size_t bytes = static_cast<size_t>(a.count) * DtypeBytes(a.dtype);
  const MemRange reads[] = {{a.a_dev, bytes}, {a.b_dev, bytes}};
  const MemRange writes[] = {{a.output_dev, bytes}};
  context_->BeforeLaunch(reads, 2, writes, 1);
  Check(ogle_hip_add(&a, context_->stream()), "ogle_hip_add");
}
void Program::RunBatchNorm(const OgleBatchNormArgs& a) const {
  const size_t bytes = static_cast<size_t>(a.outer) * a.channels * DtypeBytes(a.dtype);
  const size_t vec = static_cast<size_t>(a.channels) * sizeof(float);
  const MemRange reads[] = {{a.input_dev, bytes}, {a.gamma_dev, vec}, {a.beta_dev, vec},
                            {a.mean_dev, vec}, {a.var_dev, vec}};
  const MemRange writes[] = {{a.output_dev, bytes}};
  context_->BeforeLaunch(reads, 5, writes, 1);
  Check(ogle_hip_batchnorm(&a, context_->stream()), "ogle_hip_batchnorm");
}
void Program::RunGemm(const OgleGemmArgs& a) const {
  const size_t f = sizeof(float);
  const size_t c_bytes = a.c_dev == nullptr ? 0 : (a.c_rank == 2 ? static_cast<size_t>(a.m) * a.n : static_cast<size_t>(a.n)) * f;
  const MemRange reads[] = {{a.a_dev, static_cast<size_t>(a.m) * a.k * f},
                            {a.b_dev, static_cast<size_t>(a.k) * a.n * f},
                            {a.c_dev, c_bytes}};
  const MemRange writes[] = {{a.y_dev, static_cast<size_t>(a.m) * a.n * f},
                             {a.workspace_dev, a.workspace_dev != nullptr ? a.workspace_bytes : 0}};
  context_->BeforeLaunch(reads, 3, writes, 2);
  Check(ogle_hip_gemm(&a, context_->stream()), "ogle_hip_gemm");
}

}  // namespace opengl
