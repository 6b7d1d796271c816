// C ABI of the kernel library: argument validation, the kernel registry and the
// dispatch from op-level entry points to the HIP launchers.
#include <cstring>
#include <string>
#include <utility>
#include <vector>

#include "common.h"

namespace ogle {

static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

static thread_local int64_t g_launches = 0;

// Kernel timing state of the calling thread: one (start, stop) event pair per launch, in
// launch order; a device operation that is not a kernel holds a null pair.
struct TimingState {
  bool on = false;
  std::vector<std::pair<hipEvent_t, hipEvent_t>> events;
};
static thread_local TimingState g_timing;

bool next_timing_events(hipEvent_t* start, hipEvent_t* stop) {
  if (!g_timing.on) return false;
  hipEvent_t e0 = nullptr, e1 = nullptr;
  if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) {
    if (e0 != nullptr) (void)hipEventDestroy(e0);
    g_timing.on = false;  // cannot time: fall back to plain launches
    return false;
  }
  g_timing.events.emplace_back(e0, e1);
  *start = e0;
  *stop = e1;
  return true;
}

void note_launch() {
  ++g_launches;
  if (g_timing.on) g_timing.events.emplace_back(nullptr, nullptr);
}

int32_t check_launch(const char* kernel) {
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("%s: launch failed: %s", kernel, hipGetErrorString(e));
    return OGLE_ERR_LAUNCH;
  }
  ++g_launches;
  return OGLE_OK;
}

namespace {

// Registry: shader stem -> kernel family.  The flag bits mirror the build
// options the reference composes (conv2d.cc:54-62).
enum Family {
  FAM_CONV = 1, FAM_CONV_DW = 2, FAM_CONV_PW = 3, FAM_CONV_GRP = 4,
  FAM_POOL = 5, FAM_CONCAT = 6, FAM_DECODER = 7, FAM_TRANSPOSE = 8, FAM_RESHAPE = 9,
  FAM_ELTWISE = 10, FAM_GEMM = 11
};
enum Flags { FLAG_BIAS = 1, FLAG_CLIP = 2, FLAG_RELU = 4, FLAG_ANY4 = 8 };

struct Entry {
  const char* name;
  int family;
  int base_flags;
};

const Entry kRegistry[] = {
    {"conv2d", FAM_CONV, 0},
    {"conv2d_any4", FAM_CONV, FLAG_ANY4},
    {"conv2d_dw", FAM_CONV_DW, 0},
    {"conv2d_dw_any4", FAM_CONV_DW, FLAG_ANY4},
    {"conv2d_pw", FAM_CONV_PW, 0},
    {"conv2d_pw_any4", FAM_CONV_PW, FLAG_ANY4},
    {"conv2d_grp", FAM_CONV_GRP, 0},
    {"pool", FAM_POOL, 0},
    {"pool_any4", FAM_POOL, FLAG_ANY4},
    {"concat_multi", FAM_CONCAT, 0},
    {"decoder", FAM_DECODER, 0},
    {"transpose", FAM_TRANSPOSE, 0},
    {"transpose_any4", FAM_TRANSPOSE, FLAG_ANY4},
    {"reshape", FAM_RESHAPE, 0},
    {"reshape_any4", FAM_RESHAPE, FLAG_ANY4},
    {"binary", FAM_ELTWISE, 0},
    {"relu", FAM_ELTWISE, 0},
    {"clip", FAM_ELTWISE, 0},
    {"batchnorm", FAM_ELTWISE, 0},
    {"batchnorm_any4", FAM_ELTWISE, FLAG_ANY4},
    {"gemm", FAM_GEMM, 0},
};
constexpr int kRegistrySize = sizeof(kRegistry) / sizeof(kRegistry[0]);

bool positive(int v) { return v > 0; }

const char kSplitNeedsMfma[] =
    "a second destination (output2_dev) and an image stride (out_image_stride) are only "
    "supported by the MFMA implicit-GEMM kernels: "
    "group 1, in_c % 4 == 0 (fp16: % 8), kernel_size^2 * in_c >= 32";

// True for arguments only the implicit-GEMM kernels can serve.
bool needs_mfma(const OgleConvArgs& a) {
  return a.output2_dev != nullptr ||
         (a.out_image_stride != 0 && a.out_image_stride != (int64_t)a.out_h * a.out_w * a.out_c);
}

// launch_conv_direct for the batch entry point: it writes one dense output.
int32_t direct_no_split(const OgleConvArgs& a, hipStream_t s) {
  if (needs_mfma(a)) return fail(OGLE_ERR_UNSUPPORTED, kSplitNeedsMfma);
  return launch_conv_direct(a, s);
}

// Byte extents of a convolution's tensors.  A span is `count` runs of `run` bytes whose
// starts lie `stride` bytes apart (count 1: one plain range); an output written with
// out_image_stride is one run per image.
struct Span {
  const void* ptr;
  size_t run, stride;
  long count;
};
size_t elem_bytes(const OgleConvArgs& a) { return a.dtype == OGLE_F16 ? 2 : 4; }
Span plain(const void* p, size_t bytes) { return Span{p, bytes, 0, 1}; }
Span input_span(const OgleConvArgs& a) {
  return plain(a.input_dev, (size_t)a.n * a.in_h * a.in_w * a.in_c * elem_bytes(a));
}
Span output_span(const OgleConvArgs& a) {
  const int c = a.output2_dev != nullptr ? a.out_c_split : a.out_c;
  const size_t image = (size_t)a.out_h * a.out_w * c * elem_bytes(a);
  if (a.out_image_stride == 0 || a.n == 1 || (size_t)a.out_image_stride * elem_bytes(a) == image)
    return plain(a.output_dev, image * a.n);
  return Span{a.output_dev, image, (size_t)a.out_image_stride * elem_bytes(a), a.n};
}
Span output2_span(const OgleConvArgs& a) {
  if (a.output2_dev == nullptr) return plain(nullptr, 0);
  return plain(a.output2_dev,
               (size_t)a.n * a.out_h * a.out_w * (a.out_c - a.out_c_split) * elem_bytes(a));
}
Span workspace_span(const OgleConvArgs& a) { return plain(a.workspace_dev, a.workspace_bytes); }
// True if the two spans share a byte.  Two spans of the same stride are compared by where
// their runs lie inside one period (exact when both cover the same images, otherwise on
// the safe side); other strided pairs run by run.
bool overlap(const Span& a, const Span& b) {
  if (a.ptr == nullptr || b.ptr == nullptr || a.run == 0 || b.run == 0) return false;
  const uintptr_t a0 = reinterpret_cast<uintptr_t>(a.ptr), b0 = reinterpret_cast<uintptr_t>(b.ptr);
  const uintptr_t a1 = a0 + (size_t)(a.count - 1) * a.stride + a.run;
  const uintptr_t b1 = b0 + (size_t)(b.count - 1) * b.stride + b.run;
  if (!(a0 < b1 && b0 < a1)) return false;
  if (a.count == 1 && b.count == 1) return true;
  if (a.count > 1 && b.count > 1) {
    if (a.stride != b.stride || a.run > a.stride || b.run > b.stride) return true;
    const size_t d = b0 >= a0 ? (b0 - a0) % a.stride : (a.stride - (a0 - b0) % a.stride) % a.stride;
    return d < a.run || d + b.run > a.stride;
  }
  const Span& many = a.count > 1 ? a : b;
  const Span& one = a.count > 1 ? b : a;
  const uintptr_t m0 = reinterpret_cast<uintptr_t>(many.ptr), o0 = reinterpret_cast<uintptr_t>(one.ptr);
  for (long i = 0; i < many.count; ++i) {
    const uintptr_t r0 = m0 + (size_t)i * many.stride;
    if (r0 < o0 + one.run && o0 < r0 + many.run) return true;
  }
  return false;
}

int32_t validate_conv(const OgleConvArgs* a, const char* who) {
  if (a == nullptr) return fail(OGLE_ERR_INVALID_ARG, "null args");
  if (!a->input_dev || !a->filter_dev || !a->output_dev) {
    set_error("%s: null device pointer", who);
    return OGLE_ERR_INVALID_ARG;
  }
  if (!positive(a->n) || !positive(a->in_h) || !positive(a->in_w) || !positive(a->in_c) ||
      !positive(a->out_c) || !positive(a->kernel_size) || !positive(a->stride) ||
      a->padding < 0 || !positive(a->dilation) || !positive(a->group)) {
    set_error("%s: non-positive shape or attribute", who);
    return OGLE_ERR_INVALID_ARG;
  }
  if (a->dtype != OGLE_F32 && a->dtype != OGLE_F16) {
    set_error("%s: unknown dtype %d", who, a->dtype);
    return OGLE_ERR_INVALID_ARG;
  }
  if (a->workspace_dev == nullptr && a->workspace_bytes != 0) {
    set_error("%s: workspace_bytes without workspace_dev", who);
    return OGLE_ERR_INVALID_ARG;
  }
  if (a->act < OGLE_ACT_NONE || a->act > OGLE_ACT_RELU) {
    set_error("%s: unknown activation %d", who, a->act);
    return OGLE_ERR_INVALID_ARG;
  }
  // Output size rule of Conv2DKernel::InferOutputShape (conv2d.cc:191-193).
  const int keff = a->kernel_size * a->dilation - a->dilation + 1;
  const int oh = (a->in_h - keff + 2 * a->padding) / a->stride + 1;
  const int ow = (a->in_w - keff + 2 * a->padding) / a->stride + 1;
  if (oh != a->out_h || ow != a->out_w || oh <= 0 || ow <= 0) {
    set_error("%s: output %dx%d does not follow from input %dx%d k%d s%d p%d d%d (expect %dx%d)",
              who, a->out_h, a->out_w, a->in_h, a->in_w, a->kernel_size, a->stride, a->padding,
              a->dilation, oh, ow);
    return OGLE_ERR_INVALID_ARG;
  }
  if (a->output2_dev != nullptr && (a->out_c_split <= 0 || a->out_c_split >= a->out_c)) {
    set_error("%s: out_c_split %d must lie strictly between 0 and out_c %d", who, a->out_c_split,
              a->out_c);
    return OGLE_ERR_INVALID_ARG;
  }
  if (a->out_image_stride != 0) {
    if (a->out_image_stride < (int64_t)a->out_h * a->out_w * a->out_c) {
      set_error("%s: out_image_stride %lld is less than one image's %d x %d x %d outputs", who,
                (long long)a->out_image_stride, a->out_h, a->out_w, a->out_c);
      return OGLE_ERR_INVALID_ARG;
    }
    if (a->output2_dev != nullptr) {
      set_error("%s: out_image_stride cannot be combined with output2_dev", who);
      return OGLE_ERR_INVALID_ARG;
    }
  }
  if (a->in_c % a->group != 0 || a->out_c % a->group != 0) {
    set_error("%s: channels %d -> %d not divisible by group %d", who, a->in_c, a->out_c, a->group);
    return OGLE_ERR_INVALID_ARG;
  }
  return OGLE_OK;
}

}  // namespace
}  // namespace ogle

using namespace ogle;

extern "C" {

int32_t ogle_hip_abi_version(void) { return 101; }

int64_t ogle_hip_launch_count(void) { return g_launches; }

int32_t ogle_hip_kernel_timing_begin(void) {
  for (auto& e : g_timing.events) {
    if (e.first != nullptr) (void)hipEventDestroy(e.first);
    if (e.second != nullptr) (void)hipEventDestroy(e.second);
  }
  g_timing.events.clear();
  g_timing.on = true;
  return OGLE_OK;
}

int64_t ogle_hip_kernel_timing_end(float* microseconds, int64_t capacity) {
  g_timing.on = false;
  const int64_t n = (int64_t)g_timing.events.size();
  int32_t status = OGLE_OK;
  for (int64_t i = 0; i < n; ++i) {
    auto& e = g_timing.events[i];
    float ms = 0.f;
    if (e.first != nullptr) {
      if (hipEventSynchronize(e.second) != hipSuccess ||
          hipEventElapsedTime(&ms, e.first, e.second) != hipSuccess) {
        set_error("kernel_timing_end: event %lld could not be read", (long long)i);
        status = OGLE_ERR_LAUNCH;
      }
      (void)hipEventDestroy(e.first);
      (void)hipEventDestroy(e.second);
    }
    if (microseconds != nullptr && i < capacity) microseconds[i] = ms * 1e3f;
  }
  g_timing.events.clear();
  return status != OGLE_OK ? status : n;
}

const char* ogle_hip_last_error(void) { return g_error; }

const char* ogle_hip_status_string(int32_t status) {
  switch (status) {
    case OGLE_OK: return "ok";
    case OGLE_ERR_INVALID_ARG: return "invalid argument";
    case OGLE_ERR_UNSUPPORTED: return "unsupported";
    case OGLE_ERR_LAUNCH: return "launch failed";
    case OGLE_ERR_NOT_FOUND: return "not found";
    case OGLE_ERR_NO_DEVICE: return "no device";
    default: return "unknown status";
  }
}

int32_t ogle_hip_registry_size(void) { return kRegistrySize; }

const char* ogle_hip_registry_name(int32_t index) {
  if (index < 0 || index >= kRegistrySize) return nullptr;
  return kRegistry[index].name;
}

int32_t ogle_hip_registry_lookup(const char* name, const char* options, int32_t* handle) {
  if (name == nullptr || handle == nullptr) return fail(OGLE_ERR_INVALID_ARG, "null name/handle");
  for (int i = 0; i < kRegistrySize; ++i) {
    if (std::strcmp(kRegistry[i].name, name) != 0) continue;
    int flags = kRegistry[i].base_flags;
    if (options != nullptr) {
      if (std::strstr(options, "USE_BIAS")) flags |= FLAG_BIAS;
      if (std::strstr(options, "USE_CLIP")) flags |= FLAG_CLIP;
      if (std::strstr(options, "USE_RELU")) flags |= FLAG_RELU;
    }
    *handle = (kRegistry[i].family << 8) | flags;
    return OGLE_OK;
  }
  set_error("registry: no kernel named '%s'", name);
  return OGLE_ERR_NOT_FOUND;
}

int32_t ogle_hip_sync(ogle_stream_t stream) {
  const hipError_t e = hipStreamSynchronize(as_stream(stream));
  if (e != hipSuccess) {
    set_error("sync: %s", hipGetErrorString(e));
    return OGLE_ERR_LAUNCH;
  }
  return OGLE_OK;
}

int64_t ogle_hip_packed_filter_elems(int32_t layout, int32_t o, int32_t i, int32_t kh,
                                     int32_t kw) {
  if (o <= 0 || i <= 0 || kh <= 0 || kw <= 0) return -1;
  if (layout == OGLE_FILTER_OHWI) return (int64_t)o * i * kh * kw;
  if (layout == OGLE_FILTER_HWC) return i == 1 ? (int64_t)o * kh * kw : -1;
  return -1;
}

int32_t ogle_hip_pack_filter(const float* oihw_dev, void* packed_dev, int32_t layout,
                             int32_t dtype, int32_t o, int32_t i, int32_t kh, int32_t kw,
                             ogle_stream_t stream) {
  if (!oihw_dev || !packed_dev) return fail(OGLE_ERR_INVALID_ARG, "pack_filter: null pointer");
  if (ogle_hip_packed_filter_elems(layout, o, i, kh, kw) < 0)
    return fail(OGLE_ERR_INVALID_ARG, "pack_filter: bad layout or shape");
  if (dtype != OGLE_F32 && dtype != OGLE_F16)
    return fail(OGLE_ERR_INVALID_ARG, "pack_filter: unknown dtype");
  return launch_pack_filter(oihw_dev, packed_dev, layout, dtype, o, i, kh, kw, as_stream(stream));
}

int32_t ogle_hip_convert(const void* src_dev, int32_t src_dtype, void* dst_dev,
                         int32_t dst_dtype, int64_t count, ogle_stream_t stream) {
  if (count < 0 || (count > 0 && (!src_dev || !dst_dev)))
    return fail(OGLE_ERR_INVALID_ARG, "convert: null pointer or negative count");
  if ((src_dtype != OGLE_F32 && src_dtype != OGLE_F16) ||
      (dst_dtype != OGLE_F32 && dst_dtype != OGLE_F16))
    return fail(OGLE_ERR_INVALID_ARG, "convert: unknown dtype");
  return launch_convert(src_dev, src_dtype, dst_dev, dst_dtype, count, as_stream(stream));
}

size_t ogle_hip_conv_workspace_bytes(const OgleConvArgs* a) {
  if (a == nullptr) return 0;
  OgleConvArgs q = *a;  // a size query needs no buffers: only shapes are validated
  static char dummy;
  q.input_dev = q.filter_dev = &dummy;
  q.output_dev = &dummy;
  q.workspace_dev = nullptr;
  q.workspace_bytes = 0;
  if (validate_conv(&q, "conv_workspace_bytes") != OGLE_OK) return 0;
  if (q.group == q.in_c && q.group == q.out_c && q.group != 1) return 0;  // depthwise
  return conv_igemm_workspace_bytes(q);
}

int32_t ogle_hip_conv_takes_image_stride(const OgleConvArgs* a) {
  if (a == nullptr) return 0;
  OgleConvArgs q = *a;  // pointers are not looked at: only shapes are validated
  static char dummy;
  q.input_dev = q.filter_dev = &dummy;
  q.output_dev = &dummy;
  q.output2_dev = nullptr;
  q.out_image_stride = 0;
  q.workspace_dev = nullptr;
  q.workspace_bytes = 0;
  if (validate_conv(&q, "conv_takes_image_stride") != OGLE_OK) return 0;
  return conv_igemm_takes(q) ? 1 : 0;
}

int32_t ogle_hip_conv2d(const OgleConvArgs* a, ogle_stream_t stream) {
  int32_t st = validate_conv(a, "conv2d");
  if (st != OGLE_OK) return st;
  if (a->group == 1) {
    st = launch_conv_igemm(*a, as_stream(stream));
    if (st != OGLE_ERR_UNSUPPORTED) return st;
  }
  if (needs_mfma(*a)) return fail(OGLE_ERR_UNSUPPORTED, kSplitNeedsMfma);
  return launch_conv_direct(*a, as_stream(stream));
}

int32_t ogle_hip_conv2d_noalloc(const OgleConvArgs* a, ogle_stream_t stream) {
  int32_t st = validate_conv(a, "conv2d_noalloc");
  if (st != OGLE_OK) return st;
  if (a->workspace_dev != nullptr || a->workspace_bytes != 0)
    return fail(OGLE_ERR_INVALID_ARG,
                "conv2d_noalloc: workspace_dev must be NULL (the scratch is built in)");
  if (a->group == 1) {
    st = launch_conv_igemm_static_scratch(*a, as_stream(stream));
    if (st != OGLE_ERR_UNSUPPORTED) return st;
  }
  if (needs_mfma(*a)) return fail(OGLE_ERR_UNSUPPORTED, kSplitNeedsMfma);
  return launch_conv_direct(*a, as_stream(stream));
}

namespace {
int32_t conv2d_batch_impl(const OgleConvArgs* args, int32_t count, int32_t* reduce_pending,
                          ogle_stream_t stream);
}

int32_t ogle_hip_conv2d_batch(const OgleConvArgs* args, int32_t count, ogle_stream_t stream) {
  return conv2d_batch_impl(args, count, nullptr, stream);
}

int32_t ogle_hip_conv2d_batch_begin(const OgleConvArgs* args, int32_t count,
                                    int32_t* reduce_pending, ogle_stream_t stream) {
  if (count > 0 && reduce_pending == nullptr)
    return fail(OGLE_ERR_INVALID_ARG, "conv2d_batch_begin: reduce_pending is required");
  return conv2d_batch_impl(args, count, reduce_pending, stream);
}

int32_t ogle_hip_conv2d_batch_finish(const OgleConvArgs* args, int32_t count, ogle_stream_t stream) {
  if (count < 0 || (count > 0 && args == nullptr))
    return fail(OGLE_ERR_INVALID_ARG, "conv2d_batch_finish: null args or negative count");
  for (int i = 0; i < count; ++i) {
    const int32_t st = validate_conv(&args[i], "conv2d_batch_finish");
    if (st != OGLE_OK) return st;
  }
  return launch_conv_reduce(args, count, as_stream(stream));
}

namespace {
int32_t conv2d_batch_impl(const OgleConvArgs* args, int32_t count, int32_t* reduce_pending,
                          ogle_stream_t stream) {
  if (count < 0 || (count > 0 && args == nullptr))
    return fail(OGLE_ERR_INVALID_ARG, "conv2d_batch: null args or negative count");
  for (int i = 0; i < count; ++i) {
    const int32_t st = validate_conv(&args[i], "conv2d_batch");
    if (st != OGLE_OK) return st;
    for (int j = 0; j < i; ++j) {
      const OgleConvArgs &p = args[i], &q = args[j];
      if (overlap(input_span(p), output_span(q)) || overlap(input_span(q), output_span(p)) ||
          overlap(output_span(p), output_span(q)))
        return fail(OGLE_ERR_INVALID_ARG, "conv2d_batch: the convolutions depend on each other");
      if (overlap(output2_span(p), input_span(q)) || overlap(output2_span(q), input_span(p)) ||
          overlap(output2_span(p), output_span(q)) || overlap(output2_span(q), output_span(p)) ||
          overlap(output2_span(p), output2_span(q)))
        return fail(OGLE_ERR_INVALID_ARG, "conv2d_batch: the convolutions depend on each other");
      if (overlap(workspace_span(p), workspace_span(q)))
        return fail(OGLE_ERR_INVALID_ARG, "conv2d_batch: two convolutions share one workspace");
      if (overlap(workspace_span(p), output_span(q)) || overlap(workspace_span(q), output_span(p)) ||
          overlap(workspace_span(p), input_span(q)) || overlap(workspace_span(q), input_span(p)))
        return fail(OGLE_ERR_INVALID_ARG,
                    "conv2d_batch: a workspace overlaps another convolution's tensor");
    }
  }
  return launch_conv_batch(args, count, as_stream(stream), direct_no_split, reduce_pending);
}
}  // namespace

int32_t ogle_hip_dwconv2d(const OgleConvArgs* a, ogle_stream_t stream) {
  int32_t st = validate_conv(a, "dwconv2d");
  if (st != OGLE_OK) return st;
  // conv2d.cc:27-29,41: depthwise means group == C_in (== C_out).
  if (a->group != a->in_c || a->out_c != a->in_c) {
    set_error("dwconv2d: group %d must equal in_c %d and out_c %d", a->group, a->in_c, a->out_c);
    return OGLE_ERR_INVALID_ARG;
  }
  if (needs_mfma(*a)) return fail(OGLE_ERR_UNSUPPORTED, kSplitNeedsMfma);
  return launch_conv_dw(*a, as_stream(stream));
}

int32_t ogle_hip_pwconv_gemm(const OgleConvArgs* a, ogle_stream_t stream) {
  int32_t st = validate_conv(a, "pwconv_gemm");
  if (st != OGLE_OK) return st;
  // conv2d.cc:37: the pointwise shader is chosen only for 1x1, g1, d1, s1, p0.
  if (a->kernel_size != 1 || a->group != 1 || a->dilation != 1 || a->stride != 1 ||
      a->padding != 0) {
    set_error("pwconv_gemm: needs kernel 1, group 1, dilation 1, stride 1, padding 0");
    return OGLE_ERR_INVALID_ARG;
  }
  st = launch_conv_igemm(*a, as_stream(stream));
  if (st != OGLE_ERR_UNSUPPORTED) return st;
  if (needs_mfma(*a)) return fail(OGLE_ERR_UNSUPPORTED, kSplitNeedsMfma);
  return launch_conv_direct(*a, as_stream(stream));
}

int32_t ogle_hip_pool2d(const OglePoolArgs* a, ogle_stream_t stream) {
  if (a == nullptr) return fail(OGLE_ERR_INVALID_ARG, "pool2d: null args");
  if (!a->input_dev || !a->output_dev) return fail(OGLE_ERR_INVALID_ARG, "pool2d: null pointer");
  if (!positive(a->n) || !positive(a->in_h) || !positive(a->in_w) || !positive(a->c) ||
      !positive(a->kernel_size) || !positive(a->stride) || a->padding < 0)
    return fail(OGLE_ERR_INVALID_ARG, "pool2d: non-positive shape or attribute");
  if (a->pool_type < OGLE_POOL_MAX || a->pool_type > OGLE_POOL_GLOBAL_AVG)
    return fail(OGLE_ERR_INVALID_ARG, "pool2d: unknown pool_type");
  if (a->dtype != OGLE_F32 && a->dtype != OGLE_F16)
    return fail(OGLE_ERR_INVALID_ARG, "pool2d: unknown dtype");
  if (a->pool_type == OGLE_POOL_GLOBAL_AVG &&
      (a->in_h != a->in_w || a->kernel_size != a->in_h || a->stride != 1 || a->padding != 0))
    return fail(OGLE_ERR_INVALID_ARG,
                "pool2d: global average needs a square input, kernel = H, stride 1, padding 0");
  // pool.cc:94-96
  const int oh = (a->in_h - a->kernel_size + 2 * a->padding) / a->stride + 1;
  const int ow = (a->in_w - a->kernel_size + 2 * a->padding) / a->stride + 1;
  if (oh != a->out_h || ow != a->out_w || oh <= 0 || ow <= 0) {
    set_error("pool2d: output %dx%d does not follow from the input (expect %dx%d)", a->out_h,
              a->out_w, oh, ow);
    return OGLE_ERR_INVALID_ARG;
  }
  return launch_pool(*a, as_stream(stream));
}

int32_t ogle_hip_concat(const OgleConcatArgs* a, ogle_stream_t stream) {
  if (a == nullptr) return fail(OGLE_ERR_INVALID_ARG, "concat: null args");
  if (a->n_inputs < 1 || a->n_inputs > OGLE_CONCAT_MAX_INPUTS) {
    set_error("concat: %d inputs (1..%d allowed)", a->n_inputs, OGLE_CONCAT_MAX_INPUTS);
    return OGLE_ERR_INVALID_ARG;
  }
  if (a->outer < 0 || a->inner < 0) return fail(OGLE_ERR_INVALID_ARG, "concat: negative extent");
  if (a->dtype != OGLE_F32 && a->dtype != OGLE_F16)
    return fail(OGLE_ERR_INVALID_ARG, "concat: unknown dtype");
  int64_t total = 0;
  for (int i = 0; i < a->n_inputs; ++i) {
    if (a->axis_len[i] < 0) return fail(OGLE_ERR_INVALID_ARG, "concat: negative axis length");
    if (a->axis_len[i] > 0 && a->inputs_dev[i] == nullptr && a->outer * a->inner > 0)
      return fail(OGLE_ERR_INVALID_ARG, "concat: null input");
    total += a->axis_len[i];
  }
  if (total * a->outer * a->inner > 0 && a->output_dev == nullptr)
    return fail(OGLE_ERR_INVALID_ARG, "concat: null output");
  return launch_concat(*a, as_stream(stream));
}

int32_t ogle_hip_transpose(const OgleTransposeArgs* a, ogle_stream_t stream) {
  if (a == nullptr) return fail(OGLE_ERR_INVALID_ARG, "transpose: null args");
  if (a->dtype != OGLE_F32 && a->dtype != OGLE_F16)
    return fail(OGLE_ERR_INVALID_ARG, "transpose: unknown dtype");
  int seen = 0;
  int64_t total = 1;
  for (int d = 0; d < 4; ++d) {
    if (a->perm[d] < 0 || a->perm[d] > 3 || a->in_shape[d] < 0)
      return fail(OGLE_ERR_INVALID_ARG, "transpose: bad perm or shape");
    seen |= 1 << a->perm[d];
    total *= a->in_shape[d];
  }
  if (seen != 15) return fail(OGLE_ERR_INVALID_ARG, "transpose: perm is not a permutation");
  if (total > 0 && (!a->input_dev || !a->output_dev))
    return fail(OGLE_ERR_INVALID_ARG, "transpose: null pointer");
  return launch_transpose(*a, as_stream(stream));
}

int32_t ogle_hip_ssd_decode(const OgleDecodeArgs* a, ogle_stream_t stream) {
  if (a == nullptr) return fail(OGLE_ERR_INVALID_ARG, "ssd_decode: null args");
  if (a->batch < 0 || a->priors < 0) return fail(OGLE_ERR_INVALID_ARG, "ssd_decode: negative size");
  if ((long)a->batch * a->priors > 0 && (!a->prediction_dev || !a->anchors_dev || !a->boxes_dev))
    return fail(OGLE_ERR_INVALID_ARG, "ssd_decode: null pointer");
  // decoder.cc:82-85: anchors are either shared or one set per image.
  if (a->anchors_batch_stride != 0 && a->anchors_batch_stride != (int64_t)a->priors * 4)
    return fail(OGLE_ERR_INVALID_ARG, "ssd_decode: anchors_batch_stride must be 0 or priors*4");
  return launch_decode(*a, as_stream(stream));
}

int32_t ogle_hip_ssd_detect(const OgleDetectArgs* a, ogle_stream_t stream) {
  if (a == nullptr) return fail(OGLE_ERR_INVALID_ARG, "ssd_detect: null args");
  if (a->batch < 0 || a->priors < 0 || a->classes < 1)
    return fail(OGLE_ERR_INVALID_ARG, "ssd_detect: bad size");
  if (a->classes > 40)  // the logit slab of 256 priors must fit LDS
    return fail(OGLE_ERR_UNSUPPORTED, "ssd_detect: more than 40 classes");
  if (!a->kept_count_dev && a->batch > 0 &&
      (!a->kept_prior_dev || !a->kept_class_dev || !a->kept_score_dev || !a->kept_box_dev ||
       !a->kept_rect_dev || a->batch > 65535))
    return fail(OGLE_ERR_INVALID_ARG,
                "ssd_detect: without kept_count_dev (lists left in place) every other list is "
                "required and batch <= 65535");
  if ((long)a->batch * a->priors > 0) {
    if (!a->logits_dev) return fail(OGLE_ERR_INVALID_ARG, "ssd_detect: null logits");
    if (a->prediction_dev && !a->anchors_dev)
      return fail(OGLE_ERR_INVALID_ARG, "ssd_detect: prediction without anchors");
    if (!a->prediction_dev && !a->boxes_dev)
      return fail(OGLE_ERR_INVALID_ARG, "ssd_detect: neither prediction nor decoded boxes");
  }
  if (a->anchors_batch_stride != 0 && a->anchors_batch_stride != (int64_t)a->priors * 4)
    return fail(OGLE_ERR_INVALID_ARG, "ssd_detect: anchors_batch_stride must be 0 or priors*4");
  return launch_detect(*a, as_stream(stream));
}

namespace {
bool misaligned(const void* p, uintptr_t bytes) {
  return (reinterpret_cast<uintptr_t>(p) & (bytes - 1)) != 0;
}
bool bad_dtype(int32_t d) { return d != OGLE_F32 && d != OGLE_F16; }
}  // namespace

int32_t ogle_hip_unary(const OgleUnaryArgs* a, ogle_stream_t stream) {
  if (a == nullptr) return fail(OGLE_ERR_INVALID_ARG, "unary: null args");
  if (a->count < 0 || bad_dtype(a->dtype)) return fail(OGLE_ERR_INVALID_ARG, "unary: bad count or dtype");
  if (a->op != OGLE_UNARY_RELU && a->op != OGLE_UNARY_CLIP)
    return fail(OGLE_ERR_UNSUPPORTED, "unary: unknown op");
  if (a->count > 0 && (!a->input_dev || !a->output_dev))
    return fail(OGLE_ERR_INVALID_ARG, "unary: null device pointer");
  if (misaligned(a->input_dev, 16) || misaligned(a->output_dev, 16))
    return fail(OGLE_ERR_INVALID_ARG, "unary: pointers must be 16-byte aligned");
  return launch_unary(*a, as_stream(stream));
}

int32_t ogle_hip_add(const OgleBinaryArgs* a, ogle_stream_t stream) {
  if (a == nullptr) return fail(OGLE_ERR_INVALID_ARG, "add: null args");
  if (a->count < 0 || bad_dtype(a->dtype)) return fail(OGLE_ERR_INVALID_ARG, "add: bad count or dtype");
  if (a->count > 0 && (!a->a_dev || !a->b_dev || !a->output_dev))
    return fail(OGLE_ERR_INVALID_ARG, "add: null device pointer");
  if (misaligned(a->a_dev, 16) || misaligned(a->b_dev, 16) || misaligned(a->output_dev, 16))
    return fail(OGLE_ERR_INVALID_ARG, "add: pointers must be 16-byte aligned");
  return launch_binary(*a, as_stream(stream));
}

int32_t ogle_hip_batchnorm(const OgleBatchNormArgs* a, ogle_stream_t stream) {
  if (a == nullptr) return fail(OGLE_ERR_INVALID_ARG, "batchnorm: null args");
  if (a->outer < 0 || a->channels < 1 || bad_dtype(a->dtype))
    return fail(OGLE_ERR_INVALID_ARG, "batchnorm: bad size or dtype");
  if (a->outer > 0 && (!a->input_dev || !a->output_dev || !a->gamma_dev || !a->beta_dev ||
                       !a->mean_dev || !a->var_dev))
    return fail(OGLE_ERR_INVALID_ARG, "batchnorm: null device pointer");
  if (misaligned(a->input_dev, 16) || misaligned(a->output_dev, 16))
    return fail(OGLE_ERR_INVALID_ARG, "batchnorm: tensors must be 16-byte aligned");
  return launch_batchnorm(*a, as_stream(stream));
}

namespace {
int32_t validate_gemm(const OgleGemmArgs* a) {
  if (a == nullptr) return fail(OGLE_ERR_INVALID_ARG, "gemm: null args");
  if (a->m < 0 || a->n < 0 || a->k < 1) return fail(OGLE_ERR_INVALID_ARG, "gemm: bad size");
  if (a->c_dev != nullptr && a->c_rank != 1 && a->c_rank != 2)
    return fail(OGLE_ERR_INVALID_ARG, "gemm: c_rank must be 1 or 2");
  if (a->workspace_dev == nullptr && a->workspace_bytes != 0)
    return fail(OGLE_ERR_INVALID_ARG, "gemm: workspace_bytes without workspace_dev");
  return OGLE_OK;
}
}  // namespace

size_t ogle_hip_gemm_workspace_bytes(const OgleGemmArgs* a) {
  if (validate_gemm(a) != OGLE_OK || a->m == 0 || a->n == 0) return 0;
  return gemm_workspace_bytes(*a);
}

int32_t ogle_hip_gemm(const OgleGemmArgs* a, ogle_stream_t stream) {
  const int32_t st = validate_gemm(a);
  if (st != OGLE_OK) return st;
  if ((long)a->m * a->n > 0 && (!a->a_dev || !a->b_dev || !a->y_dev))
    return fail(OGLE_ERR_INVALID_ARG, "gemm: null device pointer");
  return launch_gemm(*a, as_stream(stream));
}

int32_t ogle_hip_ssd_topk_nms(const OgleNmsArgs* a, ogle_stream_t stream) {
  if (a == nullptr) return fail(OGLE_ERR_INVALID_ARG, "ssd_topk_nms: null args");
  if (a->batch < 0 || a->stride < 0) return fail(OGLE_ERR_INVALID_ARG, "ssd_topk_nms: bad size");
  if (a->topk < 1 || a->topk > 1024)
    return fail(OGLE_ERR_UNSUPPORTED, "ssd_topk_nms: topk must be in 1..1024");
  if (a->stride > 8192 || topk_nms_lds_bytes(a->stride, a->topk) > 64 * 1024)
    return fail(OGLE_ERR_UNSUPPORTED,  // scores and candidates of one image are staged in LDS
                "ssd_topk_nms: more than 8192 entries per image, or stride*4 + topk*28 bytes "
                "exceed 64 KB of LDS");
  if (a->batch > 0) {
    if (!a->final_count_dev)
      return fail(OGLE_ERR_INVALID_ARG, "ssd_topk_nms: final_count_dev is required");
    if (a->stride > 0 && (!a->kept_prior_dev || !a->kept_class_dev || !a->kept_score_dev ||
                          !a->kept_rect_dev))
      return fail(OGLE_ERR_INVALID_ARG, "ssd_topk_nms: null input list");
    if (!a->final_prior_dev || !a->final_class_dev || !a->final_score_dev || !a->final_rect_dev)
      return fail(OGLE_ERR_INVALID_ARG, "ssd_topk_nms: null output list");
    if ((a->kept_box_dev == nullptr) != (a->final_box_dev == nullptr))
      return fail(OGLE_ERR_INVALID_ARG, "ssd_topk_nms: kept_box_dev and final_box_dev go together");
  }
  return launch_topk_nms(*a, as_stream(stream));
}

int32_t ogle_hip_expf(const float* x_dev, float* y_dev, int64_t count, ogle_stream_t stream) {
  if (count < 0 || (count > 0 && (!x_dev || !y_dev)))
    return fail(OGLE_ERR_INVALID_ARG, "expf: null pointer or negative count");
  return launch_expf(x_dev, y_dev, count, as_stream(stream));
}

}  // extern "C"
