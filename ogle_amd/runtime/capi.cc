// C ABI over the C++ graph runtime (include/ogle_runtime.h).
#include "ogle_runtime.h"

#include <hip/hip_runtime_api.h>

#include <chrono>
#include <cstring>
#include <exception>
#include <memory>
#include <string>
#include <vector>

#include "opengl/core/fbo_session.h"
#include "opengl/core/kernel.h"
#include "opengl/core/kernel_registry.h"
#include "opengl/core/tensor.h"
#include "opengl/examples/ssd/detector.h"

using opengl::FBOSession;
using opengl::Tensor;

struct OgleSession {
  std::unique_ptr<opengl::Context> context;
  std::unique_ptr<FBOSession> session;
  std::vector<opengl::NodeTiming> timings;
  std::unique_ptr<opengl::Detector> detector;
  bool device_nms = true;
  std::vector<opengl::Context::LaunchRecord> plan;
  std::vector<float> plan_us;  // duration of every device operation of the plan, in order
  // pipelined readback: the event behind the session's last pass whose final lists were
  // copied to the detector's page-locked memory and have not been read yet
  hipEvent_t lists_ready = nullptr;
  bool lists_pending = false;
  ~OgleSession() {
    if (lists_ready != nullptr) (void)hipEventDestroy(lists_ready);
  }
};

namespace {
thread_local std::string g_error;

template <typename F>
int64_t Guard(F&& f) {
  try {
    return f();
  } catch (const std::exception& e) {
    g_error = e.what();
    return -1;
  } catch (...) {
    g_error = "unknown exception";
    return -1;
  }
}
}  // namespace

extern "C" {

const char* ogle_rt_last_error(void) { return g_error.c_str(); }

OgleSession* ogle_rt_session_create(void) {
  OgleSession* s = nullptr;
  Guard([&]() -> int64_t {
    std::unique_ptr<OgleSession> p(new OgleSession);
    p->context.reset(new opengl::Context);
    p->session.reset(new FBOSession(p->context.get()));
    s = p.release();
    return 0;
  });
  return s;
}

void ogle_rt_session_destroy(OgleSession* s) {
  if (s == nullptr) return;
  Guard([&]() -> int64_t {
    s->detector.reset();
    s->session.reset();
    s->context.reset();
    return 0;
  });
  delete s;
}

int32_t ogle_rt_load_file(OgleSession* s, const char* path) {
  return (int32_t)Guard([&]() -> int64_t {
    s->session->LoadGraph(std::string(path));
    s->detector.reset();
    return 0;
  });
}

int32_t ogle_rt_load_bytes(OgleSession* s, const void* data, size_t size) {
  return (int32_t)Guard([&]() -> int64_t {
    dlxnet::ModelProto model;
    if (!model.ParseFromArray(data, size)) {
      g_error = "not a .dlx model";
      return -1;
    }
    s->session->LoadGraph(model);
    s->detector.reset();  // its device lists belonged to the previous graph's passes
    return 0;
  });
}

int32_t ogle_rt_set_fuse_siblings(OgleSession* s, int32_t on) {
  return (int32_t)Guard([&]() -> int64_t {
    s->session->set_fuse_siblings(on != 0);
    return 0;
  });
}

int32_t ogle_rt_graph_captured(OgleSession* s, int32_t slot) {
  if (s == nullptr || slot < 0 || slot >= FBOSession::kGraphSlots) return -1;
  return s->session->graph_captured(slot) ? 1 : 0;
}

int32_t ogle_rt_hazard_conflicts(const OgleConvArgs* pending, int32_t n_pending,
                                 const void* const* read_ptrs, const size_t* read_bytes,
                                 int32_t n_reads, const void* const* write_ptrs,
                                 const size_t* write_bytes, int32_t n_writes) {
  if (n_pending < 0 || n_reads < 0 || n_writes < 0) return -1;
  std::vector<opengl::MemRange> reads, writes;
  for (int i = 0; i < n_reads; ++i) reads.push_back({read_ptrs[i], read_bytes[i]});
  for (int i = 0; i < n_writes; ++i) writes.push_back({write_ptrs[i], write_bytes[i]});
  return opengl::Context::Conflicts(pending, n_pending, reads.data(), n_reads, writes.data(),
                                    n_writes)
             ? 1
             : 0;
}

int32_t ogle_rt_conv_hazard_conflicts(const OgleConvArgs* pending, int32_t n_pending,
                                      const OgleConvArgs* next) {
  if (n_pending < 0 || next == nullptr || (n_pending > 0 && pending == nullptr)) return -1;
  opengl::MemRange reads[3], writes[3];
  opengl::Context::ConvRanges(*next, reads, writes);
  return opengl::Context::Conflicts(pending, n_pending, reads, 3, writes, 3) ? 1 : 0;
}

int32_t ogle_rt_run(OgleSession* s, int32_t n_inputs, const char* const* names,
                    const float* const* data, const int32_t* const* dims, const int32_t* ranks,
                    const char* const* dformats) {
  return (int32_t)Guard([&]() -> int64_t {
    std::vector<std::unique_ptr<Tensor>> owned;
    opengl::NamedTensorList inputs;
    for (int i = 0; i < n_inputs; ++i) {
      opengl::IntList shape(dims[i], dims[i] + ranks[i]);
      owned.emplace_back(new Tensor(Tensor::DT_FLOAT, shape, data[i], opengl::StrToFormat(dformats[i])));
      inputs.emplace_back(names[i], owned.back().get());
    }
    s->session->Run(inputs);
    return 0;
  });
}

int64_t ogle_rt_host_elements(const int32_t* dims, int32_t rank, const char* dformat) {
  return Guard([&]() -> int64_t {
    opengl::IntList shape(dims, dims + rank);
    return (int64_t)opengl::HostElements(shape, opengl::StrToFormat(dformat));
  });
}

int32_t ogle_rt_compute(OgleSession* s) {
  return (int32_t)Guard([&]() -> int64_t {
    s->session->Compute();
    return 0;
  });
}

int32_t ogle_rt_compute_graph(OgleSession* s) {
  return (int32_t)Guard([&]() -> int64_t {
    if (!s->session->graph_captured()) s->session->CaptureGraph();
    s->session->LaunchGraph();
    return 0;
  });
}

int32_t ogle_rt_sync(OgleSession* s) {
  return (int32_t)Guard([&]() -> int64_t {
    s->context->Finish();
    return 0;
  });
}

int32_t ogle_rt_time_compute(OgleSession* s, int32_t warmup, int32_t iters, int32_t use_graph,
                             int32_t with_detect, int32_t sync_each, float* ms_each,
                             float* total_ms) {
  return (int32_t)Guard([&]() -> int64_t {
    hipStream_t st = static_cast<hipStream_t>(s->context->stream());
    opengl::DetectorOptions opt;
    opt.device_nms = s->device_nms;
    if (with_detect && !s->detector) s->detector = opengl::Detector::Create(s->session.get(), opt);
    auto detect = [&]() {
      s->detector->EnqueueDetect(opt.output_names, 300, 300);
    };
    if (with_detect) {
      detect();  // first use allocates the result buffers: keep that out of a capture
      s->context->Finish();
    }
    // slot 0: the pass alone; slot 1: the pass followed by the detector's device work
    const int slot = with_detect ? 1 : 0;
    auto pass = [&]() {
      if (use_graph) {
        if (!s->session->graph_captured(slot)) {
          if (with_detect) s->session->CaptureGraph(slot, detect);
          else s->session->CaptureGraph(slot);
        }
        s->session->LaunchGraph(slot);
      } else {
        s->session->Compute();
        if (with_detect) detect();
      }
      if (sync_each) s->context->Finish();
    };
    for (int i = 0; i < warmup; ++i) pass();
    s->context->Finish();
    std::vector<hipEvent_t> ev(iters + 1);
    for (auto& e : ev)
      if (hipEventCreate(&e) != hipSuccess) LOG(FATAL) << "hipEventCreate failed";
    (void)hipEventRecord(ev[0], st);
    for (int i = 0; i < iters; ++i) {
      pass();
      (void)hipEventRecord(ev[i + 1], st);
    }
    s->context->Finish();
    float total = 0.f;
    (void)hipEventElapsedTime(&total, ev[0], ev[iters]);
    if (total_ms) *total_ms = total;
    if (ms_each)
      for (int i = 0; i < iters; ++i) (void)hipEventElapsedTime(&ms_each[i], ev[i], ev[i + 1]);
    for (auto& e : ev) (void)hipEventDestroy(e);
    return 0;
  });
}

int32_t ogle_rt_launch_plan(OgleSession* s, int32_t with_detect) {
  return (int32_t)Guard([&]() -> int64_t {
    opengl::DetectorOptions opt;
    opt.device_nms = s->device_nms;
    if (with_detect && !s->detector) {
      s->detector = opengl::Detector::Create(s->session.get(), opt);
      s->detector->EnqueueDetect(opt.output_names, 300, 300);  // first use allocates
      s->context->Finish();
    }
    s->context->Finish();
    s->context->set_launch_log(true);
    (void)ogle_hip_kernel_timing_begin();
    try {
      s->session->Compute();
      if (with_detect) s->detector->EnqueueDetect(opt.output_names, 300, 300);
      s->context->Flush();
    } catch (...) {
      s->context->set_launch_log(false);
      (void)ogle_hip_kernel_timing_end(nullptr, 0);
      throw;
    }
    s->plan = s->context->launch_log();
    s->context->set_launch_log(false);
    int64_t dispatches = 0;
    for (const auto& r : s->plan) dispatches += r.dispatches;
    std::vector<float> us(static_cast<size_t>(dispatches > 0 ? dispatches : 1), 0.f);
    const int64_t timed = ogle_hip_kernel_timing_end(us.data(), dispatches);
    s->context->Finish();
    CHECK(timed == dispatches) << "kernel timing saw " << timed << " device operations, the launch log "
                               << dispatches << " (" << ogle_hip_last_error() << ")";
    s->plan_us.assign(us.begin(), us.begin() + dispatches);
    return (int64_t)s->plan.size();
  });
}

int32_t ogle_rt_launch_plan_entry(OgleSession* s, int32_t i, const char** label,
                                  int32_t* dispatches, float* microseconds, int32_t capacity) {
  if (s == nullptr || i < 0 || i >= (int32_t)s->plan.size()) return -1;
  if (label) *label = s->plan[i].label.c_str();
  if (dispatches) *dispatches = s->plan[i].dispatches;
  size_t at = 0;
  for (int32_t j = 0; j < i; ++j) at += s->plan[j].dispatches;
  for (int32_t k = 0; k < s->plan[i].dispatches && k < capacity && microseconds != nullptr; ++k)
    microseconds[k] = s->plan_us[at + k];
  return 0;
}

void* ogle_rt_alloc_pinned(size_t bytes) {
  void* p = nullptr;
  if (bytes == 0 || hipHostMalloc(&p, bytes, hipHostMallocDefault) != hipSuccess) return nullptr;
  return p;
}

void ogle_rt_free_pinned(void* p) {
  if (p != nullptr) (void)hipHostFree(p);
}

int32_t ogle_rt_time_pipelined(OgleSession** sessions, int32_t n, int32_t warmup, int32_t iters,
                               int32_t with_detect, const char* input_name,
                               const void* const* host_inputs, float* total_ms) {
  return (int32_t)Guard([&]() -> int64_t {
    CHECK(sessions != nullptr && n >= 1 && n <= 16) << "1..16 sessions";
    const int slot = with_detect ? 1 : 0;
    std::vector<void*> dev_input(n, nullptr);
    std::vector<size_t> input_bytes(n, 0);
    if (host_inputs != nullptr) {
      CHECK(input_name != nullptr) << "input_name is required with host_inputs";
      for (int i = 0; i < n; ++i) {
        CHECK(sessions[i] != nullptr && host_inputs[i] != nullptr) << "null session or host input";
        Tensor* t = sessions[i]->session->FindTensorByName(input_name);
        CHECK(t != nullptr && t->device_ptr() != nullptr)
            << "input '" << input_name << "' is not resident: Run the session once first";
        dev_input[i] = t->device_ptr();
        input_bytes[i] = t->num_elements() * sizeof(float);
      }
    }
    for (int i = 0; i < n; ++i) {
      OgleSession* s = sessions[i];
      CHECK(s != nullptr && s->session != nullptr) << "null session";
      if (with_detect) {
        opengl::DetectorOptions opt;
        opt.device_nms = s->device_nms;
        if (!s->detector) s->detector = opengl::Detector::Create(s->session.get(), opt);
        auto detect = [s, opt]() { s->detector->EnqueueDetect(opt.output_names, 300, 300); };
        if (!s->session->graph_captured(slot)) {
          detect();  // first use allocates the result buffers: keep that out of the capture
          s->context->Finish();
          s->session->CaptureGraph(slot, detect);
        }
      } else if (!s->session->graph_captured(slot)) {
        s->session->CaptureGraph(slot);
      }
    }
    auto idle = [&]() {
      for (int i = 0; i < n; ++i) sessions[i]->context->Finish();
    };
    auto step = [&](int i) {
      OgleSession* s = sessions[i % n];
      if (host_inputs != nullptr) {
        const hipError_t e =
            hipMemcpyAsync(dev_input[i % n], host_inputs[i % n], input_bytes[i % n],
                           hipMemcpyHostToDevice, static_cast<hipStream_t>(s->context->stream()));
        if (e != hipSuccess) LOG(FATAL) << "input upload: " << hipGetErrorString(e);
      }
      s->session->LaunchGraph(slot);
    };
    for (int i = 0; i < warmup; ++i) step(i);
    idle();
    const auto t0 = std::chrono::steady_clock::now();
    for (int i = 0; i < iters; ++i) step(i);
    idle();
    const auto t1 = std::chrono::steady_clock::now();
    if (total_ms) *total_ms = std::chrono::duration<float, std::milli>(t1 - t0).count();
    return 0;
  });
}

int32_t ogle_rt_profile(OgleSession* s) {
  return (int32_t)Guard([&]() -> int64_t {
    s->session->RunProfiled(&s->timings);
    return (int64_t)s->timings.size();
  });
}

int32_t ogle_rt_profile_entry(OgleSession* s, int32_t i, const char** label, const char** type,
                              float* ms) {
  if (i < 0 || i >= (int32_t)s->timings.size()) {
    g_error = "profile entry out of range";
    return -1;
  }
  if (label) *label = s->timings[i].name.c_str();
  if (type) *type = s->timings[i].type.c_str();
  if (ms) *ms = s->timings[i].ms;
  return 0;
}

int32_t ogle_rt_tensor_shape(OgleSession* s, const char* name, int32_t* dims) {
  return (int32_t)Guard([&]() -> int64_t {
    Tensor* t = s->session->FindTensorByName(name);
    if (t == nullptr) {
      g_error = std::string("tensor '") + name + "' is not allocated";
      return -1;
    }
    const auto& shape = t->shape();
    for (size_t i = 0; i < shape.size() && i < 8; ++i) dims[i] = shape[i];
    return (int64_t)shape.size();
  });
}

int32_t ogle_rt_tensor_dformat(OgleSession* s, const char* name) {
  return (int32_t)Guard([&]() -> int64_t {
    Tensor* t = s->session->FindTensorByName(name);
    if (t == nullptr) {
      g_error = std::string("tensor '") + name + "' is not allocated";
      return -1;
    }
    return (int64_t)t->dformat();
  });
}

void* ogle_rt_tensor_device_ptr(OgleSession* s, const char* name) {
  void* p = nullptr;
  Guard([&]() -> int64_t {
    Tensor* t = s->session->FindTensorByName(name);
    p = t && t->outer_stride_bytes() == 0 ? t->device_ptr() : nullptr;
    return 0;
  });
  return p;
}

void* ogle_rt_stream(OgleSession* s) {
  void* p = nullptr;
  Guard([&]() -> int64_t {
    p = s->context->stream();
    return 0;
  });
  return p;
}

int64_t ogle_rt_get_output(OgleSession* s, const char* name, const char* dformat, float* dst,
                           int64_t capacity) {
  return Guard([&]() -> int64_t {
    opengl::TensorList outs;
    s->session->GetOutputs({name}, {dformat}, &outs);
    std::unique_ptr<Tensor> host(outs[0]);
    const int64_t n = (int64_t)host->AllocatedElements();  // padded for the stride-4 tags
    if (n > capacity) {
      g_error = "output buffer too small";
      return -1;
    }
    std::memcpy(dst, host->host(), n * sizeof(float));
    return n;
  });
}

int64_t ogle_rt_reserialize(const void* data, size_t size, void* out, int64_t capacity) {
  return Guard([&]() -> int64_t {
    dlxnet::ModelProto model;
    if (!model.ParseFromArray(data, size)) {
      g_error = "not a .dlx model";
      return -1;
    }
    const std::string bytes = model.SerializeAsString();
    if ((int64_t)bytes.size() > capacity) {
      g_error = "output buffer too small";
      return -1;
    }
    std::memcpy(out, bytes.data(), bytes.size());
    return (int64_t)bytes.size();
  });
}

int64_t ogle_rt_model_debug_string(const void* data, size_t size, char* out, int64_t capacity) {
  return Guard([&]() -> int64_t {
    dlxnet::ModelProto model;
    if (!model.ParseFromArray(data, size)) {
      g_error = "not a .dlx model";
      return -1;
    }
    const std::string text = model.DebugString();
    if ((int64_t)text.size() + 1 > capacity) {
      g_error = "output buffer too small";
      return -1;
    }
    std::memcpy(out, text.c_str(), text.size() + 1);
    return (int64_t)text.size();
  });
}

int32_t ogle_rt_num_kernels(OgleSession* s) { return s->session->num_kernels(); }

int32_t ogle_rt_set_device_nms(OgleSession* s, int32_t on) {
  return (int32_t)Guard([&]() -> int64_t {
    s->device_nms = on != 0;
    s->session->DropGraph(1);
    s->detector.reset();
    return 0;
  });
}

int32_t ogle_rt_set_reorder(OgleSession* s, int32_t on) {
  return (int32_t)Guard([&]() -> int64_t {
    s->session->set_reorder(on != 0);
    return 0;
  });
}

const char* ogle_rt_issue_order_name(OgleSession* s, int32_t i) {
  static thread_local std::string name;
  const auto names = s->session->IssueOrder();
  if (i < 0 || i >= (int32_t)names.size()) return nullptr;
  name = names[i];
  return name.c_str();
}

int32_t ogle_rt_registered_kernel_count(void) {
  return (int32_t)opengl::KernelRegistry::Global()->RegisteredNames().size();
}

const char* ogle_rt_registered_kernel_name(int32_t i) {
  static thread_local std::string name;
  const auto names = opengl::KernelRegistry::Global()->RegisteredNames();
  if (i < 0 || i >= (int32_t)names.size()) return nullptr;
  name = names[i];
  return name.c_str();
}

namespace {
int64_t CopyDetections(const std::vector<std::vector<opengl::BoxInfo>>& result, OgleDetection* out,
                       int64_t capacity) {
  int64_t n = 0;
  for (size_t b = 0; b < result.size(); ++b)
    for (const auto& info : result[b]) {
      if (n < capacity) {
        OgleDetection& d = out[n];
        d.image = (int32_t)b;
        d.prior = info.index;
        d.class_id = info.class_name;
        d.score = info.score;
        d.x = info.box.x; d.y = info.box.y; d.width = info.box.width; d.height = info.box.height;
        d.cx = info.cx; d.cy = info.cy;
      }
      ++n;
    }
  return n;
}
}  // namespace

int64_t ogle_rt_detect(OgleSession* s, const float* images, const int32_t* dims,
                       const char* input_name, const char* cls_name, const char* box_name,
                       const char* anchors_name, float score_threshold, float nms_threshold,
                       int32_t topk, int32_t raw_width, int32_t raw_height, OgleDetection* out,
                       int64_t capacity) {
  return Guard([&]() -> int64_t {
    opengl::DetectorOptions opt;
    if (input_name) opt.input_names = {input_name};
    if (cls_name) opt.output_names[0] = cls_name;
    if (box_name) opt.output_names[1] = box_name;
    if (anchors_name) opt.output_names[2] = anchors_name;
    opt.score_threshold = score_threshold;
    opt.nms_threshold = nms_threshold;
    opt.topk = topk;
    opt.device_nms = s->device_nms;
    // a graph recorded with the previous detector's buffers must not outlive them
    s->session->DropGraph(1);
    s->detector = opengl::Detector::Create(s->session.get(), opt);
    opengl::IntList shape(dims, dims + 4);
    Tensor input(Tensor::DT_FLOAT, shape, images, dlxnet::TensorProto::NHWC);
    std::vector<std::vector<opengl::BoxInfo>> result;
    s->detector->Detect(&input, raw_width, raw_height, &result);
    return CopyDetections(result, out, capacity);
  });
}

namespace {
constexpr int kReadbackSlot = 2;  // graph slot: the pass, the detector's work, the copy of its lists

// Waits for the session's last pass launched with the lists copy (its event only, not the
// stream) and reads the lists from page-locked memory.
void CollectLists(OgleSession* s, std::vector<std::vector<opengl::BoxInfo>>* out) {
  CHECK(s->detector != nullptr && s->detector->host_copy_enabled() && s->lists_ready != nullptr)
      << "no pass with a copy of its detection lists has been launched on this session";
  if (s->lists_pending) {
    const hipError_t e = hipEventSynchronize(s->lists_ready);
    if (e != hipSuccess) LOG(FATAL) << "hipEventSynchronize: " << hipGetErrorString(e);
    s->lists_pending = false;
  }
  s->detector->FinalFromHostCopy(out);
}
}  // namespace

int32_t ogle_rt_time_pipelined_readback(OgleSession** sessions, int32_t n, int32_t warmup,
                                        int32_t iters, float* total_ms, int64_t* detections) {
  return (int32_t)Guard([&]() -> int64_t {
    CHECK(sessions != nullptr && n >= 1 && n <= 16) << "1..16 sessions";
    for (int i = 0; i < n; ++i) {
      OgleSession* s = sessions[i];
      CHECK(s != nullptr && s->session != nullptr) << "null session";
      opengl::DetectorOptions opt;
      opt.device_nms = true;  // the lists that are copied are the device's final ones
      if (!s->detector) s->detector = opengl::Detector::Create(s->session.get(), opt);
      CHECK(s->device_nms) << "the pipelined readback copies the device's final lists: "
                              "ogle_rt_set_device_nms(session, 1)";
      auto detect = [s, opt]() { s->detector->EnqueueDetect(opt.output_names, 300, 300); };
      if (!s->session->graph_captured(kReadbackSlot)) {
        s->detector->EnableHostCopy();
        detect();  // first use allocates the result buffers and the page-locked copy: not under capture
        s->context->Finish();
        CHECK(s->detector->UsesDeviceNms() && s->detector->host_copy_enabled())
            << "the detector's outputs do not fit the device top-k + NMS";
        s->session->CaptureGraph(kReadbackSlot, detect);
      }
      if (s->lists_ready == nullptr &&
          hipEventCreateWithFlags(&s->lists_ready, hipEventDisableTiming) != hipSuccess)
        LOG(FATAL) << "hipEventCreate failed";
    }
    std::vector<std::vector<opengl::BoxInfo>> lists;
    int64_t seen = 0;
    auto step = [&](int i) {
      OgleSession* s = sessions[i % n];
      // the copy of the next pass lands where the last one's lists are: read those first
      if (s->lists_pending) {
        CollectLists(s, &lists);
        for (const auto& image : lists) seen += (int64_t)image.size();
      }
      s->session->LaunchGraph(kReadbackSlot);
      const hipError_t e = hipEventRecord(s->lists_ready, static_cast<hipStream_t>(s->context->stream()));
      if (e != hipSuccess) LOG(FATAL) << "hipEventRecord: " << hipGetErrorString(e);
      s->lists_pending = true;
    };
    auto drain = [&]() {
      for (int i = 0; i < n; ++i)
        if (sessions[i]->lists_pending) {
          CollectLists(sessions[i], &lists);
          for (const auto& image : lists) seen += (int64_t)image.size();
        }
      for (int i = 0; i < n; ++i) sessions[i]->context->Finish();
    };
    for (int i = 0; i < warmup; ++i) step(i);
    drain();
    seen = 0;
    const auto t0 = std::chrono::steady_clock::now();
    for (int i = 0; i < iters; ++i) step(i);
    // the lists of every session's last pass stay unread for ogle_rt_pipelined_results:
    // wait for them, count them, but leave them marked as the session's current lists
    for (int i = 0; i < n; ++i) {
      OgleSession* s = sessions[i];
      if (!s->lists_pending) continue;
      CollectLists(s, &lists);
      for (const auto& image : lists) seen += (int64_t)image.size();
    }
    for (int i = 0; i < n; ++i) sessions[i]->context->Finish();
    const auto t1 = std::chrono::steady_clock::now();
    if (total_ms) *total_ms = std::chrono::duration<float, std::milli>(t1 - t0).count();
    if (detections) *detections = seen;
    return 0;
  });
}

int64_t ogle_rt_pipelined_results(OgleSession* s, OgleDetection* out, int64_t capacity) {
  return Guard([&]() -> int64_t {
    std::vector<std::vector<opengl::BoxInfo>> result;
    CollectLists(s, &result);
    return CopyDetections(result, out, capacity);
  });
}

int64_t ogle_rt_detect_results(OgleSession* s, OgleDetection* out, int64_t capacity) {
  return Guard([&]() -> int64_t {
    CHECK(s->detector != nullptr) << "no detector work has been enqueued on this session";
    std::vector<std::vector<opengl::BoxInfo>> result;
    if (s->detector->UsesDeviceNms()) {
      s->detector->ReadbackFinal(&result);
    } else {
      s->detector->Readback();
      s->detector->HostTopkNms(&result);
    }
    return CopyDetections(result, out, capacity);
  });
}

}  // extern "C"
