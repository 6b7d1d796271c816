#include "opengl/core/fbo_session.h"

#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <cstdlib>
#include <fstream>
#include <map>
#include <set>
#include <sstream>

#include "opengl/core/kernel.h"
#include "opengl/core/kernel_registry.h"
#include "opengl/core/tensor.h"
#include "opengl/utils/logging.h"

namespace opengl {

#define OGLE_HIP_CALL(expr)                                                       \
  do {                                                                            \
    const hipError_t e__ = (expr);                                                \
    if (e__ != hipSuccess) LOG(FATAL) << #expr << ": " << hipGetErrorString(e__); \
  } while (0)

FBOSession::FBOSession(Context* context) : context_(context) {
  context_->Reset();
  const char* env = std::getenv("OGLE_REORDER");
  if (env != nullptr && env[0] != '\0' && env[0] != '0') reorder_ = true;
  env = std::getenv("OGLE_SIBLING_FUSION");
  if (env != nullptr && env[0] != '\0' && env[0] != '0') fuse_siblings_ = true;
}

FBOSession::~FBOSession() {
  for (int i = 0; i < kGraphSlots; ++i) {
    if (graph_exec_[i] != nullptr)
      (void)hipGraphExecDestroy(static_cast<hipGraphExec_t>(graph_exec_[i]));
    if (graph_[i] != nullptr) (void)hipGraphDestroy(static_cast<hipGraph_t>(graph_[i]));
  }
  // Views must go before the buffers they alias; both are plain frees, so order
  // only matters for tidiness: release in reverse creation order.
  for (auto it = total_tensors_.rbegin(); it != total_tensors_.rend(); ++it) it->reset();
}

void FBOSession::LoadGraph(std::string model_path) {
  std::ifstream in(model_path, std::ios::binary);
  CHECK(in.good()) << "Load Graph " << model_path << " Failed: cannot open file";
  std::stringstream buffer;
  buffer << in.rdbuf();
  const std::string bytes = buffer.str();
  dlxnet::ModelProto model;
  CHECK(model.ParseFromString(bytes)) << "Load Graph " << model_path << " Failed: not a .dlx model";
  LoadGraph(model);
}

void FBOSession::LoadGraph(const ::dlxnet::ModelProto& model_proto) {
  // A session that has already run holds device state that refers to the old graph's
  // tensors: deferred convolutions, recorded hipGraphs (their kernel arguments are the
  // old buffers' addresses) and the issue order's Kernel pointers.  All of it goes
  // before the tensors are released.
  if (finalized_) context_->Finish();
  for (int slot = 0; slot < kGraphSlots; ++slot) DropGraph(slot);
  order_.clear();
  ready_.clear();
  finalized_ = false;
  graph_created_ = false;
  computed_once_ = false;
  model_ = model_proto;
  kernels_.clear();
  total_tensors_.clear();
  tensor_name_index_.clear();
  default_input_sizes_.clear();
  const dlxnet::GraphProto& graph = model_.graph();
  total_tensors_.resize(graph.tensor_names_size());
  for (int i = 0; i < graph.tensor_names_size(); ++i) tensor_name_index_[graph.tensor_names(i)] = i;

  for (const dlxnet::NodeProto& node : graph.node()) {
    if (node.type() == "Input") {
      // Remembers the model's own spatial size (fbo_session.cc:102-111); no kernel.
      const auto& dims = node.attr().input_attr().dims();
      CHECK_GE(dims.size(), 2u) << "Input node '" << node.name() << "' needs at least 2 dims";
      for (size_t i = dims.size() - 2; i < dims.size(); ++i) default_input_sizes_.push_back(dims[i]);
      continue;
    }
    Kernel* kernel = nullptr;
    KernelRegistry::Global()->CreateKernel(node.type(), &kernel, context_);
    if (kernel == nullptr) LOG(FATAL) << "unsupported kernel name " << node.type();
    std::unique_ptr<Kernel> owned(kernel);
    for (auto idx : node.input_index())
      CHECK(idx >= 0 && idx < graph.tensor_names_size()) << "node '" << node.name()
                                                         << "' input index out of range";
    for (auto idx : node.output_index())
      CHECK(idx >= 0 && idx < graph.tensor_names_size()) << "node '" << node.name()
                                                         << "' output index out of range";
    kernel->Setup(node, this);
    kernels_.push_back(std::move(owned));
  }
  finalized_ = false;
  graph_created_ = true;
}

void FBOSession::Setup(const NamedTensorList& inputs_cpu) {
  CHECK(graph_created_) << "No Graph Loaded!";
  for (const auto& named : inputs_cpu) {
    const Tensor* input_cpu = named.second;
    auto it = tensor_name_index_.find(named.first);
    if (it == tensor_name_index_.end()) LOG(FATAL) << "tensor_name: " << named.first << " Cannot Find";
    const int index = it->second;
    if (!finalized_) {
      total_tensors_[index].reset(new Tensor(Tensor::DT_FLOAT, input_cpu->shape(),
                                             Tensor::DEVICE_BUFFER,
                                             FormatToStride4(input_cpu->dformat())));
    } else {
      // The input shape is fixed after the first Run (allow_resized_ is never set).
      CHECK(allow_resized_ || total_tensors_[index]->shape() == input_cpu->shape())
          << "input '" << named.first << "' changed shape after the session was finalized";
    }
    context_->CopyCPUTensorToDevice(input_cpu, total_tensors_[index].get());
  }
  if (finalized_) return;

  ready_.assign(total_tensors_.size(), false);
  for (size_t i = 0; i < kernels_.size(); ++i) {
    Kernel* kernel = kernels_[i].get();
    kernel->input_tensors_.clear();
    kernel->output_tensors_.clear();
    for (int idx : kernel->input_tensor_indexes_) {
      Tensor* t = total_tensors_[idx].get();
      CHECK(t != nullptr) << "input tensor is uninitialized of kernel index: " << i << " ("
                          << kernel->kernel_type() << " '" << kernel->kernel_name() << "')";
      kernel->input_tensors_.push_back(t);
    }
    kernel->SelectKernel(kernel->input_tensors_);
    kernel->SetupProgram(context_->CreateProgram(kernel->kernel_fname(), kernel->build_options()));

    TensorShapeList output_shapes;
    kernel->InferOutputShape(kernel->input_tensors_, output_shapes);
    CHECK_GT(output_shapes.size(), 0u);
    CHECK_EQ(output_shapes.size(), kernel->output_tensor_indexes_.size())
        << kernel->kernel_type() << " '" << kernel->kernel_name() << "'";
    for (size_t j = 0; j < output_shapes.size(); ++j) {
      const DataFormat dformat = kernel->GetOutputDFormat(static_cast<int>(j));
      const int alias = kernel->OutputAliasesInput(static_cast<int>(j));
      Tensor* out = nullptr;
      if (alias >= 0) {
        out = new Tensor(kernel->input_tensors_[alias], output_shapes[j], dformat);
      } else {
        out = new Tensor(Tensor::DT_FLOAT, output_shapes[j], Tensor::DEVICE_BUFFER, dformat);
      }
      total_tensors_[kernel->output_tensor_indexes_[j]].reset(out);
      kernel->output_tensors_.push_back(out);
    }
    if (CheckKernelReady(kernel)) {
      // Constants and constant-only subgraphs run once, here (fbo_session.cc:240-244).
      kernel->Compute();
      context_->Flush();
      UpdateKernelReady(kernel);
    }
  }
  FuseSiblings();
  PlaceInputsInOutputs();
  BuildSchedule();
  finalized_ = true;
}

// Live nodes that read the same tensor are offered to each other (Kernel::TryAbsorb): a
// pair that agrees runs as one launch from then on.  File order is kept: the absorbing
// node is the earlier one, so everything that reads either output still comes after the
// launch that fills it.
void FBOSession::FuseSiblings() {
  if (!fuse_siblings_) return;
  for (size_t i = 0; i < kernels_.size(); ++i) {
    Kernel* a = kernels_[i].get();
    if (CheckKernelReady(a) || a->absorbed() || a->input_tensor_indexes_.empty()) continue;
    for (size_t j = i + 1; j < kernels_.size(); ++j) {
      Kernel* b = kernels_[j].get();
      if (CheckKernelReady(b) || b->absorbed() || b->input_tensor_indexes_.empty()) continue;
      if (a->input_tensor_indexes_[0] != b->input_tensor_indexes_[0]) continue;
      if (a->kernel_type() != b->kernel_type()) continue;
      if (a->TryAbsorb(b)) break;
    }
  }
}

// Where a node's output is nothing but its inputs side by side (Kernel::
// InputPlacementInOutput: a Concat), the producers of those inputs are pointed at their
// places inside the output, so that the node has nothing left to copy.  With a single
// slice before the concat axis (the SSD box and class concats at batch 1) an input's place
// is one dense range; with several (the same concats at batch > 1) it is one run per
// slice, the runs a whole output slice apart, and the producer must be able to write its
// images that far apart (Kernel::CanWriteOuterSlicesApart: a convolution on the MFMA
// path) and be read by nothing but this node, since every other kernel assumes dense
// inputs.  An input qualifies if, looking through nodes that only re-interpret memory, it
// is the whole output of a live node with its own allocation that has not been placed
// already; its place (and the distance between runs) must be 16-byte aligned unless the
// producer is a convolution whose channel count is not a multiple of four (those store
// element by element).  All inputs of the node must qualify.  Every tensor that aliases
// a moved allocation is re-pointed with it.
void FBOSession::PlaceInputsInOutputs() {
  std::map<int, std::pair<Kernel*, int>> producer;  // tensor index -> (kernel, output slot)
  for (auto& k : kernels_)
    for (size_t j = 0; j < k->output_tensor_indexes_.size(); ++j)
      producer[k->output_tensor_indexes_[j]] = {k.get(), static_cast<int>(j)};
  // The allocation a tensor's memory belongs to: the tensor itself, or, for the output of
  // a node that only re-interprets memory, the root of the input it aliases.
  auto root_of = [&](int idx) {
    for (;;) {
      auto it = producer.find(idx);
      if (it == producer.end()) return idx;
      const int alias = it->second.first->OutputAliasesInput(it->second.second);
      if (alias < 0) return idx;
      idx = it->second.first->input_tensor_indexes_[alias];
    }
  };
  // True if a node other than `self` computes on the memory of allocation `root`.
  auto has_other_reader = [&](int root, const Kernel* self) {
    for (auto& other : kernels_) {
      if (other.get() == self) continue;
      bool view = !other->output_tensor_indexes_.empty();
      for (size_t j = 0; j < other->output_tensor_indexes_.size(); ++j)
        if (other->OutputAliasesInput(static_cast<int>(j)) < 0) view = false;
      if (view) continue;  // only passes the memory on; its consumers are looked at themselves
      for (int in : other->input_tensor_indexes_)
        if (root_of(in) == root) return true;
    }
    return false;
  };
  std::set<int> placed;
  for (auto& kp : kernels_) {
    Kernel* k = kp.get();
    if (CheckKernelReady(k)) continue;
    const Kernel::Placement pl = k->InputPlacementInOutput();
    const std::vector<size_t>& offsets = pl.offsets;
    if (offsets.empty() || offsets.size() != k->input_tensor_indexes_.size()) continue;
    Tensor* out = k->output_tensors_[0];
    if (!out->owns_device_buffer()) continue;
    const bool apart = pl.outer_count > 1;
    std::vector<int> roots;
    bool ok = true;
    for (size_t i = 0; i < offsets.size() && ok; ++i) {
      int idx = k->input_tensor_indexes_[i];
      Kernel* pk = nullptr;
      for (;;) {
        auto it = producer.find(idx);
        if (it == producer.end()) { ok = false; break; }  // a graph input
        pk = it->second.first;
        const int alias = pk->OutputAliasesInput(it->second.second);
        if (alias < 0) break;
        idx = pk->input_tensor_indexes_[alias];
      }
      if (!ok) break;
      Tensor* root = total_tensors_[idx].get();
      const uintptr_t place = reinterpret_cast<uintptr_t>(out->device_ptr()) + offsets[i];
      // A place that is only 4-byte aligned suits a convolution that stores element by
      // element, but every other kernel reads 16-byte vectors from the tensor's start:
      // the exception holds only if this node is the allocation's sole reader.
      const bool sole = !has_other_reader(idx, k);
      const bool by_element = pk->kernel_type() == "Conv" && root->shape().back() % 4 != 0 && sole;
      const bool aligned = place % 16 == 0 && (!apart || pl.outer_stride % 16 == 0);
      ok = !CheckKernelReady(pk) && root->owns_device_buffer() && placed.count(idx) == 0 &&
           std::find(roots.begin(), roots.end(), idx) == roots.end() &&
           root->num_elements() == k->input_tensors_[i]->num_elements() &&
           (aligned || (by_element && place % 4 == 0 && pl.outer_stride % 4 == 0)) &&
           (!apart || (sole && pk->CanWriteOuterSlicesApart(pl.outer_count)));
      roots.push_back(idx);
    }
    if (!ok) continue;
    for (size_t i = 0; i < offsets.size(); ++i) {
      Tensor* root = total_tensors_[roots[i]].get();
      void* const old = root->device_ptr();
      void* const place = static_cast<unsigned char*>(out->device_ptr()) + offsets[i];
      for (auto& t : total_tensors_)
        if (t && t.get() != root && t->mem_type() == Tensor::DEVICE_BUFFER &&
            !t->owns_device_buffer() && t->device_ptr() == old)
          t->Rebind(place, pl.outer_count, pl.outer_stride);
      root->Rebind(place, pl.outer_count, pl.outer_stride);
      placed.insert(roots[i]);
    }
    k->set_inputs_in_place(true);
  }
  // Every kernel but a placed node and the views on its inputs assumes dense inputs.
  for (auto& kp : kernels_) {
    Kernel* k = kp.get();
    if (CheckKernelReady(k) || k->inputs_in_place()) continue;
    bool view = !k->output_tensor_indexes_.empty();
    for (size_t j = 0; j < k->output_tensor_indexes_.size(); ++j)
      if (k->OutputAliasesInput(static_cast<int>(j)) < 0) view = false;
    if (view) continue;
    for (const Tensor* t : k->input_tensors_)
      CHECK(t == nullptr || t->outer_stride_bytes() == 0)
          << "node " << k->kernel_name() << " would read a tensor whose images lie apart";
  }
}

// Issue order of a pass: file order, unless reordering was asked for.  The context defers
// convolutions and launches the deferred ones as one grid when something needs a result; in
// file order the SSD heads all come last and fill the chip by themselves while the chain of
// small feature-extractor convolutions before them runs one under-filled launch after
// another.  A head only needs its feature map, so it may be issued any time between
// that map's launch and its own place in the file.  With reordering this pass simulates the
// context's flush rule over the file order to find the launch groups, then moves
// each convolution that has such slack to the group (within its window) where it
// adds least to the estimated pass time: a group costs max(launch floor, work /
// throughput), so under-filled groups absorb work for free.  A moved node is issued
// just before the node that triggers its new group's launch.  Data dependencies are
// still enforced by the context at run time, whatever this order is.
void FBOSession::BuildSchedule() {
  order_.clear();
  std::vector<Kernel*> live;
  for (auto& kernel : kernels_)
    if (!CheckKernelReady(kernel.get())) live.push_back(kernel.get());
  const int n = static_cast<int>(live.size());

  // every deferrable node's scratch fits at once, so a batch is never cut short
  size_t scratch = 0;
  for (Kernel* k : live)
    if (k->Deferrable()) scratch += (k->ScratchBytes() + 255) & ~size_t(255);
  if (scratch > 0) context_->ReserveWorkspace(scratch);

  if (!reorder_) {
    order_ = live;
    return;
  }

  // producer of every tensor, looking through nodes that only re-interpret memory
  std::map<int, int> producer;  // tensor index -> position in `live` (views resolved)
  std::vector<bool> is_view(n, false);
  std::vector<std::vector<int>> deps(n);
  for (int i = 0; i < n; ++i) {
    Kernel* k = live[i];
    for (int t : k->input_tensor_indexes_) {
      auto it = producer.find(t);
      if (it != producer.end()) deps[i].push_back(it->second);
    }
    bool view = !k->output_tensor_indexes_.empty();
    for (size_t j = 0; j < k->output_tensor_indexes_.size(); ++j)
      if (k->OutputAliasesInput(static_cast<int>(j)) < 0) view = false;
    is_view[i] = view;
    for (size_t j = 0; j < k->output_tensor_indexes_.size(); ++j) {
      int src = i;
      if (k->absorbed()) {
        // filled by the sibling's launch, which comes earlier in the file
        for (int q = 0; q < i; ++q)
          if (live[q] == k->absorbed_by()) src = q;
      } else if (view) {
        const int in = k->input_tensor_indexes_[k->OutputAliasesInput(static_cast<int>(j))];
        auto it = producer.find(in);
        src = it != producer.end() ? it->second : -1;
      }
      if (src >= 0) producer[k->output_tensor_indexes_[j]] = src;
    }
  }

  // groups under the context's flush rule, in file order
  constexpr int kMaxBatch = 16;
  std::vector<int> group(n, -1);
  std::vector<int> trigger;  // trigger[g]: position whose issue launches group g (n: end of pass)
  {
    std::set<int> pending;
    auto depends_on_pending = [&](int i) {
      for (int d : deps[i])
        if (pending.count(d)) return true;
      return false;
    };
    for (int i = 0; i < n; ++i) {
      if (is_view[i] || live[i]->absorbed()) continue;
      const bool defer = live[i]->Deferrable();
      if (!pending.empty() &&
          (depends_on_pending(i) || (defer && static_cast<int>(pending.size()) >= kMaxBatch))) {
        trigger.push_back(i);
        pending.clear();
      }
      if (defer) {
        pending.insert(i);
        group[i] = static_cast<int>(trigger.size());
      }
    }
    trigger.push_back(n);  // whatever is left goes out at the end of the pass
  }
  const int groups = static_cast<int>(trigger.size());

  // cost model: microseconds at a sustained MFMA rate, with a floor per launch
  constexpr double kMacPerUs = 45e6;  // ~90 TFLOP/s
  constexpr double kFloorUs = 10.0;  // a small dependent launch (reductions are finished together later)
  std::vector<double> load(groups, 0.0);
  std::vector<int> members(groups, 0);
  for (int i = 0; i < n; ++i)
    if (group[i] >= 0) {
      load[group[i]] += live[i]->WorkEstimate() / kMacPerUs;
      ++members[group[i]];
    }
  auto cost = [&](double us) { return std::max(kFloorUs, us); };

  std::vector<int> placed(group);
  std::vector<std::vector<int>> moved(groups);  // nodes to issue just before trigger[g]
  for (int i = 0; i < n; ++i) {
    if (group[i] < 0) continue;
    int earliest = 0;
    for (int d : deps[i]) {
      int g;
      if (group[d] >= 0) {
        g = placed[d] + 1;  // after the launch that produces it
      } else {
        // a directly launched node at position d is on the stream before every group
        // whose trigger comes after it
        g = static_cast<int>(std::upper_bound(trigger.begin(), trigger.end(), d) - trigger.begin());
      }
      earliest = std::max(earliest, g);
    }
    const int home = group[i];
    if (earliest >= home) continue;
    const double w = live[i]->WorkEstimate() / kMacPerUs;
    int best = home;
    double best_delta = cost(load[home]) - cost(load[home] - w);
    for (int g = home - 1; g >= earliest; --g) {
      if (members[g] >= kMaxBatch) continue;
      const double delta = cost(load[g] + w) - cost(load[g]);
      if (delta < best_delta - 1e-9) {
        best_delta = delta;
        best = g;
      }
    }
    if (best != home) {
      load[home] -= w;
      --members[home];
      load[best] += w;
      ++members[best];
      placed[i] = best;
      moved[best].push_back(i);
    }
  }

  std::vector<bool> is_moved(n, false);
  for (const auto& list : moved)
    for (int i : list) is_moved[i] = true;
  int g = 0;
  for (int i = 0; i <= n; ++i) {
    while (g < groups && trigger[g] == i) {
      for (int m : moved[g]) order_.push_back(live[m]);
      ++g;
    }
    if (i < n && !is_moved[i]) order_.push_back(live[i]);
  }
  CHECK_EQ(order_.size(), live.size());
}

std::vector<std::string> FBOSession::IssueOrder() const {
  std::vector<std::string> names;
  for (const Kernel* k : order_) names.push_back(k->kernel_name());
  return names;
}

void FBOSession::Compute() {
  CHECK(finalized_) << "Please Setup Session First";
  for (Kernel* kernel : order_) {
    kernel->Compute();
  }
  context_->Flush();  // convolutions still deferred at the end of the pass
  computed_once_ = true;
}

void FBOSession::Run(const NamedTensorList& inputs_cpu) {
  Setup(inputs_cpu);
  Compute();
}

void FBOSession::RunProfiled(std::vector<NodeTiming>* timings) {
  CHECK(finalized_) << "Please Setup Session First";
  hipStream_t s = static_cast<hipStream_t>(context_->stream());
  // file order, every node whole: per-node timing wants nothing deferred across nodes
  std::vector<Kernel*> live;
  for (auto& kernel : kernels_)
    if (!CheckKernelReady(kernel.get())) live.push_back(kernel.get());
  std::vector<hipEvent_t> ev(live.size() + 1);
  for (auto& e : ev) OGLE_HIP_CALL(hipEventCreate(&e));
  OGLE_HIP_CALL(hipEventRecord(ev[0], s));
  for (size_t i = 0; i < live.size(); ++i) {
    live[i]->Compute();
    context_->Flush();
    OGLE_HIP_CALL(hipEventRecord(ev[i + 1], s));
  }
  OGLE_HIP_CALL(hipStreamSynchronize(s));
  computed_once_ = true;
  timings->clear();
  for (size_t i = 0; i < live.size(); ++i) {
    float ms = 0.f;
    OGLE_HIP_CALL(hipEventElapsedTime(&ms, ev[i], ev[i + 1]));
    timings->push_back({live[i]->kernel_name() + "#" + live[i]->kernel_type() + "#",
                        live[i]->kernel_type(), ms});
  }
  for (auto& e : ev) (void)hipEventDestroy(e);
}

void FBOSession::CaptureGraph(int slot, const std::function<void()>& after_pass) {
  CHECK(finalized_) << "Please Setup Session First";
  CHECK(slot >= 0 && slot < kGraphSlots) << "graph slot";
  if (graph_exec_[slot] != nullptr) return;
  hipStream_t s = static_cast<hipStream_t>(context_->stream());
  if (!computed_once_) {
    // The first pass packs filters and may grow the workspace (allocations), which
    // must not happen inside a capture: make that pass eagerly.
    Compute();
  }
  OGLE_HIP_CALL(hipStreamSynchronize(s));
  hipGraph_t graph = nullptr;
  OGLE_HIP_CALL(hipStreamBeginCapture(s, hipStreamCaptureModeThreadLocal));
  try {
    Compute();
    if (after_pass) {
      after_pass();
      context_->Flush();
    }
  } catch (...) {
    (void)hipStreamEndCapture(s, &graph);
    if (graph != nullptr) (void)hipGraphDestroy(graph);
    throw;
  }
  OGLE_HIP_CALL(hipStreamEndCapture(s, &graph));
  hipGraphExec_t exec = nullptr;
  OGLE_HIP_CALL(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0));
  graph_[slot] = graph;
  graph_exec_[slot] = exec;
}

void FBOSession::DropGraph(int slot) {
  CHECK(slot >= 0 && slot < kGraphSlots) << "graph slot";
  if (graph_exec_[slot] == nullptr) return;
  context_->Finish();
  (void)hipGraphExecDestroy(static_cast<hipGraphExec_t>(graph_exec_[slot]));
  (void)hipGraphDestroy(static_cast<hipGraph_t>(graph_[slot]));
  graph_exec_[slot] = nullptr;
  graph_[slot] = nullptr;
}

void FBOSession::LaunchGraph(int slot) {
  CHECK(slot >= 0 && slot < kGraphSlots && graph_exec_[slot] != nullptr) << "CaptureGraph first";
  OGLE_HIP_CALL(hipGraphLaunch(static_cast<hipGraphExec_t>(graph_exec_[slot]),
                               static_cast<hipStream_t>(context_->stream())));
}

bool FBOSession::CheckKernelReady(const Kernel* kernel) {
  if (kernel->ForceReady()) return true;
  for (int id : kernel->input_tensor_indexes_)
    if (!ready_[id]) return false;
  return true;
}

void FBOSession::UpdateKernelReady(const Kernel* kernel) {
  for (int id : kernel->output_tensor_indexes_) ready_[id] = true;
}

void FBOSession::GetOutputs(const TensorNameList& output_names, const StringList& output_dformats,
                            TensorList* outputs) {
  CHECK_EQ(output_names.size(), output_dformats.size());
  if (outputs->size() < output_names.size()) outputs->resize(output_names.size(), nullptr);
  for (size_t i = 0; i < output_names.size(); ++i) {
    Tensor* gpu_tensor = FindTensorByName(output_names[i]);
    CHECK(gpu_tensor != nullptr) << "tensor '" << output_names[i] << "' was never produced";
    const DataFormat dformat = StrToFormat(output_dformats[i]);
    if (outputs->at(i) == nullptr) {
      // The caller owns the host tensors GetOutputs creates (fbo_session.cc:294).
      outputs->at(i) = new Tensor(Tensor::DT_FLOAT, gpu_tensor->shape(), Tensor::HOST_MEMORY, dformat);
    } else {
      CHECK(outputs->at(i)->shape() == gpu_tensor->shape()) << "reused output tensor has another shape";
    }
    context_->CopyDeviceTensorToCPU(gpu_tensor, outputs->at(i));
  }
}

std::string FBOSession::DebugString() const {
  return "ModelProto: " + model_.DebugString() + "\n";
}

Tensor* FBOSession::FindTensorByName(const std::string& tensor_name) {
  auto it = tensor_name_index_.find(tensor_name);
  if (it == tensor_name_index_.end()) LOG(FATAL) << "tensor_name: " << tensor_name << " Cannot Find";
  return FindTensorById(it->second);
}

Tensor* FBOSession::FindTensorById(int id) {
  CHECK_GE(id, 0);
  CHECK_LT(id, static_cast<int>(total_tensors_.size()));
  return total_tensors_[id].get();
}

}  // namespace opengl
