// Graph executor: loads a .dlx model, creates one Kernel per node, allocates every
// tensor once on the first Run and then replays the kernels in file order.
//
// Public interface and behaviour follow ogl_runtime/opengl/core/fbo_session.h:11-90
// and fbo_session.cc:62-325: nodes run in proto order (the converter emits them
// topologically sorted), "Input" nodes have no kernel, constants and constant-only
// subgraphs are computed once during Setup (the ready_ flags), only the first Run
// allocates.  Additions for a launch-bound GPU: Compute() replays the kernels
// without re-uploading inputs, RunProfiled() brackets every node with HIP events,
// CaptureGraph()/LaunchGraph() replay the whole run as one hipGraph.  On request
// (set_reorder(true) or OGLE_REORDER=1) the convolutions whose results are not needed at
// once (the SSD heads) are issued earlier than their place in the file, next to a
// convolution of the serial chain, so that the two share one grid; results are the same
// either way, and with the present kernels file order is the faster one (all heads in
// one grid), so it is the default.
#ifndef OPENGL_CORE_FBO_SESSION_H_
#define OPENGL_CORE_FBO_SESSION_H_

#include <functional>
#include <string>
#include <vector>

#include "opengl/core/context.h"
#include "opengl/core/dlxnet.h"
#include "opengl/core/types.h"

namespace opengl {

struct NodeTiming {
  std::string name;  // "<node>#<type>#", the label the reference's TraceMe uses
  std::string type;
  float ms;
};

class FBOSession {
 public:
  explicit FBOSession(Context* context);
  FBOSession() : FBOSession(GetContext()) {}
  virtual ~FBOSession();

  void LoadGraph(const ::dlxnet::ModelProto& model_proto);
  void LoadGraph(std::string model_path);

  // Allocates (first call only) and uploads the named host inputs.
  void Setup(const NamedTensorList& inputs_cpu);
  // Setup + one pass over the kernels.  Asynchronous: GetOutputs is the sync point.
  void Run(const NamedTensorList& inputs_cpu);
  // One pass over the kernels with the inputs already on the device.
  void Compute();
  // Compute() with a HIP event pair around every node; returns after the pass.
  void RunProfiled(std::vector<NodeTiming>* timings);

  // Records one Compute() pass into a hipGraph (once per slot) and replays it.
  // `after_pass`, if given, enqueues more work on the context's stream (a detector's
  // post-processing) that is recorded into the same graph; it must not allocate.
  static constexpr int kGraphSlots = 3;
  void CaptureGraph(int slot = 0, const std::function<void()>& after_pass = {});
  void LaunchGraph(int slot = 0);
  bool graph_captured(int slot = 0) const { return graph_exec_[slot] != nullptr; }
  // Forgets a recorded graph (after the stream has drained), e.g. because buffers
  // its `after_pass` work used are about to be released.
  void DropGraph(int slot);

  void GetOutputs(const TensorNameList& output_names, const StringList& output_dformats,
                  TensorList* outputs);

  std::string DebugString() const;
  Context* context() const { return context_; }
  bool IsONNX() const { return model_.producer_name() == "ONNX"; }
  Tensor* FindTensorByName(const std::string& name);
  Tensor* FindTensorById(int id);
  bool allow_resized() const { return allow_resized_; }
  void set_allow_resized(bool flag) { allow_resized_ = flag; }
  const IntList& default_input_sizes() const { return default_input_sizes_; }
  int num_kernels() const { return static_cast<int>(kernels_.size()); }
  // Whether Setup may move deferrable convolutions ahead of their file position.
  // Takes effect at the first Run.
  void set_reorder(bool on) { reorder_ = on; }
  bool reorder() const { return reorder_; }
  // Whether Setup may run two Conv nodes that read the same tensor with the same
  // attributes as one launch (OGLE_SIBLING_FUSION=1 also switches it on).  Off by
  // default: a fused pair fetches its input once, but its wide tile cannot share a grid
  // with the small convolutions of a serial chain the way the two separate heads do, and
  // on MobileNet-SSD at batch 16 the pass measured 5 % slower with it.  Takes effect at
  // the first Run.
  void set_fuse_siblings(bool on) { fuse_siblings_ = on; }
  bool fuse_siblings() const { return fuse_siblings_; }
  // Node names in the order Compute() issues them (after the first Run).
  std::vector<std::string> IssueOrder() const;

 private:
  bool CheckKernelReady(const Kernel* kernel);
  void FuseSiblings();
  void PlaceInputsInOutputs();
  void BuildSchedule();
  void UpdateKernelReady(const Kernel* kernel);

  Context* context_;
  OwnedKernelList kernels_;
  dlxnet::ModelProto model_;
  OwnedTensorList total_tensors_;
  bool finalized_ = false;
  bool graph_created_ = false;
  bool computed_once_ = false;  // a full eager pass has run since the graph was loaded
  NamedIndex tensor_name_index_;
  std::vector<bool> ready_;
  bool allow_resized_ = false;
  bool reorder_ = false;
  bool fuse_siblings_ = false;
  std::vector<Kernel*> order_;  // the per-pass kernels in issue order (not owned)
  IntList default_input_sizes_;
  void* graph_[kGraphSlots] = {};       // hipGraph_t
  void* graph_exec_[kGraphSlots] = {};  // hipGraphExec_t
};

}  // namespace opengl

#endif  // OPENGL_CORE_FBO_SESSION_H_
