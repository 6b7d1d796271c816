// Device context: the stream, host<->device tensor copies and the program cache.
// Counterpart of ogl_runtime/opengl/core/context.h:26-62 with HIP in place of GL.
#ifndef OPENGL_CORE_CONTEXT_H_
#define OPENGL_CORE_CONTEXT_H_

#include <map>
#include <memory>
#include <string>
#include <vector>

#include "opengl/core/program.h"
#include "opengl/core/tensor.h"
#include "opengl/core/types.h"

namespace opengl {

// A byte range of device memory, [ptr, ptr + bytes); with count > 1, that many ranges of
// `bytes` whose starts lie `stride` bytes apart (a convolution output written one image at
// a time into a larger tensor).
struct MemRange {
  const void* ptr;
  size_t bytes;
  size_t stride = 0;
  size_t count = 1;
};

class Context {
 public:
  Context();
  ~Context();

  // The HIP stream every kernel of this context is launched on (a hipStream_t),
  // taken on first use so that graph loading and validation need no device.  The first four
  // contexts alive on a device share a pool of streams that were created together, which
  // keeps them on different hardware queues whatever other streams the process creates.
  void* stream();

  // Looks `kernel_fname` (a shader stem such as "conv2d_pw") up in the HIP kernel
  // registry; programs are cached by name + build options and owned by the context
  // (context.cc:288-313 of the reference).
  Program* CreateProgram(const std::string& kernel_fname, const std::string& build_options = "");

  // Host -> device.  Both sides are dense row-major over the logical shape (NHWC
  // images, ANY tensors, OIHW filters), so this is one copy.
  void CopyCPUTensorToDevice(const Tensor* cpu_tensor, Tensor* device_tensor);
  // Device -> host, converting to the host tensor's dformat; synchronises.
  void CopyDeviceTensorToCPU(const Tensor* device_tensor, Tensor* cpu_tensor);

  // Scratch memory for the kernels launched on this context's stream.  Each call
  // returns a slice that no other deferred convolution is using; slices are recycled
  // when the deferred batch is launched.  A request that does not fit launches the
  // batch first and, if it still does not fit, waits for the stream and reallocates
  // (not possible while the stream is being captured: ReserveWorkspace beforehand).
  void* Workspace(size_t bytes);
  void ReserveWorkspace(size_t bytes);
  size_t workspace_bytes() const { return workspace_bytes_; }

  // Deferred convolutions.  Dense and pointwise Conv nodes are not launched one by
  // one: they are collected and go out through ogle_hip_conv2d_batch, so that
  // mutually independent convolutions (the SSD heads next to the feature-extractor
  // chain) share a grid.  A batch is launched as soon as anything depends on it.
  // Dependencies are found by byte-range overlap: every launch names the [ptr, ptr +
  // bytes) ranges it reads and writes, and a range that overlaps what a deferred
  // convolution writes (or, for a write, anything it reads or writes: input, filter,
  // bias, output, workspace) launches the batch first.  A buffer that merely encloses a
  // deferred convolution's output (a concat output whose slices the convolutions write
  // in place) is therefore seen, wherever it starts.  BeforeConv does this for the
  // coming convolution (and also launches a full batch), BeforeLaunch for any other
  // kernel; copies and waits always flush.
  void BeforeConv(const OgleConvArgs& args);
  void BeforeLaunch(const MemRange* reads, int n_reads, const MemRange* writes, int n_writes);
  // The overlap rule itself, on plain data (no device needed): true if a launch with
  // these reads and writes must wait for one of `pending`.
  static bool Conflicts(const OgleConvArgs* pending, int n_pending, const MemRange* reads,
                        int n_reads, const MemRange* writes, int n_writes);
  // The ranges a convolution reads (input, filter, bias) and writes (output, workspace,
  // second output).
  static void ConvRanges(const OgleConvArgs& a, MemRange reads[3], MemRange writes[3]);
  void EnqueueConv(const OgleConvArgs& args);
  // Launches everything that is still held back: the deferred convolutions and the
  // reductions left pending (below).
  void Flush();
  void set_batching(bool on) {
    Flush();
    batching_ = on;
  }
  size_t pending_convs() const { return pending_.size() + unreduced_.size(); }

  // Launch log.  While it is switched on, every call into the kernel library is recorded
  // with the node(s) it was made for and the number of device operations it became
  // (ogle_hip_launch_count before and after): the dispatch sequence of a pass, in order.
  // Deferred convolutions are recorded when their batch goes out, as one entry that names
  // every node of the batch (they share grids).  A trace of the replayed pass has exactly
  // this sequence per replay.
  struct LaunchRecord {
    std::string label;  // "<node>#<type>#", several joined with '+'
    int dispatches;
  };
  void set_launch_log(bool on) {
    log_launches_ = on;
    launch_log_.clear();
  }
  const std::vector<LaunchRecord>& launch_log() const { return launch_log_; }
  // The node whose Compute is running: the label of what it launches.  With
  // OGLE_ROCTX=1 the node is also bracketed by a roctx range of that name (the
  // reference's per-node TraceMe scopes, fbo_session.cc:128-151), if the roctx
  // library can be loaded.
  void BeginNode(const std::string& label);
  void EndNode();
  // Brackets one call into the kernel library made outside a node (the detector).
  void LogLaunches(const std::string& label, int64_t count_before);

  void Finish();  // glFinish: waits for the stream
  void Reset() {}

 private:
  void* stream_ = nullptr;
  bool stream_pooled_ = false;
  int stream_device_ = 0;
  void* workspace_ = nullptr;
  size_t workspace_bytes_ = 0;
  size_t workspace_used_ = 0;
  // Launches the deferred convolutions (ogle_hip_conv2d_batch_begin).  Convolutions whose
  // plan splits K leave their partial sums in their workspace slice and move to
  // unreduced_: their reduction is only launched when something touches their output,
  // bias or workspace (FinishReductions with those ranges) or at Flush, so that all
  // reductions still open at that point share one grid.  Workspace slices are recycled
  // once nothing is pending or unreduced.  LaunchPendingThatConflict launches only the
  // deferred convolutions that touch the given ranges: deferred convolutions never depend
  // on each other (one that would is only queued after the ones it conflicts with have
  // been launched), so the rest can wait for more company.
  void LaunchPending();
  void LaunchPendingThatConflict(const MemRange* reads, int n_reads, const MemRange* writes,
                                 int n_writes);
  void LaunchBatch(std::vector<OgleConvArgs>& batch, std::vector<std::string>& labels);
  void FinishReductions(const MemRange* reads, int n_reads, const MemRange* writes, int n_writes,
                        bool all);
  std::vector<OgleConvArgs> pending_;
  std::vector<std::string> pending_labels_;
  std::vector<OgleConvArgs> unreduced_;
  std::vector<std::string> unreduced_labels_;
  bool batching_ = true;
  bool log_launches_ = false;
  std::vector<LaunchRecord> launch_log_;
  std::string current_label_;
  int64_t node_count_before_ = 0;
  std::map<std::string, std::unique_ptr<Program>> programs_;
};

// Process-wide context (context.cc:316-319 of the reference).
Context* GetContext();

}  // namespace opengl

#endif  // OPENGL_CORE_CONTEXT_H_
