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

// A byte range of device memory, [ptr, ptr + bytes).
struct MemRange {
  const void* ptr;
  size_t bytes;
};

class Context {
 public:
  Context();
  ~Context();

  // The HIP stream every kernel of this context is launched on (a hipStream_t),
  // created on first use so that graph loading and validation need no device.
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
  void Flush();
  void set_batching(bool on) {
    Flush();
    batching_ = on;
  }
  size_t pending_convs() const { return pending_.size(); }

  void Finish();  // glFinish: waits for the stream
  void Reset() {}

 private:
  void* stream_ = nullptr;
  void* workspace_ = nullptr;
  size_t workspace_bytes_ = 0;
  size_t workspace_used_ = 0;
  std::vector<OgleConvArgs> pending_;
  bool batching_ = true;
  std::map<std::string, std::unique_ptr<Program>> programs_;
};

// Process-wide context (context.cc:316-319 of the reference).
Context* GetContext();

}  // namespace opengl

#endif  // OPENGL_CORE_CONTEXT_H_
