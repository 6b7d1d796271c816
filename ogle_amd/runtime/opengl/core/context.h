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
  // chain) share a grid.  A batch is launched as soon as anything depends on it:
  // BeforeConv flushes if the coming convolution touches a deferred one's buffers (or
  // the batch is full), BeforeLaunch does the same for any other kernel given the
  // buffers it reads and writes; copies and waits always flush.
  void BeforeConv(const void* input, const void* filter, const void* bias, const void* output);
  void BeforeLaunch(const void* const* reads, int n_reads, const void* const* writes, int n_writes);
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
  // True if `p` lies inside a buffer a deferred convolution writes (`written`) or
  // reads or writes (`!written`).
  bool TouchesPending(const void* p, bool written_only) const;
  std::vector<OgleConvArgs> pending_;
  bool batching_ = true;
  std::map<std::string, std::unique_ptr<Program>> programs_;
};

// Process-wide context (context.cc:316-319 of the reference).
Context* GetContext();

}  // namespace opengl

#endif  // OPENGL_CORE_CONTEXT_H_
