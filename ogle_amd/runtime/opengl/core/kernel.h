// Base class of every graph op: the drop-in boundary of the runtime.
//
// The virtuals and their call order are those of the reference
// (ogl_runtime/opengl/core/kernel.h:15-123; driven by FBOSession::Setup/Run,
// fbo_session.cc:201-245,140-153): Setup -> SetupAttr, then once per session
// SelectKernel -> (program lookup) -> InferOutputShape, then Compute per run.
// SelectKernel now names an entry of the HIP kernel registry instead of a GLSL
// source; kernel_fname() / build_options() keep their meaning as the lookup key.
#ifndef OPENGL_CORE_KERNEL_H_
#define OPENGL_CORE_KERNEL_H_

#include <cstddef>
#include <string>
#include <vector>

#include "opengl/core/dlxnet.h"
#include "opengl/core/types.h"
#include "opengl/utils/logging.h"

namespace opengl {
class Program;
class FBOSession;

class Kernel {
 public:
  explicit Kernel(Context* context);
  virtual ~Kernel();

  virtual void SetupProgram(Program* program);
  // Enqueues the op's device work on the context's stream.
  virtual void Compute(TensorList& inputs, TensorList& outputs) = 0;
  virtual void SetupAttr(const dlxnet::Attribute& attr) = 0;
  virtual void Setup(const dlxnet::NodeProto& node_proto, FBOSession* session);
  void Compute();

  DataFormat GetOutputDFormat(int i) const;
  DataFormat GetRequestInputDFormat(int i) const;
  std::string DebugString() const;

  // Output shapes from input shapes; ops that need input values or formats
  // (Reshape, Concat, Decoder) override the tensor overload instead.
  virtual void InferOutputShape(TensorShapeList& inputs, TensorShapeList& outputs) = 0;
  virtual void InferOutputShape(const TensorList& inputs, TensorShapeList& output_shapes);

  void set_kernel_name(const std::string& name) { kernel_name_ = name; }
  void set_kernel_type(const std::string& name) { kernel_type_ = name; }
  std::string kernel_name() const { return kernel_name_; }
  std::string kernel_type() const { return kernel_type_; }
  void set_session(FBOSession* session) { session_ = session; }
  FBOSession* session() const { return session_; }

  // A kernel that must run during Setup even though its inputs are not constant
  // (ShapeKernel in the reference, shape.h:19).
  virtual bool ForceReady() const { return false; }
  const std::string kernel_fname() const { return kernel_fname_; }
  std::string build_options() const { return build_options_; }
  void set_build_options(const std::string& opt) { build_options_ = opt; }
  virtual void SelectKernel(const TensorList& inputs) { (void)inputs; }

  // Index of the input whose device buffer output `i` may share (the op is a pure
  // re-interpretation of dense memory), or -1.  Not in the reference, where every
  // layout change is a draw call; with linear NHWC buffers Reshape and an identity
  // Transpose move no data.  Consulted by the executor after InferOutputShape.
  virtual int OutputAliasesInput(int i) const {
    (void)i;
    return -1;
  }

  // If output 0 is nothing but the inputs placed side by side, where every input lies
  // inside it (the session may then have the inputs produced in place, and the node has
  // nothing left to copy); `offsets` empty otherwise.  The output is `outer_count` slices
  // of `outer_stride` bytes, and input i fills bytes [offsets[i], offsets[i] + its size /
  // outer_count) of every slice: one slice for a concatenation over the first axis that
  // is not 1, one per image for the SSD concatenations over axis 1 at batch > 1.  Valid
  // after InferOutputShape.
  struct Placement {
    std::vector<size_t> offsets;
    size_t outer_count = 1;
    size_t outer_stride = 0;
  };
  virtual Placement InputPlacementInOutput() const { return {}; }
  // True if this node can write output 0 as `count` equal runs whose starts lie further
  // apart than a run is long (Tensor::outer_stride_bytes) instead of densely.
  virtual bool CanWriteOuterSlicesApart(size_t count) const {
    (void)count;
    return false;
  }
  // Set by the session once every input has been placed inside output 0.
  void set_inputs_in_place(bool v) { inputs_in_place_ = v; }
  bool inputs_in_place() const { return inputs_in_place_; }

  // Sibling fusion, not in the reference: two nodes that read the same tensor with the
  // same attributes may run as one launch that fetches the input once (the box and the
  // class head of an SSD feature map).  TryAbsorb asks this node to take over `other`'s
  // work as well; on success `other` has been told (Absorbed) and its Compute does
  // nothing from then on, this node's Compute also fills `other`'s output.  Called by the
  // executor once all tensors are bound, before the schedule is built.
  virtual bool TryAbsorb(Kernel* other) {
    (void)other;
    return false;
  }
  bool absorbed() const { return absorbed_by_ != nullptr; }
  const Kernel* absorbed_by() const { return absorbed_by_; }

  // Scheduling hints, also not in the reference (one draw call per node, in file
  // order).  The launch of a deferrable node may be held back and merged with other
  // deferrable nodes into one grid; WorkEstimate is its device work in multiply-adds
  // including tile padding, ScratchBytes the workspace its launch plan wants.  Valid
  // once the executor has bound the node's tensors.
  virtual bool Deferrable() const { return false; }
  virtual double WorkEstimate() const { return 0.0; }
  virtual size_t ScratchBytes() const { return 0; }

 protected:
  Program* program_ = nullptr;  // not owned (the context owns programs)
  Context* context_;            // not owned
  std::string kernel_fname_;
  std::vector<Tensor*> input_tensors_;   // not owned
  std::vector<Tensor*> output_tensors_;  // not owned
  std::vector<int> input_tensor_indexes_;
  std::vector<int> output_tensor_indexes_;
  std::vector<DataFormat> request_tensor_dformats_;
  std::vector<DataFormat> output_tensor_dformats_;
  friend class FBOSession;
  std::string kernel_name_;
  std::string kernel_type_;
  std::string build_options_;
  FBOSession* session_ = nullptr;
  Kernel* absorbed_by_ = nullptr;  // the sibling that does this node's work, if any
  bool inputs_in_place_ = false;
};

}  // namespace opengl

#endif  // OPENGL_CORE_KERNEL_H_
