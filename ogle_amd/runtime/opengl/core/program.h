// A resolved device kernel: what Context::CreateProgram returns.
//
// In the reference a Program is a compiled GLSL shader that Kernel::Compute feeds
// with uniforms and then draws (ogl_runtime/opengl/core/program.h:17-103).  Here
// it is a handle into the HIP kernel registry plus the stream to launch on; the
// Run* methods take the argument struct of the C ABI and enqueue the launch.
// A non-zero status from the C ABI is fatal, as a GL error is in the reference
// (OPENGL_CALL, ogl_runtime/opengl/utils/macros.h:16-20).
#ifndef OPENGL_CORE_PROGRAM_H_
#define OPENGL_CORE_PROGRAM_H_

#include <string>

#include "ogle_hip.h"
#include "opengl/core/types.h"

namespace opengl {

class Program {
 public:
  Program(const std::string& name, const std::string& options, int32_t handle, Context* context)
      : name_(name), options_(options), handle_(handle), context_(context) {}

  const std::string& name() const { return name_; }
  const std::string& options() const { return options_; }
  int32_t handle() const { return handle_; }
  bool has_option(const char* define) const { return options_.find(define) != std::string::npos; }

  void Activate() const {}  // glUseProgram has no counterpart

  void RunConv2d(const OgleConvArgs& args) const;
  void RunDepthwise(const OgleConvArgs& args) const;
  void RunPointwise(const OgleConvArgs& args) const;
  void RunPool(const OglePoolArgs& args) const;
  void RunConcat(const OgleConcatArgs& args) const;
  void RunDecode(const OgleDecodeArgs& args) const;
  void RunTranspose(const OgleTransposeArgs& args) const;
  void RunUnary(const OgleUnaryArgs& args) const;
  void RunAdd(const OgleBinaryArgs& args) const;
  void RunBatchNorm(const OgleBatchNormArgs& args) const;
  void RunGemm(const OgleGemmArgs& args) const;

 private:
  void Check(int32_t status, const char* what) const;
  std::string name_;
  std::string options_;
  int32_t handle_;
  Context* context_;
};

}  // namespace opengl

#endif  // OPENGL_CORE_PROGRAM_H_
