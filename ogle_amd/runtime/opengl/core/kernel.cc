#include "opengl/core/kernel.h"

#include <sstream>

#include "opengl/core/context.h"
#include "opengl/core/fbo_session.h"
#include "opengl/core/tensor.h"

namespace opengl {

Kernel::Kernel(Context* context) : context_(context) {}
Kernel::~Kernel() {}

void Kernel::SetupProgram(Program* program) { program_ = program; }

void Kernel::Setup(const dlxnet::NodeProto& node, FBOSession* session) {
  kernel_name_ = node.name();
  kernel_type_ = node.type();
  session_ = session;
  input_tensor_indexes_.assign(node.input_index().begin(), node.input_index().end());
  output_tensor_indexes_.assign(node.output_index().begin(), node.output_index().end());
  SetupAttr(node.attr());
}

void Kernel::Compute() {
  struct Scope {  // closes the node's range also when Compute throws
    Context* c;
    ~Scope() { c->EndNode(); }
  };
  context_->BeginNode(kernel_name_ + "#" + kernel_type_ + "#");
  Scope scope{context_};
  Compute(input_tensors_, output_tensors_);
}

DataFormat Kernel::GetOutputDFormat(int i) const {
  CHECK_GE(i, 0);
  CHECK_LT(i, static_cast<int>(output_tensor_dformats_.size()))
      << kernel_type_ << " '" << kernel_name_ << "' declared no format for output " << i;
  return output_tensor_dformats_[i];
}

DataFormat Kernel::GetRequestInputDFormat(int i) const {
  CHECK_GE(i, 0);
  CHECK_LT(i, static_cast<int>(request_tensor_dformats_.size()));
  return request_tensor_dformats_[i];
}

void Kernel::InferOutputShape(const TensorList& inputs, TensorShapeList& output_shapes) {
  TensorShapeList input_shapes;
  for (const Tensor* t : inputs) input_shapes.push_back(t->shape());
  InferOutputShape(input_shapes, output_shapes);
}

std::string Kernel::DebugString() const {
  std::ostringstream ss;
  ss << kernel_type_ << " '" << kernel_name_ << "':";
  auto dump = [&](const std::vector<int>& ids) {
    for (int id : ids) {
      const Tensor* t = session_ ? session_->FindTensorById(id) : nullptr;
      ss << " [" << id << "]";
      if (t != nullptr) {
        ss << "(";
        for (size_t k = 0; k < t->shape().size(); ++k) ss << (k ? " " : "") << t->shape()[k];
        ss << ")";
      }
    }
  };
  dump(input_tensor_indexes_);
  ss << " ->";
  dump(output_tensor_indexes_);
  return ss.str();
}

}  // namespace opengl
