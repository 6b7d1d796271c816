#include "opengl/core/kernel_registry.h"

#include <algorithm>

namespace opengl {

KernelRegistry* KernelRegistry::Global() {
  static KernelRegistry* registry = new KernelRegistry;
  return registry;
}

void KernelRegistry::RegisterKernel(std::string kernel_name, KernelFactory kernel_factory) {
  kernel_map_[kernel_name] = std::move(kernel_factory);
}

void KernelRegistry::CreateKernel(std::string kernel_name, Kernel** kernel, Context* context) {
  *kernel = nullptr;
  auto it = kernel_map_.find(kernel_name);
  if (it != kernel_map_.end()) it->second(kernel, context);
}

bool KernelRegistry::HasKernel(const std::string& kernel_name) const {
  return kernel_map_.count(kernel_name) != 0;
}

StringList KernelRegistry::RegisteredNames() const {
  StringList names;
  for (const auto& kv : kernel_map_) names.push_back(kv.first);
  std::sort(names.begin(), names.end());
  return names;
}

}  // namespace opengl
