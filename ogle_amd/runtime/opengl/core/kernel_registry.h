// Op-type string -> Kernel factory.  Same registration macro and key strings as
// ogl_runtime/opengl/core/kernel_registry.h:9-42 ("Conv", "MaxPool", "Concat", ...).
#ifndef OPENGL_CORE_KERNEL_REGISTRY_H_
#define OPENGL_CORE_KERNEL_REGISTRY_H_

#include <string>

#include "opengl/core/types.h"

namespace opengl {

class KernelRegistry {
 public:
  void RegisterKernel(std::string kernel_name, KernelFactory kernel_factory);
  // Leaves *kernel null when no factory is registered under kernel_name.
  void CreateKernel(std::string kernel_name, Kernel** kernel, Context* context);
  bool HasKernel(const std::string& kernel_name) const;
  StringList RegisteredNames() const;
  static KernelRegistry* Global();

 private:
  KernelRegistry() {}
  KernelMap kernel_map_;
};

namespace registry {
template <typename T>
class KernelRegisterHelper {
 public:
  explicit KernelRegisterHelper(const char* kernel_name) {
    KernelRegistry::Global()->RegisterKernel(
        kernel_name, [](Kernel** kernel, Context* context) { *kernel = new T(context); });
  }
};
}  // namespace registry
}  // namespace opengl

#define REGISTER_KERNEL_UNIQ(ctr, Class, class_name) \
  static ::opengl::registry::KernelRegisterHelper<Class> __register##ctr(class_name)
#define REGISTER_KERNEL_UNIQ_HELPER(ctr, Class, name) REGISTER_KERNEL_UNIQ(ctr, Class, name)
#define REGISTER_KERNEL(Class) REGISTER_KERNEL_UNIQ_HELPER(__COUNTER__, Class, #Class)
#define REGISTER_KERNEL_WITH_NAME(Class, class_name) \
  REGISTER_KERNEL_UNIQ_HELPER(__COUNTER__, Class, class_name)

#endif  // OPENGL_CORE_KERNEL_REGISTRY_H_
