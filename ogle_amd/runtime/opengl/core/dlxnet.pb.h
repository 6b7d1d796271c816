// Compatibility name: the reference includes the protoc-generated
// "opengl/core/dlxnet.pb.h"; the hand-written schema classes stand in for it.
#ifndef OPENGL_CORE_DLXNET_PB_H_
#define OPENGL_CORE_DLXNET_PB_H_
#include "opengl/core/dlxnet.h"
#endif
