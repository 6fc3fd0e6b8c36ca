// What Context::cublas_handle() points at in this build: device scratch owned by
// the context for the level-1 routines whose signature carries no Workspace
// (BlasSasum, shadow/core/blas.hpp:91-92).  The reference's cuBLAS handle owned
// such a workspace itself (shadow/core/context.cu:38-45 creates the handle per
// context); here the slot carries the buffer directly, so the Context interface
// of shadow/core/context.hpp:11-29 stays as it is.  One stream per context, so
// one user at a time.
#ifndef SHADOW_AMD_HOST_LEVEL1_HANDLE_HPP_
#define SHADOW_AMD_HOST_LEVEL1_HANDLE_HPP_

#include <cstddef>

namespace Shadow {

struct Level1Handle {
  void* scratch = nullptr;  // device memory, allocated with the context, freed with it
  size_t bytes = 0;
};

}  // namespace Shadow

#endif  // SHADOW_AMD_HOST_LEVEL1_HANDLE_HPP_
