// Launch-side constants and error capture shared by the kernel files.
#ifndef SHADOW_AMD_CSRC_LAUNCH_H_
#define SHADOW_AMD_CSRC_LAUNCH_H_

#include <hip/hip_runtime.h>

#include <cstdint>

namespace shdw {

// Grid cap for the grid-stride streaming kernels: 8 workgroups of 256 lanes per
// CU on 256 CUs keeps 32 wave64 resident per CU, the most gfx950 holds.
constexpr uint32_t kMaxStreamGrid = 256 * 8;

// Shadow checks cudaPeekAtLastError() after every launch
// (e.g. shadow/core/blas.cu:20); here the error is also cleared so that one bad
// launch does not fail every later call.
inline int launch_status() { return static_cast<int>(hipGetLastError()); }

}  // namespace shdw

#endif  // SHADOW_AMD_CSRC_LAUNCH_H_
