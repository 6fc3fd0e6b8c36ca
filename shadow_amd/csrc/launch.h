// Launch-side constants and error capture shared by the kernel files.
#ifndef SHADOW_AMD_CSRC_LAUNCH_H_
#define SHADOW_AMD_CSRC_LAUNCH_H_

#include <hip/hip_runtime.h>

#include <cstdint>

namespace shdw {

// Workgroups of kBlock (256) lanes needed for `work` lane-tasks.  Counts are
// int32, so this never exceeds 2^23 + 1 workgroups.
inline uint32_t grid_for(uint32_t work) { return (work + 255u) / 256u; }
// The same for kStream (64) lanes: at most 2^25 + 1 workgroups.
inline uint32_t stream_grid(uint32_t work) { return (work + 63u) / 64u; }

// Shadow checks cudaPeekAtLastError() after every launch
// (e.g. shadow/core/blas.cu:20); here the error is also cleared so that one bad
// launch does not fail every later call.
inline int launch_status() { return static_cast<int>(hipGetLastError()); }

// Device memory owned by the library (reduce.hip): the partial results of
// shdw_hip_reduce_static.  Resolves its address on the current device, once per
// device; returns 0 or an error code.
int library_scratch_prepare();

// Max over every row of x [rows][len] with Reduce's kernels (reduce.hip), if that
// takes a single stage and so no workspace: then *rc holds the launch result and
// the return value is true.
bool reduce_rows_max(uint32_t rows, uint32_t len, const float* x, float* y, hipStream_t st, int* rc);
bool reduce_rows_max_applies(uint32_t rows, uint32_t len);  // whether it would (host only)

}  // namespace shdw

#endif  // SHADOW_AMD_CSRC_LAUNCH_H_
