// Reduce kernel interface: shadow/operators/kernels/reduce.hpp:21-36.
#ifndef SHADOW_AMD_HOST_KERNELS_REDUCE_HPP_
#define SHADOW_AMD_HOST_KERNELS_REDUCE_HPP_

#include "shadow/kernel.hpp"

namespace Shadow {

namespace Vision {
// The reference passes device index lists (shadow/operators/kernels/reduce.hpp:9-15);
// here the HOST shape and axis list are enough, the kernels derive their own
// addressing.  `workspace` is device scratch of at least
// shdw_hip_reduce_workspace_bytes() bytes (may be null when that is 0).
template <DeviceType D, typename T>
void Reduce(const T* in_data, const int* in_shape, int num_axes, const int* axes, int num_reduce,
            int operation, T* out_data, void* workspace, size_t workspace_bytes,
            Context* context);
}  // namespace Vision

enum { kProd = 0, kSum = 1, kMax = 2, kMin = 3, kAvg = 4, kLpNorm1 = 5, kLpNorm2 = 6 };

class ReduceKernel : public Kernel {
 public:
  virtual void Run(const std::shared_ptr<Blob>& input, std::shared_ptr<Blob>& output,
                   Workspace* ws, int operation, const VecInt& axes) = 0;
};

}  // namespace Shadow

#endif  // SHADOW_AMD_HOST_KERNELS_REDUCE_HPP_
