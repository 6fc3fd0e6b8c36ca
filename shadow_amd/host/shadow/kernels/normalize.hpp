// Normalize kernel interface: shadow/operators/kernels/normalize.hpp:8-44
// (without the per-column scratch argument, see softmax.hpp).
#ifndef SHADOW_AMD_HOST_KERNELS_NORMALIZE_HPP_
#define SHADOW_AMD_HOST_KERNELS_NORMALIZE_HPP_

#include "shadow/kernel.hpp"

namespace Shadow {

namespace Vision {
template <DeviceType D, typename T>
void Normalize(const T* in_data, int outer_num, int dim, int inner_num, float p, float eps,
               T* out_data, Context* context);
}  // namespace Vision

class NormalizeKernel : public Kernel {
 public:
  virtual void Run(const std::shared_ptr<Blob>& input, std::shared_ptr<Blob>& output,
                   Workspace* ws, float p, int axis, float eps) = 0;
};

}  // namespace Shadow

#endif  // SHADOW_AMD_HOST_KERNELS_NORMALIZE_HPP_
