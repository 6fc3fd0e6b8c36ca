// Softmax kernel interface: shadow/operators/kernels/softmax.hpp:8-46.  The
// reference's per-column scratch argument is gone: the device kernels keep the
// column maximum and sum in registers or LDS.
#ifndef SHADOW_AMD_HOST_KERNELS_SOFTMAX_HPP_
#define SHADOW_AMD_HOST_KERNELS_SOFTMAX_HPP_

#include "shadow/kernel.hpp"

namespace Shadow {

namespace Vision {
template <DeviceType D, typename T>
void Softmax(const T* in_data, int outer_num, int dim, int inner_num, T* out_data,
             Context* context);
}  // namespace Vision

class SoftmaxKernel : public Kernel {
 public:
  virtual void Run(const std::shared_ptr<Blob>& input, std::shared_ptr<Blob>& output,
                   Workspace* ws, int axis) = 0;
};

}  // namespace Shadow

#endif  // SHADOW_AMD_HOST_KERNELS_SOFTMAX_HPP_
