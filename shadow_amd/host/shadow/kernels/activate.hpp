// Activate kernel interface: shadow/operators/kernels/activate.hpp:8-42.
#ifndef SHADOW_AMD_HOST_KERNELS_ACTIVATE_HPP_
#define SHADOW_AMD_HOST_KERNELS_ACTIVATE_HPP_

#include "shadow/kernel.hpp"

namespace Shadow {

namespace Vision {
template <DeviceType D, typename T>
void Activate(const T* in_data, T* out_data, int count, int type, float slope, Context* context);

template <DeviceType D, typename T>
void PRelu(const T* in_data, T* out_data, const VecInt& in_shape, bool channel_shared,
           const T* slope_data, Context* context);
}  // namespace Vision

enum {
  kPRelu = 0, kRelu = 1, kLeaky = 2, kSigmoid = 3, kSoftPlus = 4, kTanh = 5, kRelu6 = 6,
  kHardSwish = 7, kGelu = 8
};

class ActivateKernel : public Kernel {
 public:
  // `slope` is the second input blob of PRelu, nullptr for every other type.
  virtual void Run(const std::shared_ptr<Blob>& input, const std::shared_ptr<Blob>& slope,
                   std::shared_ptr<Blob>& output, Workspace* ws, int activate_type,
                   float slope_val) = 0;
};

}  // namespace Shadow

#endif  // SHADOW_AMD_HOST_KERNELS_ACTIVATE_HPP_
