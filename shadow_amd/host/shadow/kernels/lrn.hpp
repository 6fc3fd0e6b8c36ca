// LRN kernel interface: shadow/operators/kernels/lrn.hpp:8-48.
#ifndef SHADOW_AMD_HOST_KERNELS_LRN_HPP_
#define SHADOW_AMD_HOST_KERNELS_LRN_HPP_

#include "shadow/kernel.hpp"

namespace Shadow {

namespace Vision {
// Across channels.  scale_data is the reference's scratch blob of the input's
// size; the device kernel keeps a window in LDS instead and never touches it
// (nullptr is fine).
template <DeviceType D, typename T>
void LRN(const T* in_data, const VecInt& in_shape, int size, float alpha, float beta, float k,
         T* scale_data, T* out_data, Context* context);
}  // namespace Vision

class LRNKernel : public Kernel {
 public:
  virtual void Run(const std::shared_ptr<Blob>& input, std::shared_ptr<Blob>& output, Workspace* ws,
                   int size, float alpha, float beta, float k) = 0;
};

}  // namespace Shadow

#endif  // SHADOW_AMD_HOST_KERNELS_LRN_HPP_
