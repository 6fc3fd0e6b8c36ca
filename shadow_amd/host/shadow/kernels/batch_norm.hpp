// BatchNorm kernel interface: shadow/operators/kernels/batch_norm.hpp:8-54.
#ifndef SHADOW_AMD_HOST_KERNELS_BATCH_NORM_HPP_
#define SHADOW_AMD_HOST_KERNELS_BATCH_NORM_HPP_

#include "shadow/kernel.hpp"

namespace Shadow {

namespace Vision {
// index = (i / inner_num) % channel
template <DeviceType D, typename T>
void BatchNorm(const float* in_data, int count, const float* mean_data,
               const float* variance_data, int channel, int inner_num, float scale_factor,
               float eps, float* out_data, Context* context);
}  // namespace Vision

class BatchNormKernel : public Kernel {
 public:
  virtual void Run(const std::shared_ptr<Blob>& input, const std::shared_ptr<Blob>& mean,
                   const std::shared_ptr<Blob>& variance, std::shared_ptr<Blob>& output,
                   Workspace* ws, float scale_factor, float eps) = 0;
};

}  // namespace Shadow

#endif  // SHADOW_AMD_HOST_KERNELS_BATCH_NORM_HPP_
