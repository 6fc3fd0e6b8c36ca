// Scale kernel interface: shadow/operators/kernels/scale.hpp:8-39.
#ifndef SHADOW_AMD_HOST_KERNELS_SCALE_HPP_
#define SHADOW_AMD_HOST_KERNELS_SCALE_HPP_

#include "shadow/kernel.hpp"

namespace Shadow {

namespace Vision {
// index = (i / inner_num) % scale_num
template <DeviceType D, typename T>
void ScaleBias(const T* in_data, int count, const T* scale_data, const T* bias_data,
               int scale_num, int inner_num, T* out_data, Context* context);
template <DeviceType D, typename T>
void Scale(const T* in_data, int count, const T* scale_data, int scale_num, int inner_num,
           T* out_data, Context* context);
template <DeviceType D, typename T>
void Bias(const T* in_data, int count, const T* bias_data, int scale_num, int inner_num,
          T* out_data, Context* context);
}  // namespace Vision

class ScaleKernel : public Kernel {
 public:
  // parameters are blobs; either may be nullptr but not both
  virtual void Run(const std::shared_ptr<Blob>& input, const std::shared_ptr<Blob>& scale,
                   const std::shared_ptr<Blob>& bias, std::shared_ptr<Blob>& output,
                   Workspace* ws, int axis) = 0;
  // parameters are per-channel host values (either may be empty but not both)
  virtual void Run(const std::shared_ptr<Blob>& input, std::shared_ptr<Blob>& output,
                   Workspace* ws, int axis, const VecFloat& scale_value,
                   const VecFloat& bias_value) = 0;
};

}  // namespace Shadow

#endif  // SHADOW_AMD_HOST_KERNELS_SCALE_HPP_
