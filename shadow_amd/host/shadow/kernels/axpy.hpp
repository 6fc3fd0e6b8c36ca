// Axpy kernel interface: shadow/operators/kernels/axpy.hpp:8-50.
#ifndef SHADOW_AMD_HOST_KERNELS_AXPY_HPP_
#define SHADOW_AMD_HOST_KERNELS_AXPY_HPP_

#include "shadow/kernel.hpp"

namespace Shadow {

namespace Vision {
// out[n, :] = y[n, :] + alpha[n] * x[n, :] for n < outer_num
template <DeviceType D, typename T>
void Axpy(const float* alpha_data, const float* x_data, const float* y_data, int outer_num,
          int inner_num, float* out_data, Context* context);
}  // namespace Vision

class AxpyKernel : public Kernel {
 public:
  virtual void Run(const std::shared_ptr<Blob>& alpha, const std::shared_ptr<Blob>& x,
                   const std::shared_ptr<Blob>& y, std::shared_ptr<Blob>& output,
                   Workspace* ws) = 0;
};

}  // namespace Shadow

#endif  // SHADOW_AMD_HOST_KERNELS_AXPY_HPP_
