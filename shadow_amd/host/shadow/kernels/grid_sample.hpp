// GridSample kernel interface: shadow/operators/kernels/grid_sample.hpp:8-50.
#ifndef SHADOW_AMD_HOST_KERNELS_GRID_SAMPLE_HPP_
#define SHADOW_AMD_HOST_KERNELS_GRID_SAMPLE_HPP_

#include "shadow/kernel.hpp"

namespace Shadow {

namespace Vision {
// mode 0 nearest, 1 bilinear; padding_mode 0 zeros, 1 border
template <DeviceType D, typename T>
void GridSample(const T* in_data, const VecInt& in_shape, const float* grid_data, int mode,
                int padding_mode, const VecInt& out_shape, T* out_data, Context* context);
}  // namespace Vision

class GridSampleKernel : public Kernel {
 public:
  virtual void Run(const std::shared_ptr<Blob>& input, const std::shared_ptr<Blob>& grid,
                   std::shared_ptr<Blob>& output, Workspace* ws, int mode, int padding_mode) = 0;
};

}  // namespace Shadow

#endif  // SHADOW_AMD_HOST_KERNELS_GRID_SAMPLE_HPP_
