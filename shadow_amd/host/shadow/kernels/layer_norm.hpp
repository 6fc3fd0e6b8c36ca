// LayerNorm kernel interface: shadow/operators/kernels/layer_norm.hpp:8-18.
#ifndef SHADOW_AMD_HOST_KERNELS_LAYER_NORM_HPP_
#define SHADOW_AMD_HOST_KERNELS_LAYER_NORM_HPP_

#include "shadow/kernels/group_norm.hpp"

namespace Shadow {

class LayerNormKernel : public Kernel {
 public:
  virtual void Run(const std::shared_ptr<Blob>& input, const std::shared_ptr<Blob>& scale,
                   const std::shared_ptr<Blob>& bias, std::shared_ptr<Blob>& output,
                   Workspace* ws, const VecInt& normalized_shape, float eps) = 0;
};

}  // namespace Shadow

#endif  // SHADOW_AMD_HOST_KERNELS_LAYER_NORM_HPP_
