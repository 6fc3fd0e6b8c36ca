// Eltwise kernel interface: shadow/operators/kernels/eltwise.hpp:9-16.
#ifndef SHADOW_AMD_HOST_KERNELS_ELTWISE_HPP_
#define SHADOW_AMD_HOST_KERNELS_ELTWISE_HPP_

#include "shadow/blas.hpp"
#include "shadow/kernel.hpp"

namespace Shadow {

enum { kProd = 0, kSum = 1, kMax = 2, kMin = 3 };

class EltwiseKernel : public Kernel {
 public:
  virtual void Run(const std::vector<std::shared_ptr<Blob>>& inputs,
                   std::shared_ptr<Blob>& output, Workspace* ws, int operation,
                   const VecFloat& coeff) = 0;
};

}  // namespace Shadow

#endif  // SHADOW_AMD_HOST_KERNELS_ELTWISE_HPP_
