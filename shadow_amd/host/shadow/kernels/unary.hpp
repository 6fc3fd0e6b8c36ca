// Unary kernel interface: shadow/operators/kernels/unary.hpp:9-32.
#ifndef SHADOW_AMD_HOST_KERNELS_UNARY_HPP_
#define SHADOW_AMD_HOST_KERNELS_UNARY_HPP_

#include "shadow/blas.hpp"
#include "shadow/kernel.hpp"

namespace Shadow {

enum {
  kAbs = 0, kSquare = 1, kSqrt = 2, kLog = 3, kExp = 4, kSin = 5, kCos = 6, kTan = 7,
  kAsin = 8, kAcos = 9, kAtan = 10, kFloor = 11, kCeil = 12, kNeg = 13, kReciprocal = 14
};

class UnaryKernel : public Kernel {
 public:
  virtual void Run(const std::shared_ptr<Blob>& input, std::shared_ptr<Blob>& output,
                   Workspace* ws, int operation) = 0;
};

}  // namespace Shadow

#endif  // SHADOW_AMD_HOST_KERNELS_UNARY_HPP_
