// Binary kernel interface: shadow/operators/kernels/binary.hpp:23-35.
#ifndef SHADOW_AMD_HOST_KERNELS_BINARY_HPP_
#define SHADOW_AMD_HOST_KERNELS_BINARY_HPP_

#include "shadow/blas.hpp"
#include "shadow/kernel.hpp"

namespace Shadow {

namespace Vision {
// Numpy-style broadcast of `scalar_data` against `in_data`.  Unlike the CUDA
// version (shadow/operators/kernels/binary.cu:28-64) the three rank-aligned
// shape arrays are HOST pointers: they are folded into kernel arguments.
template <DeviceType D, typename T>
void BroadcastBinary(const T* in_data, const int* in_shape, const T* scalar_data,
                     const int* scalar_shape, int operation, int num_axes, int count,
                     const int* out_shape, T* out_data, Context* context);
}  // namespace Vision

enum { kAdd = 0, kSub = 1, kMul = 2, kDiv = 3, kPow = 4, kMax = 5, kMin = 6 };

class BinaryKernel : public Kernel {
 public:
  // input (op) scalar_value
  virtual void Run(const std::shared_ptr<Blob>& input, std::shared_ptr<Blob>& output,
                   Workspace* ws, int operation, float scalar_value) = 0;
  // input (op) scalar; shapes are equal, or rank-aligned and broadcastable
  virtual void Run(const std::shared_ptr<Blob>& input, const std::shared_ptr<Blob>& scalar,
                   std::shared_ptr<Blob>& output, Workspace* ws, int operation,
                   bool need_broadcast) = 0;
};

}  // namespace Shadow

#endif  // SHADOW_AMD_HOST_KERNELS_BINARY_HPP_
