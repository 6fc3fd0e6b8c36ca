// Blas:: free functions with the template signatures of shadow/core/blas.hpp:10-75
// (elementwise part and level 1).  Only <DeviceType::kGPU, float> is
// instantiated (src/blas_hip.cpp); each call enqueues one shdw_hip_* kernel on
// the context's stream and returns.  Sgemv/Sgemm are dense contractions and are
// not part of this layer.
#ifndef SHADOW_AMD_HOST_BLAS_HPP_
#define SHADOW_AMD_HOST_BLAS_HPP_

#include "device.hpp"

namespace Shadow {
namespace Blas {

template <DeviceType D, typename T>
void Set(int n, T val, T* y, int offy, Context* context);

#define SHADOW_BLAS_BINARY(name)                                                               \
  template <DeviceType D, typename T>                                                          \
  void name(int n, const T* a, int offa, const T* b, int offb, T* y, int offy, Context* ctx);  \
  template <DeviceType D, typename T>                                                          \
  void name(int n, const T* a, int offa, float alpha, T* y, int offy, Context* ctx);
SHADOW_BLAS_BINARY(Add)
SHADOW_BLAS_BINARY(Sub)
SHADOW_BLAS_BINARY(Mul)
SHADOW_BLAS_BINARY(Div)
SHADOW_BLAS_BINARY(Pow)
SHADOW_BLAS_BINARY(Max)
SHADOW_BLAS_BINARY(Min)
#undef SHADOW_BLAS_BINARY

#define SHADOW_BLAS_UNARY(name)       \
  template <DeviceType D, typename T> \
  void name(int n, const T* a, int offa, T* y, int offy, Context* ctx);
SHADOW_BLAS_UNARY(Abs)
SHADOW_BLAS_UNARY(Square)
SHADOW_BLAS_UNARY(Sqrt)
SHADOW_BLAS_UNARY(Log)
SHADOW_BLAS_UNARY(Exp)
SHADOW_BLAS_UNARY(Sin)
SHADOW_BLAS_UNARY(Cos)
SHADOW_BLAS_UNARY(Tan)
SHADOW_BLAS_UNARY(Asin)
SHADOW_BLAS_UNARY(Acos)
SHADOW_BLAS_UNARY(Atan)
SHADOW_BLAS_UNARY(Floor)
SHADOW_BLAS_UNARY(Ceil)
SHADOW_BLAS_UNARY(Neg)
SHADOW_BLAS_UNARY(Reciprocal)
#undef SHADOW_BLAS_UNARY

template <DeviceType D, typename T>
void BlasSscal(int n, float alpha, T* x, int offx, Context* context);
template <DeviceType D, typename T>
void BlasScopy(int n, const T* x, int offx, T* y, int offy, Context* context);
template <DeviceType D, typename T>
void BlasSaxpy(int n, float alpha, const T* x, int offx, T* y, int offy, Context* context);
// *y is a HOST float; the call returns after the value has arrived.
template <DeviceType D, typename T>
void BlasSasum(int n, const T* x, int offx, float* y, Context* context);

}  // namespace Blas
}  // namespace Shadow

#endif  // SHADOW_AMD_HOST_BLAS_HPP_
