// Blas::X<DeviceType::kGPU, float>: one shdw_hip_* launch each, on the context's
// stream.  Replaces the macro-generated CUDA kernels and cuBLAS level-1 calls of
// shadow/core/blas.cu:11-138.
#include "shadow/blas.hpp"

#include "level1_handle.hpp"
#include "shadow_hip.h"

namespace Shadow {
namespace Blas {

namespace {
constexpr DeviceType G = DeviceType::kGPU;
inline void* stream_of(Context* ctx) { return ctx != nullptr ? ctx->stream() : nullptr; }
}  // namespace

template <>
void Set<G, float>(int n, float val, float* y, int offy, Context* ctx) {
  SHADOW_HIP_CHECK(shdw_hip_set(n, val, y + offy, stream_of(ctx)));
}

#define SHADOW_DEFINE_BINARY(name, code)                                                       \
  template <>                                                                                  \
  void name<G, float>(int n, const float* a, int offa, const float* b, int offb, float* y,     \
                      int offy, Context* ctx) {                                                \
    SHADOW_HIP_CHECK(shdw_hip_binary(code, n, a + offa, b + offb, y + offy, stream_of(ctx)));  \
  }                                                                                            \
  template <>                                                                                  \
  void name<G, float>(int n, const float* a, int offa, float alpha, float* y, int offy,        \
                      Context* ctx) {                                                          \
    SHADOW_HIP_CHECK(shdw_hip_binary_scalar(code, n, a + offa, alpha, y + offy, stream_of(ctx))); \
  }
SHADOW_DEFINE_BINARY(Add, SHDW_BINARY_ADD)
SHADOW_DEFINE_BINARY(Sub, SHDW_BINARY_SUB)
SHADOW_DEFINE_BINARY(Mul, SHDW_BINARY_MUL)
SHADOW_DEFINE_BINARY(Div, SHDW_BINARY_DIV)
SHADOW_DEFINE_BINARY(Pow, SHDW_BINARY_POW)
SHADOW_DEFINE_BINARY(Max, SHDW_BINARY_MAX)
SHADOW_DEFINE_BINARY(Min, SHDW_BINARY_MIN)
#undef SHADOW_DEFINE_BINARY

#define SHADOW_DEFINE_UNARY(name, code)                                                    \
  template <>                                                                              \
  void name<G, float>(int n, const float* a, int offa, float* y, int offy, Context* ctx) { \
    SHADOW_HIP_CHECK(shdw_hip_unary(code, n, a + offa, y + offy, stream_of(ctx)));         \
  }
SHADOW_DEFINE_UNARY(Abs, SHDW_UNARY_ABS)
SHADOW_DEFINE_UNARY(Square, SHDW_UNARY_SQUARE)
SHADOW_DEFINE_UNARY(Sqrt, SHDW_UNARY_SQRT)
SHADOW_DEFINE_UNARY(Log, SHDW_UNARY_LOG)
SHADOW_DEFINE_UNARY(Exp, SHDW_UNARY_EXP)
SHADOW_DEFINE_UNARY(Sin, SHDW_UNARY_SIN)
SHADOW_DEFINE_UNARY(Cos, SHDW_UNARY_COS)
SHADOW_DEFINE_UNARY(Tan, SHDW_UNARY_TAN)
SHADOW_DEFINE_UNARY(Asin, SHDW_UNARY_ASIN)
SHADOW_DEFINE_UNARY(Acos, SHDW_UNARY_ACOS)
SHADOW_DEFINE_UNARY(Atan, SHDW_UNARY_ATAN)
SHADOW_DEFINE_UNARY(Floor, SHDW_UNARY_FLOOR)
SHADOW_DEFINE_UNARY(Ceil, SHDW_UNARY_CEIL)
SHADOW_DEFINE_UNARY(Neg, SHDW_UNARY_NEG)
SHADOW_DEFINE_UNARY(Reciprocal, SHDW_UNARY_RECIPROCAL)
#undef SHADOW_DEFINE_UNARY

template <>
void BlasSscal<G, float>(int n, float alpha, float* x, int offx, Context* ctx) {
  SHADOW_HIP_CHECK(shdw_hip_scal(n, alpha, x + offx, stream_of(ctx)));
}

template <>
void BlasScopy<G, float>(int n, const float* x, int offx, float* y, int offy, Context* ctx) {
  SHADOW_HIP_CHECK(shdw_hip_copy(n, x + offx, y + offy, stream_of(ctx)));
}

template <>
void BlasSaxpy<G, float>(int n, float alpha, const float* x, int offx, float* y, int offy,
                         Context* ctx) {
  SHADOW_HIP_CHECK(shdw_hip_axpy(n, alpha, x + offx, y + offy, stream_of(ctx)));
}

template <>
void BlasSasum<G, float>(int n, const float* x, int offx, float* y, Context* ctx) {
  // The signature has no Workspace to borrow scratch from (it did not need one
  // on top of cuBLAS): the partial sums live in the scratch behind the context's
  // cublas_handle() slot, which is allocated with the context.  The reference calls this once per batch item
  // (kernels/ssd_normalize.hpp:51-57); an allocation per call would stall the
  // device every time.
  CHECK_NOTNULL(ctx);
  const int shape[1] = {n}, axes[1] = {0};
  const size_t bytes = shdw_hip_reduce_workspace_bytes(1, shape, 1, axes) + 16;
  const Level1Handle* handle = static_cast<const Level1Handle*>(ctx->cublas_handle());
  CHECK_NOTNULL(handle);
  CHECK_LE(bytes, handle->bytes) << "BlasSasum: the context's level-1 scratch is too small";
  SHADOW_HIP_CHECK(shdw_hip_asum(n, x + offx, y, handle->scratch, bytes, stream_of(ctx)));
}

}  // namespace Blas
}  // namespace Shadow
