// GroupNorm / InstanceNorm / LayerNorm: x viewed as [outer][inner] rows; every
// row is shifted by its mean and divided by sqrt(variance + eps), then an
// optional per-channel scale and bias is applied.
//
// Shadow computes both statistics with its plain-loop Sgemv against a vector of
// ones: (float) of an fp64 running sum of the fp32 products alpha * v with
// alpha = 1 / inner (shadow/core/blas.cpp:238-247), five launches and three
// scratch blobs per call (shadow/operators/kernels/group_norm.hpp:41-86).  Here
// one workgroup owns a row and does everything in one launch: fp64 partial sums
// per lane, combined through LDS.  The fp64 additions are associated
// differently from the reference's front-to-back loop; the sums are then
// rounded to fp32 once, so the statistics (and with them every output) come out
// identical unless an fp64 sum lands within ~1e-16 relative of an fp32 rounding
// boundary.  Rows of up to 4096 elements stay in registers between the three
// passes (one HBM read, one write); longer rows are re-read, from L2.
#include <hip/hip_runtime.h>

#include "../../include/shadow_hip.h"
#include "device_common.h"
#include "launch.h"

#pragma clang fp contract(off)

namespace shdw {

struct NormArgs {
  uint32_t inner;
  float alpha, eps;
  const float* scale;  // nullptr: no affine step
  const float* bias;
  FastDiv f_scale_inner, f_scale_num;  // channel = (i / scale_inner) % scale_num
};

// Sum over the workgroup, result in every lane.  `slots` holds one double per wave.
SHDW_DEVICE double block_sum(double v, double* slots) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off);
  __syncthreads();  // slots may still be read from the previous sum
  if ((threadIdx.x & 63) == 0) slots[threadIdx.x >> 6] = v;
  __syncthreads();
  double total = slots[0];
#pragma unroll
  for (int w = 1; w < kBlock / kWave; ++w) total += slots[w];
  return total;
}

SHDW_DEVICE float norm_affine(const NormArgs& p, uint32_t i, float v) {
  if (p.scale == nullptr) return v;
  const uint32_t q = fd_div(i, p.f_scale_inner);
  const uint32_t c = q - fd_div(q, p.f_scale_num) * p.f_scale_num.d;
  const float t = v * p.scale[c];
  return t + p.bias[c];
}

// REGS > 0: the row (<= REGS * 4 * kBlock elements, inner % 4 == 0, 16-byte
// aligned) is held in REGS vectors per lane.  REGS < 0: longer rows of that
// kind, three passes with 128-bit accesses.  REGS == 0: any row, three passes
// with scalar accesses.
template <int REGS>
__global__ __launch_bounds__(kBlock) void norm_rows_kernel(const float* x, float* y, NormArgs p) {
  __shared__ double slots[kBlock / kWave];
  const uint64_t base = static_cast<uint64_t>(blockIdx.x) * p.inner;
  const float* xr = x + base;
  float* yr = y + base;
  if (REGS > 0) {
    constexpr int R = REGS > 0 ? REGS : 1;
    const uint32_t nvec = p.inner / 4;
    v4f reg[R];
#pragma unroll
    for (int k = 0; k < R; ++k) {
      const uint32_t v = k * kBlock + threadIdx.x;
      if (v < nvec) reg[k] = load4_stream(xr + 4ull * v);
    }
    double acc = 0;
#pragma unroll
    for (int k = 0; k < R; ++k) {
      if (k * kBlock + threadIdx.x < nvec) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float t = p.alpha * reg[k][j];
          acc += static_cast<double>(t);
        }
      }
    }
    const float mean = static_cast<float>(block_sum(acc, slots));
    acc = 0;
#pragma unroll
    for (int k = 0; k < R; ++k) {
      if (k * kBlock + threadIdx.x < nvec) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float val = reg[k][j] - mean;
          reg[k][j] = val;
          const float sq = val * val;
          const float t = p.alpha * sq;
          acc += static_cast<double>(t);
        }
      }
    }
    const float variance = static_cast<float>(block_sum(acc, slots));
    const float ve = variance + p.eps;
    const float denom = __builtin_sqrtf(ve);
#pragma unroll
    for (int k = 0; k < R; ++k) {
      const uint32_t v = k * kBlock + threadIdx.x;
      if (v < nvec) {
        v4f r;
#pragma unroll
        for (int j = 0; j < 4; ++j)
          r[j] = norm_affine(p, static_cast<uint32_t>(base) + 4 * v + j, reg[k][j] / denom);
        store4_stream(yr + 4ull * v, r);
      }
    }
  } else if (REGS < 0) {
    // Long rows, 128-bit accesses; passes two and three find the row in L2.
    const uint32_t nvec = p.inner / 4;
    double acc = 0;
    for (uint32_t v = threadIdx.x; v < nvec; v += kBlock) {
      const v4f q = load4(xr + 4ull * v);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float a = p.alpha * q[j];
        acc += static_cast<double>(a);
      }
    }
    const float mean = static_cast<float>(block_sum(acc, slots));
    acc = 0;
    for (uint32_t v = threadIdx.x; v < nvec; v += kBlock) {
      const v4f q = load4(xr + 4ull * v);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float val = q[j] - mean;
        const float sq = val * val;
        const float a = p.alpha * sq;
        acc += static_cast<double>(a);
      }
    }
    const float variance = static_cast<float>(block_sum(acc, slots));
    const float ve = variance + p.eps;
    const float denom = __builtin_sqrtf(ve);
    for (uint32_t v = threadIdx.x; v < nvec; v += kBlock) {
      const v4f q = load4(xr + 4ull * v);
      v4f r;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float val = q[j] - mean;
        r[j] = norm_affine(p, static_cast<uint32_t>(base) + 4 * v + j, val / denom);
      }
      store4_stream(yr + 4ull * v, r);
    }
  } else {
    double acc = 0;
    for (uint32_t t = threadIdx.x; t < p.inner; t += kBlock) {
      const float a = p.alpha * xr[t];
      acc += static_cast<double>(a);
    }
    const float mean = static_cast<float>(block_sum(acc, slots));
    acc = 0;
    for (uint32_t t = threadIdx.x; t < p.inner; t += kBlock) {
      const float val = xr[t] - mean;
      const float sq = val * val;
      const float a = p.alpha * sq;
      acc += static_cast<double>(a);
    }
    const float variance = static_cast<float>(block_sum(acc, slots));
    const float ve = variance + p.eps;
    const float denom = __builtin_sqrtf(ve);
    for (uint32_t t = threadIdx.x; t < p.inner; t += kBlock) {
      const float val = xr[t] - mean;
      yr[t] = norm_affine(p, static_cast<uint32_t>(base) + t, val / denom);
    }
  }
}

}  // namespace shdw

using namespace shdw;

extern "C" {

int shdw_hip_group_norm(int outer_num, int inner_num, float eps, const float* x,
                        const float* scale, const float* bias, int scale_num, int scale_inner,
                        float* y, void* stream) {
  if (outer_num < 0 || inner_num < 0) return SHDW_E_INVALID_ARGUMENT;
  const int64_t count = static_cast<int64_t>(outer_num) * inner_num;
  if (count > INT32_MAX) return SHDW_E_INVALID_ARGUMENT;
  if (count == 0) return SHDW_OK;
  if (!x || !y || (scale == nullptr) != (bias == nullptr)) return SHDW_E_INVALID_ARGUMENT;
  if (scale && (scale_num < 1 || scale_inner < 1)) return SHDW_E_INVALID_ARGUMENT;
  NormArgs p;
  p.inner = static_cast<uint32_t>(inner_num);
  p.alpha = 1.f / inner_num;
  p.eps = eps;
  p.scale = scale;
  p.bias = bias;
  p.f_scale_inner = make_fastdiv(static_cast<uint32_t>(scale ? scale_inner : 1));
  p.f_scale_num = make_fastdiv(static_cast<uint32_t>(scale ? scale_num : 1));
  hipStream_t st = static_cast<hipStream_t>(stream);
  const uint32_t grid = static_cast<uint32_t>(outer_num);
  const bool vec = inner_num % 4 == 0 && aligned16(x) && aligned16(y);
  const int vecs = (inner_num / 4 + kBlock - 1) / kBlock;
  if (vec && vecs <= 1)
    norm_rows_kernel<1><<<grid, kBlock, 0, st>>>(x, y, p);
  else if (vec && vecs <= 2)
    norm_rows_kernel<2><<<grid, kBlock, 0, st>>>(x, y, p);
  else if (vec && vecs <= 4)
    norm_rows_kernel<4><<<grid, kBlock, 0, st>>>(x, y, p);
  else if (vec)
    norm_rows_kernel<-1><<<grid, kBlock, 0, st>>>(x, y, p);
  else
    norm_rows_kernel<0><<<grid, kBlock, 0, st>>>(x, y, p);
  return launch_status();
}

}  // extern "C"
