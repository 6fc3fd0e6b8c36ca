// The ResNet bottleneck tail in one launch: per-channel Scale, residual add
// (Eltwise SUM), ReLU and the global average over the trailing `inner`
// elements.  x and the residual are read once, y is written once and the
// pooled value falls out of the same registers; run as four operators the
// same data crosses HBM 8 times instead of 3.
//
// One wave64 owns one (n, c) row.  Arithmetic per element is exactly the
// operator sequence: t = x*s; t = t + b; u = 0 + 1*t; u = u + 1*r;
// y = u > 0 ? u : 0; the row sum is fp64 and rounded once after the divide.
#include <hip/hip_runtime.h>

#include "../../include/shadow_hip.h"
#include "device_common.h"
#include "launch.h"

#pragma clang fp contract(off)

namespace shdw {

// The operator sequence on one element.  HAS_SCALE / HAS_BIAS: which parameter
// blobs the Scale operator has (Vision::ScaleBias, Scale or Bias); RES_FIRST: the
// residual is the Eltwise operator's first input and the scaled value its second.
template <bool HAS_SCALE, bool HAS_BIAS, bool RES_FIRST>
SHDW_DEVICE float tail_element(float x, float s, float b, float r) {
  float t = x;
  if (HAS_SCALE) t = t * s;
  if (HAS_BIAS) t = t + b;
  // Eltwise SUM with unit coefficients: Set(0), then y += 1 * input, input by input
  const float first = 1.0f * (RES_FIRST ? r : t), second = 1.0f * (RES_FIRST ? t : r);
  float u = 0.0f + first;
  u = u + second;
  return u > 0 ? u : 0;
}

SHDW_DEVICE double wave_sum_f64(double v) {
  v += dpp_f64<kDppXor1>(v);
  v += dpp_f64<kDppXor2>(v);
  v += dpp_f64<kDppHalfMirror>(v);
  v += dpp_f64<kDppMirror>(v);
  v += __shfl_xor(v, 16, kWave);
  v += __shfl_xor(v, 32, kWave);
  return v;
}

constexpr uint32_t kTailRunLog2 = 2;

template <bool VEC, bool WRITE_Y, bool MEAN, bool HAS_SCALE, bool HAS_BIAS, bool RES_FIRST>
__global__ __launch_bounds__(kBlock) void scale_residual_relu_rowmean_kernel(
    const float* x, const float* scale, const float* bias, const float* res, float* y,
    float* mean, uint32_t rows, uint32_t inner, FastDiv num) {
  const uint32_t lane = threadIdx.x & (kWave - 1);
  // Four workgroups in a row (16 rows, 64 bytes of means) on one XCD: measured
  // on [64,1024,14,14], 26.1 us with the workgroups dealt out one by one, 25.4 us
  // in runs of 4, 8 or 16, 25.9 us with each XCD on one contiguous eighth.
  const uint32_t group = xcd_runs(blockIdx.x, gridDim.x, kTailRunLog2);
  const uint32_t row = group * (kBlock / kWave) + threadIdx.x / kWave;
  if (row >= rows) return;  // wave-uniform
  const uint32_t c = row - fd_div(row, num) * num.d;
  const float s = HAS_SCALE ? scale[c] : 1.0f, b = HAS_BIAS ? bias[c] : 0.0f;
  const size_t base = static_cast<size_t>(row) * inner;
  double sum = 0.0;
  if (VEC) {
    const uint32_t nv = inner / 4;
    for (uint32_t i = lane; i < nv; i += kWave) {
      const v4f vx = load4_stream(x + base + 4ull * i);
      const v4f vr = load4_stream(res + base + 4ull * i);
      v4f o;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        o[j] = tail_element<HAS_SCALE, HAS_BIAS, RES_FIRST>(vx[j], s, b, vr[j]);
        if (MEAN) sum += static_cast<double>(o[j]);
      }
      if (WRITE_Y) store4_stream(y + base + 4ull * i, o);
    }
  } else {
    for (uint32_t i = lane; i < inner; i += kWave) {
      const float o = tail_element<HAS_SCALE, HAS_BIAS, RES_FIRST>(x[base + i], s, b, res[base + i]);
      if (MEAN) sum += static_cast<double>(o);
      if (WRITE_Y) y[base + i] = o;
    }
  }
  if (!MEAN) return;
  sum = wave_sum_f64(sum);
  if (lane == 0) mean[row] = static_cast<float>(sum / static_cast<double>(static_cast<int>(inner)));
}

}  // namespace shdw

using namespace shdw;

namespace {

template <bool HAS_SCALE, bool HAS_BIAS, bool RES_FIRST>
int launch_tail(uint32_t rows, uint32_t inner, FastDiv num, const float* x, const float* scale, const float* bias,
                const float* residual, float* y, float* mean, bool vec, hipStream_t st) {
  const uint32_t grid = (rows + kBlock / kWave - 1) / (kBlock / kWave);
#define SHDW_LAUNCH(V, W, M)                                                                              \
  scale_residual_relu_rowmean_kernel<V, W, M, HAS_SCALE, HAS_BIAS, RES_FIRST><<<grid, kBlock, 0, st>>>(   \
      x, scale, bias, residual, y, mean, rows, inner, num)
  if (vec) {
    if (y && mean) SHDW_LAUNCH(true, true, true);
    else if (y) SHDW_LAUNCH(true, true, false);
    else SHDW_LAUNCH(true, false, true);
  } else {
    if (y && mean) SHDW_LAUNCH(false, true, true);
    else if (y) SHDW_LAUNCH(false, true, false);
    else SHDW_LAUNCH(false, false, true);
  }
#undef SHDW_LAUNCH
  return launch_status();
}

}  // namespace

extern "C" int shdw_hip_scale_residual_relu(int n, int scale_num, int inner_num, const float* x,
                                            const float* scale, const float* bias,
                                            const float* residual, int residual_first, float* y,
                                            float* mean, void* stream) {
  if (n < 0 || scale_num < 1 || inner_num < 1 || !x || (!scale && !bias) || !residual || (!y && !mean))
    return SHDW_E_INVALID_ARGUMENT;
  if (n % inner_num != 0) return SHDW_E_INVALID_ARGUMENT;
  if (n == 0) return SHDW_OK;
  const uint32_t rows = static_cast<uint32_t>(n / inner_num);
  const uint32_t inner = static_cast<uint32_t>(inner_num);
  const FastDiv num = make_fastdiv(static_cast<uint32_t>(scale_num));
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool vec = inner % 4 == 0 && aligned16(x) && aligned16(residual) && (!y || aligned16(y));
#define SHDW_FORM(S, B)                                                                                       \
  (residual_first ? launch_tail<S, B, true>(rows, inner, num, x, scale, bias, residual, y, mean, vec, st)     \
                  : launch_tail<S, B, false>(rows, inner, num, x, scale, bias, residual, y, mean, vec, st))
  if (scale && bias) return SHDW_FORM(true, true);
  if (scale) return SHDW_FORM(true, false);
  return SHDW_FORM(false, true);
#undef SHDW_FORM
}

extern "C" int shdw_hip_scale_residual_relu_rowmean(int n, int scale_num, int inner_num,
                                                    const float* x, const float* scale,
                                                    const float* bias, const float* residual,
                                                    float* y, float* mean, void* stream) {
  if (!scale || !bias || !mean) return SHDW_E_INVALID_ARGUMENT;
  return shdw_hip_scale_residual_relu(n, scale_num, inner_num, x, scale, bias, residual, 0, y, mean, stream);
}
