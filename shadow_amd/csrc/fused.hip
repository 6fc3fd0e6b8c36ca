// The ResNet bottleneck tail in one launch: per-channel Scale, residual add
// (Eltwise SUM), ReLU and the global average over the trailing `inner`
// elements.  x and the residual are read once, y is written once and the
// pooled value falls out of the same registers; run as four operators the
// same data crosses HBM 8 times instead of 3.
//
// One wave64 owns one (n, c) row.  Arithmetic per element is exactly the
// operator sequence: t = x*s; t = t + b; u = 0 + 1*t; u = u + 1*r;
// y = u > 0 ? u : 0; the row sum is fp64 and rounded once after the divide.
// With a BatchNorm in front of the Scale (how a Caffe-style model holds the
// normalisation) x is (x - m) / d first, m and d the channel's as
// Vision::BatchNorm forms them.
#include <hip/hip_runtime.h>

#include "../../include/shadow_hip.h"
#include "device_common.h"
#include "launch.h"

#pragma clang fp contract(off)

namespace shdw {

// The operator sequence on one element.  HAS_SCALE / HAS_BIAS: which parameter
// blobs the Scale operator has (Vision::ScaleBias, Scale or Bias); RES_FIRST: the
// residual is the Eltwise operator's first input and the scaled value its second.
template <bool NORM, bool HAS_SCALE, bool HAS_BIAS, bool RES_FIRST>
SHDW_DEVICE float tail_element(float x, float m, float d, float s, float b, float r) {
  float t = x;
  if (NORM) t = (t - m) / d;
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

// The BatchNorm in front of the Scale: stored statistics, one pair per channel,
// and the factor and eps of shadow/operators/kernels/batch_norm.cu:9-34.
struct TailNorm {
  const float* mean;
  const float* variance;
  float scale_factor, eps;
};

template <bool VEC, bool WRITE_Y, bool MEAN, bool NORM, bool HAS_SCALE, bool HAS_BIAS, bool RES_FIRST>
__global__ __launch_bounds__(kBlock) void scale_residual_relu_rowmean_kernel(
    const float* x, TailNorm norm, const float* scale, const float* bias, const float* res, float* y,
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
  float m = 0.0f, d = 1.0f;
  if (NORM) {
    m = norm.mean[c] * norm.scale_factor;
    d = __builtin_sqrtf(__builtin_fabsf(norm.variance[c] * norm.scale_factor) + norm.eps);
  }
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
        o[j] = tail_element<NORM, HAS_SCALE, HAS_BIAS, RES_FIRST>(vx[j], m, d, s, b, vr[j]);
        if (MEAN) sum += static_cast<double>(o[j]);
      }
      if (WRITE_Y) store4_stream(y + base + 4ull * i, o);
    }
  } else {
    for (uint32_t i = lane; i < inner; i += kWave) {
      const float o = tail_element<NORM, HAS_SCALE, HAS_BIAS, RES_FIRST>(x[base + i], m, d, s, b, res[base + i]);
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

template <bool NORM, bool HAS_SCALE, bool HAS_BIAS, bool RES_FIRST>
int launch_tail(uint32_t rows, uint32_t inner, FastDiv num, const float* x, const TailNorm& norm, const float* scale,
                const float* bias, const float* residual, float* y, float* mean, bool vec, hipStream_t st) {
  const uint32_t grid = (rows + kBlock / kWave - 1) / (kBlock / kWave);
#define SHDW_LAUNCH(V, W, M)                                                                                  \
  scale_residual_relu_rowmean_kernel<V, W, M, NORM, HAS_SCALE, HAS_BIAS, RES_FIRST><<<grid, kBlock, 0, st>>>( \
      x, norm, scale, bias, residual, y, mean, rows, inner, num)
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

// norm == nullptr: no BatchNorm in front.  scale_num is then the Scale operator's
// parameter count; with a BatchNorm it is the channel count, which both operators share.
int run_tail(int n, int scale_num, int inner_num, const float* x, const TailNorm* norm, const float* scale,
             const float* bias, const float* residual, int residual_first, float* y, float* mean, void* stream) {
  if (n < 0 || scale_num < 1 || inner_num < 1 || !x || (!scale && !bias) || !residual || (!y && !mean))
    return SHDW_E_INVALID_ARGUMENT;
  if (norm && (!norm->mean || !norm->variance)) return SHDW_E_INVALID_ARGUMENT;
  if (n % inner_num != 0) return SHDW_E_INVALID_ARGUMENT;
  if (n == 0) return SHDW_OK;
  const uint32_t rows = static_cast<uint32_t>(n / inner_num);
  const uint32_t inner = static_cast<uint32_t>(inner_num);
  const FastDiv num = make_fastdiv(static_cast<uint32_t>(scale_num));
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool vec = inner % 4 == 0 && aligned16(x) && aligned16(residual) && (!y || aligned16(y));
  const TailNorm none{nullptr, nullptr, 1.0f, 0.0f};
#define SHDW_SIDE(N, S, B)                                                                                          \
  (residual_first ? launch_tail<N, S, B, true>(rows, inner, num, x, norm ? *norm : none, scale, bias, residual, y,  \
                                               mean, vec, st)                                                       \
                  : launch_tail<N, S, B, false>(rows, inner, num, x, norm ? *norm : none, scale, bias, residual, y, \
                                                mean, vec, st))
#define SHDW_FORM(S, B) (norm ? SHDW_SIDE(true, S, B) : SHDW_SIDE(false, S, B))
  if (scale && bias) return SHDW_FORM(true, true);
  if (scale) return SHDW_FORM(true, false);
  return SHDW_FORM(false, true);
#undef SHDW_FORM
#undef SHDW_SIDE
}

}  // namespace

extern "C" int shdw_hip_scale_residual_relu(int n, int scale_num, int inner_num, const float* x,
                                            const float* scale, const float* bias,
                                            const float* residual, int residual_first, float* y,
                                            float* mean, void* stream) {
  return run_tail(n, scale_num, inner_num, x, nullptr, scale, bias, residual, residual_first, y, mean, stream);
}

extern "C" int shdw_hip_batch_norm_scale_residual_relu(int n, int channel, int inner_num, const float* x,
                                                       const float* stat_mean, const float* stat_variance,
                                                       float scale_factor, float eps, const float* scale,
                                                       const float* bias, const float* residual,
                                                       int residual_first, float* y, float* mean, void* stream) {
  const TailNorm norm{stat_mean, stat_variance, scale_factor, eps};
  return run_tail(n, channel, inner_num, x, &norm, scale, bias, residual, residual_first, y, mean, stream);
}

extern "C" int shdw_hip_scale_residual_relu_rowmean(int n, int scale_num, int inner_num,
                                                    const float* x, const float* scale,
                                                    const float* bias, const float* residual,
                                                    float* y, float* mean, void* stream) {
  if (!scale || !bias || !mean) return SHDW_E_INVALID_ARGUMENT;
  return shdw_hip_scale_residual_relu(n, scale_num, inner_num, x, scale, bias, residual, 0, y, mean, stream);
}
