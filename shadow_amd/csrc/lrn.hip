// LRN across channels (shadow/operators/kernels/lrn.cpp:9-60, lrn.cu).
//
// The reference walks the channels of one (batch, h, w) position with a running
// fp32 sum of squares -- the entering square is added, then the one that leaves
// the window is subtracted -- writes scale = k + sum * (alpha / size) into a
// scratch blob, and multiplies x by powf(scale, -beta) in a second pass.  The
// order of the additions and subtractions fixes the bits, so the walk stays: one
// lane per position, channel after channel.  What goes is the scratch blob and
// the second pass: the window's values wait in LDS (a column of `size` floats per
// lane, no two lanes share a bank row), the centre of the window is multiplied as
// soon as its scale is known, x is read once and y written once.  Neighbouring
// lanes hold neighbouring positions, so every load and store of a wave is one run
// of 256 bytes.  y may be x: a lane has read every channel it still needs before
// it writes the one behind them.
#include <hip/hip_runtime.h>

#include <climits>

#include "../../include/shadow_hip.h"
#include "device_common.h"
#include "launch.h"
#include "libm_exact.h"

#pragma clang fp contract(off)

namespace shdw {

// Windows of up to 63 channels: 63 KB of LDS for the 256 lanes of a workgroup.
constexpr int kLrnMaxSize = 63;

__global__ __launch_bounds__(kBlock) void lrn_across_channels_kernel(
    const float* x, float* y, uint32_t positions, uint32_t step, uint32_t channels, FastDiv f_step,
    uint32_t size, float alpha_over_size, float neg_beta, float k) {
  extern __shared__ float window[];  // [size][kBlock]
  const uint32_t p = blockIdx.x * kBlock + threadIdx.x;
  if (p >= positions) return;  // no barrier below: a lane only meets its own column
  const uint32_t b = fd_div(p, f_step);
  const size_t base = static_cast<size_t>(b) * channels * step + (p - b * step);
  const float* in = x + base;
  float* out = y + base;
  float* mine = window + threadIdx.x;
  const uint32_t post = (size - 1) / 2;
  float accum = 0.f;
  uint32_t slot_head = 0, slot_mid = 0;  // head % size and (head - post) % size
  float entering = in[0];
  for (uint32_t head = 0; head < channels + post; ++head) {
    const float v = entering;
    if (head + 1 < channels) entering = in[static_cast<size_t>(head + 1) * step];  // on its way during the powf
    if (head < channels) accum += v * v;
    if (head >= size) {  // channel head - size lives where channel head goes
      const float leaving = mine[slot_head * kBlock];
      accum -= leaving * leaving;
    }
    if (head < channels) mine[slot_head * kBlock] = v;
    slot_head = slot_head + 1 == size ? 0 : slot_head + 1;
    if (head >= post) {
      const float scale = k + accum * alpha_over_size;
      const float centre = mine[slot_mid * kBlock];
      out[static_cast<size_t>(head - post) * step] = centre * libm::exact_powf(scale, neg_beta, libm::kExp2fTab);
      slot_mid = slot_mid + 1 == size ? 0 : slot_mid + 1;
    }
  }
}

}  // namespace shdw

using namespace shdw;

extern "C" int shdw_hip_lrn(const int* in_shape, int size, float alpha, float beta, float k, const float* x,
                            float* y, void* stream) {
  if (!in_shape || size < 1 || size % 2 == 0) return SHDW_E_INVALID_ARGUMENT;
  long long count = 1;
  for (int d = 0; d < 4; ++d) {
    if (in_shape[d] < 0) return SHDW_E_INVALID_ARGUMENT;
    count *= in_shape[d];
    if (count > INT_MAX) return SHDW_E_UNSUPPORTED;
  }
  const int channels = in_shape[1], post = (size - 1) / 2;
  // fewer channels than lie behind the centre of a window: the reference's last
  // loop then writes in front of its scale blob
  if (channels < post) return SHDW_E_INVALID_ARGUMENT;
  if (count == 0) return SHDW_OK;
  if (!x || !y) return SHDW_E_INVALID_ARGUMENT;
  if (size > kLrnMaxSize) return SHDW_E_UNSUPPORTED;
  const uint32_t step = static_cast<uint32_t>(in_shape[2]) * static_cast<uint32_t>(in_shape[3]);
  const uint32_t positions = static_cast<uint32_t>(in_shape[0]) * step;
  const float alpha_over_size = alpha / size;  // float / int, as the reference forms it
  const size_t lds = static_cast<size_t>(size) * kBlock * sizeof(float);
  lrn_across_channels_kernel<<<grid_for(positions), kBlock, lds, static_cast<hipStream_t>(stream)>>>(
      x, y, positions, step, static_cast<uint32_t>(channels), make_fastdiv(step), static_cast<uint32_t>(size),
      alpha_over_size, -beta, k);
  return launch_status();
}
