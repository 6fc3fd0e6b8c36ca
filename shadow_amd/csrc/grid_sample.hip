// GridSample (shadow/operators/kernels/grid_sample.cpp:9-100, grid_sample.cu).
//
// grid holds an (x, y) pair in [-1, 1] per output position of a batch item, the same
// for every channel.  One lane owns one output position: it reads its pair (8 bytes,
// neighbouring lanes neighbouring pairs), works out the source cells and weights
// once, and walks the eight channels of its workgroup's share with them, so that every
// store of a wave is one run of 256 bytes; the reads go wherever the grid points.
//
// Every source index is clamped to the input plane before it is used, whatever the
// coordinate was, so no grid value can make the kernel read outside its input.
// Where the reference leaves a value to the machine (a float that fits no int) the
// result is what its x86-64 build gives: the conversion yields INT_MIN.  A NaN
// coordinate in the bilinear mode makes the reference index far outside its input;
// here the output is NaN.
#include <hip/hip_runtime.h>

#include <climits>

#include "../../include/shadow_hip.h"
#include "device_common.h"
#include "launch.h"

#pragma clang fp contract(off)

namespace shdw {

constexpr int kGridChannels = 8;  // channels per workgroup

typedef float v2f_unaligned __attribute__((ext_vector_type(2), aligned(4)));

SHDW_DEVICE int to_int_as_x86(float v) {
  return (v >= -2147483648.f && v < 2147483648.f) ? static_cast<int>(v) : INT_MIN;
}
SHDW_DEVICE int clamp_index(int v, int extent) { return v < 0 ? 0 : (v > extent - 1 ? extent - 1 : v); }
// std::min(std::max(v, 0.f), hi) as libstdc++ evaluates them: a NaN stays
SHDW_DEVICE float clamp_like_std(float v, float hi) {
  const float lower = (v < 0.f) ? 0.f : v;
  return (hi < lower) ? hi : lower;
}

// MODE 0: nearest, 1: bilinear.  PAD 0: zeros outside, 1: border.
template <int MODE, int PAD>
__global__ __launch_bounds__(kBlock) void grid_sample_kernel(const float* x, const float* grid, float* y,
                                                             uint32_t positions, uint32_t out_plane,
                                                             FastDiv f_out_plane, int channel, int in_h, int in_w,
                                                             FastDiv f_groups) {
  // Workgroups that sample neighbouring rows read the same input rows (the row below a
  // cell, and whatever the grid's warp adds): numbered so that each XCD owns a contiguous
  // range of (channel share, position group) pairs they find them in their own L2.
  // [64,256,56,56] with a grid warped by +-1.4 cells: 427 MB fetched for 207 with the
  // workgroups dealt out round-robin, 257 MB so.
  uint32_t share, group;
  fd_divmod(xcd_contiguous(blockIdx.x, gridDim.x), f_groups, share, group);
  const uint32_t p = group * kBlock + threadIdx.x;
  if (p >= positions) return;
  const uint32_t b = fd_div(p, f_out_plane);
  const uint32_t s = p - b * out_plane;
  const float gx = grid[2ull * p], gy = grid[2ull * p + 1];
  const int c0 = static_cast<int>(share) * kGridChannels;
  const int count = channel - c0 < kGridChannels ? channel - c0 : kGridChannels;
  const size_t in_plane = static_cast<size_t>(in_h) * in_w;
  const float* src = x + (static_cast<size_t>(b) * channel + c0) * in_plane;
  float* dst = y + (static_cast<size_t>(b) * channel + c0) * out_plane + s;
  const float src_h_f = (gy + 1) / 2.f * static_cast<float>(in_h - 1);
  const float src_w_f = (gx + 1) / 2.f * static_cast<float>(in_w - 1);
  if (MODE == 0) {
    int src_h = to_int_as_x86(__builtin_roundf(src_h_f));
    int src_w = to_int_as_x86(__builtin_roundf(src_w_f));
    const bool outside = PAD == 0 && (src_h < 0 || src_w < 0 || src_h > in_h - 1 || src_w > in_w - 1);
    const size_t cell = static_cast<size_t>(clamp_index(src_h, in_h)) * in_w + clamp_index(src_w, in_w);
    for (int c = 0; c < count; ++c) {
      const float v = src[c * in_plane + cell];
      dst[static_cast<size_t>(c) * out_plane] = outside ? 0.f : v;
    }
    return;
  }
  float fh = src_h_f, fw = src_w_f;
  bool outside = false;
  if (PAD == 1) {
    fh = clamp_like_std(fh, static_cast<float>(in_h) - 1.f);
    fw = clamp_like_std(fw, static_cast<float>(in_w) - 1.f);
  } else {
    outside = fh < 0 || fw < 0 || fh > static_cast<float>(in_h - 1) || fw > static_cast<float>(in_w - 1);
  }
  const bool nan = fh != fh || fw != fw;
  if (outside || nan) fh = fw = 0.f;  // nothing of the cells below is used then
  const int h0 = clamp_index(static_cast<int>(__builtin_floorf(fh)), in_h);
  const int h1 = clamp_index(static_cast<int>(__builtin_ceilf(fh)), in_h);
  const int w0 = clamp_index(static_cast<int>(__builtin_floorf(fw)), in_w);
  const int w1 = clamp_index(static_cast<int>(__builtin_ceilf(fw)), in_w);
  const float sh = fh - static_cast<float>(h0), sw = fw - static_cast<float>(w0);
  const float k0 = (1 - sh) * (1 - sw), k1 = sh * (1 - sw), k2 = (1 - sh) * sw, k3 = sh * sw;
  if (in_w >= 2) {
    // Both columns of a row in one 8-byte load: w0 and w1 are `left` and `left + 1` in some
    // order, or the same one of them (a coordinate on a cell, or clamped to the last column).
    const int left = w0 < in_w - 2 ? w0 : in_w - 2;
    const bool w0_first = w0 == left, w1_first = w1 == left;
    const size_t r0 = static_cast<size_t>(h0) * in_w + left, r1 = static_cast<size_t>(h1) * in_w + left;
    for (int c = 0; c < count; ++c) {
      const float* plane = src + c * in_plane;
      const v2f_unaligned top = *reinterpret_cast<const v2f_unaligned*>(plane + r0);
      const v2f_unaligned bottom = *reinterpret_cast<const v2f_unaligned*>(plane + r1);
      const float v0 = w0_first ? top[0] : top[1], v1 = w0_first ? bottom[0] : bottom[1];
      const float v2 = w1_first ? top[0] : top[1], v3 = w1_first ? bottom[0] : bottom[1];
      float v = k0 * v0 + k1 * v1 + k2 * v2 + k3 * v3;
      v = nan ? __builtin_nanf("") : v;
      dst[static_cast<size_t>(c) * out_plane] = outside ? 0.f : v;
    }
    return;
  }
  const size_t i0 = static_cast<size_t>(h0) * in_w + w0, i1 = static_cast<size_t>(h1) * in_w + w0;
  const size_t i2 = static_cast<size_t>(h0) * in_w + w1, i3 = static_cast<size_t>(h1) * in_w + w1;
  for (int c = 0; c < count; ++c) {
    const float* plane = src + c * in_plane;
    float v = k0 * plane[i0] + k1 * plane[i1] + k2 * plane[i2] + k3 * plane[i3];
    v = nan ? __builtin_nanf("") : v;
    dst[static_cast<size_t>(c) * out_plane] = outside ? 0.f : v;
  }
}

}  // namespace shdw

using namespace shdw;

extern "C" int shdw_hip_grid_sample(const int* in_shape, const int* out_shape, int mode, int padding_mode,
                                    const float* x, const float* grid, float* y, void* stream) {
  if (!in_shape || !out_shape || mode < 0 || mode > 1 || padding_mode < 0 || padding_mode > 1)
    return SHDW_E_INVALID_ARGUMENT;
  long long in_count = 1, out_count = 1;
  for (int d = 0; d < 4; ++d) {
    if (in_shape[d] < 0 || out_shape[d] < 0) return SHDW_E_INVALID_ARGUMENT;
    in_count *= in_shape[d];
    out_count *= out_shape[d];
    if (in_count > INT_MAX || out_count > INT_MAX) return SHDW_E_UNSUPPORTED;
  }
  if (in_shape[0] != out_shape[0] || in_shape[1] != out_shape[1]) return SHDW_E_INVALID_ARGUMENT;
  if (out_count == 0) return SHDW_OK;
  if (in_count == 0) return SHDW_E_INVALID_ARGUMENT;  // positions to fill and nothing to sample
  if (!x || !grid || !y || x == y) return SHDW_E_INVALID_ARGUMENT;
  const long long grid_count = 2ll * out_shape[0] * out_shape[2] * out_shape[3];
  if (grid_count > INT_MAX) return SHDW_E_UNSUPPORTED;
  const int channel = in_shape[1];
  const uint32_t out_plane = static_cast<uint32_t>(out_shape[2]) * static_cast<uint32_t>(out_shape[3]);
  const uint32_t positions = static_cast<uint32_t>(out_shape[0]) * out_plane;
  const uint32_t groups = grid_for(positions);
  const long long launch = static_cast<long long>(groups) * ((channel + kGridChannels - 1) / kGridChannels);
  if (launch > INT_MAX) return SHDW_E_UNSUPPORTED;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const FastDiv f = make_fastdiv(out_plane), fg = make_fastdiv(groups);
#define SHDW_GRID(M, P)                                                                                          \
  grid_sample_kernel<M, P><<<static_cast<uint32_t>(launch), kBlock, 0, st>>>(x, grid, y, positions, out_plane, f, \
                                                                             channel, in_shape[2], in_shape[3], fg)
  if (mode == 0) {
    if (padding_mode == 0) SHDW_GRID(0, 0); else SHDW_GRID(0, 1);
  } else {
    if (padding_mode == 0) SHDW_GRID(1, 0); else SHDW_GRID(1, 1);
  }
#undef SHDW_GRID
  return launch_status();
}
