// Operators that sit next to the elementwise path in a converted CNN:
//   * Axpy       out = y + alpha[row] * x          (SE-net channel gate)
//   * BatchNorm  out = (x - m[c]) / sqrt(|v[c]| + eps) with global statistics
//   * Pooling    2-D / 3-D max and average windows
// Axpy and BatchNorm stream one 128-bit vector per lane like the Scale kernels.
// Pooling gives every output element to one lane, which walks its window in the
// reference's order: the fp32 running sum of an average window is
// order-dependent and this keeps it bit-identical.  Windows that cover a whole
// plane (global pooling) go through LDS so that global loads stay coalesced.
#include <hip/hip_runtime.h>

#include <cfloat>

#include "../../include/shadow_hip.h"
#include "device_common.h"
#include "launch.h"

#pragma clang fp contract(off)

namespace shdw {

// ---------------------------------------------------------------------------
// Axpy rows and BatchNorm: per-row parameters, two flavours of one kernel.
// ---------------------------------------------------------------------------
struct AxpyRows {
  const float* alpha;
  const float* y;
  SHDW_DEVICE v4f load_other(uint64_t off) const { return load4_stream(y + off); }
  SHDW_DEVICE float other(uint64_t off) const { return y[off]; }
  struct Row {
    float a;
  };
  SHDW_DEVICE Row row(uint32_t r) const { return {alpha[r]}; }
  SHDW_DEVICE float apply(float x, float yv, const Row& p) const {
    const float t = p.a * x;
    return yv + t;
  }
  static constexpr bool kTwoInputs = true;
};

struct BatchNormRows {
  const float* mean;
  const float* variance;
  float scale_factor, eps;
  FastDiv channel;
  SHDW_DEVICE v4f load_other(uint64_t) const { return v4f{0, 0, 0, 0}; }
  SHDW_DEVICE float other(uint64_t) const { return 0.f; }
  struct Row {
    float m, d;
  };
  SHDW_DEVICE Row row(uint32_t r) const {
    const uint32_t c = r - fd_div(r, channel) * channel.d;
    const float m = mean[c] * scale_factor;
    const float v = __builtin_fabsf(variance[c] * scale_factor) + eps;
    return {m, __builtin_sqrtf(v)};
  }
  SHDW_DEVICE float apply(float x, float, const Row& p) const { return (x - p.m) / p.d; }
  static constexpr bool kTwoInputs = false;
};

// ROWVEC: inner % 4 == 0, the four elements of a vector share a row.
template <class P, bool ROWVEC>
__global__ __launch_bounds__(kBlock) void rows_vec_kernel(P p, const float* x, float* out,
                                                           uint32_t n4, uint32_t n, FastDiv inner) {
  const uint32_t i = blockIdx.x * kBlock + threadIdx.x;
  if (i < n4) {
    const v4f vx = load4_stream(x + 4ull * i);
    const v4f vo = p.load_other(4ull * i);
    v4f r;
    if (ROWVEC) {
      const typename P::Row rp = p.row(fd_div(4 * i, inner));
#pragma unroll
      for (int j = 0; j < 4; ++j) r[j] = p.apply(vx[j], vo[j], rp);
    } else {
      // Most vectors still lie inside one row: fetch its parameters once and
      // only the lanes whose vector straddles a boundary look up a second row.
      const uint32_t r0 = fd_div(4 * i, inner);
      const typename P::Row rp0 = p.row(r0);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint32_t rj = fd_div(4 * i + j, inner);
        r[j] = p.apply(vx[j], vo[j], rj == r0 ? rp0 : p.row(rj));
      }
    }
    store4_stream(out + 4ull * i, r);
  } else if (i == n4) {
    for (uint32_t t = 4 * n4; t < n; ++t) out[t] = p.apply(x[t], p.other(t), p.row(fd_div(t, inner)));
  }
}

template <class P>
__global__ __launch_bounds__(kBlock) void rows_scalar_kernel(P p, const float* x, float* out,
                                                              uint32_t n, FastDiv inner) {
  const uint32_t i = blockIdx.x * kBlock + threadIdx.x;
  if (i < n) out[i] = p.apply(x[i], p.other(i), p.row(fd_div(i, inner)));
}

template <class P>
static int launch_rows(const P& p, uint32_t n, uint32_t inner, const float* x, const float* other,
                       float* out, hipStream_t st) {
  const FastDiv fi = make_fastdiv(inner);
  if (aligned16(x) && aligned16(out) && (!P::kTwoInputs || aligned16(other))) {
    const uint32_t n4 = n / 4;
    const uint32_t grid = grid_for(n4 + 1);
    if (inner % 4 == 0)
      rows_vec_kernel<P, true><<<grid, kBlock, 0, st>>>(p, x, out, n4, n, fi);
    else
      rows_vec_kernel<P, false><<<grid, kBlock, 0, st>>>(p, x, out, n4, n, fi);
  } else {
    rows_scalar_kernel<P><<<grid_for(n), kBlock, 0, st>>>(p, x, out, n, fi);
  }
  return launch_status();
}

// ---------------------------------------------------------------------------
// Pooling.
// ---------------------------------------------------------------------------
struct PoolArgs {
  int in_d, in_h, in_w;
  int out_d, out_h, out_w;
  int kd, kh, kw;
  int sd, sh, sw;
  int pd, ph, pw;
  FastDiv f_out_w, f_out_h, f_out_d;
};

// std::max(max_val, value) of libstdc++: keeps max_val unless max_val < value.
SHDW_DEVICE float pool_max(float max_val, float value) { return max_val < value ? value : max_val; }

template <bool MAX, bool THREE_D>
__global__ __launch_bounds__(kBlock) void pool_window_kernel(const float* x, float* y, uint32_t n_out,
                                                              PoolArgs p) {
  const uint32_t i = blockIdx.x * kBlock + threadIdx.x;
  if (i >= n_out) return;
  uint32_t rest, w, h, d = 0;
  fd_divmod(i, p.f_out_w, rest, w);
  fd_divmod(rest, p.f_out_h, rest, h);
  if (THREE_D) fd_divmod(rest, p.f_out_d, rest, d);
  const float* plane =
      x + static_cast<uint64_t>(rest) * (static_cast<uint64_t>(p.in_d) * p.in_h * p.in_w);
  int dstart = THREE_D ? static_cast<int>(d) * p.sd - p.pd : 0;
  int hstart = static_cast<int>(h) * p.sh - p.ph;
  int wstart = static_cast<int>(w) * p.sw - p.pw;
  int dend = THREE_D ? min(dstart + p.kd, p.in_d + p.pd) : 1;
  int hend = min(hstart + p.kh, p.in_h + p.ph);
  int wend = min(wstart + p.kw, p.in_w + p.pw);
  const int pool_size = (dend - dstart) * (hend - hstart) * (wend - wstart);
  dstart = max(dstart, 0), hstart = max(hstart, 0), wstart = max(wstart, 0);
  dend = min(dend, p.in_d), hend = min(hend, p.in_h), wend = min(wend, p.in_w);
  float max_val = -FLT_MAX, sum_val = 0.f;
  for (int pd = dstart; pd < dend; ++pd) {
    for (int ph = hstart; ph < hend; ++ph) {
      const float* row = plane + (static_cast<int64_t>(pd) * p.in_h + ph) * p.in_w;
      for (int pw = wstart; pw < wend; ++pw) {
        const float v = row[pw];
        if (MAX)
          max_val = pool_max(max_val, v);
        else
          sum_val += v;
      }
    }
  }
  y[i] = MAX ? max_val : sum_val / static_cast<float>(pool_size);
}

// 2-D windows through LDS.  A workgroup owns `band` consecutive output rows of
// one plane.  The input rows they touch are one contiguous span of the plane,
// copied with 128-bit loads; every input element is then fetched from HBM/L2
// once per band instead of once per overlapping window, and the window walks
// read LDS.  Order inside a window is unchanged.
constexpr int kBandTileFloats = 8192;  // upper bound of the dynamic LDS tile (32 KB)
constexpr int kBandBatch = 4;
constexpr int kPoolBandOutputs = 512;  // outputs a workgroup aims for (measured best of 256..4096)

struct BandArgs {
  int in_h, in_w, out_h, out_w;
  int kh, kw, sh, sw, ph, pw;
  int band, bands_per_plane;
  FastDiv f_out_w, f_bands;
};

// K > 0: square K x K window, walked fully unrolled with the out-of-range
// cells predicated off (same cells, same order as the clipped loops) so that
// all LDS reads of a window are in flight together.  K = 0: any window.
template <bool MAX, int K>
__global__ __launch_bounds__(kBlock) void pool_band_kernel(const float* x, float* y, BandArgs p) {
  extern __shared__ __align__(16) float tile[];  // rows of one band, at most kBandTileFloats
  uint32_t plane, b;
  fd_divmod(blockIdx.x, p.f_bands, plane, b);
  const int h0 = static_cast<int>(b) * p.band;
  const int nh = min(p.band, p.out_h - h0);
  const int r_lo = max(h0 * p.sh - p.ph, 0);
  const int r_hi = min((h0 + nh - 1) * p.sh - p.ph + p.kh, p.in_h);
  const uint32_t span = r_hi > r_lo ? static_cast<uint32_t>(r_hi - r_lo) * p.in_w : 0u;
  const float* src = x + static_cast<uint64_t>(plane) * p.in_h * p.in_w + static_cast<uint64_t>(r_lo) * p.in_w;
  if (aligned16_device(src)) {
    const uint32_t nvec = span / 4;
    for (uint32_t v0 = 0; v0 < nvec; v0 += kBandBatch * kBlock) {
      v4f reg[kBandBatch];
#pragma unroll
      for (int k = 0; k < kBandBatch; ++k) {
        const uint32_t v = v0 + k * kBlock + threadIdx.x;
        if (v < nvec) reg[k] = load4_stream(src + 4ull * v);
      }
#pragma unroll
      for (int k = 0; k < kBandBatch; ++k) {
        const uint32_t v = v0 + k * kBlock + threadIdx.x;
        if (v < nvec) *reinterpret_cast<v4f*>(tile + 4 * v) = reg[k];
      }
    }
    for (uint32_t t = 4 * nvec + threadIdx.x; t < span; t += kBlock) tile[t] = src[t];
  } else {
    for (uint32_t t0 = 0; t0 < span; t0 += kBandBatch * kBlock) {
      float reg[kBandBatch];
#pragma unroll
      for (int k = 0; k < kBandBatch; ++k) {
        const uint32_t t = t0 + k * kBlock + threadIdx.x;
        if (t < span) reg[k] = __builtin_nontemporal_load(src + t);
      }
#pragma unroll
      for (int k = 0; k < kBandBatch; ++k) {
        const uint32_t t = t0 + k * kBlock + threadIdx.x;
        if (t < span) tile[t] = reg[k];
      }
    }
  }
  __syncthreads();
  float* dst = y + (static_cast<uint64_t>(plane) * p.out_h + h0) * p.out_w;
  const uint32_t outs = static_cast<uint32_t>(nh) * p.out_w;
  for (uint32_t o = threadIdx.x; o < outs; o += kBlock) {
    uint32_t hl, w;
    fd_divmod(o, p.f_out_w, hl, w);
    int hstart = (h0 + static_cast<int>(hl)) * p.sh - p.ph;
    int wstart = static_cast<int>(w) * p.sw - p.pw;
    int hend = min(hstart + p.kh, p.in_h + p.ph);
    int wend = min(wstart + p.kw, p.in_w + p.pw);
    const int pool_size = (hend - hstart) * (wend - wstart);
    hstart = max(hstart, 0), wstart = max(wstart, 0);
    hend = min(hend, p.in_h), wend = min(wend, p.in_w);
    float max_val = -FLT_MAX, sum_val = 0.f;
    if (K > 0) {
      const int h_first = (h0 + static_cast<int>(hl)) * p.sh - p.ph;
      const int w_first = static_cast<int>(w) * p.sw - p.pw;
      float cell[K > 0 ? K * K : 1];
#pragma unroll
      for (int i = 0; i < K; ++i) {
#pragma unroll
        for (int j = 0; j < K; ++j) {
          const int ph = h_first + i, pw = w_first + j;
          const bool inside = ph >= hstart && ph < hend && pw >= wstart && pw < wend;
          cell[i * K + j] = inside ? tile[(ph - r_lo) * p.in_w + pw] : 0.f;
        }
      }
#pragma unroll
      for (int i = 0; i < K; ++i) {
#pragma unroll
        for (int j = 0; j < K; ++j) {
          const int ph = h_first + i, pw = w_first + j;
          const bool inside = ph >= hstart && ph < hend && pw >= wstart && pw < wend;
          if (inside) {
            if (MAX)
              max_val = pool_max(max_val, cell[i * K + j]);
            else
              sum_val += cell[i * K + j];
          }
        }
      }
    } else {
      for (int ph = hstart; ph < hend; ++ph) {
        const float* row = tile + (ph - r_lo) * p.in_w;
        for (int pw = wstart; pw < wend; ++pw) {
          const float v = row[pw];
          if (MAX)
            max_val = pool_max(max_val, v);
          else
            sum_val += v;
        }
      }
    }
    dst[o] = MAX ? max_val : sum_val / static_cast<float>(pool_size);
  }
}

// Output rows per workgroup, or 0 when a single output row's input rows do not
// fit the tile (the direct kernel handles that).
static int plan_pool_band(const PoolArgs& p, int target_outputs) {
  const int rows_cap = kBandTileFloats / p.in_w;
  if (rows_cap < p.kh) return 0;
  const int band_cap = (rows_cap - p.kh) / p.sh + 1;
  int band = (target_outputs + p.out_w - 1) / p.out_w;
  band = band < 1 ? 1 : band;
  band = band > band_cap ? band_cap : band;
  return band > p.out_h ? p.out_h : band;
}

// Whole-plane windows: x is [rows][len], one output per row.  A workgroup owns
// ROWS consecutive rows; they pass through LDS in chunks of `chunk` columns
// (coalesced loads by all lanes), then lane r folds row r element by element.
// The row pitch in LDS is odd, so the per-lane walks hit distinct banks.
constexpr int kPlaneTileFloats = 12608;  // 256 rows x 49 or 64 rows x 197

inline int plane_pitch_cap(int rows_per_group) { return kPlaneTileFloats / rows_per_group; }

constexpr int kPlaneBatch = 8;  // global loads a lane keeps in flight while staging

template <bool MAX, int ROWS>
__global__ __launch_bounds__(kBlock) void pool_plane_kernel(const float* x, float* y, uint32_t rows,
                                                             uint32_t len, uint32_t chunk,
                                                             FastDiv f_chunk, FastDiv f_last,
                                                             float pool_size) {
  __shared__ float tile[kPlaneTileFloats];
  const uint32_t row0 = blockIdx.x * ROWS;
  const uint32_t nrows = min(static_cast<uint32_t>(ROWS), rows - row0);
  const uint32_t pitch = chunk | 1u;
  const float* base = x + static_cast<uint64_t>(row0) * len;
  float max_val = -FLT_MAX, sum_val = 0.f;
  for (uint32_t c0 = 0; c0 < len; c0 += chunk) {
    const bool last = c0 + chunk > len;
    const uint32_t cols = last ? len - c0 : chunk;
    const FastDiv fc = last ? f_last : f_chunk;
    const uint32_t cells = nrows * cols;
    if (cols == len && aligned16_device(base)) {
      // The rows are one contiguous span: 128-bit loads, a batch in flight per
      // lane, then scattered into the padded LDS rows.
      const uint32_t nvec = cells / 4;
      for (uint32_t v0 = 0; v0 < nvec; v0 += kPlaneBatch * kBlock) {
        v4f reg[kPlaneBatch];
#pragma unroll
        for (int k = 0; k < kPlaneBatch; ++k) {
          const uint32_t v = v0 + k * kBlock + threadIdx.x;
          if (v < nvec) reg[k] = load4_stream(base + 4ull * v);
        }
#pragma unroll
        for (int k = 0; k < kPlaneBatch; ++k) {
          const uint32_t v = v0 + k * kBlock + threadIdx.x;
          if (v < nvec) {
            uint32_t r, c;
            fd_divmod(4 * v, fc, r, c);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              tile[r * pitch + c] = reg[k][j];
              if (++c == cols) c = 0, ++r;
            }
          }
        }
      }
      for (uint32_t t = 4 * nvec + threadIdx.x; t < cells; t += kBlock) {
        uint32_t r, c;
        fd_divmod(t, fc, r, c);
        tile[r * pitch + c] = base[t];
      }
    } else {
      for (uint32_t t0 = 0; t0 < cells; t0 += kPlaneBatch * kBlock) {
        float reg[kPlaneBatch];
        uint32_t slot[kPlaneBatch];
#pragma unroll
        for (int k = 0; k < kPlaneBatch; ++k) {
          const uint32_t t = t0 + k * kBlock + threadIdx.x;
          if (t < cells) {
            uint32_t r, c;
            fd_divmod(t, fc, r, c);
            slot[k] = r * pitch + c;
            reg[k] = __builtin_nontemporal_load(base + static_cast<uint64_t>(r) * len + c0 + c);
          }
        }
#pragma unroll
        for (int k = 0; k < kPlaneBatch; ++k) {
          const uint32_t t = t0 + k * kBlock + threadIdx.x;
          if (t < cells) tile[slot[k]] = reg[k];
        }
      }
    }
    __syncthreads();
    if (threadIdx.x < nrows) {
      const float* mine = tile + threadIdx.x * pitch;
      for (uint32_t c = 0; c < cols; ++c) {
        const float v = mine[c];
        if (MAX)
          max_val = pool_max(max_val, v);
        else
          sum_val += v;
      }
    }
    __syncthreads();
  }
  if (threadIdx.x < nrows) y[row0 + threadIdx.x] = MAX ? max_val : sum_val / pool_size;
}

template <bool MAX>
static void launch_pool_plane(const float* x, float* y, uint32_t rows, uint32_t len,
                              hipStream_t st) {
  // 256 rows per workgroup only when that still leaves a few workgroups per CU.
  const int group = rows >= 256u * 1024u ? 256 : 64;
  const uint32_t cap = static_cast<uint32_t>(plane_pitch_cap(group));  // odd
  const uint32_t chunk = (len | 1u) <= cap ? len : cap - 1;
  const uint32_t tail = len % chunk;
  const FastDiv fc = make_fastdiv(chunk), fl = make_fastdiv(tail ? tail : chunk);
  const float size = static_cast<float>(static_cast<int>(len));
  const uint32_t grid = (rows + group - 1) / group;
  if (group == 256)
    pool_plane_kernel<MAX, 256><<<grid, kBlock, 0, st>>>(x, y, rows, len, chunk, fc, fl, size);
  else
    pool_plane_kernel<MAX, 64><<<grid, kBlock, 0, st>>>(x, y, rows, len, chunk, fc, fl, size);
}

static int check_pool_dims(int n, const int* in_shape, const int* out_shape) {
  int64_t in_count = 1, out_count = 1;
  for (int k = 0; k < n; ++k) {
    if (in_shape[k] < 0 || out_shape[k] < 0) return SHDW_E_INVALID_ARGUMENT;
    in_count *= in_shape[k];
    out_count *= out_shape[k];
    if (in_count > INT32_MAX || out_count > INT32_MAX) return SHDW_E_INVALID_ARGUMENT;
  }
  if (in_shape[0] != out_shape[0] || in_shape[1] != out_shape[1]) return SHDW_E_INVALID_ARGUMENT;
  return SHDW_OK;
}

static int run_pooling(bool three_d, const int* in_shape, int pool_type, const int* kernel,
                       const int* stride, const int* pad, const int* out_shape, const float* x,
                       float* y, hipStream_t st) {
  const int nsp = three_d ? 3 : 2;
  if (!in_shape || !out_shape || pool_type < 0 || pool_type > 1) return SHDW_E_INVALID_ARGUMENT;
  const int rc = check_pool_dims(nsp + 2, in_shape, out_shape);
  if (rc != SHDW_OK) return rc;
  for (int k = 0; k < nsp; ++k)
    if (kernel[k] < 1 || stride[k] < 1 || pad[k] < 0) return SHDW_E_INVALID_ARGUMENT;
  int64_t out_count = 1, in_count = 1;
  for (int k = 0; k < nsp + 2; ++k) out_count *= out_shape[k], in_count *= in_shape[k];
  if (out_count == 0) return SHDW_OK;
  if (!x || !y || in_count == 0) return SHDW_E_INVALID_ARGUMENT;

  // One window that is exactly the unpadded plane: rows of contiguous elements.
  bool whole_plane = true;
  int64_t plane = 1;
  for (int k = 0; k < nsp; ++k) {
    whole_plane = whole_plane && out_shape[k + 2] == 1 && pad[k] == 0 && kernel[k] == in_shape[k + 2];
    plane *= in_shape[k + 2];
  }
  if (whole_plane && plane >= 8) {
    const uint32_t rows = static_cast<uint32_t>(out_count);
    if (pool_type == 0)
      launch_pool_plane<true>(x, y, rows, static_cast<uint32_t>(plane), st);
    else
      launch_pool_plane<false>(x, y, rows, static_cast<uint32_t>(plane), st);
    return launch_status();
  }

  PoolArgs p;
  const int o = three_d ? 1 : 0;
  p.in_d = three_d ? in_shape[2] : 1, p.in_h = in_shape[2 + o], p.in_w = in_shape[3 + o];
  p.out_d = three_d ? out_shape[2] : 1, p.out_h = out_shape[2 + o], p.out_w = out_shape[3 + o];
  p.kd = three_d ? kernel[0] : 1, p.kh = kernel[o], p.kw = kernel[o + 1];
  p.sd = three_d ? stride[0] : 1, p.sh = stride[o], p.sw = stride[o + 1];
  p.pd = three_d ? pad[0] : 0, p.ph = pad[o], p.pw = pad[o + 1];
  p.f_out_w = make_fastdiv(static_cast<uint32_t>(p.out_w));
  p.f_out_h = make_fastdiv(static_cast<uint32_t>(p.out_h));
  p.f_out_d = make_fastdiv(static_cast<uint32_t>(p.out_d));
  const uint32_t n_out = static_cast<uint32_t>(out_count);
  const int band = three_d ? 0 : plan_pool_band(p, kPoolBandOutputs);
  if (band > 0) {
    BandArgs a;
    a.in_h = p.in_h, a.in_w = p.in_w, a.out_h = p.out_h, a.out_w = p.out_w;
    a.kh = p.kh, a.kw = p.kw, a.sh = p.sh, a.sw = p.sw, a.ph = p.ph, a.pw = p.pw;
    a.band = band;
    a.bands_per_plane = (p.out_h + band - 1) / band;
    a.f_out_w = p.f_out_w;
    a.f_bands = make_fastdiv(static_cast<uint32_t>(a.bands_per_plane));
    const int64_t groups = static_cast<int64_t>(in_shape[0]) * in_shape[1] * a.bands_per_plane;
    const int tile_rows = min((band - 1) * p.sh + p.kh, p.in_h);
    const size_t lds = static_cast<size_t>(tile_rows) * p.in_w * sizeof(float);
    if (groups <= INT32_MAX) {
      const uint32_t g = static_cast<uint32_t>(groups);
      const int k = p.kh == p.kw && (p.kh == 2 || p.kh == 3) ? p.kh : 0;
      if (pool_type == 0) {
        if (k == 3)
          pool_band_kernel<true, 3><<<g, kBlock, lds, st>>>(x, y, a);
        else if (k == 2)
          pool_band_kernel<true, 2><<<g, kBlock, lds, st>>>(x, y, a);
        else
          pool_band_kernel<true, 0><<<g, kBlock, lds, st>>>(x, y, a);
      } else {
        if (k == 3)
          pool_band_kernel<false, 3><<<g, kBlock, lds, st>>>(x, y, a);
        else if (k == 2)
          pool_band_kernel<false, 2><<<g, kBlock, lds, st>>>(x, y, a);
        else
          pool_band_kernel<false, 0><<<g, kBlock, lds, st>>>(x, y, a);
      }
      return launch_status();
    }
  }
  const uint32_t grid = grid_for(n_out);
  if (three_d) {
    if (pool_type == 0)
      pool_window_kernel<true, true><<<grid, kBlock, 0, st>>>(x, y, n_out, p);
    else
      pool_window_kernel<false, true><<<grid, kBlock, 0, st>>>(x, y, n_out, p);
  } else {
    if (pool_type == 0)
      pool_window_kernel<true, false><<<grid, kBlock, 0, st>>>(x, y, n_out, p);
    else
      pool_window_kernel<false, false><<<grid, kBlock, 0, st>>>(x, y, n_out, p);
  }
  return launch_status();
}

}  // namespace shdw

using namespace shdw;

extern "C" {

int shdw_hip_axpy_rows(int outer_num, int inner_num, const float* alpha, const float* x,
                       const float* y, float* out, void* stream) {
  if (outer_num < 0 || inner_num < 0) return SHDW_E_INVALID_ARGUMENT;
  const int64_t n = static_cast<int64_t>(outer_num) * inner_num;
  if (n > INT32_MAX) return SHDW_E_INVALID_ARGUMENT;
  if (n == 0) return SHDW_OK;
  if (!alpha || !x || !y || !out) return SHDW_E_INVALID_ARGUMENT;
  AxpyRows p{alpha, y};
  return launch_rows(p, static_cast<uint32_t>(n), static_cast<uint32_t>(inner_num), x, y, out,
                     static_cast<hipStream_t>(stream));
}

int shdw_hip_batch_norm(int n, int channel, int inner_num, const float* x, const float* mean,
                        const float* variance, float scale_factor, float eps, float* y,
                        void* stream) {
  if (n < 0 || channel < 1 || inner_num < 1) return SHDW_E_INVALID_ARGUMENT;
  if (n == 0) return SHDW_OK;
  if (!x || !mean || !variance || !y) return SHDW_E_INVALID_ARGUMENT;
  BatchNormRows p{mean, variance, scale_factor, eps, make_fastdiv(static_cast<uint32_t>(channel))};
  return launch_rows(p, static_cast<uint32_t>(n), static_cast<uint32_t>(inner_num), x, nullptr, y,
                     static_cast<hipStream_t>(stream));
}

int shdw_hip_pooling2d(const int* in_shape, int pool_type, int kernel_h, int kernel_w,
                       int stride_h, int stride_w, int pad_h, int pad_w, const int* out_shape,
                       const float* x, float* y, void* stream) {
  const int kernel[2] = {kernel_h, kernel_w}, stride[2] = {stride_h, stride_w},
            pad[2] = {pad_h, pad_w};
  return run_pooling(false, in_shape, pool_type, kernel, stride, pad, out_shape, x, y,
                     static_cast<hipStream_t>(stream));
}

int shdw_hip_pooling3d(const int* in_shape, int pool_type, int kernel_d, int kernel_h,
                       int kernel_w, int stride_d, int stride_h, int stride_w, int pad_d,
                       int pad_h, int pad_w, const int* out_shape, const float* x, float* y,
                       void* stream) {
  const int kernel[3] = {kernel_d, kernel_h, kernel_w}, stride[3] = {stride_d, stride_h, stride_w},
            pad[3] = {pad_d, pad_h, pad_w};
  return run_pooling(true, in_shape, pool_type, kernel, stride, pad, out_shape, x, y,
                     static_cast<hipStream_t>(stream));
}

}  // extern "C"
