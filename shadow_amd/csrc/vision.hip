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

#include <algorithm>
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
  SHDW_DEVICE v4f load_other(uint64_t off) const { return load4_stream_any(y + off); }
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

// BatchNorm followed by Scale over the same channel axis and, optionally, ReLU:
// the three operators' arithmetic, element by element, in one pass.
template <bool HAS_SCALE, bool HAS_BIAS, bool RELU>
struct BatchNormScaleRows {
  const float* mean;
  const float* variance;
  const float* scale;
  const float* bias;
  float scale_factor, eps;
  FastDiv channel;
  SHDW_DEVICE v4f load_other(uint64_t) const { return v4f{0, 0, 0, 0}; }
  SHDW_DEVICE float other(uint64_t) const { return 0.f; }
  struct Row {
    float m, d, s, b;
  };
  SHDW_DEVICE Row row(uint32_t r) const {
    const uint32_t c = r - fd_div(r, channel) * channel.d;
    const float m = mean[c] * scale_factor;
    const float v = __builtin_fabsf(variance[c] * scale_factor) + eps;
    return {m, __builtin_sqrtf(v), HAS_SCALE ? scale[c] : 1.f, HAS_BIAS ? bias[c] : 0.f};
  }
  SHDW_DEVICE float apply(float x, float, const Row& p) const {
    float t = (x - p.m) / p.d;    // BatchNorm
    if (HAS_SCALE) t = t * p.s;   // Scale: multiply, then add
    if (HAS_BIAS) t = t + p.b;
    if (RELU) t = t > 0 ? t : 0;  // Activate(relu)
    return t;
  }
  static constexpr bool kTwoInputs = false;
};

// ROWVEC: inner % 4 == 0, the four elements of a vector share a row.
template <class P, bool ROWVEC>
__global__ __launch_bounds__(kStream) void rows_vec_kernel(P p, const float* x, float* out,
                                                           uint32_t n4, uint32_t n, FastDiv inner) {
  const uint32_t i = blockIdx.x * kStream + threadIdx.x;
  if (i < n4) {
    const v4f vx = load4_stream_any(x + 4ull * i);
    const v4f vo = p.load_other(4ull * i);
    v4f r;
    if (ROWVEC) {
      const typename P::Row rp = p.row(fd_div(4 * i, inner));
#pragma unroll
      for (int j = 0; j < 4; ++j) r[j] = p.apply(vx[j], vo[j], rp);
    } else {
      // One division per vector.  Rows of four and more: the vector ends in the
      // next row at the furthest, so the parameters of two rows serve it (the
      // second is the first again where the vector lies inside one row); a
      // division and a test per element ran BatchNorm over 7x7 maps at 24 us
      // per 51 MB against 17 us for rows of whole vectors.  Shorter rows: the
      // row steps along with the elements.
      const uint32_t r0 = fd_div(4 * i, inner);
      const uint32_t left = (r0 + 1) * inner.d - 4 * i;  // elements of the vector in row r0: 1 ..
      if (inner.d >= 4) {
        const typename P::Row rp0 = p.row(r0), rp1 = p.row(left < 4 ? r0 + 1 : r0);
#pragma unroll
        for (int j = 0; j < 4; ++j) r[j] = p.apply(vx[j], vo[j], static_cast<uint32_t>(j) < left ? rp0 : rp1);
      } else {
        uint32_t row = r0, togo = left;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          r[j] = p.apply(vx[j], vo[j], p.row(row));
          if (--togo == 0) ++row, togo = inner.d;
        }
      }
    }
    store4_stream_any(out + 4ull * i, r);
  } else if (i == n4) {
    for (uint32_t t = 4 * n4; t < n; ++t) out[t] = p.apply(x[t], p.other(t), p.row(fd_div(t, inner)));
  }
}

template <class P>
static int launch_rows(const P& p, uint32_t n, uint32_t inner, const float* x, const float* other,
                       float* out, hipStream_t st) {
  const FastDiv fi = make_fastdiv(inner);
  const uint32_t n4 = n / 4;  // any float pointers: the 128-bit accesses need dword alignment only
  const uint32_t grid = stream_grid(n4 + 1);
  if (inner % 4 == 0)
    rows_vec_kernel<P, true><<<grid, kStream, 0, st>>>(p, x, out, n4, n, fi);
  else
    rows_vec_kernel<P, false><<<grid, kStream, 0, st>>>(p, x, out, n4, n, fi);
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
//
// LDS layout: rows of pitch = pad_l + in_w + pad_r, plus one spare row.  The pad
// cells and the spare row hold the fold's neutral value (lowest() for max, +0
// for the sum: the running sum starts at +0 and can never become -0, so adding
// +0 leaves it unchanged bit for bit).  A window cell left or right of the
// input reads a pad cell, a cell above or below reads the spare row, and the
// unrolled K x K walk needs no predicates at all.
constexpr int kBandTileFloats = 8192;  // upper bound of the dynamic LDS tile (32 KB)
constexpr int kBandBatch = 4;
constexpr int kBandMaxPad = 64;        // wider clipping goes to the direct kernel
constexpr int kPoolBandOutputs = 512;  // outputs a workgroup aims for (measured best of 256..4096)
constexpr int kBandWideMinCols = 3;    // windows this wide at a column stride of 1: four outputs per lane

struct BandArgs {
  int in_h, in_w, out_h, out_w;
  int kh, kw, sh, sw, ph, pw;
  int band, bands_per_plane, w_shift;
  int wide;  // a lane walks four neighbouring outputs (w_shift then counts quads of outputs)
  int pad_l, pitch, tile_rows;  // data rows in the tile; the spare row is row tile_rows
  uint32_t total_bands, bands_per_group;
  FastDiv f_bands, f_in_w;
};

// Where band g of the launch lies: plane, first output row, row count, and the
// contiguous span of input rows it reads.
struct BandSpan {
  uint32_t plane;
  int h0, nh, r_lo, r_hi;
  uint32_t span;
  const float* src;
};

SHDW_DEVICE BandSpan band_span(const BandArgs& p, const float* x, uint32_t g) {
  BandSpan s;
  uint32_t b;
  fd_divmod(g, p.f_bands, s.plane, b);
  s.h0 = static_cast<int>(b) * p.band;
  s.nh = min(p.band, p.out_h - s.h0);
  s.r_lo = max(s.h0 * p.sh - p.ph, 0);
  s.r_hi = max(min((s.h0 + s.nh - 1) * p.sh - p.ph + p.kh, p.in_h), s.r_lo);
  s.span = static_cast<uint32_t>(s.r_hi - s.r_lo) * p.in_w;
  s.src = x + static_cast<uint64_t>(s.plane) * p.in_h * p.in_w + static_cast<uint64_t>(s.r_lo) * p.in_w;
  return s;
}

// LDS offset of element t of a band's span.
SHDW_DEVICE uint32_t band_slot(const BandArgs& p, uint32_t t) {
  uint32_t r, c;
  fd_divmod(t, p.f_in_w, r, c);
  return r * p.pitch + p.pad_l + c;
}

// K > 0: square K x K window, fully unrolled, all LDS reads in flight together.
// K = 0: any window, clipped loops.
template <bool MAX, int K>
SHDW_DEVICE void band_windows(const float* tile, float* y, const BandArgs& p, const BandSpan& bs) {
  // Lane -> (output row, output column) by shift and mask: w_lanes is a power
  // of two >= min(out_w, 256).  A lane keeps its column(s), so everything that
  // depends on the column only is computed once per lane, not once per output.
  float* dst = y + (static_cast<uint64_t>(bs.plane) * p.out_h + bs.h0) * p.out_w;
  const int w_lanes = 1 << p.w_shift;
  const int h_step = kBlock >> p.w_shift;
  const int h_lane = static_cast<int>(threadIdx.x) >> p.w_shift;
  const int spare = p.tile_rows * p.pitch;
  for (int w = static_cast<int>(threadIdx.x) & (w_lanes - 1); w < p.out_w; w += w_lanes) {
    const int w_first = w * p.sw - p.pw;
    const int w_end_pad = min(w_first + p.kw, p.in_w + p.pw);
    const int wstart = max(w_first, 0), wend = min(w_end_pad, p.in_w);
    for (int hl = h_lane; hl < bs.nh; hl += h_step) {
      const int h_first = (bs.h0 + hl) * p.sh - p.ph;
      const int h_end_pad = min(h_first + p.kh, p.in_h + p.ph);
      float max_val = -FLT_MAX, sum_val = 0.f;
      if (K > 0) {
        float cell[K > 0 ? K * K : 1];
#pragma unroll
        for (int i = 0; i < K; ++i) {
          const int ri = h_first + i;
          const int row = ri >= bs.r_lo && ri < bs.r_hi ? (ri - bs.r_lo) * p.pitch : spare;
          const float* cells = tile + row + p.pad_l + w_first;
#pragma unroll
          for (int j = 0; j < K; ++j) cell[i * K + j] = cells[j];
        }
#pragma unroll
        for (int c = 0; c < K * K; ++c) {
          if (MAX)
            max_val = pool_max(max_val, cell[c]);
          else
            sum_val += cell[c];
        }
      } else {
        const int hstart = max(h_first, 0), hend = min(h_end_pad, p.in_h);
        for (int ph = hstart; ph < hend; ++ph) {
          const float* row = tile + (ph - bs.r_lo) * p.pitch + p.pad_l;
          for (int pw = wstart; pw < wend; ++pw) {
            const float v = row[pw];
            if (MAX)
              max_val = pool_max(max_val, v);
            else
              sum_val += v;
          }
        }
      }
      const int pool_size = (h_end_pad - h_first) * (w_end_pad - w_first);
      dst[hl * p.out_w + w] = MAX ? max_val : sum_val / static_cast<float>(pool_size);
    }
  }
}

// Windows of three and more columns at a column stride of one: a lane takes four
// neighbouring outputs of a row and reads the kw + 3 cells under them once per
// window row, handing each to the outputs it belongs to, in place of 4 kw reads
// (the walks are bound by their LDS reads: 5x5 on 112x112 planes 77 us per
// 51 MB, 25 reads an output).  Every output still receives its cells row by
// row and left to right.  The four outputs start at a column w with w = pw
// (mod 4): their cells then start on a 16-byte boundary of the tile and come
// as 128-bit reads, neighbouring lanes on neighbouring banks (single floats at
// a lane stride of four met the same bank four at a time: 43 us).  The first
// quad of a row may so begin left of column 0 and the last end right of
// out_w - 1; those outputs read the padding, the next row or the eight floats
// behind the tile, and are not stored.
template <bool MAX, int K>
SHDW_DEVICE void band_windows_wide(const float* tile, float* y, const BandArgs& p, const BandSpan& bs) {
  float* dst = y + (static_cast<uint64_t>(bs.plane) * p.out_h + bs.h0) * p.out_w;
  const int q_lanes = 1 << p.w_shift;
  const int h_step = kBlock >> p.w_shift;
  const int h_lane = static_cast<int>(threadIdx.x) >> p.w_shift;
  const int spare = p.tile_rows * p.pitch;
  const int kh = K > 0 ? K : p.kh, kw = K > 0 ? K : p.kw;
  const int lead = p.pad_l - p.pw;  // outputs of the first quad left of column 0: 0 .. 3
  const int quads = (p.out_w + lead + 3) >> 2;
  for (int q = static_cast<int>(threadIdx.x) & (q_lanes - 1); q < quads; q += q_lanes) {
    const int w = 4 * q - lead, w_first = w - p.pw;  // sw == 1; pad_l + w_first = 4 q
    for (int hl = h_lane; hl < bs.nh; hl += h_step) {
      const int h_first = (bs.h0 + hl) * p.sh - p.ph;
      const int rows_pad = min(h_first + p.kh, p.in_h + p.ph) - h_first;
      float acc[4];
#pragma unroll
      for (int o = 0; o < 4; ++o) acc[o] = MAX ? -FLT_MAX : 0.f;
      for (int i = 0; i < kh; ++i) {
        const int ri = h_first + i;
        const int row = ri >= bs.r_lo && ri < bs.r_hi ? (ri - bs.r_lo) * p.pitch : spare;
        const v4f* cells = reinterpret_cast<const v4f*>(tile + row + 4 * q);
        if (K > 0) {
          constexpr int kVecs = (K + 3 + 3) / 4;
          float c[4 * kVecs];
#pragma unroll
          for (int t = 0; t < kVecs; ++t) {
            const v4f v = cells[t];
#pragma unroll
            for (int e = 0; e < 4; ++e) c[4 * t + e] = v[e];
          }
#pragma unroll
          for (int j = 0; j < K; ++j) {
#pragma unroll
            for (int o = 0; o < 4; ++o) acc[o] = MAX ? pool_max(acc[o], c[o + j]) : acc[o] + c[o + j];
          }
        } else {
          v4f cur = cells[0];
          for (int j0 = 0; j0 < kw; j0 += 4) {
            const v4f next = cells[(j0 >> 2) + 1];
            float c[8] = {cur[0], cur[1], cur[2], cur[3], next[0], next[1], next[2], next[3]};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              if (j0 + j < kw) {
#pragma unroll
                for (int o = 0; o < 4; ++o) acc[o] = MAX ? pool_max(acc[o], c[o + j]) : acc[o] + c[o + j];
              }
            }
            cur = next;
          }
        }
      }
      float* out = dst + hl * p.out_w + w;
#pragma unroll
      for (int o = 0; o < 4; ++o) {
        if (w + o >= 0 && w + o < p.out_w) {
          const int cols_pad = min(w_first + o + p.kw, p.in_w + p.pw) - (w_first + o);
          out[o] = MAX ? acc[o] : acc[o] / static_cast<float>(rows_pad * cols_pad);
        }
      }
    }
  }
}

// A workgroup walks `bands_per_group` consecutive bands.  PIPE (every span
// starts 16-byte aligned and in_w % 4 == 0): the next band's 128-bit loads are
// issued into registers before the current band's windows are walked, so HBM
// requests stay in flight during the LDS phase.  Otherwise each band is staged
// on its own with scalar loads.
constexpr int kBandMaxRegs = kBandTileFloats / 4 / kBlock;  // vectors per lane for a full tile
static_assert(kBandMaxRegs == 8, "the launch switch covers up to 8 staged vectors per lane");
constexpr uint32_t kBandGroupsWanted = 4096;
constexpr uint32_t kBandMaxWalk = 16;

// REGS: 128-bit vectors a lane stages per band (PIPE only; 0 otherwise).
template <bool MAX, int K, int REGS>
__global__ __launch_bounds__(kBlock) void pool_band_kernel(const float* x, float* y, BandArgs p) {
  constexpr bool PIPE = REGS > 0;
  constexpr int kBandRegs = PIPE ? REGS : 1;
  extern __shared__ __align__(16) float tile[];  // (tile_rows + 1) x pitch
  const uint32_t g0 = blockIdx.x * p.bands_per_group;
  const uint32_t g1 = min(g0 + p.bands_per_group, p.total_bands);
  {
    const float neutral = MAX ? -FLT_MAX : 0.f;
    const uint32_t cells = static_cast<uint32_t>(p.tile_rows + 1) * p.pitch;  // multiple of 4
    for (uint32_t t = 4 * threadIdx.x; t < cells; t += 4 * kBlock)
      *reinterpret_cast<v4f*>(tile + t) = v4f{neutral, neutral, neutral, neutral};
  }
  __syncthreads();
  if (PIPE) {
    v4f reg[kBandRegs];
    BandSpan cur = band_span(p, x, g0);
#pragma unroll
    for (int k = 0; k < kBandRegs; ++k) {
      const uint32_t v = k * kBlock + threadIdx.x;
      if (4 * v < cur.span) reg[k] = load4_stream(cur.src + 4ull * v);
    }
    for (uint32_t g = g0; g < g1; ++g) {
#pragma unroll
      for (int k = 0; k < kBandRegs; ++k) {
        const uint32_t v = k * kBlock + threadIdx.x;
        if (4 * v < cur.span) *reinterpret_cast<v4f*>(tile + band_slot(p, 4 * v)) = reg[k];
      }
      __syncthreads();
      const BandSpan walk = cur;
      if (g + 1 < g1) {
        cur = band_span(p, x, g + 1);
#pragma unroll
        for (int k = 0; k < kBandRegs; ++k) {
          const uint32_t v = k * kBlock + threadIdx.x;
          if (4 * v < cur.span) reg[k] = load4_stream(cur.src + 4ull * v);
        }
      }
      if (p.wide) band_windows_wide<MAX, K>(tile, y, p, walk);
      else band_windows<MAX, K>(tile, y, p, walk);
      __syncthreads();  // the tile is rewritten next
    }
  } else {
    for (uint32_t g = g0; g < g1; ++g) {
      const BandSpan bs = band_span(p, x, g);
      for (uint32_t t0 = 0; t0 < bs.span; t0 += kBandBatch * kBlock) {
        float reg[kBandBatch];
#pragma unroll
        for (int k = 0; k < kBandBatch; ++k) {
          const uint32_t t = t0 + k * kBlock + threadIdx.x;
          if (t < bs.span) reg[k] = __builtin_nontemporal_load(bs.src + t);
        }
#pragma unroll
        for (int k = 0; k < kBandBatch; ++k) {
          const uint32_t t = t0 + k * kBlock + threadIdx.x;
          if (t < bs.span) tile[band_slot(p, t)] = reg[k];
        }
      }
      __syncthreads();
      if (p.wide) band_windows_wide<MAX, K>(tile, y, p, bs);
      else band_windows<MAX, K>(tile, y, p, bs);
      __syncthreads();
    }
  }
}

// Fills the band geometry; returns false when the direct kernel must be used
// (rows too wide for the tile, or windows that overhang the input by more than
// kBandMaxPad columns, which only an inconsistent out_shape can ask for).
static bool plan_pool_band(const PoolArgs& p, int target_outputs, BandArgs* a) {
  const int over_r = (p.out_w - 1) * p.sw - p.pw + p.kw - p.in_w;
  const int pad_l = (p.pw + 3) & ~3, pad_r = over_r > 0 ? (over_r + 3) & ~3 : 0;
  if (pad_l > kBandMaxPad || pad_r > kBandMaxPad) return false;
  const int pitch = pad_l + ((p.in_w + 3) & ~3) + pad_r;
  const int rows_cap = kBandTileFloats / pitch - 1;  // one row is the spare
  if (rows_cap < p.kh) return false;
  const int band_cap = (rows_cap - p.kh) / p.sh + 1;
  const bool wide = p.sw == 1 && p.kw >= kBandWideMinCols && p.out_w >= 16;
  if (wide) target_outputs *= 4;
  int band = (target_outputs + p.out_w - 1) / p.out_w;
  band = band < 1 ? 1 : band;
  band = band > band_cap ? band_cap : band;
  band = band > p.out_h ? p.out_h : band;
  const int w_units = wide ? (p.out_w + pad_l - p.pw + 3) / 4 : p.out_w;  // what a lane takes along a row
  int w_shift = 0;
  while ((1 << w_shift) < w_units && w_shift < 8) ++w_shift;
  const int h_step = kBlock >> w_shift;  // output rows a workgroup walks at a time
  if (band > h_step && band < p.out_h) band -= band % h_step;
  a->in_h = p.in_h, a->in_w = p.in_w, a->out_h = p.out_h, a->out_w = p.out_w;
  a->kh = p.kh, a->kw = p.kw, a->sh = p.sh, a->sw = p.sw, a->ph = p.ph, a->pw = p.pw;
  a->band = band;
  a->bands_per_plane = (p.out_h + band - 1) / band;
  a->w_shift = w_shift;
  a->wide = wide ? 1 : 0;
  a->pad_l = pad_l, a->pitch = pitch;
  a->tile_rows = min((band - 1) * p.sh + p.kh, p.in_h);
  a->f_bands = make_fastdiv(static_cast<uint32_t>(a->bands_per_plane));
  a->f_in_w = make_fastdiv(static_cast<uint32_t>(p.in_w));
  return true;
}

// Windows of 3x3 (pad 0 or 1) or 2x2 (no pad) at stride 2 over rows of a multiple
// of four columns, out_w = in_w / 2 (the stem pooling of a classifier in either
// rounding of the output size; VGG-style halving): no staging.  A lane owns two
// neighbouring outputs of one row: their windows lie in the columns 4v ... 4v+3
// of two or three input rows, one 128-bit load per row (a wave's loads are whole
// rows of consecutive vectors), plus, for three columns, the one column before
// (pad 1) or after (pad 0) them, which the neighbouring lane loads as part of
// its own vector: it comes from that lane's register (a wave shift), and only
// the lane at the wave's end fetches it from memory.  Cells outside the input take
// the fold's neutral value, as the padding of the band tile does, and every window
// is folded row by row, left to right.  (Four outputs per lane from two
// vectors per row, so that a load instruction covers every other 16 bytes, ran
// at 59 us on [64,64,112,112] where the band kernel takes 49 and this one 43;
// workgroups of 64 or 1024 lanes 47 to 48 us, XCD-contiguous numbering no change.)
struct HalveArgs {
  int in_h, in_w, out_h, out_w;
  FastDiv f_pairs;  // lanes per output row: in_w / 4
  FastDiv f_out_h;
};

constexpr int kHalveLanes = kBlock;

// Lane i receives `from` of lane i - 1 (SHIFT = -1) or i + 1 (SHIFT = +1) of its
// wave; the lane at the wave's end keeps `own`.  Whole-wave shifts are DPP
// controls of the GFX9 family only (gfx950 has them; GFX10 and later do not).
#if defined(__HIP_DEVICE_COMPILE__) && !defined(__gfx950__)
#error "vision.hip: wave_shr / wave_shl DPP controls are used as gfx950 provides them"
#endif
template <int SHIFT>
SHDW_DEVICE float neighbour(float own, float from) {
  constexpr int kWaveShr1 = 0x138, kWaveShl1 = 0x130;
  return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(own), __float_as_int(from),
                                                    SHIFT < 0 ? kWaveShr1 : kWaveShl1, 0xf, 0xf, false));
}

template <bool MAX, int K, int PAD>
__global__ __launch_bounds__(kHalveLanes) void pool_halve_kernel(const float* x, float* y, uint32_t tasks,
                                                                 HalveArgs p) {
  const uint32_t t = blockIdx.x * kHalveLanes + threadIdx.x;
  if (t >= tasks) return;
  uint32_t rest, v, plane, r;
  fd_divmod(t, p.f_pairs, rest, v);
  fd_divmod(rest, p.f_out_h, plane, r);
  constexpr int kCells = K == 3 ? 5 : 4;  // columns under the two windows
  constexpr int kAt = (K == 3 && PAD) ? 1 : 0;  // where column 4v sits among the cells
  const float neutral = MAX ? -FLT_MAX : 0.f;
  const int h_first = 2 * static_cast<int>(r) - PAD;
  const float* img = x + plane * static_cast<uint32_t>(p.in_h * p.in_w) + 4 * v;
  // The one column beside the vector belongs to the neighbouring lane's vector (the
  // lanes of a wave walk along a row); only the lane at the wave's end fetches it.
  constexpr int kHaloCol = PAD ? -1 : 4;  // relative to column 4v
  const int halo_abs = 4 * static_cast<int>(v) + kHaloCol;
  const bool halo_valid = K == 3 && halo_abs >= 0 && halo_abs < p.in_w;
  const uint32_t lane = threadIdx.x & (kWave - 1);
  const bool fetch_halo = halo_valid && lane == (PAD ? 0u : static_cast<uint32_t>(kWave - 1));
  float acc[2];
  acc[0] = acc[1] = MAX ? -FLT_MAX : 0.f;
#pragma unroll
  for (int i = 0; i < K; ++i) {
    const int ri = h_first + i;
    const bool row_valid = ri >= 0 && ri < p.in_h;
    const float* row = img + min(max(ri, 0), p.in_h - 1) * p.in_w;
    const v4f q = load4(row);
    float cells[kCells];
#pragma unroll
    for (int e = 0; e < 4; ++e) cells[kAt + e] = q[e];
    if (K == 3) {
      float own = neutral;
      if (fetch_halo) own = row[kHaloCol];
      const float h = PAD ? neighbour<-1>(own, q[3]) : neighbour<+1>(own, q[0]);
      cells[PAD ? 0 : 4] = halo_valid ? h : neutral;
    }
    // a row above or below the input leaves the running values as they are,
    // which is what folding the neutral value into them does
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      float next = acc[j];
#pragma unroll
      for (int k = 0; k < K; ++k) next = MAX ? pool_max(next, cells[2 * j + k]) : next + cells[2 * j + k];
      acc[j] = row_valid ? next : acc[j];
    }
  }
  float res[2];
  const int h_end_pad = min(h_first + K, p.in_h + PAD);
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int w_first = 2 * (2 * static_cast<int>(v) + j) - PAD;
    const int w_end_pad = min(w_first + K, p.in_w + PAD);
    const int pool_size = (h_end_pad - h_first) * (w_end_pad - w_first);
    res[j] = MAX ? acc[j] : acc[j] / static_cast<float>(pool_size);
  }
  typedef float v2f __attribute__((ext_vector_type(2)));
  float* dst = y + ((plane * static_cast<uint32_t>(p.out_h) + r) * static_cast<uint32_t>(p.out_w) + 2 * v);
  __builtin_nontemporal_store(v2f{res[0], res[1]}, reinterpret_cast<v2f*>(dst));
}

// 3x3 windows at stride 1 with one cell of padding (the output as large as the
// input; rows of a multiple of four columns): a lane owns four neighbouring outputs
// of one row, whose windows lie in its own vector of three input rows and in the
// columns left and right of it, which are elements of the neighbouring lanes'
// vectors (wave shifts; the lanes at the two ends of a wave fetch theirs).  One
// 128-bit load per input row, one 128-bit store.
template <bool MAX>
__global__ __launch_bounds__(kHalveLanes) void pool_same_kernel(const float* x, float* y, uint32_t tasks,
                                                                HalveArgs p) {
  // runs of eight workgroups on one XCD: every input row is read for three output rows
  const uint32_t t = xcd_runs(blockIdx.x, gridDim.x, 3) * kHalveLanes + threadIdx.x;
  if (t >= tasks) return;
  uint32_t rest, v, plane, r;
  fd_divmod(t, p.f_pairs, rest, v);
  fd_divmod(rest, p.f_out_h, plane, r);
  const float neutral = MAX ? -FLT_MAX : 0.f;
  const uint32_t lane = threadIdx.x & (kWave - 1);
  const bool left_valid = v > 0, right_valid = 4 * v + 4 < static_cast<uint32_t>(p.in_w);
  const bool fetch_left = left_valid && lane == 0, fetch_right = right_valid && lane == kWave - 1;
  const float* img = x + plane * static_cast<uint32_t>(p.in_h * p.in_w) + 4 * v;
  const int h_first = static_cast<int>(r) - 1;
  float acc[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) acc[j] = MAX ? -FLT_MAX : 0.f;
#pragma unroll
  for (int i = 0; i < 3; ++i) {
    const int ri = h_first + i;
    const bool row_valid = ri >= 0 && ri < p.in_h;
    const float* row = img + min(max(ri, 0), p.in_h - 1) * p.in_w;
    const v4f q = load4(row);
    float own_l = neutral, own_r = neutral;
    if (fetch_left) own_l = row[-1];
    if (fetch_right) own_r = row[4];
    const float hl = neighbour<-1>(own_l, q[3]), hr = neighbour<+1>(own_r, q[0]);
    const float cells[6] = {left_valid ? hl : neutral, q[0], q[1], q[2], q[3], right_valid ? hr : neutral};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float next = acc[j];
#pragma unroll
      for (int k = 0; k < 3; ++k) next = MAX ? pool_max(next, cells[j + k]) : next + cells[j + k];
      acc[j] = row_valid ? next : acc[j];
    }
  }
  v4f res;
  const int h_end_pad = min(h_first + 3, p.in_h + 1);
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int w_first = 4 * static_cast<int>(v) + j - 1;
    const int w_end_pad = min(w_first + 3, p.in_w + 1);
    const int pool_size = (h_end_pad - h_first) * (w_end_pad - w_first);
    res[j] = MAX ? acc[j] : acc[j] / static_cast<float>(pool_size);
  }
  store4_stream(y + ((plane * static_cast<uint32_t>(p.out_h) + r) * static_cast<uint32_t>(p.out_w) + 4 * v), res);
}

static bool pool_same_applies(const PoolArgs& p, const float* x, const float* y, bool planning) {
  if (p.kh != 3 || p.kw != 3 || p.sh != 1 || p.sw != 1 || p.ph != 1 || p.pw != 1) return false;
  if (p.in_w % 4 != 0 || p.out_w != p.in_w || p.out_h != p.in_h) return false;
  return planning || (aligned16(x) && aligned16(y));
}

// True when the kernel above applies to p (2-D).
static bool pool_halve_applies(const PoolArgs& p, const float* x, const float* y, bool planning) {
  if (p.kh != p.kw || p.sh != 2 || p.sw != 2 || p.ph != p.pw) return false;
  if (!((p.kh == 3 && p.pw <= 1) || (p.kh == 2 && p.pw == 0))) return false;
  if (p.in_w % 4 != 0 || p.out_w * 2 != p.in_w || p.in_h < 1) return false;
  return planning || (aligned16(x) && aligned16(y));
}

// Planes too small to keep a workgroup busy (14x14 and 7x7 maps with 3x3 / 2x2 /
// 5x5 .. 13x13 windows): with a workgroup per band of one plane, a 7x7 plane
// gives 49 outputs to 256 lanes (3x3 stride 1 on [128,2048,7,7]: 179 us per
// 51 MB).  Here a workgroup takes `planes` consecutive planes, one contiguous
// span of x, into LDS, each with its padding in place: ph rows above, pw
// columns left, and as many below and to the right as the last window reaches
// over, all holding the fold's neutral value (lowest() for max, +0 for the sum:
// the running sum starts at +0 and can never become -0, so adding +0 leaves it
// unchanged bit for bit).  A lane then walks the window of one output after the
// other, rows and columns in ascending order, without a test.
//
// Max windows of 16 and more cells (5x5 .. 13x13 at stride 1: the pyramid
// pooling of detection heads) are folded in two steps, SEP: first the maximum of
// every window-wide piece of every row into a second LDS array, then down the
// window's rows of that array, kh + kw comparisons for an output instead of
// kh * kw.  pool_max never takes a NaN and keeps the earlier of equal values
// (+0 and -0), so the result of the row-major walk is the earliest largest cell,
// and that is what the two steps return as well: the earliest of a row, then the
// earliest row.
constexpr int kSmallPlanesTileFloats = 12288;  // 48 KB: three workgroups per CU
constexpr int kSmallPlanesMaxOutputs = 512;    // larger planes go to the band kernel
constexpr int kSeparableMinCells = 16;         // max windows from this size on fold rows first

struct SmallPlanesArgs {
  int in_h, in_w, out_h, out_w, kh, kw, sh, sw, ph, pw;
  int pitch, plane_lds;  // padded row and plane in LDS, in floats
  int rows_lds;          // padded rows of a plane
  uint32_t planes, total_planes;
  FastDiv f_plane_in, f_in_w, f_plane_out, f_out_w, f_row_maxima;  // the last: rows_lds * out_w; for the
                                                                   // wide average: output quads per plane
  FastDiv f_quads_w;  // wide average: output quads per row
  FastDiv f_out_quads;  // maximum by quads: output quads per plane (f_row_maxima: row-maximum quads per plane)
  bool quads_max;       // the maximum by quads applies
};

// SEP with MAX false is the wide average at a column stride of one: a lane takes four
// neighbouring outputs of a row and reads every cell of their 4 + kw - 1 columns once per
// window row, adding it to the sums it belongs to - each sum still receives its cells row by
// row and left to right - in place of 4 kw reads (13x13 on 14x14 maps: 256 us per 51 MB, all
// of it LDS reads).  The tile has eight spare floats behind it for the reads of a row's last,
// partly empty quad.
template <bool MAX, int K, bool SEP = false>
__global__ __launch_bounds__(kBlock) void pool_small_planes_kernel(const float* x, float* y, SmallPlanesArgs a) {
  extern __shared__ __align__(16) float tile[];  // planes * plane_lds floats, a multiple of 4
  const uint32_t first = blockIdx.x * a.planes;
  const uint32_t np = min(a.planes, a.total_planes - first);
  const uint32_t plane_in = a.f_plane_in.d, plane_out = a.f_plane_out.d;
  {
    const float neutral = MAX ? -FLT_MAX : 0.f;
    const uint32_t cells = a.planes * static_cast<uint32_t>(a.plane_lds);
    for (uint32_t t = 4 * threadIdx.x; t < cells; t += 4 * kBlock)
      *reinterpret_cast<v4f*>(tile + t) = v4f{neutral, neutral, neutral, neutral};
  }
  __syncthreads();
  const float* xs = x + static_cast<uint64_t>(first) * plane_in;
  const uint32_t span = np * plane_in, nvec = span / 4;
  auto slot = [&](uint32_t t) -> uint32_t {
    uint32_t pl, rem, r, c;
    fd_divmod(t, a.f_plane_in, pl, rem);
    fd_divmod(rem, a.f_in_w, r, c);
    return pl * a.plane_lds + (r + a.ph) * a.pitch + a.pw + c;
  };
  for (uint32_t v0 = 0; v0 < nvec; v0 += 4 * kBlock) {
    v4f reg[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const uint32_t v = v0 + k * kBlock + threadIdx.x;
      if (v < nvec) reg[k] = load4_stream_any(xs + 4ull * v);
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const uint32_t v = v0 + k * kBlock + threadIdx.x;
      if (v < nvec) {
        // one division per vector: the following elements step along the row and wrap into the
        // next row (past the right padding) or the next plane (past the bottom padding)
        uint32_t pl, rem, r, c;
        fd_divmod(4 * v, a.f_plane_in, pl, rem);
        fd_divmod(rem, a.f_in_w, r, c);
        uint32_t at = pl * a.plane_lds + (r + a.ph) * a.pitch + a.pw + c;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          tile[at] = reg[k][j];
          ++at;
          if (++c == static_cast<uint32_t>(a.in_w)) {
            c = 0, at += a.pitch - a.in_w;
            if (++r == static_cast<uint32_t>(a.in_h)) r = 0, at += a.plane_lds - a.in_h * a.pitch;
          }
        }
      }
    }
  }
  if (4 * nvec + threadIdx.x < span) tile[slot(4 * nvec + threadIdx.x)] = xs[4 * nvec + threadIdx.x];
  __syncthreads();
  float* ys = y + static_cast<uint64_t>(first) * plane_out;
  const uint32_t outputs = np * plane_out;
  if (SEP && !MAX) {
    const uint32_t quads_w = (static_cast<uint32_t>(a.out_w) + 3) / 4, per_plane = a.out_h * quads_w;
    const FastDiv f_quads = a.f_row_maxima, f_quads_w = a.f_quads_w;  // per plane, per row
    for (uint32_t t = threadIdx.x; t < np * per_plane; t += kBlock) {
      uint32_t pl, rem, oh, q;
      fd_divmod(t, f_quads, pl, rem);
      fd_divmod(rem, f_quads_w, oh, q);
      const uint32_t ow = 4 * q;
      const float* win = tile + pl * a.plane_lds + (oh * a.sh) * a.pitch + ow;  // sw == 1
      float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
      const int kw = a.kw;
      for (int i = 0; i < a.kh; ++i) {
        const float* row = win + i * a.pitch;
        // cells 0 .. kw+2 of the row piece; cell j belongs to the windows j-3 .. j of the four
        if (K > 0) {
          // the window width known: all reads of the row piece are asked for before the first sum
          // waits for one (a lane otherwise waits out the LDS latency once per cell, with three
          // waves per SIMD to cover it)
          // (as 128-bit pieces: the launch keeps the pitch a multiple of four floats for these widths,
          // and a lane's first column is one; single floats four columns apart from lane to lane meet
          // in a quarter of the banks)
          constexpr int kPieces = (K + 3 + 3) / 4;
          float v[4 * kPieces];
#pragma unroll
          for (int q4 = 0; q4 < kPieces; ++q4) {
            const v4f piece = *reinterpret_cast<const v4f*>(row + 4 * q4);
#pragma unroll
            for (int e = 0; e < 4; ++e) v[4 * q4 + e] = piece[e];
          }
#pragma unroll
          for (int j = 0; j < K + 3; ++j) {
            if (j < K) s0 += v[j];
            if (j >= 1 && j < K + 1) s1 += v[j];
            if (j >= 2 && j < K + 2) s2 += v[j];
            if (j >= 3) s3 += v[j];
          }
          continue;
        }
        float v0 = row[0], v1 = row[1], v2 = row[2];
        s0 += v0;
        s0 += v1, s1 += v1;
        s0 += v2, s1 += v2, s2 += v2;
        for (int j = 3; j < kw; ++j) {
          const float v = row[j];
          s0 += v, s1 += v, s2 += v, s3 += v;
        }
        v0 = row[kw], v1 = row[kw + 1], v2 = row[kw + 2];
        s1 += v0, s2 += v0, s3 += v0;
        s2 += v1, s3 += v1;
        s3 += v2;
      }
      const float sums[4] = {s0, s1, s2, s3};
      const int h_first = static_cast<int>(oh) * a.sh - a.ph;
      const int rows_in = min(h_first + a.kh, a.in_h + a.ph) - h_first;
      float* dst = ys + pl * plane_out + oh * a.out_w + ow;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        if (ow + k < static_cast<uint32_t>(a.out_w)) {
          const int w_first = static_cast<int>(ow + k) - a.pw;
          const int pool_size = rows_in * (min(w_first + kw, a.in_w + a.pw) - w_first);
          dst[k] = sums[k] / static_cast<float>(pool_size);
        }
      }
    }
    return;
  }
  if (SEP && K > 0) {
    // The two-step maximum for square K x K windows at a column stride of one, four neighbouring outputs
    // per lane: a row piece of K + 3 cells is read once as 128-bit pieces (the pitch is a multiple of four
    // floats) and gives four row maxima, which share the fold of the cells 3 .. K - 1; the leftmost of equal
    // maxima wins in every partial fold, as in the fold cell by cell.  The row maxima lie as quads,
    // [plane][padded row][quad], so the second step reads a column of K quads.
    float* row_maxima = tile + a.planes * static_cast<uint32_t>(a.plane_lds);
    const uint32_t quads_w = a.f_quads_w.d;
    const uint32_t pieces = np * a.f_row_maxima.d;  // rows_lds * quads_w per plane
    for (uint32_t t = threadIdx.x; t < pieces; t += kBlock) {
      uint32_t pl, rem, r, q;
      fd_divmod(t, a.f_row_maxima, pl, rem);
      fd_divmod(rem, a.f_quads_w, r, q);
      const float* row = tile + pl * a.plane_lds + r * a.pitch + 4 * q;
      constexpr int kPieces = (K + 3 + 3) / 4;
      float v[4 * kPieces];
#pragma unroll
      for (int q4 = 0; q4 < kPieces; ++q4) {
        const v4f piece = *reinterpret_cast<const v4f*>(row + 4 * q4);
#pragma unroll
        for (int e = 0; e < 4; ++e) v[4 * q4 + e] = piece[e];
      }
      float core = -FLT_MAX;
#pragma unroll
      for (int j = 3; j < K; ++j) core = pool_max(core, v[j]);
      const float lo = -FLT_MAX;
      v4f m;
      m[0] = pool_max(pool_max(pool_max(pool_max(lo, v[0]), v[1]), v[2]), core);
      m[1] = pool_max(pool_max(pool_max(pool_max(lo, v[1]), v[2]), core), v[K]);
      m[2] = pool_max(pool_max(pool_max(pool_max(lo, v[2]), core), v[K]), v[K + 1]);
      m[3] = pool_max(pool_max(pool_max(pool_max(lo, core), v[K]), v[K + 1]), v[K + 2]);
      *reinterpret_cast<v4f*>(row_maxima + 4 * t) = m;
    }
    __syncthreads();
    const uint32_t out_quads = np * a.f_out_quads.d;  // out_h * quads_w per plane
    for (uint32_t t = threadIdx.x; t < out_quads; t += kBlock) {
      uint32_t pl, rem, oh, q;
      fd_divmod(t, a.f_out_quads, pl, rem);
      fd_divmod(rem, a.f_quads_w, oh, q);
      const float* col = row_maxima + 4 * ((pl * a.rows_lds + oh * a.sh) * quads_w + q);
      v4f v[K > 0 ? K : 1];
#pragma unroll
      for (int i = 0; i < K; ++i) v[i] = *reinterpret_cast<const v4f*>(col + 4 * i * quads_w);
      v4f m = {-FLT_MAX, -FLT_MAX, -FLT_MAX, -FLT_MAX};
#pragma unroll
      for (int i = 0; i < K; ++i)
#pragma unroll
        for (int k = 0; k < 4; ++k) m[k] = pool_max(m[k], v[i][k]);
      float* dst = ys + pl * plane_out + oh * a.out_w + 4 * q;
#pragma unroll
      for (int k = 0; k < 4; ++k)
        if (4 * q + k < static_cast<uint32_t>(a.out_w)) dst[k] = m[k];
    }
    return;
  }
  if (SEP) {
    float* row_maxima = tile + a.planes * static_cast<uint32_t>(a.plane_lds);  // [plane][padded row][out_w]
    const uint32_t per_plane = a.f_row_maxima.d, pieces = np * per_plane;
    for (uint32_t t = threadIdx.x; t < pieces; t += kBlock) {
      uint32_t pl, rem, r, ow;
      fd_divmod(t, a.f_row_maxima, pl, rem);
      fd_divmod(rem, a.f_out_w, r, ow);
      const float* piece = tile + pl * a.plane_lds + r * a.pitch + ow * a.sw;
      float max_val = -FLT_MAX;
      for (int j = 0; j < a.kw; ++j) max_val = pool_max(max_val, piece[j]);
      row_maxima[t] = max_val;
    }
    __syncthreads();
    for (uint32_t o = threadIdx.x; o < outputs; o += kBlock) {
      uint32_t pl, rem, oh, ow;
      fd_divmod(o, a.f_plane_out, pl, rem);
      fd_divmod(rem, a.f_out_w, oh, ow);
      const float* win = row_maxima + pl * per_plane + (oh * a.sh) * a.out_w + ow;
      float max_val = -FLT_MAX;
      for (int i = 0; i < a.kh; ++i) max_val = pool_max(max_val, win[i * a.out_w]);
      ys[o] = max_val;
    }
    return;
  }
  for (uint32_t o = threadIdx.x; o < outputs; o += kBlock) {
    uint32_t pl, rem, oh, ow;
    fd_divmod(o, a.f_plane_out, pl, rem);
    fd_divmod(rem, a.f_out_w, oh, ow);
    const float* win = tile + pl * a.plane_lds + (oh * a.sh) * a.pitch + ow * a.sw;
    float max_val = -FLT_MAX, sum_val = 0.f;
    if (K > 0) {
      float cell[K > 0 ? K * K : 1];
#pragma unroll
      for (int i = 0; i < K; ++i)
#pragma unroll
        for (int j = 0; j < K; ++j) cell[i * K + j] = win[i * a.pitch + j];
#pragma unroll
      for (int c = 0; c < K * K; ++c) {
        if (MAX)
          max_val = pool_max(max_val, cell[c]);
        else
          sum_val += cell[c];
      }
    } else {
      for (int i = 0; i < a.kh; ++i) {
        const float* row = win + i * a.pitch;
        for (int j = 0; j < a.kw; ++j) {
          const float v = row[j];
          if (MAX)
            max_val = pool_max(max_val, v);
          else
            sum_val += v;
        }
      }
    }
    if (MAX) {
      ys[o] = max_val;
    } else {
      const int h_first = static_cast<int>(oh) * a.sh - a.ph, w_first = static_cast<int>(ow) * a.sw - a.pw;
      const int pool_size = (min(h_first + a.kh, a.in_h + a.ph) - h_first) * (min(w_first + a.kw, a.in_w + a.pw) - w_first);
      ys[o] = sum_val / static_cast<float>(pool_size);
    }
  }
}

// Window widths whose row pieces the kernels for four outputs per lane unroll and read as 128-bit pieces.
static bool wide_unrolled(int kw) { return kw == 5 || kw == 7 || kw == 9 || kw == 13; }

// Fills `a` and returns true where the kernel above applies: several padded
// planes fit the tile and one plane alone would leave lanes idle.
static bool plan_small_planes(const PoolArgs& p, int64_t total_planes, bool max_pool, SmallPlanesArgs* a,
                              bool* separable) {
  const int64_t plane_out = static_cast<int64_t>(p.out_h) * p.out_w, plane_in = static_cast<int64_t>(p.in_h) * p.in_w;
  // the two-step maximum is worth whole planes of up to 32 x 32 as well (13x13 windows on
  // 26x26 maps: 64 us per 51 MB; the band kernel, which walks every cell of every window,
  // takes 369 us for the average over the same windows)
  const bool wide_max = max_pool && p.kh * p.kw >= kSeparableMinCells;
  // ... and so is the average that reads every cell once for four neighbouring outputs (13x13 on
  // 26x26 maps: 369 us through the band kernel)
  const bool wide_avg = !max_pool && p.kh * p.kw >= kSeparableMinCells && p.sw == 1 && p.kw >= 4;
  if (plane_out > (wide_max || wide_avg ? 2 : 1) * kSmallPlanesMaxOutputs || plane_out < 1 || total_planes > INT32_MAX)
    return false;
  const int over_b = std::max(0, (p.out_h - 1) * p.sh - p.ph + p.kh - p.in_h);
  const int over_r = std::max(0, (p.out_w - 1) * p.sw - p.pw + p.kw - p.in_w);
  const int64_t rows_lds = static_cast<int64_t>(p.ph) + p.in_h + over_b;
  const int64_t quads_w = (static_cast<int64_t>(p.out_w) + 3) / 4;
  int64_t pitch = static_cast<int64_t>(p.pw) + p.in_w + over_r;
  // the maximum by quads where its wider rows leave room for two planes
  const int64_t pitch4 = (pitch + 3) & ~int64_t{3};
  const bool quads_max = wide_max && p.sw == 1 && p.kh == p.kw && wide_unrolled(p.kw) &&
                         (rows_lds * pitch4 + rows_lds * 4 * quads_w) * 2 <= kSmallPlanesTileFloats;
  if (wide_avg) pitch = wide_unrolled(p.kw) ? pitch4 : pitch | 1;
  if (quads_max) pitch = pitch4;
  int64_t plane_lds = rows_lds * pitch;
  plane_lds = (plane_lds + 3) & ~int64_t{3};
  if (plane_lds * 2 > kSmallPlanesTileFloats) return false;
  const int64_t row_maxima = wide_avg ? 0 : rows_lds * (quads_max ? 4 * quads_w : p.out_w);
  *separable = wide_avg || (wide_max && (plane_lds + row_maxima) * 2 <= kSmallPlanesTileFloats);
  if (plane_out > kSmallPlanesMaxOutputs && !*separable) return false;
  int64_t planes = kSmallPlanesTileFloats / (plane_lds + (*separable ? row_maxima : 0));
  const int64_t want = (4 * kBlock + plane_out - 1) / plane_out;  // about four outputs per lane
  planes = std::min(planes, std::max<int64_t>(2, want));
  if (planes >= 4) planes &= ~int64_t{3};  // whole 128-bit pieces wherever the plane count allows
  a->in_h = p.in_h, a->in_w = p.in_w, a->out_h = p.out_h, a->out_w = p.out_w;
  a->kh = p.kh, a->kw = p.kw, a->sh = p.sh, a->sw = p.sw, a->ph = p.ph, a->pw = p.pw;
  a->pitch = static_cast<int>(pitch), a->plane_lds = static_cast<int>(plane_lds);
  a->rows_lds = static_cast<int>(rows_lds);
  const uint32_t qw = static_cast<uint32_t>(quads_w);
  a->f_row_maxima = make_fastdiv(wide_avg ? p.out_h * qw : static_cast<uint32_t>(quads_max ? rows_lds * qw : row_maxima));
  a->f_quads_w = make_fastdiv(qw);
  a->f_out_quads = make_fastdiv(p.out_h * qw);
  a->quads_max = quads_max;
  a->planes = static_cast<uint32_t>(planes), a->total_planes = static_cast<uint32_t>(total_planes);
  a->f_plane_in = make_fastdiv(static_cast<uint32_t>(plane_in));
  a->f_in_w = make_fastdiv(static_cast<uint32_t>(p.in_w));
  a->f_plane_out = make_fastdiv(static_cast<uint32_t>(plane_out));
  a->f_out_w = make_fastdiv(static_cast<uint32_t>(p.out_w));
  return true;
}

// Whole-plane windows: x is [rows][len], one output per row.  A workgroup owns
// `group` consecutive rows (as many as fit the tile, at most one per lane); they
// pass through LDS (coalesced 128-bit loads by all lanes), then lane r folds
// row r element by element.  The row pitch in LDS is odd, so the per-lane walks
// hit distinct banks.  Rows longer than the tile are staged in column chunks.
// Measured on 51 MB inputs: 49 KB tiles (256 rows of 7x7, 64 rows of 14x14) beat
// 13 KB tiles by 8 % and 25 %: what the large tile loses in resident workgroups
// it gains by having every lane of the workgroup fold a row.
constexpr int kPlaneTileFloats = 12608;  // 256 rows x 49 or 64 rows x 197
constexpr int kPlaneMaxGroup = 256;      // rows per workgroup (one lane folds one row)
constexpr int kPlaneChunkRows = 64;      // rows per workgroup when rows are chunked

constexpr int kPlaneBatch = 8;  // global loads a lane keeps in flight while staging
constexpr int kPlaneFold = 8;   // LDS reads a lane keeps in flight while folding

template <bool MAX>
__global__ __launch_bounds__(kBlock) void pool_plane_kernel(const float* x, float* y, uint32_t rows,
                                                             uint32_t len, uint32_t group,
                                                             uint32_t chunk, FastDiv f_chunk,
                                                             FastDiv f_last, float pool_size) {
  __shared__ float tile[kPlaneTileFloats];
  const uint32_t row0 = blockIdx.x * group;
  const uint32_t nrows = min(group, rows - row0);
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
      // Eight LDS reads in flight per step of the (inherently serial) fold.
      const float* mine = tile + threadIdx.x * pitch;
      uint32_t c = 0;
      for (; c + kPlaneFold <= cols; c += kPlaneFold) {
        float v[kPlaneFold];
#pragma unroll
        for (int k = 0; k < kPlaneFold; ++k) v[k] = mine[c + k];
#pragma unroll
        for (int k = 0; k < kPlaneFold; ++k) {
          if (MAX)
            max_val = pool_max(max_val, v[k]);
          else
            sum_val += v[k];
        }
      }
      for (; c < cols; ++c) {
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
  uint32_t group, chunk;
  const uint32_t pitch = len | 1u;
  if (pitch <= kPlaneTileFloats) {  // whole rows: as many as fit the tile
    group = kPlaneTileFloats / pitch;
    group = group > kPlaneMaxGroup ? kPlaneMaxGroup : group;
    if (group >= 4) group &= ~3u;  // keeps every workgroup's first row 16-byte aligned
    chunk = len;
  } else {
    group = kPlaneChunkRows;
    chunk = (kPlaneTileFloats / kPlaneChunkRows - 1) | 1u;  // odd: it is the LDS pitch too
  }
  const uint32_t tail = len % chunk;
  const FastDiv fc = make_fastdiv(chunk), fl = make_fastdiv(tail ? tail : chunk);
  const float size = static_cast<float>(static_cast<int>(len));
  const uint32_t grid = (rows + group - 1) / group;
  pool_plane_kernel<MAX><<<grid, kBlock, 0, st>>>(x, y, rows, len, group, chunk, fc, fl, size);
}

// Whole-plane average over rows of any length, without a barrier: every wave of a
// workgroup works by itself on G consecutive rows, which it walks in chunks of
// W = 4096 / G columns.  All lanes fetch a chunk (16 vectors each, 16 KB per wave)
// and lay it down in the wave's LDS rows; lane g < G then adds row g's columns in
// index order (an fp32 running sum has no other order; a dependent addition takes
// six clocks, so a row of 3136 takes 8 us whatever else happens) while the next
// chunk is already on its way.  A wave never waits for another wave, so a CU's
// eight resident waves overlap each other's fetches and folds.  G shrinks as the
// rows get longer and fewer: what matters is enough waves in flight (16 KB each)
// to cover HBM's latency, not how many lanes of a wave fold.  The four waves of a
// workgroup exist for their placement only: one per SIMD.  Single-wave
// workgroups were measured to pile up on one SIMD of a CU when only four of
// them fit the launch, and waves that share a SIMD take turns at every addition.
// The LDS pitch of W + 4 floats keeps 128-bit accesses aligned and puts the
// folding lanes on distinct banks.
constexpr int kStreamVectors = 16;  // per lane and chunk
constexpr int kStreamWaves = kBlock / kWave;

template <int G>
__global__ __launch_bounds__(kBlock) void pool_rows_stream_kernel(const float* x, float* y, uint32_t rows,
                                                                   uint32_t len, float pool_size) {
  constexpr uint32_t W = 256u * kStreamVectors / G, VW = W / 4, PITCH = W + 4;
  __shared__ __align__(16) float tiles[kStreamWaves * G * PITCH];
  const uint32_t lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  float* tile = tiles + wave * (G * PITCH);
  const uint32_t row0 = (blockIdx.x * kStreamWaves + wave) * G;
  if (row0 >= rows) return;  // the whole wave
  v4f reg[kStreamVectors];
  auto request = [&](uint32_t c0) {
#pragma unroll
    for (int i = 0; i < kStreamVectors; ++i) {
      const uint32_t v = lane + kWave * i;
      const uint32_t g = v / VW, c = c0 + 4 * (v % VW);
      if (row0 + g >= rows || c >= len) continue;
      const float* src = x + static_cast<uint64_t>(row0 + g) * len + c;
      if (c + 4 <= len) {
        reg[i] = __builtin_nontemporal_load(reinterpret_cast<const v4f_unaligned*>(src));
      } else {
#pragma unroll
        for (int k = 0; k < 3; ++k)
          if (c + k < len) reg[i][k] = __builtin_nontemporal_load(src + k);
      }
    }
  };
  float sum = 0.f;
  request(0);
  for (uint32_t c0 = 0; c0 < len; c0 += W) {
#pragma unroll
    for (int i = 0; i < kStreamVectors; ++i) {
      const uint32_t v = lane + kWave * i;
      *reinterpret_cast<v4f*>(tile + (v / VW) * PITCH + 4 * (v % VW)) = reg[i];
    }
    __builtin_amdgcn_wave_barrier();
    if (c0 + W < len) request(c0 + W);
    if (lane < G) {
      const uint32_t cols = min(W, len - c0);
      const float* mine = tile + lane * PITCH;
      // 64 values per step, read with sixteen 128-bit reads and then added in order.  One set of
      // registers: with two sets taking turns (the next step's reads behind this step's additions) the
      // compiler copied one set into the other every turn, 32 moves per 64 additions, and a wave
      // alone on its SIMD issues an instruction every 2.8 ns whatever it is; the LDS latency that is
      // exposed instead is a twentieth of a step's additions.
      constexpr int kAhead = 16, kStep = 4 * kAhead;
      uint32_t c = 0;
      for (; c + kStep <= cols; c += kStep) {
        v4f q[kAhead];
#pragma unroll
        for (int k = 0; k < kAhead; ++k) q[k] = *reinterpret_cast<const v4f*>(mine + c + 4 * k);
#pragma unroll
        for (int k = 0; k < kStep; ++k) sum += q[k / 4][k % 4];
      }
      for (; c < cols; ++c) sum += mine[c];
    }
    __builtin_amdgcn_wave_barrier();
  }
  if (lane < G && row0 + lane < rows) y[row0 + lane] = sum / pool_size;
}

// From this row length on the whole-plane average takes the streaming kernel
// (per 51 MB, against pool_plane_kernel: 28x28 planes 15.1 / 23.5 us, 56x56 planes
// 24.6 / 59 us; 14x14 planes 13.2 / 14.2 us but 45.8 / 42.0 us per 205 MB, 7x7 planes
// 12.6 / 12.7 and 44.1 / 39.6 us).
constexpr int kPlaneStreamMinLen = 256;
// Few rows as well: a wave per row walks at 5 ns per element where the workgroup form above, which stages
// a chunk, meets at a barrier and then walks it, takes 10 to 18 ([1,3,224,224]: 252 us against 630 us,
// 64 planes of 56x56: 29 against 30).
// Rows per wave: as many as leave 1536 waves and more (six per CU), so long and few rows get a wave
// each.  Measured per 51 MB: 16x16 planes 10.2 us with 32 rows per wave (12.7 with 16), 20x20 11.7 with
// 16 (14.6 with 8), 28x28 13.1 with 8 (17.2 with 4, 13.7 with 16), 40x40 16.6 with 4 (21.7 with 2),
// 56x56 21.3 with 2 (26.3 with 4, 33.9 with 1).
static int stream_rows_per_wave(uint32_t rows) {
  int g = 1;
  while (g < 64 && rows / static_cast<uint32_t>(2 * g) >= 1536u) g <<= 1;
  return g;
}

static void launch_pool_rows_stream(const float* x, float* y, uint32_t rows, uint32_t len, hipStream_t st) {
  const float size = static_cast<float>(static_cast<int>(len));
  const int g = stream_rows_per_wave(rows);
  const uint32_t per_wg = static_cast<uint32_t>(g) * kStreamWaves;
  const uint32_t grid = (rows + per_wg - 1) / per_wg;
  switch (g) {
    case 64: pool_rows_stream_kernel<64><<<grid, kBlock, 0, st>>>(x, y, rows, len, size); break;
    case 32: pool_rows_stream_kernel<32><<<grid, kBlock, 0, st>>>(x, y, rows, len, size); break;
    case 16: pool_rows_stream_kernel<16><<<grid, kBlock, 0, st>>>(x, y, rows, len, size); break;
    case 8: pool_rows_stream_kernel<8><<<grid, kBlock, 0, st>>>(x, y, rows, len, size); break;
    case 4: pool_rows_stream_kernel<4><<<grid, kBlock, 0, st>>>(x, y, rows, len, size); break;
    case 2: pool_rows_stream_kernel<2><<<grid, kBlock, 0, st>>>(x, y, rows, len, size); break;
    default: pool_rows_stream_kernel<1><<<grid, kBlock, 0, st>>>(x, y, rows, len, size);
  }
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

// The decision of run_pooling, handed back instead of a launch when `want` is set
// (shdw_hip_pooling2d_plan).
struct PoolPlan {
  int path = SHDW_PATH_NONE, variant = 0;
  uint32_t grid = 0;
  bool want = false;
  bool chosen(int p, int v, uint32_t g) {
    path = p, variant = v, grid = g;
    return want;
  }
};

static int run_pooling(bool three_d, const int* in_shape, int pool_type, const int* kernel,
                       const int* stride, const int* pad, const int* out_shape, const float* x,
                       float* y, hipStream_t st, PoolPlan* pl) {
  const int nsp = three_d ? 3 : 2;
  if (!in_shape || !out_shape || pool_type < 0 || pool_type > 1) return SHDW_E_INVALID_ARGUMENT;
  const int rc = check_pool_dims(nsp + 2, in_shape, out_shape);
  if (rc != SHDW_OK) return rc;
  for (int k = 0; k < nsp; ++k)
    if (kernel[k] < 1 || stride[k] < 1 || pad[k] < 0) return SHDW_E_INVALID_ARGUMENT;
  int64_t out_count = 1, in_count = 1;
  for (int k = 0; k < nsp + 2; ++k) out_count *= out_shape[k], in_count *= in_shape[k];
  if (out_count == 0) return SHDW_OK;
  if (in_count == 0 || (!pl->want && (!x || !y))) return SHDW_E_INVALID_ARGUMENT;

  // One window that is exactly the unpadded plane: rows of contiguous elements.
  bool whole_plane = true;
  int64_t plane = 1;
  for (int k = 0; k < nsp; ++k) {
    whole_plane = whole_plane && out_shape[k + 2] == 1 && pad[k] == 0 && kernel[k] == in_shape[k + 2];
    plane *= in_shape[k + 2];
  }
  if (whole_plane && plane >= 8) {
    const uint32_t rows = static_cast<uint32_t>(out_count);
    if (pool_type == 0) {
      // The running maximum of a plane is Reduce's Max over a row: the same
      // std::max(v, x) walk from -FLT_MAX, which those kernels take in parallel
      // (per 51 MB: 3x3 planes 10.9 us against 19.1 us here, 7x7 10.3 / 12.9,
      // 14x14 10.1 / 16.5, 56x56 10.7 / 99).
      int rc = SHDW_OK;
      if (pl->want) {
        pl->chosen(reduce_rows_max_applies(rows, static_cast<uint32_t>(plane)) ? SHDW_PATH_POOL_PLANE_REDUCE
                                                                               : SHDW_PATH_POOL_PLANE, 0, 0);
        return SHDW_OK;
      }
      if (reduce_rows_max(rows, static_cast<uint32_t>(plane), x, y, st, &rc)) return rc;
      launch_pool_plane<true>(x, y, rows, static_cast<uint32_t>(plane), st);
    } else if (plane >= kPlaneStreamMinLen) {
      if (pl->chosen(SHDW_PATH_POOL_PLANE_STREAM, 0, 0)) return SHDW_OK;
      launch_pool_rows_stream(x, y, rows, static_cast<uint32_t>(plane), st);
    } else {
      if (pl->chosen(SHDW_PATH_POOL_PLANE, 0, 0)) return SHDW_OK;
      launch_pool_plane<false>(x, y, rows, static_cast<uint32_t>(plane), st);
    }
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
  SmallPlanesArgs sp;
  bool separable = false;
  if (!three_d && plan_small_planes(p, static_cast<int64_t>(in_shape[0]) * in_shape[1], pool_type == 0, &sp, &separable)) {
    const uint32_t grid = (sp.total_planes + sp.planes - 1) / sp.planes;
    const int k = p.kh == p.kw && (p.kh == 2 || p.kh == 3) ? p.kh : 0;
    const int unrolled = !separable ? k : (pool_type == 0 ? (sp.quads_max ? p.kw : 0) : (wide_unrolled(p.kw) ? p.kw : 0));
    if (pl->chosen(SHDW_PATH_POOL_SMALL_PLANES, (separable ? 100 : 0) + unrolled, grid)) return SHDW_OK;
    if (separable && pool_type == 0) {
      const size_t both = static_cast<size_t>(sp.planes) * (sp.plane_lds + (sp.quads_max ? 4 : 1) * sp.f_row_maxima.d) * sizeof(float);
      switch (sp.quads_max ? p.kw : 0) {  // the common square windows at a column stride of one: by quads
        case 5: pool_small_planes_kernel<true, 5, true><<<grid, kBlock, both, st>>>(x, y, sp); break;
        case 7: pool_small_planes_kernel<true, 7, true><<<grid, kBlock, both, st>>>(x, y, sp); break;
        case 9: pool_small_planes_kernel<true, 9, true><<<grid, kBlock, both, st>>>(x, y, sp); break;
        case 13: pool_small_planes_kernel<true, 13, true><<<grid, kBlock, both, st>>>(x, y, sp); break;
        default: pool_small_planes_kernel<true, 0, true><<<grid, kBlock, both, st>>>(x, y, sp);
      }
      return launch_status();
    }
    if (separable) {  // the wide average: eight spare floats behind the planes
      const size_t spare = (static_cast<size_t>(sp.planes) * sp.plane_lds + 8) * sizeof(float);
      switch (wide_unrolled(p.kw) ? p.kw : 0) {
        case 5: pool_small_planes_kernel<false, 5, true><<<grid, kBlock, spare, st>>>(x, y, sp); break;
        case 7: pool_small_planes_kernel<false, 7, true><<<grid, kBlock, spare, st>>>(x, y, sp); break;
        case 9: pool_small_planes_kernel<false, 9, true><<<grid, kBlock, spare, st>>>(x, y, sp); break;
        case 13: pool_small_planes_kernel<false, 13, true><<<grid, kBlock, spare, st>>>(x, y, sp); break;
        default: pool_small_planes_kernel<false, 0, true><<<grid, kBlock, spare, st>>>(x, y, sp);
      }
      return launch_status();
    }
    const size_t lds = static_cast<size_t>(sp.planes) * sp.plane_lds * sizeof(float);
#define SHDW_SMALL(MAXV)                                                                      \
  do {                                                                                        \
    if (k == 3) pool_small_planes_kernel<MAXV, 3><<<grid, kBlock, lds, st>>>(x, y, sp);       \
    else if (k == 2) pool_small_planes_kernel<MAXV, 2><<<grid, kBlock, lds, st>>>(x, y, sp);  \
    else pool_small_planes_kernel<MAXV, 0><<<grid, kBlock, lds, st>>>(x, y, sp);              \
  } while (0)
    if (pool_type == 0) SHDW_SMALL(true); else SHDW_SMALL(false);
#undef SHDW_SMALL
    return launch_status();
  }
  if (!three_d && pool_halve_applies(p, x, y, pl->want)) {
    const uint32_t tasks = n_out / 2;
    const uint32_t grid = (tasks + kHalveLanes - 1) / kHalveLanes;
    if (pl->chosen(SHDW_PATH_POOL_HALVE, p.kh, grid)) return SHDW_OK;
    HalveArgs h;
    h.in_h = p.in_h, h.in_w = p.in_w, h.out_h = p.out_h, h.out_w = p.out_w;
    h.f_pairs = make_fastdiv(static_cast<uint32_t>(p.out_w / 2));
    h.f_out_h = make_fastdiv(static_cast<uint32_t>(p.out_h));
#define SHDW_HALVE(KV, PV)                                                                     \
  do {                                                                                         \
    if (pool_type == 0) pool_halve_kernel<true, KV, PV><<<grid, kHalveLanes, 0, st>>>(x, y, tasks, h); \
    else pool_halve_kernel<false, KV, PV><<<grid, kHalveLanes, 0, st>>>(x, y, tasks, h);       \
  } while (0)
    if (p.kh == 2) SHDW_HALVE(2, 0);
    else if (p.pw == 0) SHDW_HALVE(3, 0);
    else SHDW_HALVE(3, 1);
#undef SHDW_HALVE
    return launch_status();
  }
  if (!three_d && pool_same_applies(p, x, y, pl->want)) {
    const uint32_t tasks = n_out / 4;
    const uint32_t grid = (tasks + kHalveLanes - 1) / kHalveLanes;
    if (pl->chosen(SHDW_PATH_POOL_SAME, 3, grid)) return SHDW_OK;
    HalveArgs h;
    h.in_h = p.in_h, h.in_w = p.in_w, h.out_h = p.out_h, h.out_w = p.out_w;
    h.f_pairs = make_fastdiv(static_cast<uint32_t>(p.in_w / 4));
    h.f_out_h = make_fastdiv(static_cast<uint32_t>(p.out_h));
    if (pool_type == 0) pool_same_kernel<true><<<grid, kHalveLanes, 0, st>>>(x, y, tasks, h);
    else pool_same_kernel<false><<<grid, kHalveLanes, 0, st>>>(x, y, tasks, h);
    return launch_status();
  }
  BandArgs a;
  if (!three_d && plan_pool_band(p, kPoolBandOutputs, &a)) {
    const int64_t groups = static_cast<int64_t>(in_shape[0]) * in_shape[1] * a.bands_per_plane;
    const size_t lds = (static_cast<size_t>(a.tile_rows + 1) * a.pitch + 8) * sizeof(float);  // eight spare: band_windows_wide
    if (groups <= INT32_MAX) {
      a.total_bands = static_cast<uint32_t>(groups);
      // Enough workgroups to fill the chip a few times over, then longer walks.
      uint32_t per = a.total_bands / kBandGroupsWanted;
      per = per < 1 ? 1 : (per > kBandMaxWalk ? kBandMaxWalk : per);
      a.bands_per_group = per;
      const uint32_t g = (a.total_bands + per - 1) / per;
      const bool pipe = p.in_w % 4 == 0 && aligned16(x);
      const int k = p.kh == p.kw && (p.kh == 2 || p.kh == 3 || (p.kh == 5 && a.wide)) ? p.kh : 0;
      const int vecs = (a.tile_rows * p.in_w / 4 + kBlock - 1) / kBlock;  // per lane and band
      const int regs = !pipe ? 0 : (vecs <= 2 ? 2 : (vecs <= 3 ? 3 : (vecs <= 4 ? 4 : (vecs <= 6 ? 6 : 8))));
      if (pl->chosen(SHDW_PATH_POOL_BAND, 100 * regs + k, g)) return SHDW_OK;
#define SHDW_LAUNCH_BAND(MAXV, KV)                                                              \
  do {                                                                                           \
    switch (regs) {                                                                              \
      case 0: pool_band_kernel<MAXV, KV, 0><<<g, kBlock, lds, st>>>(x, y, a); break;             \
      case 2: pool_band_kernel<MAXV, KV, 2><<<g, kBlock, lds, st>>>(x, y, a); break;             \
      case 3: pool_band_kernel<MAXV, KV, 3><<<g, kBlock, lds, st>>>(x, y, a); break;             \
      case 4: pool_band_kernel<MAXV, KV, 4><<<g, kBlock, lds, st>>>(x, y, a); break;             \
      case 6: pool_band_kernel<MAXV, KV, 6><<<g, kBlock, lds, st>>>(x, y, a); break;             \
      default: pool_band_kernel<MAXV, KV, 8><<<g, kBlock, lds, st>>>(x, y, a); break;            \
    }                                                                                            \
  } while (0)
      if (pool_type == 0) {
        if (k == 3)
          SHDW_LAUNCH_BAND(true, 3);
        else if (k == 5)
          SHDW_LAUNCH_BAND(true, 5);
        else if (k == 2)
          SHDW_LAUNCH_BAND(true, 2);
        else
          SHDW_LAUNCH_BAND(true, 0);
      } else {
        if (k == 3)
          SHDW_LAUNCH_BAND(false, 3);
        else if (k == 5)
          SHDW_LAUNCH_BAND(false, 5);
        else if (k == 2)
          SHDW_LAUNCH_BAND(false, 2);
        else
          SHDW_LAUNCH_BAND(false, 0);
      }
#undef SHDW_LAUNCH_BAND
      return launch_status();
    }
  }
  const uint32_t grid = grid_for(n_out);
  if (pl->chosen(SHDW_PATH_POOL_WINDOW, 0, grid)) return SHDW_OK;
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

int shdw_hip_batch_norm_scale(int n, int channel, int inner_num, const float* x, const float* mean,
                              const float* variance, float scale_factor, float eps, const float* scale,
                              const float* bias, int relu, float* y, void* stream) {
  if (n < 0 || channel < 1 || inner_num < 1 || (!scale && !bias)) return SHDW_E_INVALID_ARGUMENT;
  if (n == 0) return SHDW_OK;
  if (!x || !mean || !variance || !y) return SHDW_E_INVALID_ARGUMENT;
  const FastDiv fc = make_fastdiv(static_cast<uint32_t>(channel));
  hipStream_t st = static_cast<hipStream_t>(stream);
  const uint32_t count = static_cast<uint32_t>(n), inner = static_cast<uint32_t>(inner_num);
#define SHDW_BNS(S, B, R)                                                                       \
  do {                                                                                          \
    BatchNormScaleRows<S, B, R> p{mean, variance, scale, bias, scale_factor, eps, fc};          \
    return launch_rows(p, count, inner, x, nullptr, y, st);                                     \
  } while (0)
  if (scale && bias) {
    if (relu) SHDW_BNS(true, true, true); else SHDW_BNS(true, true, false);
  } else if (scale) {
    if (relu) SHDW_BNS(true, false, true); else SHDW_BNS(true, false, false);
  } else {
    if (relu) SHDW_BNS(false, true, true); else SHDW_BNS(false, true, false);
  }
#undef SHDW_BNS
}

int shdw_hip_pooling2d(const int* in_shape, int pool_type, int kernel_h, int kernel_w,
                       int stride_h, int stride_w, int pad_h, int pad_w, const int* out_shape,
                       const float* x, float* y, void* stream) {
  const int kernel[2] = {kernel_h, kernel_w}, stride[2] = {stride_h, stride_w},
            pad[2] = {pad_h, pad_w};
  PoolPlan pl;
  return run_pooling(false, in_shape, pool_type, kernel, stride, pad, out_shape, x, y,
                     static_cast<hipStream_t>(stream), &pl);
}

int shdw_hip_pooling2d_plan(const int* in_shape, int pool_type, int kernel_h, int kernel_w,
                            int stride_h, int stride_w, int pad_h, int pad_w, const int* out_shape,
                            int* path, int* variant, unsigned* grid) {
  const int kernel[2] = {kernel_h, kernel_w}, stride[2] = {stride_h, stride_w},
            pad[2] = {pad_h, pad_w};
  PoolPlan pl;
  pl.want = true;
  const int rc = run_pooling(false, in_shape, pool_type, kernel, stride, pad, out_shape, nullptr, nullptr,
                             nullptr, &pl);
  if (rc != SHDW_OK) return rc;
  if (path) *path = pl.path;
  if (variant) *variant = pl.variant;
  if (grid) *grid = pl.grid;
  return SHDW_OK;
}

int shdw_hip_pooling3d(const int* in_shape, int pool_type, int kernel_d, int kernel_h,
                       int kernel_w, int stride_d, int stride_h, int stride_w, int pad_d,
                       int pad_h, int pad_w, const int* out_shape, const float* x, float* y,
                       void* stream) {
  const int kernel[3] = {kernel_d, kernel_h, kernel_w}, stride[3] = {stride_d, stride_h, stride_w},
            pad[3] = {pad_d, pad_h, pad_w};
  PoolPlan pl;
  return run_pooling(true, in_shape, pool_type, kernel, stride, pad, out_shape, x, y,
                     static_cast<hipStream_t>(stream), &pl);
}

}  // extern "C"
