// Softmax and Normalize: x viewed as [outer][dim][inner]; a statistic is folded
// over `dim` for every (outer, inner) column and then applied to the column.
//
// Shadow folds each column front to back (an fp32 running sum for Softmax, an
// fp64 one for Normalize); both are order-dependent, so a column is always
// folded by ONE lane in that order and the results match bit for bit.  Two
// layouts keep the global accesses coalesced around that constraint:
//   * columns : inner >= 64 (or a slab too large for LDS).  Lane = column,
//               neighbouring lanes read neighbouring addresses.
//   * slab    : inner < 64.  One workgroup per outer index copies its
//               contiguous [dim][inner] slab into LDS with all lanes, `inner`
//               lanes fold the columns out of LDS, all lanes write back.
// The elementwise parts (exp, divide) are done by every lane in both layouts.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cfloat>

#include "../../include/shadow_hip.h"
#include "device_common.h"
#include "launch.h"
#include "libm_exact.h"

#pragma clang fp contract(off)

namespace shdw {

constexpr int kSlabMaxFloats = 15 * 1024;  // slab + per-column statistics, 60 KB of LDS: two workgroups per CU (whole
                                           // slabs of up to 156 KB, one workgroup per CU, ran at half the speed of the
                                           // chunked kernels that take the larger ones now)

// std::max(a, b) of libstdc++: b only when a < b.
SHDW_DEVICE float std_max(float a, float b) { return a < b ? b : a; }

// ---------------------------------------------------------------------------
// Softmax (shadow/operators/kernels/softmax.cpp:10-42)
// ---------------------------------------------------------------------------
// Any column length: a lane walks its column three times (max, exp and running
// sum, divide).  kColumnBatch loads are issued before the first is consumed so
// that a lane keeps that many requests in flight, and a workgroup is a single
// wave: long columns mean few of them, and 64 columns per workgroup spread them
// over four times as many CUs.  Neighbouring waves share the cache lines their
// 256-byte rows straddle, hence the XCD-contiguous order.  Every fold keeps the
// reference's index order.
constexpr int kColumnBatch = 16;

__global__ __launch_bounds__(kWave) void softmax_columns_kernel(const float* x, float* y,
                                                                 uint32_t columns, uint32_t dim,
                                                                 FastDiv f_inner) {
  __shared__ uint64_t tab[32];
  if (threadIdx.x < 32) tab[threadIdx.x] = libm::kExp2fTab[threadIdx.x];
  __syncthreads();
  const uint32_t i = xcd_contiguous(blockIdx.x, gridDim.x) * kWave + threadIdx.x;
  if (i >= columns) return;
  uint32_t n, s;
  fd_divmod(i, f_inner, n, s);
  const uint32_t inner = f_inner.d;
  const uint64_t base = static_cast<uint64_t>(n) * dim * inner + s;
  const float* xc = x + base;
  float* yc = y + base;
  float max_val = -FLT_MAX;
  for (uint32_t c0 = 0; c0 < dim; c0 += kColumnBatch) {
    float v[kColumnBatch];
#pragma unroll
    for (int u = 0; u < kColumnBatch; ++u)
      if (c0 + u < dim) v[u] = xc[static_cast<uint64_t>(c0 + u) * inner];
#pragma unroll
    for (int u = 0; u < kColumnBatch; ++u)
      if (c0 + u < dim) max_val = std_max(v[u], max_val);
  }
  float sum = 0.f;
  // Whole batches run without the `c < dim` test: a tested row is a basic block
  // of its own and the exp chains of different blocks are not interleaved.
  uint32_t c0 = 0;
  for (; c0 + kColumnBatch <= dim; c0 += kColumnBatch) {
    float v[kColumnBatch];
#pragma unroll
    for (int u = 0; u < kColumnBatch; ++u) v[u] = xc[static_cast<uint64_t>(c0 + u) * inner];
#pragma unroll
    for (int u = 0; u < kColumnBatch; ++u) v[u] = libm::exact_expf(v[u] - max_val, tab);
#pragma unroll
    for (int u = 0; u < kColumnBatch; ++u) {
      yc[static_cast<uint64_t>(c0 + u) * inner] = v[u];
      sum += v[u];
    }
  }
  if (c0 < dim) {
    float v[kColumnBatch];
#pragma unroll
    for (int u = 0; u < kColumnBatch; ++u)
      if (c0 + u < dim) v[u] = xc[static_cast<uint64_t>(c0 + u) * inner];
#pragma unroll
    for (int u = 0; u < kColumnBatch; ++u) {
      if (c0 + u < dim) {
        const float e = libm::exact_expf(v[u] - max_val, tab);
        yc[static_cast<uint64_t>(c0 + u) * inner] = e;
        sum += e;
      }
    }
  }
  for (c0 = 0; c0 + kColumnBatch <= dim; c0 += kColumnBatch) {
    float v[kColumnBatch];
#pragma unroll
    for (int u = 0; u < kColumnBatch; ++u) v[u] = yc[static_cast<uint64_t>(c0 + u) * inner];
#pragma unroll
    for (int u = 0; u < kColumnBatch; ++u) v[u] = v[u] / sum;
#pragma unroll
    for (int u = 0; u < kColumnBatch; ++u)
      __builtin_nontemporal_store(v[u], yc + static_cast<uint64_t>(c0 + u) * inner);
  }
  if (c0 < dim) {
    float v[kColumnBatch];
#pragma unroll
    for (int u = 0; u < kColumnBatch; ++u)
      if (c0 + u < dim) v[u] = yc[static_cast<uint64_t>(c0 + u) * inner];
#pragma unroll
    for (int u = 0; u < kColumnBatch; ++u)
      if (c0 + u < dim) __builtin_nontemporal_store(v[u] / sum, yc + static_cast<uint64_t>(c0 + u) * inner);
  }
}

// Same layout for dim <= DMAX: the column lives in registers, so x is read once
// and y written once, and all of a lane's loads are in flight together.
// The first DFULL rows exist for every column this instance is launched for
// (DFULL < dim <= DMAX) and run as straight-line code, which lets the compiler
// interleave the exp chains of neighbouring rows; only the last DMAX - DFULL
// rows carry the `c < dim` test (each guarded row is a basic block of its own).
template <int DMAX, int DFULL>
__global__ __launch_bounds__(kBlock) void softmax_columns_reg_kernel(const float* x, float* y,
                                                                      uint32_t columns,
                                                                      uint32_t dim,
                                                                      FastDiv f_inner) {
  __shared__ uint64_t tab[32];
  if (threadIdx.x < 32) tab[threadIdx.x] = libm::kExp2fTab[threadIdx.x];
  __syncthreads();
  const uint32_t i = xcd_contiguous(blockIdx.x, gridDim.x) * kBlock + threadIdx.x;  // neighbours share straddled lines
  if (i >= columns) return;
  uint32_t n, s;
  fd_divmod(i, f_inner, n, s);
  const uint32_t inner = f_inner.d;
  const uint64_t base = static_cast<uint64_t>(n) * dim * inner + s;
  const float* xc = x + base;
  float* yc = y + base;
  float v[DMAX];
#pragma unroll
  for (int c = 0; c < DMAX; ++c)
    if (c < DFULL || c < dim) v[c] = __builtin_nontemporal_load(xc + static_cast<uint64_t>(c) * inner);
  float max_val = -FLT_MAX;
#pragma unroll
  for (int c = 0; c < DMAX; ++c)
    if (c < DFULL || c < dim) max_val = std_max(v[c], max_val);
  float sum = 0.f;
#pragma unroll
  for (int c = 0; c < DMAX; ++c) {
    if (c < DFULL || c < dim) {
      v[c] = libm::exact_expf(v[c] - max_val, tab);
      sum += v[c];
    }
  }
#pragma unroll
  for (int c = 0; c < DMAX; ++c)
    if (c < DFULL || c < dim) __builtin_nontemporal_store(v[c] / sum, yc + static_cast<uint64_t>(c) * inner);
}

// Copy a contiguous slab into LDS through `f`: 128-bit loads, eight in flight per
// lane, where the slab starts on a 16-byte boundary, single floats elsewhere.
constexpr int kSlabBatch = 8;
template <class F>
SHDW_DEVICE void stage_slab(float* lds, const float* xs, uint32_t slab, F f) {
  uint32_t done = 0;
  if ((reinterpret_cast<uintptr_t>(xs) & 15) == 0) {
    const v4f* x4 = reinterpret_cast<const v4f*>(xs);
    v4f* l4 = reinterpret_cast<v4f*>(lds);
    const uint32_t quads = slab / 4;
    for (uint32_t t0 = 0; t0 < quads; t0 += kSlabBatch * kBlock) {
      v4f reg[kSlabBatch];
#pragma unroll
      for (int k = 0; k < kSlabBatch; ++k) {
        const uint32_t t = t0 + k * kBlock + threadIdx.x;
        if (t < quads) reg[k] = x4[t];
      }
#pragma unroll
      for (int k = 0; k < kSlabBatch; ++k) {
        const uint32_t t = t0 + k * kBlock + threadIdx.x;
        if (t < quads) l4[t] = v4f{f(reg[k][0]), f(reg[k][1]), f(reg[k][2]), f(reg[k][3])};
      }
    }
    done = 4 * quads;
  }
  for (uint32_t t0 = done; t0 < slab; t0 += kSlabBatch * kBlock) {
    float reg[kSlabBatch];
#pragma unroll
    for (int k = 0; k < kSlabBatch; ++k) {
      const uint32_t t = t0 + k * kBlock + threadIdx.x;
      if (t < slab) reg[k] = xs[t];
    }
#pragma unroll
    for (int k = 0; k < kSlabBatch; ++k) {
      const uint32_t t = t0 + k * kBlock + threadIdx.x;
      if (t < slab) lds[t] = f(reg[k]);
    }
  }
}

// Rows 0 .. n-1 of a column in LDS (`stride` floats apart) handed to `fold` in
// index order, sixteen reads in flight and then their folds.  One set of
// registers: two sets taking turns (the next batch on its way while this one is
// folded) had the compiler copy one set into the other every turn, and the
// walking wave, which is often alone on its SIMD, pays every instruction it
// issues; the LDS latency exposed between batches costs less (7-12 % on the
// walk-bound shapes, columns of 1000 and 4096).
template <class F>
SHDW_DEVICE void walk_column(const float* col, uint32_t stride, uint32_t n, F&& fold) {
  constexpr int kBatch = 16;
  uint32_t c = 0;
  for (; c + kBatch <= n; c += kBatch) {
    const float* at = col + c * stride;
    float v[kBatch];
#pragma unroll
    for (int k = 0; k < kBatch; ++k) v[k] = at[k * stride];
#pragma unroll
    for (int k = 0; k < kBatch; ++k) fold(v[k]);
  }
  for (; c < n; ++c) fold(col[c * stride]);
}

// The same for the strides the tall kernels have (16, 32 or 64 floats): with the stride a constant the
// sixteen reads of a batch share one address register and differ in their immediate offsets, one
// instruction less per element for the walking lane.
template <class F>
SHDW_DEVICE void walk_column_tile(const float* col, uint32_t width, uint32_t n, F&& fold) {
  if (width == 16) walk_column(col, 16, n, fold);
  else if (width == 32) walk_column(col, 32, n, fold);
  else walk_column(col, 64, n, fold);
}

// ... and for the small position counts of the slab kernels (a column per position, `inner` floats apart).
template <class F>
SHDW_DEVICE void walk_column_inner(const float* col, uint32_t inner, uint32_t n, F&& fold) {
  switch (inner) {
    case 1: walk_column(col, 1, n, fold); break;
    case 2: walk_column(col, 2, n, fold); break;
    case 3: walk_column(col, 3, n, fold); break;
    case 4: walk_column(col, 4, n, fold); break;
    case 7: walk_column(col, 7, n, fold); break;
    case 8: walk_column(col, 8, n, fold); break;
    case 16: walk_column(col, 16, n, fold); break;
    case 49: walk_column(col, 49, n, fold); break;
    default: walk_column(col, inner, n, fold);
  }
}

// Any-order maximum over the workgroup.  Only valid where the order cannot
// show: see softmax_slab_kernel.
SHDW_DEVICE float block_max_any_order(float m, float* scratch4) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) m = std_max(__shfl_xor(m, off), m);
  if ((threadIdx.x & 63) == 0) scratch4[threadIdx.x >> 6] = m;
  __syncthreads();
  m = scratch4[0];
#pragma unroll
  for (int w = 1; w < kBlock / kWave; ++w) m = std_max(scratch4[w], m);
  return m;
}

// Front-to-back sum of lds[0..n) by the calling lane, 128-bit LDS reads.
template <class ACC>
SHDW_DEVICE ACC sequential_sum(const float* lds, uint32_t n) {
  ACC sum = 0;
  const v4f* l4 = reinterpret_cast<const v4f*>(lds);
  const uint32_t q = n / 4;
#pragma unroll 8
  for (uint32_t c = 0; c < q; ++c) {
    const v4f v = l4[c];
    sum += static_cast<ACC>(v[0]);
    sum += static_cast<ACC>(v[1]);
    sum += static_cast<ACC>(v[2]);
    sum += static_cast<ACC>(v[3]);
  }
  for (uint32_t c = 4 * q; c < n; ++c) sum += static_cast<ACC>(lds[c]);
  return sum;
}

// inner == 1 takes the maximum with all lanes in any order.  That is exact:
// the value of the maximum does not depend on the order unless the column
// holds a NaN, and then every output is NaN whatever maximum was used (the
// NaN's own term poisons the sum); the sign of a zero maximum cannot reach the
// output because exp(+-0) = 1 and x - (+-0) = x for x != 0.
__global__ __launch_bounds__(kBlock) void softmax_slab_kernel(const float* x, float* y,
                                                               uint32_t dim, FastDiv f_inner) {
  extern __shared__ __align__(16) float lds[];
  __shared__ uint64_t tab[32];
  __shared__ float wave_max[kBlock / kWave];
  __shared__ float part[kBlock];
  const uint32_t inner = f_inner.d;
  const uint32_t slab = dim * inner;
  float* stat = lds + slab;
  const float* xs = x + static_cast<uint64_t>(blockIdx.x) * slab;
  float* ys = y + static_cast<uint64_t>(blockIdx.x) * slab;
  if (threadIdx.x < 32) tab[threadIdx.x] = libm::kExp2fTab[threadIdx.x];
  stage_slab(lds, xs, slab, [](float v) { return v; });
  __syncthreads();
  if (inner == 1) {
    float m = -FLT_MAX;
    for (uint32_t t = threadIdx.x; t < slab; t += kBlock) m = std_max(lds[t], m);
    m = block_max_any_order(m, wave_max);
    for (uint32_t t = threadIdx.x; t < slab; t += kBlock) lds[t] = libm::exact_expf(lds[t] - m, tab);
    __syncthreads();
    if (threadIdx.x == 0) stat[0] = sequential_sum<float>(lds, slab);
    __syncthreads();
    const float sum = stat[0];
    for (uint32_t t = threadIdx.x; t < slab; t += kBlock) ys[t] = lds[t] / sum;
    return;
  }
  // inner < 64 here.  The maxima in any order as well (a NaN in a column makes all
  // of that column NaN whatever maximum was used): 256 / inner lanes per column
  // take every lanes-th row, lane s folds their partials.
  const uint32_t lanes = kBlock / inner;
  {
    uint32_t g, s;
    fd_divmod(threadIdx.x, f_inner, g, s);
    if (g < lanes) {
      float max_val = -FLT_MAX;
      const uint32_t n = g < dim ? (dim - g + lanes - 1) / lanes : 0;
      walk_column(lds + g * inner + s, lanes * inner, n, [&](float v) { max_val = std_max(v, max_val); });
      part[threadIdx.x] = max_val;
    }
  }
  __syncthreads();
  if (threadIdx.x < inner) {
    float max_val = -FLT_MAX;
    for (uint32_t g = 0; g < lanes; ++g) max_val = std_max(part[g * inner + threadIdx.x], max_val);
    stat[threadIdx.x] = max_val;
  }
  __syncthreads();
  for (uint32_t t = threadIdx.x; t < slab; t += kBlock) {
    const uint32_t s = t - fd_div(t, f_inner) * inner;
    lds[t] = libm::exact_expf(lds[t] - stat[s], tab);
  }
  __syncthreads();
  if (threadIdx.x < inner) {
    float sum = 0.f;
    walk_column_inner(lds + threadIdx.x, inner, dim, [&](float v) { sum += v; });
    stat[threadIdx.x] = sum;
  }
  __syncthreads();
  for (uint32_t t = threadIdx.x; t < slab; t += kBlock) {
    const uint32_t s = t - fd_div(t, f_inner) * inner;
    ys[t] = lds[t] / stat[s];
  }
}

// ---------------------------------------------------------------------------
// Normalize (shadow/operators/kernels/normalize.cpp:10-43)
//   PMODE 1: sum |x|          2: sqrt(sum |x|^2)      0: (sum |x|^p)^(1/p)
// SSDNormalize over channels (shadow/operators/kernels/ssd_normalize.cpp:14-28,
// squares from Blas::Square, ssd_normalize.hpp:47) shares the kernels:
//   PMODE 3: (float) sqrt((double) sum x^2 + eps) in fp64, no lower bound, and
//            the optional scale of ssd_normalize.hpp:68-80 applied to the quotient.
// ---------------------------------------------------------------------------
enum SsdScale { kSsdNoScale = 0, kSsdSharedScale = 1, kSsdChannelScale = 2 };

// SM is kSsdNoScale for Normalize; c is the channel (the position in the column).
template <int SM>
SHDW_DEVICE float ssd_scaled(float v, const float* scale, uint32_t c) {
  if (SM == kSsdSharedScale) return v * scale[0];
  if (SM == kSsdChannelScale) return v * scale[c];
  return v;
}

template <int PMODE>
SHDW_DEVICE double norm_term(float v, float p) {
  const float a = __builtin_fabsf(v);
  if (PMODE == 1) return static_cast<double>(a);
  if (PMODE == 2) {
    const float sq = a * a;  // fp32 product, widened afterwards
    return static_cast<double>(sq);
  }
  if (PMODE == 3) {
    const float sq = v * v;
    return static_cast<double>(sq);
  }
  return static_cast<double>(libm::exact_powf(a, p, libm::kExp2fTab));
}

template <int PMODE>
SHDW_DEVICE float norm_finish(double acc, float p, float eps) {
  float val;
  if (PMODE == 3) return static_cast<float>(__builtin_sqrt(acc + static_cast<double>(eps)));
  if (PMODE == 1) {
    val = static_cast<float>(acc);
  } else if (PMODE == 2) {
    val = __builtin_sqrtf(static_cast<float>(acc));
  } else {
    const float inv = 1.f / p;
    val = libm::exact_powf(static_cast<float>(acc), inv, libm::kExp2fTab);
  }
  return std_max(val, eps);
}

// Any column length: a lane walks its column twice (the second time from cache
// where the column still is there), launched like softmax_columns_kernel.

template <int PMODE, int SM = kSsdNoScale>
__global__ __launch_bounds__(kWave) void normalize_columns_kernel(const float* x, float* y,
                                                                   uint32_t columns, uint32_t dim,
                                                                   FastDiv f_inner, float p,
                                                                   float eps,
                                                                   const float* scale = nullptr) {
  const uint32_t i = xcd_contiguous(blockIdx.x, gridDim.x) * kWave + threadIdx.x;
  if (i >= columns) return;
  uint32_t n, s;
  fd_divmod(i, f_inner, n, s);
  const uint32_t inner = f_inner.d;
  const uint64_t base = static_cast<uint64_t>(n) * dim * inner + s;
  const float* xc = x + base;
  float* yc = y + base;
  double acc = 0;
  for (uint32_t c0 = 0; c0 < dim; c0 += kColumnBatch) {
    float v[kColumnBatch];
#pragma unroll
    for (int u = 0; u < kColumnBatch; ++u)
      if (c0 + u < dim) v[u] = xc[static_cast<uint64_t>(c0 + u) * inner];
#pragma unroll
    for (int u = 0; u < kColumnBatch; ++u)
      if (c0 + u < dim) acc += norm_term<PMODE>(v[u], p);
  }
  const float div = norm_finish<PMODE>(acc, p, eps);
  uint32_t c0 = 0;
  for (; c0 + kColumnBatch <= dim; c0 += kColumnBatch) {  // whole batches: no per-row test between the divisions
    float v[kColumnBatch];
#pragma unroll
    for (int u = 0; u < kColumnBatch; ++u) v[u] = xc[static_cast<uint64_t>(c0 + u) * inner];
#pragma unroll
    for (int u = 0; u < kColumnBatch; ++u) v[u] = ssd_scaled<SM>(v[u] / div, scale, c0 + u);
#pragma unroll
    for (int u = 0; u < kColumnBatch; ++u)
      __builtin_nontemporal_store(v[u], yc + static_cast<uint64_t>(c0 + u) * inner);
  }
  if (c0 < dim) {
    float v[kColumnBatch];
#pragma unroll
    for (int u = 0; u < kColumnBatch; ++u)
      if (c0 + u < dim) v[u] = xc[static_cast<uint64_t>(c0 + u) * inner];
#pragma unroll
    for (int u = 0; u < kColumnBatch; ++u)
      if (c0 + u < dim)
        __builtin_nontemporal_store(ssd_scaled<SM>(v[u] / div, scale, c0 + u), yc + static_cast<uint64_t>(c0 + u) * inner);
  }
}

template <int PMODE, int DMAX, int SM = kSsdNoScale>
__global__ __launch_bounds__(kBlock) void normalize_columns_reg_kernel(const float* x, float* y,
                                                                        uint32_t columns,
                                                                        uint32_t dim,
                                                                        FastDiv f_inner, float p,
                                                                        float eps,
                                                                        const float* scale = nullptr) {
  const uint32_t i = xcd_contiguous(blockIdx.x, gridDim.x) * kBlock + threadIdx.x;  // neighbours share straddled lines
  if (i >= columns) return;
  uint32_t n, s;
  fd_divmod(i, f_inner, n, s);
  const uint32_t inner = f_inner.d;
  const uint64_t base = static_cast<uint64_t>(n) * dim * inner + s;
  const float* xc = x + base;
  float* yc = y + base;
  float v[DMAX];
#pragma unroll
  for (int c = 0; c < DMAX; ++c)
    if (c < dim) v[c] = __builtin_nontemporal_load(xc + static_cast<uint64_t>(c) * inner);
  double acc = 0;
#pragma unroll
  for (int c = 0; c < DMAX; ++c)
    if (c < dim) acc += norm_term<PMODE>(v[c], p);
  const float div = norm_finish<PMODE>(acc, p, eps);
#pragma unroll
  for (int c = 0; c < DMAX; ++c)
    if (c < dim)
      __builtin_nontemporal_store(ssd_scaled<SM>(v[c] / div, scale, c), yc + static_cast<uint64_t>(c) * inner);
}

// ---------------------------------------------------------------------------
// Columns of up to DMAX elements over four and more positions: a lane takes four
// neighbouring positions of one slab, every row of them as one 128-bit access on
// any dword address, and keeps its four columns in registers.  One division per
// lane in place of four, a quarter of the memory instructions of the
// column-per-lane kernels above (softmax over [2048,2,3136]: 38 us per 51 MB with
// a column per lane).  The last quad of a slab holds inner % 4 positions where
// that is not zero and moves float by float.
// ---------------------------------------------------------------------------
struct QuadLane {
  uint64_t base;  // first row, first position
  uint32_t n;     // positions that exist: 1 .. 4
};

SHDW_DEVICE QuadLane quad_lane(uint32_t i, FastDiv f_quads, uint32_t dim, uint32_t inner) {
  uint32_t slab, quad;
  fd_divmod(i, f_quads, slab, quad);
  QuadLane q;
  q.base = static_cast<uint64_t>(slab) * dim * inner + 4 * quad;
  q.n = min(4u, inner - 4 * quad);
  return q;
}

template <int DMAX>
SHDW_DEVICE void quad_load(const float* xc, const QuadLane& q, uint32_t dim, uint32_t inner, v4f (&v)[DMAX]) {
  if (q.n == 4) {
#pragma unroll
    for (int c = 0; c < DMAX; ++c)
      if (c < dim) v[c] = load4_stream_any(xc + static_cast<uint64_t>(c) * inner);
  } else {
#pragma unroll
    for (int c = 0; c < DMAX; ++c) {
      if (c < dim) {
        v[c] = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int k = 0; k < 3; ++k)
          if (static_cast<uint32_t>(k) < q.n) v[c][k] = __builtin_nontemporal_load(xc + static_cast<uint64_t>(c) * inner + k);
      }
    }
  }
}

SHDW_DEVICE void quad_store(float* at, const QuadLane& q, const v4f& r) {
  if (q.n == 4) {
    store4_stream_any(at, r);
  } else {
#pragma unroll
    for (int k = 0; k < 3; ++k)
      if (static_cast<uint32_t>(k) < q.n) __builtin_nontemporal_store(r[k], at + k);
  }
}

template <int DMAX>
__global__ __launch_bounds__(kBlock) void softmax_quads_reg_kernel(const float* x, float* y, uint32_t quads,
                                                                    uint32_t dim, uint32_t inner, FastDiv f_quads) {
  __shared__ uint64_t tab[32];
  if (threadIdx.x < 32) tab[threadIdx.x] = libm::kExp2fTab[threadIdx.x];
  __syncthreads();
  const uint32_t i = xcd_contiguous(blockIdx.x, gridDim.x) * kBlock + threadIdx.x;  // neighbours share straddled lines
  if (i >= quads) return;
  const QuadLane q = quad_lane(i, f_quads, dim, inner);
  v4f v[DMAX];
  quad_load<DMAX>(x + q.base, q, dim, inner, v);
  v4f max_val = {-FLT_MAX, -FLT_MAX, -FLT_MAX, -FLT_MAX};
#pragma unroll
  for (int c = 0; c < DMAX; ++c) {
    if (c < dim) {
#pragma unroll
      for (int k = 0; k < 4; ++k) max_val[k] = std_max(v[c][k], max_val[k]);
    }
  }
  v4f sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int c = 0; c < DMAX; ++c) {
    if (c < dim) {
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        v[c][k] = libm::exact_expf(v[c][k] - max_val[k], tab);
        sum[k] += v[c][k];
      }
    }
  }
#pragma unroll
  for (int c = 0; c < DMAX; ++c) {
    if (c < dim) {
      v4f r;
#pragma unroll
      for (int k = 0; k < 4; ++k) r[k] = v[c][k] / sum[k];
      quad_store(y + q.base + static_cast<uint64_t>(c) * inner, q, r);
    }
  }
}

template <int PMODE, int DMAX, int SM>
__global__ __launch_bounds__(kBlock) void normalize_quads_reg_kernel(const float* x, float* y, uint32_t quads,
                                                                      uint32_t dim, uint32_t inner, FastDiv f_quads,
                                                                      float p, float eps, const float* scale) {
  const uint32_t i = xcd_contiguous(blockIdx.x, gridDim.x) * kBlock + threadIdx.x;
  if (i >= quads) return;
  const QuadLane q = quad_lane(i, f_quads, dim, inner);
  v4f v[DMAX];
  quad_load<DMAX>(x + q.base, q, dim, inner, v);
  double acc[4] = {0, 0, 0, 0};
#pragma unroll
  for (int c = 0; c < DMAX; ++c) {
    if (c < dim) {
#pragma unroll
      for (int k = 0; k < 4; ++k) acc[k] += norm_term<PMODE>(v[c][k], p);
    }
  }
  float div[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) div[k] = norm_finish<PMODE>(acc[k], p, eps);
#pragma unroll
  for (int c = 0; c < DMAX; ++c) {
    if (c < dim) {
      v4f r;
#pragma unroll
      for (int k = 0; k < 4; ++k) r[k] = ssd_scaled<SM>(v[c][k] / div[k], scale, c);
      quad_store(y + q.base + static_cast<uint64_t>(c) * inner, q, r);
    }
  }
}

// The slab in LDS holds the per-element terms (|x|, |x|^2 or |x|^p, computed by
// all lanes); x itself is read again for the division, from L2.
template <int PMODE, int SM = kSsdNoScale>
__global__ __launch_bounds__(kBlock) void normalize_slab_kernel(const float* x, float* y,
                                                                 uint32_t dim, FastDiv f_inner,
                                                                 float p, float eps,
                                                                 const float* scale = nullptr) {
  extern __shared__ __align__(16) float lds[];
  const uint32_t inner = f_inner.d;
  const uint32_t slab = dim * inner;
  float* stat = lds + slab;
  const float* xs = x + static_cast<uint64_t>(blockIdx.x) * slab;
  float* ys = y + static_cast<uint64_t>(blockIdx.x) * slab;
  stage_slab(lds, xs, slab, [p](float v) { return static_cast<float>(norm_term<PMODE>(v, p)); });
  __syncthreads();
  if (inner == 1) {
    if (threadIdx.x == 0) stat[0] = norm_finish<PMODE>(sequential_sum<double>(lds, slab), p, eps);
  } else {
    if (threadIdx.x < inner) {  // inner < 64 here
      double acc = 0;
      walk_column_inner(lds + threadIdx.x, inner, dim, [&](float v) { acc += static_cast<double>(v); });
      stat[threadIdx.x] = norm_finish<PMODE>(acc, p, eps);
    }
  }
  __syncthreads();
  for (uint32_t t0 = 0; t0 < slab; t0 += kSlabBatch * kBlock) {
    float reg[kSlabBatch];
#pragma unroll
    for (int k = 0; k < kSlabBatch; ++k) {
      const uint32_t t = t0 + k * kBlock + threadIdx.x;
      if (t < slab) reg[k] = xs[t];
    }
#pragma unroll
    for (int k = 0; k < kSlabBatch; ++k) {
      const uint32_t t = t0 + k * kBlock + threadIdx.x;
      if (t < slab) {
        const uint32_t c = fd_div(t, f_inner);
        ys[t] = ssd_scaled<SM>(reg[k] / stat[t - c * inner], scale, c);
      }
    }
  }
}

// ---------------------------------------------------------------------------
// Small slabs (inner < 64, dim * inner up to 3 K floats): class scores per box
// ([batch * boxes, 21], inner = 1), per-position embeddings, 2-class maps.  One
// workgroup per slab, as the slab kernels above do it, leaves a workgroup with a
// few dozen elements (softmax over [6.4M, 2]: 5 ms per 51 MB).  Here a
// workgroup takes `group` consecutive slabs, one contiguous span: 128-bit loads
// and stores on the global side, and in LDS every slab at a pitch of
// inner * (dim | 1) floats, so that lane q = slab * inner + s, which walks the
// column (slab, s) in index order with a stride of inner floats, meets the other
// lanes of its wave on different banks (all of them where inner is a power of
// two).  The per-element work between the walks (exp, the division) is done by
// all lanes over the span as it lies.
// ---------------------------------------------------------------------------
constexpr uint32_t kPackedTileFloats = 12288;  // 48 KB: three workgroups per CU

struct PackedSpan {
  uint32_t slab, pitch, inner, ncols, cells;
  FastDiv f_slab, f_inner;
  // element t of the span -> LDS offset, column, row
  SHDW_DEVICE void place(uint32_t t, uint32_t& at, uint32_t& q, uint32_t& c) const {
    uint32_t g, rem, s;
    fd_divmod(t, f_slab, g, rem);
    fd_divmod(rem, f_inner, c, s);
    at = g * pitch + rem;
    q = g * inner + s;
  }
};

SHDW_DEVICE PackedSpan packed_span(uint32_t slabs, uint32_t dim, FastDiv f_inner, FastDiv f_slab, uint32_t group,
                                   uint32_t* first_slab) {
  PackedSpan sp;
  sp.inner = f_inner.d;
  sp.slab = dim * sp.inner;
  sp.pitch = sp.inner * (dim | 1u);
  sp.f_slab = f_slab, sp.f_inner = f_inner;
  *first_slab = blockIdx.x * group;
  const uint32_t n = min(group, slabs - *first_slab);
  sp.ncols = n * sp.inner;
  sp.cells = n * sp.slab;
  return sp;
}

// The span into LDS: four vectors in flight per lane, scattered by element
// because a vector may straddle two slabs.
SHDW_DEVICE void packed_stage_in(float* lds, const float* xs, const PackedSpan& sp) {
  const uint32_t nvec = sp.cells / 4;
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
        uint32_t g, rem;
        fd_divmod(4 * v, sp.f_slab, g, rem);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          lds[g * sp.pitch + rem] = reg[k][j];
          if (++rem == sp.slab) rem = 0, ++g;
        }
      }
    }
  }
  const uint32_t t = 4 * nvec + threadIdx.x;
  if (t < sp.cells) {
    uint32_t at, q, c;
    sp.place(t, at, q, c);
    lds[at] = xs[t];
  }
}

// Walks the four elements that start at element t of the span: one division by
// the slab and one by inner for the first, then steps.
struct PackedWalk {
  uint32_t at, q, c, s, rem;
  SHDW_DEVICE PackedWalk(const PackedSpan& sp, uint32_t t) {
    uint32_t g;
    fd_divmod(t, sp.f_slab, g, rem);
    fd_divmod(rem, sp.f_inner, c, s);
    at = g * sp.pitch + rem;
    q = g * sp.inner + s;
  }
  SHDW_DEVICE void step(const PackedSpan& sp) {
    ++at, ++q, ++s, ++rem;
    if (s == sp.inner) s = 0, q -= sp.inner, ++c;          // next row of the same slab: its columns again
    if (rem == sp.slab) rem = 0, c = 0, q += sp.inner, at += sp.pitch - sp.slab;  // next slab
  }
};

// f(value in LDS, column, row) -> new value in LDS, for the whole span.
template <class F>
SHDW_DEVICE void packed_update(float* lds, const PackedSpan& sp, F f) {
  const uint32_t nvec = (sp.cells + 3) / 4;
  for (uint32_t v = threadIdx.x; v < nvec; v += kBlock) {
    PackedWalk w(sp, 4 * v);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (4 * v + j < sp.cells) lds[w.at] = f(lds[w.at], w.q, w.c);
      w.step(sp);
    }
  }
}

// f(value in LDS, column, row) -> output element, for the whole span, 128-bit stores.
template <class F>
SHDW_DEVICE void packed_stage_out(const float* lds, float* ys, const PackedSpan& sp, F f) {
  const uint32_t nvec = sp.cells / 4;
  for (uint32_t v = threadIdx.x; v < nvec; v += kBlock) {
    PackedWalk w(sp, 4 * v);
    v4f r;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      r[j] = f(lds[w.at], w.q, w.c);
      w.step(sp);
    }
    store4_stream_any(ys + 4ull * v, r);
  }
  const uint32_t t = 4 * nvec + threadIdx.x;
  if (t < sp.cells) {
    uint32_t at, q, c;
    sp.place(t, at, q, c);
    ys[t] = f(lds[at], q, c);
  }
}

// A lane's walk down its column: batches of sixteen reads at a constant stride from sixteen rows on, a
// plain loop for the short columns (two classes, a handful of channels), which a batch would not fill.
template <class F>
SHDW_DEVICE void packed_walk(const float* col, uint32_t inner, uint32_t dim, F&& fold) {
  if (dim >= 16) {
    walk_column_inner(col, inner, dim, fold);
  } else {
#pragma unroll 4
    for (uint32_t c = 0; c < dim; ++c) fold(col[c * inner]);
  }
}

__global__ __launch_bounds__(kBlock) void softmax_packed_kernel(const float* x, float* y, uint32_t slabs,
                                                                 uint32_t dim, FastDiv f_inner, FastDiv f_slab,
                                                                 uint32_t group) {
  extern __shared__ __align__(16) float lds[];  // group * pitch floats
  __shared__ uint64_t tab[32];
  __shared__ float stat[kBlock];
  if (threadIdx.x < 32) tab[threadIdx.x] = libm::kExp2fTab[threadIdx.x];
  uint32_t first;
  const PackedSpan sp = packed_span(slabs, dim, f_inner, f_slab, group, &first);
  const uint64_t base = static_cast<uint64_t>(first) * sp.slab;
  packed_stage_in(lds, x + base, sp);
  __syncthreads();
  const uint32_t q = threadIdx.x;
  const float* col = lds + fd_div(q, f_inner) * sp.pitch + (q - fd_div(q, f_inner) * sp.inner);
  if (q < sp.ncols) {
    float m = -FLT_MAX;
    packed_walk(col, sp.inner, dim, [&](float v) { m = std_max(v, m); });
    stat[q] = m;
  }
  __syncthreads();
  packed_update(lds, sp, [&](float v, uint32_t cq, uint32_t) { return libm::exact_expf(v - stat[cq], tab); });
  __syncthreads();
  if (q < sp.ncols) {
    float sum = 0.f;
    packed_walk(col, sp.inner, dim, [&](float v) { sum += v; });
    stat[q] = sum;
  }
  __syncthreads();
  packed_stage_out(lds, y + base, sp, [&](float e, uint32_t cq, uint32_t) { return e / stat[cq]; });
}

template <int PMODE, int SM>
__global__ __launch_bounds__(kBlock) void normalize_packed_kernel(const float* x, float* y, uint32_t slabs,
                                                                   uint32_t dim, FastDiv f_inner, FastDiv f_slab,
                                                                   uint32_t group, float p, float eps,
                                                                   const float* scale) {
  extern __shared__ __align__(16) float lds[];
  __shared__ float stat[kBlock];
  uint32_t first;
  const PackedSpan sp = packed_span(slabs, dim, f_inner, f_slab, group, &first);
  const uint64_t base = static_cast<uint64_t>(first) * sp.slab;
  packed_stage_in(lds, x + base, sp);
  __syncthreads();
  const uint32_t q = threadIdx.x;
  if (q < sp.ncols) {
    const uint32_t g = fd_div(q, f_inner);
    const float* col = lds + g * sp.pitch + (q - g * sp.inner);
    double acc = 0;
    packed_walk(col, sp.inner, dim, [&](float v) { acc += norm_term<PMODE>(v, p); });
    stat[q] = norm_finish<PMODE>(acc, p, eps);
  }
  __syncthreads();
  packed_stage_out(lds, y + base, sp,
                   [&](float v, uint32_t cq, uint32_t c) { return ssd_scaled<SM>(v / stat[cq], scale, c); });
}

// Columns of 65 to 1024 elements over a wide inner extent: a workgroup owns a
// tile of TS = 64, 32 or 16 neighbouring positions with all their `dim` elements,
// 64 KB at most, so x is read from HBM once.  Each lane keeps its share of the
// tile (16 vectors of 4 positions at most) in registers and also parks it in
// LDS; wave 0 folds the TS columns from LDS in index order, one column per lane,
// and hands the TS results over in the first tile row (nobody else reads the
// tile, and the fold is done with it); after the barrier every lane finishes
// its registers.  Only one SIMD pays for the serial fold, the other waves of
// the CU keep their SIMDs free for the other resident workgroups.
//
// Rows of the tile start wherever inner and the tile offset put them, so the
// 128-bit global accesses are only 4-byte aligned (the hardware splits the ones
// that straddle a line; that is still far cheaper than four 4-byte accesses per
// lane, which run at the address-unit rate: 185 us against 84 us on
// [64,150,73,73] / [64,150,72,72]).  Neighbouring tiles share the straddled
// lines, hence the XCD-contiguous workgroup order.
constexpr int kTilePerLane = 16;  // 64 KB / (256 lanes x 16 bytes)

// ROWS says how the tile rows lie in memory:
//   kRowsSector: inner % 16 == 0, every row starts on a 64-byte boundary;
//   kRowsQuad:   inner % 4 == 0, rows start on a multiple of four positions;
//   kRowsAny:    a row may end inside a lane's four positions.
enum TileRows { kRowsSector = 0, kRowsQuad = 1, kRowsAny = 2 };

template <int TS_SHIFT, int ROWS>
struct TileLane {
  static constexpr bool TAIL = ROWS == kRowsAny;
  static constexpr uint32_t TS = 1u << TS_SHIFT;
  static constexpr uint32_t LANES_PER_ROW = TS / 4;
  static constexpr uint32_t STEP = kBlock / LANES_PER_ROW;  // rows between a lane's vectors
  uint32_t j, c0, valid;  // first position, first row, positions of j..j+3 inside the tile
  uint32_t dim, inner;

  SHDW_DEVICE TileLane(uint32_t width, uint32_t dim_, uint32_t inner_) : dim(dim_), inner(inner_) {
    j = (threadIdx.x & (LANES_PER_ROW - 1)) * 4;
    c0 = threadIdx.x / LANES_PER_ROW;
    valid = j < width ? min(4u, width - j) : 0u;
  }
  SHDW_DEVICE void load(const float* xs, v4f (&r)[kTilePerLane]) const {
    if (valid == 0) return;
#pragma unroll
    for (int u = 0; u < kTilePerLane; ++u) {
      const uint32_t c = c0 + u * STEP;
      if (c >= dim) continue;
      const float* src = xs + static_cast<uint64_t>(c) * inner + j;
      if (!TAIL || valid == 4) {
        r[u] = __builtin_nontemporal_load(reinterpret_cast<const v4f_unaligned*>(src));
      } else {
        r[u] = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int k = 0; k < 3; ++k)
          if (k < valid) r[u][k] = src[k];
      }
    }
  }
  // f(v): what the folding lanes are to find in the tile for the vector v
  template <typename F>
  SHDW_DEVICE void park(float* lds, const v4f (&r)[kTilePerLane], F f) const {
    if (valid == 0) return;
#pragma unroll
    for (int u = 0; u < kTilePerLane; ++u) {
      const uint32_t c = c0 + u * STEP;
      if (c < dim) *reinterpret_cast<v4f*>(lds + (c << TS_SHIFT) + j) = f(r[u]);
    }
  }
  SHDW_DEVICE void park(float* lds, const v4f (&r)[kTilePerLane]) const {
    park(lds, r, [](const v4f& v) { return v; });
  }
  SHDW_DEVICE void store(float* ys, uint32_t u, v4f v) const {
    const uint32_t c = c0 + u * STEP;
    float* dst = ys + static_cast<uint64_t>(c) * inner + j;
    // Rows that do not start on a 64-byte boundary end inside a sector whose
    // other part the neighbouring tile writes: with a plain store the two parts
    // merge in L2 before they go to HBM, a streaming store sends each on its own
    // (+37 % write traffic on [64,512,38,38]).  Aligned rows stream.
    if (!TAIL || valid == 4) {
      if (ROWS == kRowsSector)
        __builtin_nontemporal_store(v, reinterpret_cast<v4f_unaligned*>(dst));
      else
        *reinterpret_cast<v4f_unaligned*>(dst) = v;
    } else {
#pragma unroll
      for (int k = 0; k < 3; ++k)
        if (k < valid) dst[k] = v[k];
    }
  }
};

// Serial fold of one tile column (stride 1 << TS_SHIFT floats in LDS) by one
// lane, in index order: acc = f(acc, column[c]) for c = 0 .. dim - 1.  The
// values come in batches of 16 reads that are all requested before the first is
// folded: written as a plain loop, the compiler waits for each pair of LDS
// reads right before it uses them, and the LDS latency, not the chain of
// additions, sets the pace (about 130 clocks per two values; 512-long columns
// then take 14 us per tile).  One set of registers: the folding waves of the
// workgroups on a CU share one SIMD, and a second set that the next batch is
// read into while this one is folded costs that SIMD a move per value.
template <int TS_SHIFT, typename T, typename F>
SHDW_DEVICE T fold_tile_column(const float* column, uint32_t dim, T acc, F f) {
  constexpr int kBatch = 16;
  uint32_t c = 0;
  for (; c + kBatch <= dim; c += kBatch) {
    float v[kBatch];
#pragma unroll
    for (int u = 0; u < kBatch; ++u) v[u] = column[(c + u) << TS_SHIFT];
#pragma unroll
    for (int u = 0; u < kBatch; ++u) acc = f(acc, v[u]);
  }
  for (; c < dim; ++c) acc = f(acc, column[c << TS_SHIFT]);
  return acc;
}

// p other than 1 and 2 is not taken here: powf per element inside the serial
// fold would dominate.
template <int PMODE, int SM, int TS_SHIFT, int ROWS>
__global__ __launch_bounds__(kBlock) void normalize_tile_kernel(const float* x, float* y, uint32_t dim,
                                                                 uint32_t inner, FastDiv f_tiles, float p,
                                                                 float eps, const float* scale) {
  extern __shared__ __align__(16) float lds[];
  constexpr uint32_t TS = 1u << TS_SHIFT;
  uint32_t n, tile;
  fd_divmod(xcd_contiguous(blockIdx.x, gridDim.x), f_tiles, n, tile);
  const uint32_t p0 = tile << TS_SHIFT;
  const uint32_t width = min(TS, inner - p0);
  const uint64_t base = static_cast<uint64_t>(n) * dim * inner + p0;
  const TileLane<TS_SHIFT, ROWS> lane(width, dim, inner);
  v4f r[kTilePerLane];
  lane.load(x + base, r);
  // the tile holds the terms of the sums, fp32 values that widen exactly: the folding wave's chain sets the
  // pace of a tall, narrow tile, and every instruction taken off it is time off the tile
  lane.park(lds, r, [p](const v4f& v) {
    return v4f{static_cast<float>(norm_term<PMODE>(v[0], p)), static_cast<float>(norm_term<PMODE>(v[1], p)),
               static_cast<float>(norm_term<PMODE>(v[2], p)), static_cast<float>(norm_term<PMODE>(v[3], p))};
  });
  __syncthreads();
  if (threadIdx.x < width) {  // width <= TS <= 64: lanes of wave 0, one column each
    const float* column = lds + threadIdx.x;
    const double acc =
        fold_tile_column<TS_SHIFT>(column, dim, 0.0, [](double a, float t) { return a + static_cast<double>(t); });
    lds[threadIdx.x] = norm_finish<PMODE>(acc, p, eps);
  }
  __syncthreads();
  if (lane.valid == 0) return;
  const v4f d = *reinterpret_cast<const v4f*>(lds + lane.j);
#pragma unroll
  for (int u = 0; u < kTilePerLane; ++u) {
    const uint32_t c = lane.c0 + u * lane.STEP;
    if (c >= dim) continue;
    v4f q;
#pragma unroll
    for (int k = 0; k < 4; ++k) q[k] = ssd_scaled<SM>(r[u][k] / d[k], scale, c);
    lane.store(y + base, u, q);
  }
}

constexpr int kTileMinDim = 65, kTileMaxDim = 1024, kTileMinInner = 16;
constexpr int kTileLdsBytes = 65536;

static int tile_rows(int inner_num, const float* y) {
  if (inner_num % 16 == 0 && (reinterpret_cast<uintptr_t>(y) & 63u) == 0) return kRowsSector;
  return inner_num % 4 == 0 ? kRowsQuad : kRowsAny;
}

// Columns of 513 to 1024 rows take tiles of 16 positions (64-byte row pieces), which pay from 32 (Softmax)
// or 64 (Normalize) positions on: [127,513,196] softmax 89 -> 39 us, normalize 68 -> 31; [65,1000,196]
// 94 -> 51, 69 -> 41; below, the slab kernels stay ahead ([513,1000,25] normalize 46 against 61).
constexpr int kTileWideDim = 512, kTileMinInnerTallSoftmax = 32, kTileMinInnerTallNormalize = 64;

static bool tile_fits(int dim, int inner_num, bool softmax) {
  if (dim < kTileMinDim || dim > kTileMaxDim) return false;
  if (dim <= kTileWideDim) return inner_num >= kTileMinInner;
  return inner_num >= (softmax ? kTileMinInnerTallSoftmax : kTileMinInnerTallNormalize);
}

template <int PMODE, int SM, int TS_SHIFT>
static void launch_normalize_tile_ts(int outer_num, int dim, int inner_num, float p, float eps, const float* x,
                                     const float* scale, float* y, hipStream_t st) {
  const uint32_t tiles = (static_cast<uint32_t>(inner_num) + (1u << TS_SHIFT) - 1) >> TS_SHIFT;
  const uint32_t grid = static_cast<uint32_t>(outer_num) * tiles;
  const size_t bytes = (static_cast<size_t>(dim) << TS_SHIFT) * sizeof(float);
  const uint32_t d = static_cast<uint32_t>(dim), in = static_cast<uint32_t>(inner_num);
  const FastDiv ft = make_fastdiv(tiles);
  switch (tile_rows(inner_num, y)) {
    case kRowsSector:
      normalize_tile_kernel<PMODE, SM, TS_SHIFT, kRowsSector><<<grid, kBlock, bytes, st>>>(x, y, d, in, ft, p, eps, scale);
      break;
    case kRowsQuad:
      normalize_tile_kernel<PMODE, SM, TS_SHIFT, kRowsQuad><<<grid, kBlock, bytes, st>>>(x, y, d, in, ft, p, eps, scale);
      break;
    default:
      normalize_tile_kernel<PMODE, SM, TS_SHIFT, kRowsAny><<<grid, kBlock, bytes, st>>>(x, y, d, in, ft, p, eps, scale);
  }
}

static int normalize_tile_shift(int dim);

template <int PMODE, int SM>
static void launch_normalize_tile(int outer_num, int dim, int inner_num, float p, float eps, const float* x,
                                  const float* scale, float* y, hipStream_t st) {
  // 64 positions per tile row while the tile stays within 32 KB (four and more
  // workgroups per CU), else 32, up to 64 KB: rows of 16 positions (64 bytes)
  // cost more than the lower occupancy does.  [64,256,56,56]: 85 us with 64
  // positions (64 KB), 80 us with 32; [64,512,38,38]: 105 us with 32 (64 KB),
  // 115 us with 16.  Softmax, with its four barriers per tile, takes the widest
  // tile that fits.
  const int shift = normalize_tile_shift(dim);
  if (shift == 6)
    launch_normalize_tile_ts<PMODE, SM, 6>(outer_num, dim, inner_num, p, eps, x, scale, y, st);
  else if (shift == 5)
    launch_normalize_tile_ts<PMODE, SM, 5>(outer_num, dim, inner_num, p, eps, x, scale, y, st);
  else
    launch_normalize_tile_ts<PMODE, SM, 4>(outer_num, dim, inner_num, p, eps, x, scale, y, st);
}

// Softmax on the same tile layout (65 <= dim <= 1024).  The lanes hold x, later
// exp(x - max), in registers.  Behind the tile lie the exp table, a row that
// hands the maxima and later the sums over, and a flag.
//
// The running maximum max = std_max(x[c], max), started at -FLT_MAX, is the
// largest element whatever the order as long as no element is NaN (a NaN takes
// the maximum over and the next element takes it back, so then the order
// counts; which of two zeros wins does not change exp(x - max)).  Every lane
// therefore takes the maximum of its own rows, the STEP partial maxima per
// position meet in the first tile rows and one lane per position folds them; a
// lane that met a NaN hands a NaN over instead, and a tile with one anywhere
// parks x and walks the columns in index order like the sums.  The sum of the
// exponentials is an fp32 running sum and always walks.
template <int TS_SHIFT, int ROWS>
__global__ __launch_bounds__(kBlock) void softmax_tile_kernel(const float* x, float* y, uint32_t dim,
                                                               uint32_t inner, FastDiv f_tiles) {
  extern __shared__ __align__(16) float lds[];
  constexpr uint32_t TS = 1u << TS_SHIFT;
  using Lane = TileLane<TS_SHIFT, ROWS>;
  uint64_t* tab = reinterpret_cast<uint64_t*>(lds + (dim << TS_SHIFT));  // after the tile, 16-byte aligned
  float* handed = reinterpret_cast<float*>(tab + 32);
  uint32_t* any_nan = reinterpret_cast<uint32_t*>(handed + TS);
  if (threadIdx.x < 32) tab[threadIdx.x] = libm::kExp2fTab[threadIdx.x];
  uint32_t n, tile;
  fd_divmod(xcd_contiguous(blockIdx.x, gridDim.x), f_tiles, n, tile);
  const uint32_t p0 = tile << TS_SHIFT;
  const uint32_t width = min(TS, inner - p0);
  const uint64_t base = static_cast<uint64_t>(n) * dim * inner + p0;
  const Lane lane(width, dim, inner);
  v4f r[kTilePerLane];
  lane.load(x + base, r);
  if (lane.valid != 0) {
    v4f m = {-FLT_MAX, -FLT_MAX, -FLT_MAX, -FLT_MAX};
    bool nan[4] = {false, false, false, false};
#pragma unroll
    for (int u = 0; u < kTilePerLane; ++u) {
      if (lane.c0 + u * Lane::STEP >= dim) continue;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const float v = r[u][k];
        nan[k] |= v != v;
        m[k] = m[k] < v ? v : m[k];
      }
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) m[k] = nan[k] ? __builtin_nanf("") : m[k];
    *reinterpret_cast<v4f*>(lds + (lane.c0 << TS_SHIFT) + lane.j) = m;  // row c0 < STEP <= 64 < dim
  }
  __syncthreads();
  if (threadIdx.x < kWave) {  // all of wave 0, so that its lanes agree on the flag
    float m = -FLT_MAX;
    bool nan = false;
    if (threadIdx.x < width) {
      const uint32_t groups = min(Lane::STEP, dim);
      for (uint32_t g = 0; g < groups; ++g) {
        const float v = lds[(g << TS_SHIFT) + threadIdx.x];
        nan |= v != v;
        m = m < v ? v : m;
      }
      handed[threadIdx.x] = m;
    }
    const uint64_t seen = __builtin_amdgcn_ballot_w64(nan);
    if (threadIdx.x == 0) *any_nan = seen != 0;
  }
  __syncthreads();
  if (*any_nan != 0) {  // the whole workgroup: the maxima in index order
    lane.park(lds, r);
    __syncthreads();
    if (threadIdx.x < width) {
      const float* column = lds + threadIdx.x;
      handed[threadIdx.x] = fold_tile_column<TS_SHIFT>(column, dim, -FLT_MAX,
                                                      [](float m, float v) { return std_max(v, m); });
    }
    __syncthreads();
  }
  if (lane.valid != 0) {
    const v4f m = *reinterpret_cast<const v4f*>(handed + lane.j);
#pragma unroll
    for (int u = 0; u < kTilePerLane; ++u) {
      if (lane.c0 + u * lane.STEP >= dim) continue;
#pragma unroll
      for (int k = 0; k < 4; ++k) r[u][k] = libm::exact_expf(r[u][k] - m[k], tab);
    }
  }
  lane.park(lds, r);
  __syncthreads();  // also: every lane has its maxima before the sums replace them
  if (threadIdx.x < width) {
    const float* column = lds + threadIdx.x;
    handed[threadIdx.x] = fold_tile_column<TS_SHIFT>(column, dim, 0.f, [](float a, float v) { return a + v; });
  }
  __syncthreads();
  if (lane.valid == 0) return;
  const v4f d = *reinterpret_cast<const v4f*>(handed + lane.j);
#pragma unroll
  for (int u = 0; u < kTilePerLane; ++u) {
    if (lane.c0 + u * lane.STEP >= dim) continue;
    v4f q;
#pragma unroll
    for (int k = 0; k < 4; ++k) q[k] = r[u][k] / d[k];
    lane.store(y + base, u, q);
  }
}

constexpr size_t kExpTabBytes = 32 * sizeof(uint64_t);
constexpr size_t kSoftmaxTileExtraBytes = kExpTabBytes + 64 * sizeof(float) + 16;  // table, hand-over row, flag
// (32 positions of 512 channels, or 16 of 1024, plus the exp table: 64 KB + 256 bytes, two workgroups per CU all the same)

template <int TS_SHIFT>
static void launch_softmax_tile_ts(int outer_num, int dim, int inner_num, const float* x, float* y,
                                   hipStream_t st) {
  const uint32_t tiles = (static_cast<uint32_t>(inner_num) + (1u << TS_SHIFT) - 1) >> TS_SHIFT;
  const uint32_t grid = static_cast<uint32_t>(outer_num) * tiles;
  const size_t bytes = (static_cast<size_t>(dim) << TS_SHIFT) * sizeof(float) + kSoftmaxTileExtraBytes;
  const uint32_t d = static_cast<uint32_t>(dim), in = static_cast<uint32_t>(inner_num);
  const FastDiv ft = make_fastdiv(tiles);
  switch (tile_rows(inner_num, y)) {
    case kRowsSector: softmax_tile_kernel<TS_SHIFT, kRowsSector><<<grid, kBlock, bytes, st>>>(x, y, d, in, ft); break;
    case kRowsQuad: softmax_tile_kernel<TS_SHIFT, kRowsQuad><<<grid, kBlock, bytes, st>>>(x, y, d, in, ft); break;
    default: softmax_tile_kernel<TS_SHIFT, kRowsAny><<<grid, kBlock, bytes, st>>>(x, y, d, in, ft);
  }
}

// ---------------------------------------------------------------------------
// Rows: the statistic over the last axis (inner == 1: class scores, attention
// rows), 17 to 4096 long.  The ordered sum of a row is one lane's walk, a few
// microseconds for a thousand elements, and with a workgroup per row (the slab
// kernels) a CU has eight such walks in flight and 255 of 256 lanes wait for
// each.  Here every wave works by itself, without a barrier, on R consecutive
// rows (R a power of two, R * pitch floats of LDS: one contiguous piece of x):
// all 64 lanes stage them, 64 / R lanes share a row for the maximum (any order,
// see softmax_slab_kernel), the exponentials and the division, the first lane
// of each row adds it up front to back, and the piece goes back as it came.  A
// wave never waits for another, so a CU has 8 or 16 of them, each with R walks,
// at different points of their work.  The four waves of a workgroup exist for
// their placement, one per SIMD (see pool_rows_stream_kernel).
// ---------------------------------------------------------------------------
constexpr uint32_t kRowsMinDim = 17;

struct WaveRows {
  uint32_t dim, pitch, rows_per_wave, group_log2;  // lanes per row = 1 << group_log2
  FastDiv f_dim;
};

// The wave's rows into its tile: 128-bit loads of the contiguous piece, eight in flight, scattered
// by element (a vector may end in the next row).
SHDW_DEVICE void rows_stage_in(float* tile, const float* xs, uint32_t cells, const WaveRows& w, uint32_t lane) {
  const uint32_t nvec = cells / 4;
  for (uint32_t v0 = 0; v0 < nvec; v0 += 8 * kWave) {
    v4f reg[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const uint32_t v = v0 + k * kWave + lane;
      if (v < nvec) reg[k] = load4_stream_any(xs + 4ull * v);
    }
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const uint32_t v = v0 + k * kWave + lane;
      if (v < nvec) {
        uint32_t r, c;
        fd_divmod(4 * v, w.f_dim, r, c);
        uint32_t at = r * w.pitch + c;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          tile[at] = reg[k][j];
          ++at;
          if (++c == w.dim) c = 0, at += w.pitch - w.dim;
        }
      }
    }
  }
  const uint32_t t = 4 * nvec + lane;
  if (t < cells) {
    uint32_t r, c;
    fd_divmod(t, w.f_dim, r, c);
    tile[r * w.pitch + c] = xs[t];
  }
}

// f(value in the tile, row, column) for every element, written to the contiguous piece of y.
template <class F>
SHDW_DEVICE void rows_stage_out(const float* tile, float* ys, uint32_t cells, const WaveRows& w, uint32_t lane, F f) {
  const uint32_t nvec = cells / 4;
  for (uint32_t v = lane; v < nvec; v += kWave) {
    uint32_t r, c;
    fd_divmod(4 * v, w.f_dim, r, c);
    uint32_t at = r * w.pitch + c;
    v4f q;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      q[j] = f(tile[at], r, c);
      ++at;
      if (++c == w.dim) c = 0, ++r, at += w.pitch - w.dim;
    }
    store4_stream_any(ys + 4ull * v, q);
  }
  const uint32_t t = 4 * nvec + lane;
  if (t < cells) {
    uint32_t r, c;
    fd_divmod(t, w.f_dim, r, c);
    ys[t] = f(tile[r * w.pitch + c], r, c);
  }
}

// Softmax over rows of D = 2 .. 16 elements (two to a handful of class scores per box): a lane owns four
// whole rows, 4 * D consecutive floats, in registers.  The wave's span moves between memory and the wave's
// own tile in LDS as it lies, 128 bits per lane and access, and between the tile and the lanes' registers
// with a lane's rows at a pitch of an odd number of 128-bit pieces; no divisions, no workgroup barrier
// after the first.
//
// The same for slabs of D = dim * inner floats with inner > 1 (two classes over a few positions or anchors
// per cell): a lane owns four slabs and walks their inner columns one after the other, at a stride of inner.
template <int D>
__global__ __launch_bounds__(kBlock) void softmax_short_rows_kernel(const float* x, float* y, uint32_t rows,
                                                                     uint32_t dim, uint32_t inner) {
  constexpr uint32_t kMine = 4 * D;                          // floats of a lane
  constexpr uint32_t kPitch = kMine + (D % 2 == 0 ? 4 : 0);  // of the lanes in the tile
  constexpr uint32_t kSpan = kWave * kMine;                  // floats of a wave
  __shared__ __align__(16) float tiles[kBlock / kWave][kWave * kPitch];
  __shared__ uint64_t tab[32];
  if (threadIdx.x < 32) tab[threadIdx.x] = libm::kExp2fTab[threadIdx.x];
  __syncthreads();  // the only one
  const uint32_t lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const uint64_t total = static_cast<uint64_t>(rows) * D;
  const uint64_t first = (static_cast<uint64_t>(blockIdx.x) * (kBlock / kWave) + wave) * kSpan;
  if (first >= total) return;  // the whole wave
  const uint32_t cells = static_cast<uint32_t>(min(static_cast<uint64_t>(kSpan), total - first));
  const float* xs = x + first;
  float* ys = y + first;
  float* tile = tiles[wave];
  auto place = [](uint32_t t) { return (t / kMine) * kPitch + t % kMine; };  // element t of the span in the tile
  v4f reg[D];
  // No branch around a load (vectors past the end re-read the tensor's first): with one, the compiler
  // copied the whole register array at every join, 500 moves at D = 8 and 42 us per 51 MB in place of 25.
#pragma unroll
  for (int k = 0; k < D; ++k) {
    const uint32_t t = 4 * (k * kWave + lane);
    reg[k] = load4_stream_any(t + 4 <= cells ? xs + t : x);
  }
#pragma unroll
  for (int k = 0; k < D; ++k) {
    const uint32_t t = 4 * (k * kWave + lane);
    if (t + 4 <= cells) *reinterpret_cast<v4f*>(tile + place(t)) = reg[k];
  }
  const uint32_t rest = (cells & ~3u) + lane;  // a span that ends the tensor may end inside a vector
  if (lane < 3 && rest < cells) tile[place(rest)] = xs[rest];
  __builtin_amdgcn_wave_barrier();
  float* mine = tile + lane * kPitch;
  // A row at a time, from and to the tile: the 4 * D exponentials of a lane side by side (each a chain of
  // fp64 operations) would take over 200 registers at D = 8.
#pragma unroll 1
  for (uint32_t r = 0; r < 4; ++r) {  // rows past the end of the tensor hold what the tile held; nothing of them is stored
    float* row = mine + r * D;
    if (inner != 1) {
      for (uint32_t s = 0; s < inner; ++s) {
        float* col = row + s;
        float m = -FLT_MAX;
        for (uint32_t c = 0; c < dim; ++c) m = std_max(col[c * inner], m);
        float sum = 0.f;
        for (uint32_t c = 0; c < dim; ++c) {
          const float v = libm::exact_expf(col[c * inner] - m, tab);
          col[c * inner] = v;
          sum += v;
        }
        for (uint32_t c = 0; c < dim; ++c) col[c * inner] = col[c * inner] / sum;
      }
      continue;
    }
    float e[D];
#pragma unroll
    for (int c = 0; c < D; ++c) e[c] = row[c];
    float m = -FLT_MAX;
#pragma unroll
    for (int c = 0; c < D; ++c) m = std_max(e[c], m);
    float sum = 0.f;
#pragma unroll
    for (int c = 0; c < D; ++c) {
      e[c] = libm::exact_expf(e[c] - m, tab);
      sum += e[c];
    }
#pragma unroll
    for (int c = 0; c < D; ++c) row[c] = e[c] / sum;
  }
  __builtin_amdgcn_wave_barrier();
#pragma unroll
  for (int k = 0; k < D; ++k) {
    const uint32_t t = 4 * (k * kWave + lane);
    if (t + 4 <= cells) store4_stream_any(ys + t, *reinterpret_cast<const v4f*>(tile + place(t)));
  }
  if (lane < 3 && rest < cells) ys[rest] = tile[place(rest)];
}

template <int TILE>
__global__ __launch_bounds__(kBlock) void softmax_rows_kernel(const float* x, float* y, uint32_t rows, WaveRows w) {
  __shared__ __align__(16) float tiles[kBlock / kWave][TILE];
  __shared__ float stats[kBlock / kWave][kWave];
  __shared__ uint64_t tab[32];
  if (threadIdx.x < 32) tab[threadIdx.x] = libm::kExp2fTab[threadIdx.x];
  __syncthreads();  // the only one: from here on every wave is on its own
  const uint32_t lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  float* tile = tiles[wave];
  float* stat = stats[wave];
  const uint32_t row0 = (blockIdx.x * (kBlock / kWave) + wave) * w.rows_per_wave;
  if (row0 >= rows) return;  // the whole wave
  const uint32_t nrows = min(w.rows_per_wave, rows - row0), cells = nrows * w.dim;
  const uint64_t base = static_cast<uint64_t>(row0) * w.dim;
  rows_stage_in(tile, x + base, cells, w, lane);
  __builtin_amdgcn_wave_barrier();
  const uint32_t group = 1u << w.group_log2;
  const uint32_t r = lane >> w.group_log2, sub = lane & (group - 1);
  float* mine = tile + (r < nrows ? r : 0) * w.pitch;  // rows past the end: their lanes read row 0 and write nothing
  float m = -FLT_MAX;
  for (uint32_t c = sub; c < w.dim; c += group) m = std_max(mine[c], m);
  for (uint32_t off = 1; off < group; off <<= 1) m = std_max(__shfl_xor(m, off), m);  // all 64 lanes are here
  __builtin_amdgcn_wave_barrier();
  if (r < nrows)
    for (uint32_t c = sub; c < w.dim; c += group) mine[c] = libm::exact_expf(mine[c] - m, tab);
  __builtin_amdgcn_wave_barrier();
  if (sub == 0 && r < nrows) {
    float sum = 0.f;
    walk_column(mine, 1, w.dim, [&](float a) { sum += a; });
    stat[r] = sum;
  }
  __builtin_amdgcn_wave_barrier();
  rows_stage_out(tile, y + base, cells, w, lane, [&](float e, uint32_t rr, uint32_t) { return e / stat[rr]; });
}

// PMODE 1, 2 (Normalize) and 3 (SSDNormalize per position); the terms of the sum are formed by the walking lane.
template <int PMODE, int SM, int TILE>
__global__ __launch_bounds__(kBlock) void normalize_rows_kernel(const float* x, float* y, uint32_t rows, WaveRows w,
                                                                 float p, float eps, const float* scale) {
  __shared__ __align__(16) float tiles[kBlock / kWave][TILE];
  __shared__ float stats[kBlock / kWave][kWave];
  const uint32_t lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  float* tile = tiles[wave];
  float* stat = stats[wave];
  const uint32_t row0 = (blockIdx.x * (kBlock / kWave) + wave) * w.rows_per_wave;
  if (row0 >= rows) return;  // the whole wave
  const uint32_t nrows = min(w.rows_per_wave, rows - row0), cells = nrows * w.dim;
  const uint64_t base = static_cast<uint64_t>(row0) * w.dim;
  rows_stage_in(tile, x + base, cells, w, lane);
  __builtin_amdgcn_wave_barrier();
  const uint32_t group = 1u << w.group_log2;
  const uint32_t r = lane >> w.group_log2, sub = lane & (group - 1);
  if (sub == 0 && r < nrows) {
    double acc = 0;
    walk_column(tile + r * w.pitch, 1, w.dim, [&](float a) { acc += norm_term<PMODE>(a, p); });
    stat[r] = norm_finish<PMODE>(acc, p, eps);
  }
  __builtin_amdgcn_wave_barrier();
  rows_stage_out(tile, y + base, cells, w, lane,
                 [&](float v, uint32_t rr, uint32_t c) { return ssd_scaled<SM>(v / stat[rr], scale, c); });
}

// Rows per wave and lanes per row for the kernels above; false where they do not apply.
template <int TILE>
static bool wave_rows(int dim, WaveRows* w) {
  const uint32_t d = static_cast<uint32_t>(dim);
  uint32_t r = 1;
  while (r < kWave && 2 * r * (d | 1u) <= static_cast<uint32_t>(TILE)) r *= 2;
  w->dim = d, w->pitch = r > 1 ? (d | 1u) : d;
  if (w->pitch * r > static_cast<uint32_t>(TILE)) return false;
  w->rows_per_wave = r;
  w->group_log2 = 0;
  while ((r << w->group_log2) < kWave) ++w->group_log2;
  w->f_dim = make_fastdiv(d);
  return true;
}

// ---------------------------------------------------------------------------
// Normalize over long rows (inner == 1, more than a few hundred elements).  One
// lane walking a row costs its wave a full instruction slot per element whether
// one lane walks or sixty-four (rows of 2048 with a row per wave: 105 us per
// 51 MB, all of it the walks), and whole rows of this length leave room for one
// or two per wave in LDS.  Here a wave takes G rows and moves along them in
// equal chunks of at most W = 4096 / G columns: all lanes fetch a chunk (up to
// 16 vectors each) into the wave's tile, lane g < G folds row g's piece in
// index order, and the next chunk's requests are already out; a second pass
// scales x straight from the registers, no tile.  No barriers; four waves per
// workgroup for their placement only.  (Softmax in this form takes every
// exponential twice and came out slower than the kernels it would replace.)
// ---------------------------------------------------------------------------
constexpr int kStreamVectors = 16;  // per lane and chunk

template <int G>
struct RowStream {
  static constexpr uint32_t W = 256u * kStreamVectors / G, VW = W / 4, PITCH = W + 4;
  uint32_t rows, len, row0, lane;
  uint32_t step;  // columns per chunk: the row cut into equal pieces of at most W (a multiple of 4), not W + a rest
  SHDW_DEVICE void init(uint32_t rows_, uint32_t len_, uint32_t row0_, uint32_t lane_) {
    rows = rows_, len = len_, row0 = row0_, lane = lane_;
    const uint32_t pieces = (len + W - 1) / W;
    step = (((len + pieces - 1) / pieces) + 3) & ~3u;
  }
  // vector i of the lane's share of the chunk at column c0: its row (of the wave's G) and first column
  SHDW_DEVICE static uint32_t row_of(uint32_t lane, int i) { return (lane + kWave * i) / VW; }
  SHDW_DEVICE static uint32_t col_of(uint32_t lane, int i) { return 4 * ((lane + kWave * i) % VW); }
  SHDW_DEVICE uint32_t count(int i, uint32_t c0) const {  // elements of vector i that exist
    if (row0 + row_of(lane, i) >= rows || col_of(lane, i) >= step) return 0;
    const uint32_t c = c0 + col_of(lane, i);
    return c >= len ? 0u : min(4u, len - c);
  }
  SHDW_DEVICE uint32_t cols(uint32_t c0) const { return min(step, len - c0); }  // of the chunk at c0
  SHDW_DEVICE void request(const float* x, uint32_t c0, v4f (&reg)[kStreamVectors]) const {
#pragma unroll
    for (int i = 0; i < kStreamVectors; ++i) {
      const uint32_t n = count(i, c0);
      if (n == 0) continue;
      const float* src = x + static_cast<uint64_t>(row0 + row_of(lane, i)) * len + c0 + col_of(lane, i);
      if (n == 4) {
        reg[i] = load4_stream_any(src);
      } else {
#pragma unroll
        for (int k = 0; k < 3; ++k)
          if (static_cast<uint32_t>(k) < n) reg[i][k] = __builtin_nontemporal_load(src + k);
      }
    }
  }
  // f(vector, i) for every vector of the chunk, into the wave's tile
  template <class F>
  SHDW_DEVICE void lay_down(float* tile, const v4f (&reg)[kStreamVectors], F f) const {
#pragma unroll
    for (int i = 0; i < kStreamVectors; ++i)
      *reinterpret_cast<v4f*>(tile + row_of(lane, i) * PITCH + col_of(lane, i)) = f(reg[i], i);
  }
};

template <int PMODE, int SM, int G>
__global__ __launch_bounds__(kBlock) void normalize_rows_stream_kernel(const float* x, float* y, uint32_t rows,
                                                                        uint32_t len, float p, float eps,
                                                                        const float* scale) {
  using S = RowStream<G>;
  __shared__ __align__(16) float tiles[kBlock / kWave][G * S::PITCH];
  __shared__ float divisors[kBlock / kWave][G];
  S s;
  const uint32_t wave = threadIdx.x / kWave;
  s.init(rows, len, (blockIdx.x * (kBlock / kWave) + wave) * G, threadIdx.x % kWave);
  if (s.row0 >= rows) return;  // the whole wave
  float* tile = tiles[wave];
  const float* mine = tile + s.lane * S::PITCH;
  v4f reg[kStreamVectors];

  double acc = 0;
  s.request(x, 0, reg);
  for (uint32_t c0 = 0; c0 < len; c0 += s.step) {
    // the terms of the sums (exactly representable in fp32: they are widened fp32 values) are formed by all
    // lanes on the way into the tile; the walking lanes, whose every instruction is paid in full, only widen and add
    s.lay_down(tile, reg, [p](const v4f& v, int) {
      return v4f{static_cast<float>(norm_term<PMODE>(v[0], p)), static_cast<float>(norm_term<PMODE>(v[1], p)),
                 static_cast<float>(norm_term<PMODE>(v[2], p)), static_cast<float>(norm_term<PMODE>(v[3], p))};
    });
    __builtin_amdgcn_wave_barrier();
    if (c0 + s.step < len) s.request(x, c0 + s.step, reg);
    if (s.lane < G) walk_column(mine, 1, s.cols(c0), [&](float a) { acc += static_cast<double>(a); });
    __builtin_amdgcn_wave_barrier();
  }
  if (s.lane < G) divisors[wave][s.lane] = norm_finish<PMODE>(acc, p, eps);
  __builtin_amdgcn_wave_barrier();

  for (uint32_t c0 = 0; c0 < len; c0 += s.step) {
    s.request(x, c0, reg);
#pragma unroll
    for (int i = 0; i < kStreamVectors; ++i) {
      const uint32_t n = s.count(i, c0);
      if (n == 0) continue;
      const uint32_t g = S::row_of(s.lane, i), c = c0 + S::col_of(s.lane, i);
      const float div = divisors[wave][g];
      v4f q = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int k = 0; k < 4; ++k)
        if (static_cast<uint32_t>(k) < n) q[k] = ssd_scaled<SM>(reg[i][k] / div, scale, c + k);  // scale[] ends with the row
      float* dst = y + static_cast<uint64_t>(s.row0 + g) * len + c;
      if (n == 4) {
        store4_stream_any(dst, q);
      } else {
#pragma unroll
        for (int k = 0; k < 3; ++k)
          if (static_cast<uint32_t>(k) < n) dst[k] = q[k];
      }
    }
  }
}

constexpr int kRowsSmallTile = 2048;  // floats per wave: 16 waves per CU
constexpr int kRowsMinRows = 1024;                          // fewer rows: a workgroup per row keeps more lanes busy

static bool rows_apply(int outer_num, int dim, int inner_num) {
  return inner_num == 1 && static_cast<uint32_t>(dim) >= kRowsMinDim && outer_num >= kRowsMinRows;
}

// Normalize: from this row length on the rows move in chunks, G rows per wave (512: 34 us against 47 per 51 MB).
// Softmax stays with the rows in LDS while two rows fit a wave's tile (1000: 49 us; in chunks 62, since the
// exponentials then have to be taken twice) and with a workgroup per row beyond (4096: 62 us; in chunks 94).
constexpr int kRowsStreamMinDim = 401;
constexpr int kRowsSoftmaxMaxDim = 1023;

// Rows per wave of the streaming kernels: as many as still leave a thousand waves.
static int stream_rows(uint32_t rows, uint32_t len) {
  int best = 4;
  uint64_t best_cost = ~0ull;
  for (int g = 4; g <= 64; g *= 2) {
    if (g > 4 && rows / static_cast<uint32_t>(g) < 1024u) break;
    const uint32_t w = 256u * kStreamVectors / static_cast<uint32_t>(g);
    const uint64_t cost = static_cast<uint64_t>((len + w - 1) / w) * w;  // vector slots a row takes, filled or not
    if (cost <= best_cost) best = g, best_cost = cost;
  }
  return best;
}

template <int PMODE, int SM>
static void launch_normalize_rows_stream(uint32_t rows, uint32_t len, float p, float eps, const float* x,
                                         const float* scale, float* y, hipStream_t st) {
  const int g = stream_rows(rows, len);
  const uint32_t per_wg = static_cast<uint32_t>(g) * (kBlock / kWave), grid = (rows + per_wg - 1) / per_wg;
  switch (g) {
    case 64: normalize_rows_stream_kernel<PMODE, SM, 64><<<grid, kBlock, 0, st>>>(x, y, rows, len, p, eps, scale); break;
    case 32: normalize_rows_stream_kernel<PMODE, SM, 32><<<grid, kBlock, 0, st>>>(x, y, rows, len, p, eps, scale); break;
    case 8: normalize_rows_stream_kernel<PMODE, SM, 8><<<grid, kBlock, 0, st>>>(x, y, rows, len, p, eps, scale); break;
    case 16: normalize_rows_stream_kernel<PMODE, SM, 16><<<grid, kBlock, 0, st>>>(x, y, rows, len, p, eps, scale); break;
    default: normalize_rows_stream_kernel<PMODE, SM, 4><<<grid, kBlock, 0, st>>>(x, y, rows, len, p, eps, scale);
  }
}

// Quads of positions with their columns in registers: how many there are, 0 where the quad kernels do not apply.
constexpr int kQuadMaxDim = 4, kQuadMinInner = 16;
constexpr int kShortRowsMaxDim = 16;  // rows of up to this many elements: four to a lane
constexpr int kShortSlabMax = 9;      // slabs of dim * inner floats, inner > 1, likewise
static uint32_t quad_count(int outer_num, int dim, int inner_num, bool softmax, FastDiv* f_quads) {
  // Measured against the column-per-lane and packed kernels (per 51 MB): ahead where the per-column
  // work is small against a lane's set-up, behind from five rows on (softmax [512,8,3136] 32 us against 21)
  // and where a slab has fewer than four quads (the lanes of a wave then scatter over many lines).
  const bool whole = inner_num % 4 == 0;
  const bool apply = softmax ? (dim <= 3 || (dim == 4 && whole)) : (dim <= 2 && whole);
  if (!apply || inner_num < kQuadMinInner) return 0;
  const uint32_t per_slab = (static_cast<uint32_t>(inner_num) + 3) / 4;
  *f_quads = make_fastdiv(per_slab);
  return static_cast<uint32_t>(outer_num) * per_slab;  // at most the number of columns
}

template <int PMODE, int SM>
static void launch_normalize_quads(uint32_t quads, FastDiv fq, int dim, int inner_num, float p, float eps, const float* x,
                                   const float* scale, float* y, hipStream_t st) {
  const uint32_t d = static_cast<uint32_t>(dim), inner = static_cast<uint32_t>(inner_num);
  normalize_quads_reg_kernel<PMODE, kQuadMaxDim, SM><<<grid_for(quads), kBlock, 0, st>>>(x, y, quads, d, inner, fq, p, eps, scale);
}

static uint32_t rows_grid(uint32_t rows, const WaveRows& w) {
  const uint32_t per_group = w.rows_per_wave * (kBlock / kWave);
  return (rows + per_group - 1) / per_group;
}

template <int PMODE, int SM>
static void launch_normalize_rows(int outer_num, int dim, float p, float eps, const float* x, const float* scale,
                                  float* y, hipStream_t st) {
  WaveRows w;
  const uint32_t rows = static_cast<uint32_t>(outer_num);
  if (dim < kRowsStreamMinDim && wave_rows<kRowsSmallTile>(dim, &w))
    normalize_rows_kernel<PMODE, SM, kRowsSmallTile><<<rows_grid(rows, w), kBlock, 0, st>>>(x, y, rows, w, p, eps, scale);
  else
    launch_normalize_rows_stream<PMODE, SM>(rows, static_cast<uint32_t>(dim), p, eps, x, scale, y, st);
}

// ---------------------------------------------------------------------------
// Tall columns: more rows than the tile kernels hold in LDS and, with that, few
// columns (a softmax over 1000 or 4096 channels of a 56x56 map has 3136 per
// image), which a lane per column leaves to a handful of waves.  Here a
// workgroup owns 16, 32 or 64 neighbouring positions of one outer index and
// moves down their rows in chunks of 4096 floats with all 256 lanes.  The
// maxima are folded in any order (see softmax_slab_kernel); the ordered sums are
// walked by one lane per column out of LDS, chunk after chunk, while the loads
// of the next chunk are in flight.  x is read once per pass (Softmax: maxima,
// sums, quotients; Normalize: sums, quotients), y written once.
// ---------------------------------------------------------------------------
constexpr uint32_t kTallChunkFloats = 4096;
constexpr uint32_t kTallMinInner = 16;
constexpr int kTallAhead = 4;  // chunks requested at a time by the passes that only stream

// A lane takes four neighbouring positions of a row with one 128-bit access on
// whatever dword address they have (rows of 49 or 1001 positions start anywhere);
// where the row ends inside the four, the ones that exist move one by one.
struct TallTile {
  static constexpr int kLoads = 4;  // vectors per lane and chunk
  uint32_t dim, inner, width, rows_per_sweep, chunk_rows, row0, col;
  uint32_t valid;  // how many of the lane's four positions exist (the last tile of a row may be cut)
  uint64_t base;   // of (outer index, row 0, the lane's first position)

  SHDW_DEVICE TallTile(uint32_t dim_, uint32_t inner_, uint32_t width_log2, FastDiv f_tiles) {
    dim = dim_, inner = inner_, width = 1u << width_log2;
    const uint32_t lanes_log2 = width_log2 - 2;  // lanes per row of the tile
    rows_per_sweep = kBlock >> lanes_log2;
    chunk_rows = rows_per_sweep * kLoads;
    row0 = threadIdx.x >> lanes_log2;
    col = (threadIdx.x & ((1u << lanes_log2) - 1)) * 4;
    uint32_t n, tile;
    fd_divmod(xcd_contiguous(blockIdx.x, gridDim.x), f_tiles, n, tile);  // neighbours share cache lines
    const uint32_t p = tile * width + col;
    valid = p < inner ? min(4u, inner - p) : 0u;
    base = static_cast<uint64_t>(n) * dim * inner + p;
  }
  SHDW_DEVICE uint32_t chunks() const { return (dim + chunk_rows - 1) / chunk_rows; }
  SHDW_DEVICE uint32_t rows_in(uint32_t k) const { return min(chunk_rows, dim - k * chunk_rows); }
  SHDW_DEVICE uint32_t row(uint32_t k, int i) const { return k * chunk_rows + i * rows_per_sweep + row0; }
  SHDW_DEVICE bool has(uint32_t k, int i) const { return valid > 0 && row(k, i) < dim; }
  SHDW_DEVICE uint32_t slot(int i) const { return (i * rows_per_sweep + row0) * width + col; }
  SHDW_DEVICE void load(const float* x, uint32_t k, v4f (&v)[kLoads]) const {
#pragma unroll
    for (int i = 0; i < kLoads; ++i)
      if (has(k, i)) {
        const float* src = x + base + static_cast<uint64_t>(row(k, i)) * inner;
        if (valid == 4) {
          v[i] = load4_stream_any(src);
        } else {
#pragma unroll
          for (int e = 0; e < 3; ++e)
            if (static_cast<uint32_t>(e) < valid) v[i][e] = __builtin_nontemporal_load(src + e);
        }
      }
  }
  SHDW_DEVICE void store(float* y, uint32_t r, const v4f& q) const {
    float* dst = y + base + static_cast<uint64_t>(r) * inner;
    if (valid == 4) {
      store4_stream_any(dst, q);
    } else {
#pragma unroll
      for (int e = 0; e < 3; ++e)
        if (static_cast<uint32_t>(e) < valid) dst[e] = q[e];
    }
  }
};

__global__ __launch_bounds__(kBlock) void softmax_tall_kernel(const float* x, float* y, uint32_t dim,
                                                               uint32_t inner, uint32_t width_log2,
                                                               FastDiv f_tiles) {
  using T = TallTile;
  __shared__ __align__(16) float chunk[2][kTallChunkFloats];
  __shared__ __align__(16) float stat[64];
  __shared__ uint64_t tab[32];
  if (threadIdx.x < 32) tab[threadIdx.x] = libm::kExp2fTab[threadIdx.x];
  const T t(dim, inner, width_log2, f_tiles);
  const uint32_t chunks = t.chunks();
  v4f v[T::kLoads];

  float part[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) part[e] = -FLT_MAX;
  for (uint32_t k = 0; k < chunks; k += kTallAhead) {  // chunks past the end hold no rows
    v4f w[kTallAhead][T::kLoads];
#pragma unroll
    for (int j = 0; j < kTallAhead; ++j) t.load(x, k + j, w[j]);
#pragma unroll
    for (int j = 0; j < kTallAhead; ++j)
#pragma unroll
      for (int i = 0; i < T::kLoads; ++i)
        if (t.has(k + j, i))
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (static_cast<uint32_t>(e) < t.valid) part[e] = std_max(w[j][i][e], part[e]);
  }
  *reinterpret_cast<v4f*>(chunk[0] + t.row0 * t.width + t.col) = v4f{part[0], part[1], part[2], part[3]};
  __syncthreads();
  if (threadIdx.x < t.width) {
    float m = -FLT_MAX;
    for (uint32_t r = 0; r < t.rows_per_sweep; ++r) m = std_max(chunk[0][r * t.width + threadIdx.x], m);
    stat[threadIdx.x] = m;
  }
  __syncthreads();
  const v4f max_val = *reinterpret_cast<const v4f*>(stat + t.col);

  float sum = 0.f;
  // chunk k: its exponentials into LDS by all lanes, then the walk by one lane per
  // column while the loads of chunk k + 2 fly.  Two buffers: the slowest walker is
  // at most one chunk behind.  Positions past the end of a row hold whatever the
  // lanes had; their sums are never used.
  auto pass = [&](uint32_t k, v4f(&reg)[T::kLoads]) {
    float* buf = chunk[k & 1];
#pragma unroll
    for (int i = 0; i < T::kLoads; ++i)
      if (t.has(k, i)) {
        v4f ex;
#pragma unroll
        for (int e = 0; e < 4; ++e) ex[e] = libm::exact_expf(reg[i][e] - max_val[e], tab);
        *reinterpret_cast<v4f*>(buf + t.slot(i)) = ex;
      }
    __syncthreads();
    t.load(x, k + 2, reg);
    if (threadIdx.x < t.width) walk_column_tile(buf + threadIdx.x, t.width, t.rows_in(k), [&](float a) { sum += a; });
  };
  v4f v2[T::kLoads];
  t.load(x, 0, v);
  t.load(x, 1, v2);
  for (uint32_t k = 0; k < chunks; k += 2) {
    pass(k, v);
    if (k + 1 < chunks) pass(k + 1, v2);
  }
  __syncthreads();
  if (threadIdx.x < t.width) stat[threadIdx.x] = sum;
  __syncthreads();
  const v4f total = *reinterpret_cast<const v4f*>(stat + t.col);

  for (uint32_t k = 0; k < chunks; k += kTallAhead) {
    v4f w[kTallAhead][T::kLoads];
#pragma unroll
    for (int j = 0; j < kTallAhead; ++j) t.load(x, k + j, w[j]);
#pragma unroll
    for (int j = 0; j < kTallAhead; ++j)
#pragma unroll
      for (int i = 0; i < T::kLoads; ++i)
        if (t.has(k + j, i)) {
          v4f q;
#pragma unroll
          for (int e = 0; e < 4; ++e) q[e] = libm::exact_expf(w[j][i][e] - max_val[e], tab) / total[e];
          t.store(y, t.row(k + j, i), q);
        }
  }
}

template <int PMODE, int SM>
__global__ __launch_bounds__(kBlock) void normalize_tall_kernel(const float* x, float* y, uint32_t dim,
                                                                 uint32_t inner, uint32_t width_log2,
                                                                 FastDiv f_tiles, float p, float eps,
                                                                 const float* scale) {
  using T = TallTile;
  __shared__ __align__(16) float chunk[2][kTallChunkFloats];
  __shared__ __align__(16) float stat[64];
  const T t(dim, inner, width_log2, f_tiles);
  const uint32_t chunks = t.chunks();
  v4f v[T::kLoads];

  double acc = 0;
  auto pass = [&](uint32_t k, v4f(&reg)[T::kLoads]) {  // as in softmax_tall_kernel
    float* buf = chunk[k & 1];
#pragma unroll
    for (int i = 0; i < T::kLoads; ++i)
      if (t.has(k, i)) {
        v4f term;
#pragma unroll
        for (int e = 0; e < 4; ++e) term[e] = static_cast<float>(norm_term<PMODE>(reg[i][e], p));
        *reinterpret_cast<v4f*>(buf + t.slot(i)) = term;
      }
    __syncthreads();
    t.load(x, k + 2, reg);
    if (threadIdx.x < t.width)
      walk_column_tile(buf + threadIdx.x, t.width, t.rows_in(k), [&](float a) { acc += static_cast<double>(a); });
  };
  v4f v2[T::kLoads];
  t.load(x, 0, v);
  t.load(x, 1, v2);
  for (uint32_t k = 0; k < chunks; k += 2) {
    pass(k, v);
    if (k + 1 < chunks) pass(k + 1, v2);
  }
  __syncthreads();
  if (threadIdx.x < t.width) stat[threadIdx.x] = norm_finish<PMODE>(acc, p, eps);
  __syncthreads();
  const v4f div = *reinterpret_cast<const v4f*>(stat + t.col);

  for (uint32_t k = 0; k < chunks; k += kTallAhead) {
    v4f w[kTallAhead][T::kLoads];
#pragma unroll
    for (int j = 0; j < kTallAhead; ++j) t.load(x, k + j, w[j]);
#pragma unroll
    for (int j = 0; j < kTallAhead; ++j)
#pragma unroll
      for (int i = 0; i < T::kLoads; ++i)
        if (t.has(k + j, i)) {
          const uint32_t r = t.row(k + j, i);
          v4f q;
#pragma unroll
          for (int e = 0; e < 4; ++e) q[e] = ssd_scaled<SM>(w[j][i][e] / div[e], scale, r);
          t.store(y, r, q);
        }
  }
}

// ---------------------------------------------------------------------------
// Long slabs: columns of thousands of rows over fewer than 16 positions
// ([448][4096][7]).  The slab of an outer index is contiguous but too large to
// stay in LDS with more than one workgroup per CU (112 KB here), so it moves
// through LDS in chunks of whole rows, at most 4096 floats, as the tall kernels'
// tiles do.  A chunk is a multiple of inner floats long, so the k-th element of
// every chunk has the same position, and a lane, which always takes the same
// elements of a chunk, keeps the statistics of its sixteen positions in
// registers.
// ---------------------------------------------------------------------------
constexpr int kLongLoads = kTallChunkFloats / 4 / kBlock;  // 128-bit loads per lane and chunk
static_assert(kLongLoads == 4, "a chunk is four vectors per lane");

struct LongSlab {
  uint32_t dim, inner, chunk_rows, chunk_cells;
  const float* xs;
  float* ys;
  SHDW_DEVICE LongSlab(const float* x, float* y, uint32_t dim_, uint32_t inner_) {
    dim = dim_, inner = inner_;
    chunk_rows = kTallChunkFloats / inner, chunk_cells = chunk_rows * inner;
    const uint64_t slab = static_cast<uint64_t>(blockIdx.x) * dim * inner;
    xs = x + slab, ys = y + slab;
  }
  SHDW_DEVICE uint32_t chunks() const { return (dim + chunk_rows - 1) / chunk_rows; }
  SHDW_DEVICE uint32_t rows_in(uint32_t k) const {
    const uint32_t r0 = k * chunk_rows;
    return r0 < dim ? min(chunk_rows, dim - r0) : 0u;  // chunks past the end hold nothing
  }
  SHDW_DEVICE uint32_t cells_in(uint32_t k) const { return rows_in(k) * inner; }
  SHDW_DEVICE static uint32_t first(int i) { return 4 * (threadIdx.x + kBlock * i); }  // of vector i, in the chunk
  SHDW_DEVICE void load(uint32_t k, v4f (&v)[kLongLoads]) const {
    const uint32_t cells = cells_in(k);
    const float* src = xs + static_cast<uint64_t>(k) * chunk_cells;
#pragma unroll
    for (int i = 0; i < kLongLoads; ++i) {
      const uint32_t e = first(i);
      if (e + 4 <= cells) {
        v[i] = load4_stream_any(src + e);
      } else {
#pragma unroll
        for (int j = 0; j < 3; ++j)
          if (e + j < cells) v[i][j] = __builtin_nontemporal_load(src + e + j);
      }
    }
  }
  // q(value, vector i, element j, row in the slab) for the lane's elements of chunk k, then stored
  template <class Q>
  SHDW_DEVICE void store(uint32_t k, const v4f (&v)[kLongLoads], Q q) const {
    const uint32_t cells = cells_in(k);
    float* dst = ys + static_cast<uint64_t>(k) * chunk_cells;
#pragma unroll
    for (int i = 0; i < kLongLoads; ++i) {
      const uint32_t e = first(i);
      if (e >= cells) continue;
      v4f r;
#pragma unroll
      for (int j = 0; j < 4; ++j) r[j] = q(v[i][j], i, j);
      if (e + 4 <= cells) {
        store4_stream_any(dst + e, r);
      } else {
#pragma unroll
        for (int j = 0; j < 3; ++j)
          if (e + j < cells) dst[e + j] = r[j];
      }
    }
  }
};

__global__ __launch_bounds__(kBlock) void softmax_long_slab_kernel(const float* x, float* y, uint32_t dim,
                                                                    FastDiv f_inner) {
  __shared__ __align__(16) float chunk[2][kTallChunkFloats];
  __shared__ float stat[kBlock];
  __shared__ uint64_t tab[32];
  if (threadIdx.x < 32) tab[threadIdx.x] = libm::kExp2fTab[threadIdx.x];
  const LongSlab t(x, y, dim, f_inner.d);
  const uint32_t chunks = t.chunks(), inner = t.inner;
  uint32_t pos[kLongLoads][4];
#pragma unroll
  for (int i = 0; i < kLongLoads; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t e = LongSlab::first(i) + j;
      pos[i][j] = e - fd_div(e, f_inner) * inner;
    }
  v4f v[kLongLoads], v2[kLongLoads];

  // maxima in any order (see softmax_slab_kernel): per element slot of the chunk, then per position
  float part[kLongLoads][4];
#pragma unroll
  for (int i = 0; i < kLongLoads; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) part[i][j] = -FLT_MAX;
  auto fold_max = [&](uint32_t k, const v4f(&reg)[kLongLoads]) {
    const uint32_t cells = t.cells_in(k);
#pragma unroll
    for (int i = 0; i < kLongLoads; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (LongSlab::first(i) + j < cells) part[i][j] = std_max(reg[i][j], part[i][j]);
  };
  for (uint32_t k = 0; k < chunks; k += 2) {
    t.load(k, v);
    t.load(k + 1, v2);
    fold_max(k, v);
    fold_max(k + 1, v2);
  }
#pragma unroll
  for (int i = 0; i < kLongLoads; ++i)
    *reinterpret_cast<v4f*>(chunk[0] + LongSlab::first(i)) = v4f{part[i][0], part[i][1], part[i][2], part[i][3]};
  __syncthreads();
  if (threadIdx.x < inner) {
    float m = -FLT_MAX;
    walk_column_inner(chunk[0] + threadIdx.x, inner, t.chunk_rows, [&](float a) { m = std_max(a, m); });
    stat[threadIdx.x] = m;
  }
  __syncthreads();
  float max_val[kLongLoads][4];
#pragma unroll
  for (int i = 0; i < kLongLoads; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) max_val[i][j] = stat[pos[i][j]];

  // exponentials of a chunk into LDS by all lanes, ordered sums by one lane per position
  float sum = 0.f;
  auto pass = [&](uint32_t k, v4f(&reg)[kLongLoads]) {
    float* buf = chunk[k & 1];
#pragma unroll
    for (int i = 0; i < kLongLoads; ++i) {
      v4f ex;
#pragma unroll
      for (int j = 0; j < 4; ++j) ex[j] = libm::exact_expf(reg[i][j] - max_val[i][j], tab);
      *reinterpret_cast<v4f*>(buf + LongSlab::first(i)) = ex;  // slots past the chunk's cells are never walked
    }
    __syncthreads();
    t.load(k + 2, reg);
    if (threadIdx.x < inner) walk_column_inner(buf + threadIdx.x, inner, t.rows_in(k), [&](float a) { sum += a; });
  };
  t.load(0, v);
  t.load(1, v2);
  for (uint32_t k = 0; k < chunks; k += 2) {
    pass(k, v);
    if (k + 1 < chunks) pass(k + 1, v2);
  }
  __syncthreads();
  if (threadIdx.x < inner) stat[threadIdx.x] = sum;
  __syncthreads();
  float total[kLongLoads][4];
#pragma unroll
  for (int i = 0; i < kLongLoads; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) total[i][j] = stat[pos[i][j]];

  for (uint32_t k = 0; k < chunks; k += 2) {
    t.load(k, v);
    t.load(k + 1, v2);
    auto quotient = [&](float a, int i, int j) { return libm::exact_expf(a - max_val[i][j], tab) / total[i][j]; };
    t.store(k, v, quotient);
    t.store(k + 1, v2, quotient);
  }
}

template <int PMODE, int SM>
__global__ __launch_bounds__(kBlock) void normalize_long_slab_kernel(const float* x, float* y, uint32_t dim,
                                                                      FastDiv f_inner, float p, float eps,
                                                                      const float* scale) {
  __shared__ __align__(16) float chunk[2][kTallChunkFloats];
  __shared__ float stat[kBlock];
  const LongSlab t(x, y, dim, f_inner.d);
  const uint32_t chunks = t.chunks(), inner = t.inner;
  uint32_t pos[kLongLoads][4], row[kLongLoads][4];  // position and row inside a chunk of the lane's elements
#pragma unroll
  for (int i = 0; i < kLongLoads; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t e = LongSlab::first(i) + j;
      row[i][j] = fd_div(e, f_inner);
      pos[i][j] = e - row[i][j] * inner;
    }
  v4f v[kLongLoads], v2[kLongLoads];

  double acc = 0;
  auto pass = [&](uint32_t k, v4f(&reg)[kLongLoads]) {  // as in softmax_long_slab_kernel
    float* buf = chunk[k & 1];
#pragma unroll
    for (int i = 0; i < kLongLoads; ++i) {
      v4f term;
#pragma unroll
      for (int j = 0; j < 4; ++j) term[j] = static_cast<float>(norm_term<PMODE>(reg[i][j], p));
      *reinterpret_cast<v4f*>(buf + LongSlab::first(i)) = term;
    }
    __syncthreads();
    t.load(k + 2, reg);
    if (threadIdx.x < inner)
      walk_column_inner(buf + threadIdx.x, inner, t.rows_in(k), [&](float a) { acc += static_cast<double>(a); });
  };
  t.load(0, v);
  t.load(1, v2);
  for (uint32_t k = 0; k < chunks; k += 2) {
    pass(k, v);
    if (k + 1 < chunks) pass(k + 1, v2);
  }
  __syncthreads();
  if (threadIdx.x < inner) stat[threadIdx.x] = norm_finish<PMODE>(acc, p, eps);
  __syncthreads();
  float div[kLongLoads][4];
#pragma unroll
  for (int i = 0; i < kLongLoads; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) div[i][j] = stat[pos[i][j]];

  for (uint32_t k = 0; k < chunks; k += 2) {
    t.load(k, v);
    t.load(k + 1, v2);
    t.store(k, v, [&](float a, int i, int j) { return ssd_scaled<SM>(a / div[i][j], scale, k * t.chunk_rows + row[i][j]); });
    t.store(k + 1, v2,
            [&](float a, int i, int j) { return ssd_scaled<SM>(a / div[i][j], scale, (k + 1) * t.chunk_rows + row[i][j]); });
  }
}

// Slabs from this size on take the long-slab kernels where inner < 16 (smaller ones
// stay whole in LDS: softmax_slab_kernel, normalize_slab_kernel).
constexpr int64_t kLongSlabMinFloats = kSlabMaxFloats;

// ... and where inner >= 16 with a few hundred slabs to hand out, one per workgroup: rows that do not
// start on 64-byte boundaries (inner not a multiple of 16) cost the tall and tile kernels, which cut every
// row into pieces of 16 to 64 positions, up to half their speed, and the slab moves as it lies
// ([513,1000,25] softmax 101 -> 68 us per 51 MB, normalize 76 -> 45; [511,513,49] 79 -> 56, 55 -> 37).
// Normalize gains on aligned rows too ([782,513,32] 46 -> 36); Softmax does not ([782,513,32] 59 -> 71).
constexpr int kLongSlabMinSlabs = 192, kLongSlabMinSlabsAligned = 384;
static bool long_slab(int outer_num, int dim, int inner_num, bool softmax) {
  if (static_cast<int64_t>(dim) * inner_num <= kLongSlabMinFloats) return false;
  if (static_cast<uint32_t>(inner_num) < kTallMinInner) return true;
  if (inner_num > kBlock) return false;  // a lane per position walks the sums
  if (tile_fits(dim, inner_num, softmax)) return false;  // the tile kernels are ahead where they apply ([256,256,196]: 32 us, 65 us here)
  if (inner_num % 16 != 0) return outer_num >= kLongSlabMinSlabs;
  return !softmax && outer_num >= kLongSlabMinSlabsAligned;
}

// Where the tall kernels apply, and their launch: positions per workgroup as wide
// as still leaves a thousand workgroups.
struct TallLaunch {
  uint32_t grid, width_log2;
  FastDiv f_tiles;
};

static bool tall_launch(int outer_num, int dim, int inner_num, TallLaunch* t) {
  if (static_cast<uint32_t>(inner_num) < kTallMinInner || dim < 128) return false;
  uint32_t w = 6;
  while (w > 4 && static_cast<uint64_t>(outer_num) * ((inner_num + (1u << w) - 1) >> w) < 1024) --w;
  const uint32_t tiles = (static_cast<uint32_t>(inner_num) + (1u << w) - 1) >> w;
  t->grid = static_cast<uint32_t>(outer_num) * tiles;
  t->width_log2 = w;
  t->f_tiles = make_fastdiv(tiles);
  return true;
}

template <int PMODE, int SM>
static void launch_normalize_tall(const TallLaunch& t, int dim, int inner_num, float p, float eps, const float* x,
                                  const float* scale, float* y, hipStream_t st) {
  normalize_tall_kernel<PMODE, SM><<<t.grid, kBlock, 0, st>>>(x, y, static_cast<uint32_t>(dim),
                                                              static_cast<uint32_t>(inner_num), t.width_log2,
                                                              t.f_tiles, p, eps, scale);
}

// Shared launch geometry: slab layout when the columns are too narrow to
// coalesce and one slab (plus its statistics) fits the LDS budget.
struct ColumnGeometry {
  bool use_slab;
  uint32_t columns, slab_bytes;
};

// Slabs per workgroup of the packed kernels, 0 where they do not apply (a slab
// of more than a quarter of the tile stays with one workgroup per slab).
static uint32_t packed_group(int dim, int inner_num) {
  if (inner_num >= 64) return 0;
  const uint64_t pitch = static_cast<uint64_t>(inner_num) * (static_cast<uint32_t>(dim) | 1u);
  if (pitch * 4 > kPackedTileFloats) return 0;
  // (more than 256 columns to a workgroup, a lane walking several, measured slower for every dim but 2:
  // softmax over [1.6M,8]: 33 -> 48 us per 51 MB with 1024 columns)
  uint32_t group = std::min<uint32_t>(kBlock / inner_num, kPackedTileFloats / static_cast<uint32_t>(pitch));
  group &= ~3u;  // whole 128-bit pieces per workgroup
  // the walks are done by group * inner lanes: under 32 of them (rows of 512 and
  // more with inner = 1) the slab kernels' all-lane forms do better
  return group * inner_num >= 32 ? group : 0;
}

static size_t packed_bytes(int dim, int inner_num, uint32_t group) {
  return static_cast<size_t>(group) * inner_num * (static_cast<uint32_t>(dim) | 1u) * sizeof(float);
}

// Which family of kernels a shape goes to, for shdw_hip_softmax_plan and its
// siblings: the entry points below decide as they always do and, asked for a
// report, hand the decision back instead of launching.
struct ColumnPlan {
  int path = SHDW_PATH_NONE, variant = 0;
  uint32_t grid = 0;
  bool want = false;  // report only
  // true: the caller returns without launching
  bool chosen(int p, int v, uint32_t g) {
    path = p, variant = v, grid = g;
    return want;
  }
};

static int column_geometry(int outer_num, int dim, int inner_num, ColumnGeometry* g) {
  if (outer_num < 0 || dim < 0 || inner_num < 0) return SHDW_E_INVALID_ARGUMENT;
  const int64_t columns = static_cast<int64_t>(outer_num) * inner_num;
  const int64_t count = columns * dim;
  if (count > INT32_MAX || columns > INT32_MAX) return SHDW_E_INVALID_ARGUMENT;
  g->columns = static_cast<uint32_t>(columns);
  const int64_t slab = static_cast<int64_t>(dim) * inner_num;
  g->use_slab = inner_num < 64 && slab + inner_num <= kSlabMaxFloats;
  g->slab_bytes = static_cast<uint32_t>((slab + inner_num) * sizeof(float));
  return SHDW_OK;
}

// What launch_normalize_rows and launch_normalize_tile would launch.
static int report_normalize_rows(int outer_num, int dim, ColumnPlan* pl) {
  WaveRows w;
  const uint32_t rows = static_cast<uint32_t>(outer_num);
  if (dim < kRowsStreamMinDim && wave_rows<kRowsSmallTile>(dim, &w)) {
    pl->chosen(SHDW_PATH_ROWS, static_cast<int>(w.rows_per_wave), rows_grid(rows, w));
  } else {
    const int g = stream_rows(rows, static_cast<uint32_t>(dim));
    const uint32_t per_wg = static_cast<uint32_t>(g) * (kBlock / kWave);
    pl->chosen(SHDW_PATH_ROWS_STREAM, g, (rows + per_wg - 1) / per_wg);
  }
  return SHDW_OK;
}

static int normalize_tile_shift(int dim) {
  return dim * 64 * sizeof(float) <= kTileLdsBytes / 2 ? 6 : (dim * 32 * sizeof(float) <= kTileLdsBytes ? 5 : 4);
}

static int report_normalize_tile(int outer_num, int dim, int inner_num, ColumnPlan* pl) {
  const int shift = normalize_tile_shift(dim);
  const uint32_t tiles = (static_cast<uint32_t>(inner_num) + (1u << shift) - 1) >> shift;
  pl->chosen(SHDW_PATH_TILE, shift, static_cast<uint32_t>(outer_num) * tiles);
  return SHDW_OK;
}

static int run_softmax(int outer_num, int dim, int inner_num, const float* x, float* y, hipStream_t st,
                       ColumnPlan* pl) {
  ColumnGeometry g;
  const int rc = column_geometry(outer_num, dim, inner_num, &g);
  if (rc != SHDW_OK) return rc;
  if (g.columns == 0 || dim == 0) return SHDW_OK;
  if (!pl->want && (!x || !y)) return SHDW_E_INVALID_ARGUMENT;
  const FastDiv fi = make_fastdiv(static_cast<uint32_t>(inner_num));
  if (WaveRows w; rows_apply(outer_num, dim, inner_num) && dim <= kRowsSoftmaxMaxDim &&
                  wave_rows<kRowsSmallTile>(dim, &w)) {
    const uint32_t rows = static_cast<uint32_t>(outer_num);
    if (pl->chosen(SHDW_PATH_ROWS, static_cast<int>(w.rows_per_wave), rows_grid(rows, w))) return SHDW_OK;
    softmax_rows_kernel<kRowsSmallTile><<<pl->grid, kBlock, 0, st>>>(x, y, rows, w);
    return launch_status();
  }
  // slabs with inner > 1 walk their columns in loops, one exponential after the other: ahead of the packed
  // kernel up to nine floats ([3.2M,2,2] 58 -> 27 us per 51 MB, [1.4M,3,3] 40 -> 34), behind from twelve on
  if (dim >= 2 && inner_num <= kShortSlabMax / 2 && dim * inner_num <= (inner_num == 1 ? kShortRowsMaxDim : kShortSlabMax) &&
      outer_num >= kRowsMinRows) {
    const uint32_t rows = static_cast<uint32_t>(outer_num);
    const uint64_t per_group = 4ull * kBlock;  // rows (slabs) of a workgroup
    const uint32_t grid = static_cast<uint32_t>((rows + per_group - 1) / per_group);
    const uint32_t d = static_cast<uint32_t>(dim), inner = static_cast<uint32_t>(inner_num);
    if (pl->chosen(SHDW_PATH_SHORT_ROWS, dim * inner_num, grid)) return SHDW_OK;
    switch (dim * inner_num) {
#define SHDW_SHORT_ROWS(D) case D: softmax_short_rows_kernel<D><<<grid, kBlock, 0, st>>>(x, y, rows, d, inner); break;
      SHDW_SHORT_ROWS(2) SHDW_SHORT_ROWS(3) SHDW_SHORT_ROWS(4) SHDW_SHORT_ROWS(5) SHDW_SHORT_ROWS(6)
      SHDW_SHORT_ROWS(7) SHDW_SHORT_ROWS(8) SHDW_SHORT_ROWS(9) SHDW_SHORT_ROWS(10) SHDW_SHORT_ROWS(11)
      SHDW_SHORT_ROWS(12) SHDW_SHORT_ROWS(13) SHDW_SHORT_ROWS(14) SHDW_SHORT_ROWS(15) SHDW_SHORT_ROWS(16)
#undef SHDW_SHORT_ROWS
    }
    return launch_status();
  }
  if (FastDiv fq; const uint32_t quads = quad_count(outer_num, dim, inner_num, true, &fq)) {
    const uint32_t d = static_cast<uint32_t>(dim), inner = static_cast<uint32_t>(inner_num);
    if (pl->chosen(SHDW_PATH_QUADS, 0, grid_for(quads))) return SHDW_OK;
    softmax_quads_reg_kernel<kQuadMaxDim><<<pl->grid, kBlock, 0, st>>>(x, y, quads, d, inner, fq);
    return launch_status();
  }
  if (const uint32_t group = packed_group(dim, inner_num)) {
    const uint32_t slabs = static_cast<uint32_t>(outer_num);
    if (pl->chosen(SHDW_PATH_PACKED, static_cast<int>(group), (slabs + group - 1) / group)) return SHDW_OK;
    softmax_packed_kernel<<<pl->grid, kBlock, packed_bytes(dim, inner_num, group), st>>>(
        x, y, slabs, static_cast<uint32_t>(dim), fi, make_fastdiv(static_cast<uint32_t>(dim) * inner_num), group);
  } else if (long_slab(outer_num, dim, inner_num, true)) {
    if (pl->chosen(SHDW_PATH_LONG_SLAB, 0, static_cast<uint32_t>(outer_num))) return SHDW_OK;
    softmax_long_slab_kernel<<<outer_num, kBlock, 0, st>>>(x, y, static_cast<uint32_t>(dim), fi);
  } else if (g.use_slab) {
    if (pl->chosen(SHDW_PATH_SLAB, 0, static_cast<uint32_t>(outer_num))) return SHDW_OK;
    softmax_slab_kernel<<<outer_num, kBlock, g.slab_bytes, st>>>(x, y, static_cast<uint32_t>(dim), fi);
  } else if (dim <= 64) {
    // the tile kernel is slower here: [64,49,128,128] 115 us against 88
    const uint32_t grid = grid_for(g.columns), d = static_cast<uint32_t>(dim);
    const int dmax = dim <= 16 ? 16 : (dim <= 32 ? 32 : (dim <= 48 ? 48 : 64));
    if (pl->chosen(SHDW_PATH_COLUMNS_REG, dmax, grid)) return SHDW_OK;
    if (dmax == 16)
      softmax_columns_reg_kernel<16, 0><<<grid, kBlock, 0, st>>>(x, y, g.columns, d, fi);
    else if (dmax == 32)
      softmax_columns_reg_kernel<32, 16><<<grid, kBlock, 0, st>>>(x, y, g.columns, d, fi);
    else if (dmax == 48)
      softmax_columns_reg_kernel<48, 32><<<grid, kBlock, 0, st>>>(x, y, g.columns, d, fi);
    else
      softmax_columns_reg_kernel<64, 48><<<grid, kBlock, 0, st>>>(x, y, g.columns, d, fi);
  } else if (tile_fits(dim, inner_num, true)) {
    // the widest tile (64, 32 or 16 positions) that fits 64 KB beside the table and the hand-over row
    const int shift = dim * 64 * sizeof(float) <= kTileLdsBytes - 1024 ? 6 : (dim * 32 * sizeof(float) <= kTileLdsBytes ? 5 : 4);
    const uint32_t tiles = (static_cast<uint32_t>(inner_num) + (1u << shift) - 1) >> shift;
    if (pl->chosen(SHDW_PATH_TILE, shift, static_cast<uint32_t>(outer_num) * tiles)) return SHDW_OK;
    if (shift == 6) launch_softmax_tile_ts<6>(outer_num, dim, inner_num, x, y, st);
    else if (shift == 5) launch_softmax_tile_ts<5>(outer_num, dim, inner_num, x, y, st);
    else launch_softmax_tile_ts<4>(outer_num, dim, inner_num, x, y, st);
  } else if (TallLaunch t; tall_launch(outer_num, dim, inner_num, &t)) {
    if (pl->chosen(SHDW_PATH_TALL, static_cast<int>(t.width_log2), t.grid)) return SHDW_OK;
    softmax_tall_kernel<<<t.grid, kBlock, 0, st>>>(x, y, static_cast<uint32_t>(dim), static_cast<uint32_t>(inner_num),
                                                   t.width_log2, t.f_tiles);
  } else {
    if (pl->chosen(SHDW_PATH_COLUMNS, 0, (g.columns + kWave - 1) / kWave)) return SHDW_OK;
    softmax_columns_kernel<<<pl->grid, kWave, 0, st>>>(x, y, g.columns, static_cast<uint32_t>(dim), fi);
  }
  return launch_status();
}

static int run_normalize(int outer_num, int dim, int inner_num, float p, float eps, const float* x, float* y,
                         hipStream_t st, ColumnPlan* pl) {
  ColumnGeometry g;
  const int rc = column_geometry(outer_num, dim, inner_num, &g);
  if (rc != SHDW_OK) return rc;
  if (g.columns == 0 || dim == 0) return SHDW_OK;
  if (!pl->want && (!x || !y)) return SHDW_E_INVALID_ARGUMENT;
  const FastDiv fi = make_fastdiv(static_cast<uint32_t>(inner_num));
  const uint32_t d = static_cast<uint32_t>(dim);
  const int mode = p == 1.f ? 1 : (p == 2.f ? 2 : 0);
  if (mode != 0 && rows_apply(outer_num, dim, inner_num)) {
    if (pl->want) return report_normalize_rows(outer_num, dim, pl);
    if (mode == 1) launch_normalize_rows<1, kSsdNoScale>(outer_num, dim, p, eps, x, nullptr, y, st);
    else launch_normalize_rows<2, kSsdNoScale>(outer_num, dim, p, eps, x, nullptr, y, st);
    return launch_status();
  }
  if (FastDiv fq; const uint32_t quads = mode != 0 ? quad_count(outer_num, dim, inner_num, false, &fq) : 0) {
    if (pl->chosen(SHDW_PATH_QUADS, 0, grid_for(quads))) return SHDW_OK;
    if (mode == 1) launch_normalize_quads<1, kSsdNoScale>(quads, fq, dim, inner_num, p, eps, x, nullptr, y, st);
    else launch_normalize_quads<2, kSsdNoScale>(quads, fq, dim, inner_num, p, eps, x, nullptr, y, st);
    return launch_status();
  }
  if (const uint32_t group = packed_group(dim, inner_num)) {
    const uint32_t slabs = static_cast<uint32_t>(outer_num);
    const uint32_t grid = (slabs + group - 1) / group;
    const size_t bytes = packed_bytes(dim, inner_num, group);
    const FastDiv fs = make_fastdiv(d * inner_num);
    if (pl->chosen(SHDW_PATH_PACKED, static_cast<int>(group), grid)) return SHDW_OK;
    if (mode == 1)
      normalize_packed_kernel<1, kSsdNoScale><<<grid, kBlock, bytes, st>>>(x, y, slabs, d, fi, fs, group, p, eps, nullptr);
    else if (mode == 2)
      normalize_packed_kernel<2, kSsdNoScale><<<grid, kBlock, bytes, st>>>(x, y, slabs, d, fi, fs, group, p, eps, nullptr);
    else
      normalize_packed_kernel<0, kSsdNoScale><<<grid, kBlock, bytes, st>>>(x, y, slabs, d, fi, fs, group, p, eps, nullptr);
  } else if (long_slab(outer_num, dim, inner_num, false)) {
    if (pl->chosen(SHDW_PATH_LONG_SLAB, 0, static_cast<uint32_t>(outer_num))) return SHDW_OK;
    if (mode == 1)
      normalize_long_slab_kernel<1, kSsdNoScale><<<outer_num, kBlock, 0, st>>>(x, y, d, fi, p, eps, nullptr);
    else if (mode == 2)
      normalize_long_slab_kernel<2, kSsdNoScale><<<outer_num, kBlock, 0, st>>>(x, y, d, fi, p, eps, nullptr);
    else
      normalize_long_slab_kernel<0, kSsdNoScale><<<outer_num, kBlock, 0, st>>>(x, y, d, fi, p, eps, nullptr);
  } else if (g.use_slab) {
    if (pl->chosen(SHDW_PATH_SLAB, 0, static_cast<uint32_t>(outer_num))) return SHDW_OK;
    if (mode == 1)
      normalize_slab_kernel<1><<<outer_num, kBlock, g.slab_bytes, st>>>(x, y, d, fi, p, eps);
    else if (mode == 2)
      normalize_slab_kernel<2><<<outer_num, kBlock, g.slab_bytes, st>>>(x, y, d, fi, p, eps);
    else
      normalize_slab_kernel<0><<<outer_num, kBlock, g.slab_bytes, st>>>(x, y, d, fi, p, eps);
  } else if (mode != 0 && tile_fits(dim, inner_num, false)) {
    if (pl->want) return report_normalize_tile(outer_num, dim, inner_num, pl);
    if (mode == 1)
      launch_normalize_tile<1, kSsdNoScale>(outer_num, dim, inner_num, p, eps, x, nullptr, y, st);
    else
      launch_normalize_tile<2, kSsdNoScale>(outer_num, dim, inner_num, p, eps, x, nullptr, y, st);
  } else if (dim <= 64 && mode != 0) {
    // p = 1 and p = 2 keep short columns in registers (one read, one write);
    // the generic-p form would unroll a powf per element and stays two-pass.
    const uint32_t grid = grid_for(g.columns);
    if (pl->chosen(SHDW_PATH_COLUMNS_REG, dim <= 16 ? 16 : 64, grid)) return SHDW_OK;
    if (mode == 1) {
      if (dim <= 16)
        normalize_columns_reg_kernel<1, 16><<<grid, kBlock, 0, st>>>(x, y, g.columns, d, fi, p, eps);
      else
        normalize_columns_reg_kernel<1, 64><<<grid, kBlock, 0, st>>>(x, y, g.columns, d, fi, p, eps);
    } else {
      if (dim <= 16)
        normalize_columns_reg_kernel<2, 16><<<grid, kBlock, 0, st>>>(x, y, g.columns, d, fi, p, eps);
      else
        normalize_columns_reg_kernel<2, 64><<<grid, kBlock, 0, st>>>(x, y, g.columns, d, fi, p, eps);
    }
  } else if (TallLaunch t; tall_launch(outer_num, dim, inner_num, &t)) {
    if (pl->chosen(SHDW_PATH_TALL, static_cast<int>(t.width_log2), t.grid)) return SHDW_OK;
    if (mode == 1)
      launch_normalize_tall<1, kSsdNoScale>(t, dim, inner_num, p, eps, x, nullptr, y, st);
    else if (mode == 2)
      launch_normalize_tall<2, kSsdNoScale>(t, dim, inner_num, p, eps, x, nullptr, y, st);
    else
      launch_normalize_tall<0, kSsdNoScale>(t, dim, inner_num, p, eps, x, nullptr, y, st);
  } else {
    const uint32_t grid = (g.columns + kWave - 1) / kWave;
    if (pl->chosen(SHDW_PATH_COLUMNS, 0, grid)) return SHDW_OK;
    if (mode == 1)
      normalize_columns_kernel<1><<<grid, kWave, 0, st>>>(x, y, g.columns, d, fi, p, eps);
    else if (mode == 2)
      normalize_columns_kernel<2><<<grid, kWave, 0, st>>>(x, y, g.columns, d, fi, p, eps);
    else
      normalize_columns_kernel<0><<<grid, kWave, 0, st>>>(x, y, g.columns, d, fi, p, eps);
  }
  return launch_status();
}

}  // namespace shdw

using namespace shdw;

extern "C" {

int shdw_hip_softmax(int outer_num, int dim, int inner_num, const float* x, float* y,
                     void* stream) {
  ColumnPlan pl;
  return run_softmax(outer_num, dim, inner_num, x, y, static_cast<hipStream_t>(stream), &pl);
}

int shdw_hip_normalize(int outer_num, int dim, int inner_num, float p, float eps, const float* x,
                       float* y, void* stream) {
  ColumnPlan pl;
  return run_normalize(outer_num, dim, inner_num, p, eps, x, y, static_cast<hipStream_t>(stream), &pl);
}

static int hand_back(const ColumnPlan& pl, int* path, int* variant, unsigned* grid) {
  if (path) *path = pl.path;
  if (variant) *variant = pl.variant;
  if (grid) *grid = pl.grid;
  return SHDW_OK;
}

int shdw_hip_softmax_plan(int outer_num, int dim, int inner_num, int* path, int* variant, unsigned* grid) {
  ColumnPlan pl;
  pl.want = true;
  const int rc = run_softmax(outer_num, dim, inner_num, nullptr, nullptr, nullptr, &pl);
  return rc != SHDW_OK ? rc : hand_back(pl, path, variant, grid);
}

int shdw_hip_normalize_plan(int outer_num, int dim, int inner_num, float p, int* path, int* variant,
                            unsigned* grid) {
  ColumnPlan pl;
  pl.want = true;
  const int rc = run_normalize(outer_num, dim, inner_num, p, 1e-12f, nullptr, nullptr, nullptr, &pl);
  return rc != SHDW_OK ? rc : hand_back(pl, path, variant, grid);
}

}  // extern "C"

namespace shdw {

// SSDNormalize over the channels of every position; called from
// shdw_hip_ssd_normalize (norm.hip owns the across-spatial form).
template <int SM>
static void launch_ssd_columns(const ColumnGeometry& g, int outer_num, int dim, int inner_num, float eps,
                               const float* x, const float* scale, float* y, hipStream_t st) {
  const FastDiv fi = make_fastdiv(static_cast<uint32_t>(inner_num));
  const uint32_t d = static_cast<uint32_t>(dim);
  const uint32_t grid = grid_for(g.columns);
  if (rows_apply(outer_num, dim, inner_num)) {
    launch_normalize_rows<3, SM>(outer_num, dim, 2.f, eps, x, scale, y, st);
    return;
  }
  if (FastDiv fq; const uint32_t quads = quad_count(outer_num, dim, inner_num, false, &fq)) {
    launch_normalize_quads<3, SM>(quads, fq, dim, inner_num, 2.f, eps, x, scale, y, st);
    return;
  }
  if (const uint32_t group = packed_group(dim, inner_num)) {
    const uint32_t slabs = static_cast<uint32_t>(outer_num);
    normalize_packed_kernel<3, SM><<<(slabs + group - 1) / group, kBlock, packed_bytes(dim, inner_num, group), st>>>(
        x, y, slabs, d, fi, make_fastdiv(d * inner_num), group, 2.f, eps, scale);
  } else if (long_slab(outer_num, dim, inner_num, false))
    normalize_long_slab_kernel<3, SM><<<outer_num, kBlock, 0, st>>>(x, y, d, fi, 2.f, eps, scale);
  else if (g.use_slab)
    normalize_slab_kernel<3, SM><<<outer_num, kBlock, g.slab_bytes, st>>>(x, y, d, fi, 2.f, eps, scale);
  else if (tile_fits(dim, inner_num, false))
    launch_normalize_tile<3, SM>(outer_num, dim, inner_num, 2.f, eps, x, scale, y, st);
  else if (dim <= 16)
    normalize_columns_reg_kernel<3, 16, SM><<<grid, kBlock, 0, st>>>(x, y, g.columns, d, fi, 2.f, eps, scale);
  else if (dim <= 64)
    normalize_columns_reg_kernel<3, 64, SM><<<grid, kBlock, 0, st>>>(x, y, g.columns, d, fi, 2.f, eps, scale);
  else if (TallLaunch t; tall_launch(outer_num, dim, inner_num, &t))
    launch_normalize_tall<3, SM>(t, dim, inner_num, 2.f, eps, x, scale, y, st);
  else
    normalize_columns_kernel<3, SM><<<(g.columns + kWave - 1) / kWave, kWave, 0, st>>>(x, y, g.columns, d, fi, 2.f,
                                                                                  eps, scale);
}

int ssd_normalize_columns(int outer_num, int dim, int inner_num, float eps, const float* x,
                          const float* scale, int channel_shared, float* y, hipStream_t st) {
  ColumnGeometry g;
  const int rc = column_geometry(outer_num, dim, inner_num, &g);
  if (rc != SHDW_OK) return rc;
  if (g.columns == 0 || dim == 0) return SHDW_OK;
  if (!x || !y) return SHDW_E_INVALID_ARGUMENT;
  if (!scale)
    launch_ssd_columns<kSsdNoScale>(g, outer_num, dim, inner_num, eps, x, scale, y, st);
  else if (channel_shared)
    launch_ssd_columns<kSsdSharedScale>(g, outer_num, dim, inner_num, eps, x, scale, y, st);
  else
    launch_ssd_columns<kSsdChannelScale>(g, outer_num, dim, inner_num, eps, x, scale, y, st);
  return launch_status();
}

}  // namespace shdw
