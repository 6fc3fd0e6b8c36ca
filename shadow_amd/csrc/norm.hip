// GroupNorm / InstanceNorm / LayerNorm: x viewed as [outer][inner] rows; every
// row is shifted by its mean and divided by sqrt(variance + eps), then an
// optional per-channel scale and bias is applied.
//
// Shadow computes both statistics with its plain-loop Sgemv against a vector of
// ones: (float) of an fp64 running sum of the fp32 products alpha * v with
// alpha = 1 / inner (shadow/core/blas.cpp:238-247), five launches and three
// scratch blobs per call (shadow/operators/kernels/group_norm.hpp:41-86).  Here
// a row is owned by one wave64 (rows up to 2048 elements) or one workgroup and
// everything happens in one launch: fp64 partial sums per lane, combined by
// shuffles (and LDS across waves).  The fp64 additions are associated
// differently from the reference's front-to-back loop; the sums are then
// rounded to fp32 once, so the statistics (and with them every output) come out
// identical unless an fp64 sum lands within ~1e-16 relative of an fp32 rounding
// boundary.  Rows of up to 32768 elements stay in registers between the three
// passes (one HBM read, one write); longer rows are re-read, from L2.
//
// The kernels are close to VALU-bound (two fp64 accumulations and an IEEE
// division per element), so the affine step avoids per-element index
// arithmetic: LayerNorm's parameters are loaded as vectors by row position,
// GroupNorm's channel is computed once per 128-bit vector.
#include <hip/hip_runtime.h>

#include <algorithm>

#include "../../include/shadow_hip.h"
#include "device_common.h"
#include "launch.h"

#pragma clang fp contract(off)

namespace shdw {

enum AffineMode {
  kAffineNone = 0,
  kAffineRowPos = 1,   // parameter index = position in the row (LayerNorm)
  kAffineVector = 2,   // scale_inner % 4 == 0: one channel per aligned vector
  kAffineElement = 3,  // anything else: channel per element
  kAffineRow = 4,      // scale_inner % inner == 0: one channel per row (InstanceNorm), looked up once
};

struct NormArgs {
  uint32_t outer, inner;
  float alpha, eps;
  int affine;
  const float* scale;
  const float* bias;
  FastDiv f_scale_inner, f_scale_num;  // channel = (i / scale_inner) % scale_num
};

SHDW_DEVICE uint32_t norm_channel(const NormArgs& p, uint32_t i) {
  const uint32_t q = fd_div(i, p.f_scale_inner);
  return q - fd_div(q, p.f_scale_num) * p.f_scale_num.d;
}

SHDW_DEVICE float affine1(float v, float s, float b) {
  const float t = v * s;
  return t + b;
}

// Affine step for the aligned vector at row position `pos` (global index i).
SHDW_DEVICE v4f norm_affine4(const NormArgs& p, uint32_t i, uint32_t pos, v4f v) {
  if (p.affine == kAffineNone) return v;
  v4f r;
  if (p.affine == kAffineRowPos) {
    const v4f s = load4(p.scale + pos), b = load4(p.bias + pos);
#pragma unroll
    for (int j = 0; j < 4; ++j) r[j] = affine1(v[j], s[j], b[j]);
  } else if (p.affine == kAffineVector) {
    const uint32_t c = norm_channel(p, i);
    const float s = p.scale[c], b = p.bias[c];
#pragma unroll
    for (int j = 0; j < 4; ++j) r[j] = affine1(v[j], s, b);
  } else {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t c = norm_channel(p, i + j);
      r[j] = affine1(v[j], p.scale[c], p.bias[c]);
    }
  }
  return r;
}

// Scale and bias of the row that starts at global index `base` (kAffineRow).
struct RowAffine {
  float s, b;
};
SHDW_DEVICE RowAffine norm_row_affine(const NormArgs& p, uint32_t base) {
  RowAffine ra = {1.f, 0.f};
  if (p.affine == kAffineRow) {
    const uint32_t c = norm_channel(p, base);
    ra.s = p.scale[c], ra.b = p.bias[c];
  }
  return ra;
}
SHDW_DEVICE v4f norm_row_affine4(const RowAffine& ra, v4f v) {
  v4f r;
#pragma unroll
  for (int j = 0; j < 4; ++j) r[j] = affine1(v[j], ra.s, ra.b);
  return r;
}

SHDW_DEVICE float norm_affine1(const NormArgs& p, uint32_t i, float v) {
  if (p.affine == kAffineNone) return v;
  const uint32_t c = norm_channel(p, i);
  return affine1(v, p.scale[c], p.bias[c]);
}

SHDW_DEVICE double wave_sum(double v) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off);
  return v;
}

// Sum over the LANES lanes that own a row, result in each of them.  LANES <= 64:
// the lanes are neighbours inside one wave; more: whole waves, through `slots`.
template <int LANES>
SHDW_DEVICE double row_sum(double v, double* slots) {
  if (LANES <= 16) {
    // inside a row of 16 lanes the exchanges are DPP moves (no LDS traffic); after
    // each step the lanes that have met hold the same sum, so the mirrors of the
    // last two steps pair every lane with one from the other half
    if (LANES >= 2) v += dpp_f64<kDppXor1>(v);
    if (LANES >= 4) v += dpp_f64<kDppXor2>(v);
    if (LANES >= 8) v += dpp_f64<kDppHalfMirror>(v);
    if (LANES >= 16) v += dpp_f64<kDppMirror>(v);
    return v;
  }
  if (LANES <= kWave) {
#pragma unroll
    for (int off = LANES / 2; off >= 1; off >>= 1) v += __shfl_xor(v, off);
    return v;
  }
  v = wave_sum(v);
  __syncthreads();  // slots may still be read from the previous sum
  if ((threadIdx.x & 63) == 0) slots[threadIdx.x >> 6] = v;
  __syncthreads();
  double total = slots[0];
#pragma unroll
  for (int w = 1; w < LANES / kWave; ++w) total += slots[w];
  return total;
}

// The row (<= REGS * 4 * LANES elements) is held in REGS vectors per lane.
// LANES = 16, 32 or 64: 16, 8 or 4 rows per 256-lane workgroup, no barriers (a
// wave-per-row layout leaves 3/4 of the lanes idle on rows of 64 floats: 85 us
// per 58 MB, and rows of 49 went through the one-workgroup-per-row kernel at
// 307 us).  LANES = 256 or 1024: one row per workgroup of that size.
// TAIL = false: inner % 4 == 0 and 16-byte aligned pointers.  TAIL = true: any
// row length on any dword address; a lane's vector may end inside its four
// positions, whole vectors still move as (unaligned) 128-bit accesses.
constexpr int kBigBlock = 1024;

template <int REGS, int LANES, bool TAIL>
// Two 1024-lane workgroups per CU are 8 waves per SIMD, at most 64 registers
// per lane (the second launch bound asks for that; unasked the compiler took
// 67 and left room for one workgroup).
__global__ __launch_bounds__(LANES <= kWave ? kBlock : LANES, LANES == kBigBlock ? 8 : 1) void norm_rows_reg_kernel(
    const float* x, float* y, NormArgs p) {
  __shared__ double slots[kBigBlock / kWave];
  const uint32_t lane = LANES <= kWave ? (threadIdx.x & (LANES - 1)) : threadIdx.x;
  const uint32_t row = LANES <= kWave ? blockIdx.x * (kBlock / LANES) + threadIdx.x / LANES : blockIdx.x;
  if (LANES <= kWave && row >= p.outer) return;  // whole rows of lanes leave; no barrier in this form
  const uint64_t base = static_cast<uint64_t>(row) * p.inner;
  const float* xr = x + base;
  float* yr = y + base;
  // elements of vector k that exist: 4, or fewer at the end of a TAIL row
  auto count = [&](int k) -> uint32_t {
    const uint32_t first = 4 * (k * LANES + lane);
    return first >= p.inner ? 0u : min(4u, p.inner - first);
  };
  v4f reg[REGS];
#pragma unroll
  for (int k = 0; k < REGS; ++k) {
    const uint32_t first = 4 * (k * LANES + lane), c = count(k);
    if (c == 4) {
      reg[k] = TAIL ? load4_stream_any(xr + first) : load4_stream(xr + first);
    } else if (TAIL && c > 0) {
      reg[k] = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int j = 0; j < 3; ++j)
        if (j < c) reg[k][j] = xr[first + j];
    }
  }
  double acc = 0;
#pragma unroll
  for (int k = 0; k < REGS; ++k) {
    const uint32_t c = count(k);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (j < c) {
        const float t = p.alpha * reg[k][j];
        acc += static_cast<double>(t);
      }
    }
  }
  const float mean = static_cast<float>(row_sum<LANES>(acc, slots));
  acc = 0;
#pragma unroll
  for (int k = 0; k < REGS; ++k) {
    const uint32_t c = count(k);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (j < c) {
        const float val = reg[k][j] - mean;
        reg[k][j] = val;
        const float sq = val * val;
        const float t = p.alpha * sq;
        acc += static_cast<double>(t);
      }
    }
  }
  const float variance = static_cast<float>(row_sum<LANES>(acc, slots));
  const float ve = variance + p.eps;
  const float denom = __builtin_sqrtf(ve);
  // One lookup per row where the row shares its scale and bias; only in the
  // forms of up to 64 lanes per row (the host asks for it only there): the
  // 1024-lane form has no register to spare for it.
  constexpr bool kRowForm = LANES <= kWave;
  const bool row_affine = kRowForm && p.affine == kAffineRow;
  RowAffine ra = {1.f, 0.f};
  if (kRowForm) ra = norm_row_affine(p, static_cast<uint32_t>(base));
#pragma unroll
  for (int k = 0; k < REGS; ++k) {
    const uint32_t first = 4 * (k * LANES + lane), c = count(k);
    if (c == 0) continue;
    v4f r;
#pragma unroll
    for (int j = 0; j < 4; ++j) r[j] = reg[k][j] / denom;
    if (row_affine) r = norm_row_affine4(ra, r);
    if (!TAIL) {
      if (!row_affine) r = norm_affine4(p, static_cast<uint32_t>(base) + first, first, r);
      store4_stream(yr + first, r);
    } else {
      // any alignment: the affine parameters are looked up per element unless the row shares them
      if (!row_affine) {
#pragma unroll
        for (int j = 0; j < 4; ++j) r[j] = norm_affine1(p, static_cast<uint32_t>(base) + first + j, r[j]);
      }
      if (c == 4) {
        store4_stream_any(yr + first, r);
      } else {
#pragma unroll
        for (int j = 0; j < 3; ++j)
          if (j < c) yr[first + j] = r[j];
      }
    }
  }
}

// Rows of up to 256 elements, at least a thousand of them.  The register forms
// above give such rows 16 to 64 lanes with one vector each, and what a lane does
// once per row (two fp64 exchanges, four IEEE divisions' worth of setup, the
// square root, the parameter lookup, the vector-tail logic) then outweighs what
// it does per element: rows of 49 on 16 lanes ran at the instruction issue rate
// (258 vector instructions per wave of four rows, 32 us per 103 MB).  Giving a
// lane 16 neighbouring elements straight from global memory does not work
// either: 128-bit loads whose lanes are 64 bytes apart run at the address rate
// (53 us).  Here a workgroup's 256 / L rows, one contiguous span, pass through
// LDS as they lie, with 128-bit copies on both sides, and L lanes share a row,
// each walking its own piece of about 13 to 16 elements three times in LDS (mean,
// variance, output in place).  The lane partials of the two sums meet by DPP.
constexpr int kNormLdsMaxInner = 256;

// PADDED: inner % 4 == 0.  Such rows would start on the same few LDS banks (rows
// of 64 or 128 floats: all on one), so their pitch is the next odd number of
// 128-bit pieces, inner + 4 or inner + 8 floats (the 128-bit copies then never
// cross a row end, and 16 neighbouring rows start on 16 different banks); other
// row lengths are copied as they lie.  The pieces are an odd number of elements long for the same reason.
template <int L, bool PADDED>
__global__ __launch_bounds__(kBlock) void norm_rows_lds_kernel(const float* x, float* y, NormArgs p,
                                                                uint32_t seg, FastDiv f_inner4) {
  constexpr uint32_t kRows = kBlock / L;
  __shared__ __align__(16) float tile[kRows * (16 * L + 4)];  // 16 to 17 KB: inner <= 16 L
  __shared__ float sc[16 * L], bi[16 * L];                   // LayerNorm: scale and bias by row position
  const uint32_t inner = p.inner;
  const uint32_t pitch = PADDED ? 4 * ((inner / 4 + 1) | 1u) : inner;  // an odd number of 128-bit pieces
  const uint32_t row0 = blockIdx.x * kRows;
  const uint32_t nrows = min(kRows, p.outer - row0);
  const uint64_t base = static_cast<uint64_t>(row0) * inner;
  const float* xs = x + base;
  float* ys = y + base;
  const uint32_t cells = nrows * inner, nvec = cells / 4;
  // LDS offset of the vector that starts at element 4 v of the span
  auto slot = [&](uint32_t v) -> uint32_t {
    if (!PADDED) return 4 * v;
    const uint32_t r = fd_div(v, f_inner4);  // inner / 4 vectors per row
    return 4 * v + (pitch - inner) * r;
  };
  for (uint32_t v0 = 0; v0 < nvec; v0 += 4 * kBlock) {
    v4f reg[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const uint32_t v = min(v0 + k * kBlock + threadIdx.x, nvec - 1);  // past the end: the last piece again
      reg[k] = load4_stream_any(xs + 4ull * v);
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const uint32_t v = v0 + k * kBlock + threadIdx.x;
      if (v < nvec) *reinterpret_cast<v4f*>(tile + slot(v)) = reg[k];
    }
  }
  if (!PADDED && threadIdx.x < (cells & 3u)) tile[4 * nvec + threadIdx.x] = xs[4 * nvec + threadIdx.x];
  if (p.affine == kAffineRowPos) {
    for (uint32_t t = threadIdx.x; t < inner; t += kBlock) sc[t] = p.scale[t], bi[t] = p.bias[t];
  }
  __syncthreads();

  const uint32_t r = threadIdx.x / L, h = threadIdx.x % L;
  // rows past the end compute on whatever the tile holds and store nothing: all
  // lanes of a wave stay together for the exchanges
  const uint32_t c_begin = min(h * seg, inner), c_end = min(c_begin + seg, inner);
  const uint32_t n = c_end - c_begin;
  float* mine = tile + (r < nrows ? r : 0) * pitch + c_begin;
  double acc = 0;
  uint32_t c = 0;
  for (; c + 4 <= n; c += 4) {
    float v[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) v[k] = mine[c + k];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const float t = p.alpha * v[k];
      acc += static_cast<double>(t);
    }
  }
  for (; c < n; ++c) {
    const float t = p.alpha * mine[c];
    acc += static_cast<double>(t);
  }
  const float mean = static_cast<float>(row_sum<L>(acc, nullptr));
  acc = 0;
  for (c = 0; c + 4 <= n; c += 4) {
    float v[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) v[k] = mine[c + k];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const float val = v[k] - mean;
      const float sq = val * val;
      const float t = p.alpha * sq;
      acc += static_cast<double>(t);
    }
  }
  for (; c < n; ++c) {
    const float val = mine[c] - mean;
    const float sq = val * val;
    const float t = p.alpha * sq;
    acc += static_cast<double>(t);
  }
  const float variance = static_cast<float>(row_sum<L>(acc, nullptr));
  const float ve = variance + p.eps;
  const float denom = __builtin_sqrtf(ve);
  if (r < nrows) {
    const uint32_t first = static_cast<uint32_t>(base) + r * inner;  // global index of the row
    const RowAffine ra = norm_row_affine(p, first);
    auto finish = [&](uint32_t pos, float v) -> float {
      const float val = v - mean;
      float q = val / denom;
      if (p.affine == kAffineRow) q = affine1(q, ra.s, ra.b);
      else if (p.affine == kAffineRowPos) q = affine1(q, sc[c_begin + pos], bi[c_begin + pos]);
      else if (p.affine != kAffineNone) q = norm_affine1(p, first + c_begin + pos, q);
      return q;
    };
    for (c = 0; c + 4 <= n; c += 4) {
      float v[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) v[k] = mine[c + k];
#pragma unroll
      for (int k = 0; k < 4; ++k) v[k] = finish(c + k, v[k]);
#pragma unroll
      for (int k = 0; k < 4; ++k) mine[c + k] = v[k];
    }
    for (; c < n; ++c) mine[c] = finish(c, mine[c]);
  }
  __syncthreads();

  for (uint32_t v = threadIdx.x; v < nvec; v += kBlock)
    store4_stream_any(ys + 4ull * v, *reinterpret_cast<const v4f*>(tile + slot(v)));
  if (!PADDED && threadIdx.x < (cells & 3u)) ys[4 * nvec + threadIdx.x] = tile[4 * nvec + threadIdx.x];
}

// Any row, one workgroup per row, three passes over memory (the second and
// third find the row in L2).  VEC: inner % 4 == 0 and 16-byte aligned.
template <bool VEC>
__global__ __launch_bounds__(kBlock) void norm_rows_stream_kernel(const float* x, float* y, NormArgs p) {
  __shared__ double slots[kBlock / kWave];
  const uint64_t base = static_cast<uint64_t>(blockIdx.x) * p.inner;
  const float* xr = x + base;
  float* yr = y + base;
  const uint32_t steps = VEC ? p.inner / 4 : p.inner;
  double acc = 0;
  for (uint32_t t = threadIdx.x; t < steps; t += kBlock) {
    if (VEC) {
      const v4f q = load4(xr + 4ull * t);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float a = p.alpha * q[j];
        acc += static_cast<double>(a);
      }
    } else {
      const float a = p.alpha * xr[t];
      acc += static_cast<double>(a);
    }
  }
  const float mean = static_cast<float>(row_sum<kBlock>(acc, slots));
  acc = 0;
  for (uint32_t t = threadIdx.x; t < steps; t += kBlock) {
    if (VEC) {
      const v4f q = load4(xr + 4ull * t);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float val = q[j] - mean;
        const float sq = val * val;
        const float a = p.alpha * sq;
        acc += static_cast<double>(a);
      }
    } else {
      const float val = xr[t] - mean;
      const float sq = val * val;
      const float a = p.alpha * sq;
      acc += static_cast<double>(a);
    }
  }
  const float variance = static_cast<float>(row_sum<kBlock>(acc, slots));
  const float ve = variance + p.eps;
  const float denom = __builtin_sqrtf(ve);
  const RowAffine ra = norm_row_affine(p, static_cast<uint32_t>(base));
  for (uint32_t t = threadIdx.x; t < steps; t += kBlock) {
    if (VEC) {
      const v4f q = load4(xr + 4ull * t);
      v4f r;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float val = q[j] - mean;
        r[j] = val / denom;
      }
      r = p.affine == kAffineRow ? norm_row_affine4(ra, r)
                                 : norm_affine4(p, static_cast<uint32_t>(base) + 4 * t, 4 * t, r);
      store4_stream(yr + 4ull * t, r);
    } else {
      const float val = xr[t] - mean;
      const float q = val / denom;
      yr[t] = p.affine == kAffineRow ? affine1(q, ra.s, ra.b) : norm_affine1(p, static_cast<uint32_t>(base) + t, q);
    }
  }
}

// Rows too long and too few for a workgroup each (GroupNorm of a detector's
// feature map at batch 1: 32 rows of 320 000; one row of 12.8 M elements took
// 17 ms): every row is cut into `splits` slices, a workgroup per slice, in three
// launches that hand fp64 partial sums on through scratch memory of the caller:
//   pass 1: partial sums of alpha * x
//   pass 2: the mean from pass 1's partials, partial sums of alpha * (x - mean)^2
//   pass 3: mean and variance from the partials, then the row's slice of y.
// Every workgroup of a row folds the row's partials in the same fixed order, so
// all of them hold the same mean and variance.
template <bool VEC>
SHDW_DEVICE double slice_sum(const float* xr, uint32_t begin, uint32_t end, float alpha, bool centred, float mean) {
  double acc = 0;
  auto term = [&](float v) {
    float t;
    if (centred) {
      const float val = v - mean;
      const float sq = val * val;
      t = alpha * sq;
    } else {
      t = alpha * v;
    }
    acc += static_cast<double>(t);
  };
  if (VEC) {
    for (uint32_t t = begin / 4 + threadIdx.x; t < end / 4; t += kBlock) {
      const v4f q = load4(xr + 4ull * t);
#pragma unroll
      for (int j = 0; j < 4; ++j) term(q[j]);
    }
  } else {
    for (uint32_t t = begin + threadIdx.x; t < end; t += kBlock) term(xr[t]);
  }
  return acc;
}

// Sum of a row's `splits` partials (<= 1024), the same tree in every workgroup.
SHDW_DEVICE double fold_partials(const double* part, uint32_t splits, double* slots) {
  double acc = 0;
  for (uint32_t s = threadIdx.x; s < splits; s += kBlock) acc += part[s];
  return row_sum<kBlock>(acc, slots);
}

template <int PASS, bool VEC>
__global__ __launch_bounds__(kBlock) void norm_rows_split_kernel(const float* x, float* y, NormArgs p,
                                                                  uint32_t splits, uint32_t chunk,
                                                                  double* sums, double* squares) {
  __shared__ double slots[kBlock / kWave];
  const uint32_t row = blockIdx.x, slice = blockIdx.y;
  const uint64_t base = static_cast<uint64_t>(row) * p.inner;
  const float* xr = x + base;
  const uint32_t begin = min(slice * chunk, p.inner), end = min(begin + chunk, p.inner);
  const double* row_sums = sums + static_cast<size_t>(row) * splits;
  double* row_squares = squares + static_cast<size_t>(row) * splits;
  if (PASS == 1) {
    const double acc = row_sum<kBlock>(slice_sum<VEC>(xr, begin, end, p.alpha, false, 0.f), slots);
    if (threadIdx.x == 0) sums[static_cast<size_t>(row) * splits + slice] = acc;
    return;
  }
  const float mean = static_cast<float>(fold_partials(row_sums, splits, slots));
  if (PASS == 2) {
    const double acc = row_sum<kBlock>(slice_sum<VEC>(xr, begin, end, p.alpha, true, mean), slots);
    if (threadIdx.x == 0) row_squares[slice] = acc;
    return;
  }
  const float variance = static_cast<float>(fold_partials(row_squares, splits, slots));
  const float ve = variance + p.eps;
  const float denom = __builtin_sqrtf(ve);
  float* yr = y + base;
  const RowAffine ra = norm_row_affine(p, static_cast<uint32_t>(base));
  if (VEC) {
    for (uint32_t t = begin / 4 + threadIdx.x; t < end / 4; t += kBlock) {
      const v4f q = load4(xr + 4ull * t);
      v4f r;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float val = q[j] - mean;
        r[j] = val / denom;
      }
      r = p.affine == kAffineRow ? norm_row_affine4(ra, r)
                                 : norm_affine4(p, static_cast<uint32_t>(base) + 4 * t, 4 * t, r);
      store4_stream(yr + 4ull * t, r);
    }
  } else {
    for (uint32_t t = begin + threadIdx.x; t < end; t += kBlock) {
      const float val = xr[t] - mean;
      const float q = val / denom;
      yr[t] = p.affine == kAffineRow ? affine1(q, ra.s, ra.b) : norm_affine1(p, static_cast<uint32_t>(base) + t, q);
    }
  }
}

constexpr uint32_t kNormSplitMaxRows = 512, kNormSplitMinInner = 32768, kNormSplitMinChunk = 8192;

// Slices per row: enough for about a thousand workgroups, each with at least
// 8192 elements; 1 where rows are many or short.
static uint32_t norm_row_splits(int64_t rows, int64_t inner) {
  if (rows >= kNormSplitMaxRows || inner < kNormSplitMinInner || rows < 1) return 1;
  const int64_t by_fill = (1024 + rows - 1) / rows, by_work = inner / kNormSplitMinChunk;
  return static_cast<uint32_t>(std::max<int64_t>(1, std::min<int64_t>(std::min(by_fill, by_work), 1024)));
}

// ---------------------------------------------------------------------------
// SSDNormalize across the whole item (shadow/operators/kernels/
// ssd_normalize.hpp:47-57): the reference squares x into the output, takes
// Sasum of each item on the host (fp64 running sum, blas.cpp:229-233) and
// multiplies the item by 1 / sqrt(sum + eps), all in fp32 after the sum.  An
// item is usually megabytes long, so its sum is split over `parts` workgroups
// that each fold a fixed segment (fp64 per lane, shuffles, LDS) into a slot of
// the workspace; the second kernel adds the slots in index order, forms the
// factor and applies it, with the optional scale of ssd_normalize.hpp:68-80 in
// the same pass.  Nothing returns to the host in between.
// ---------------------------------------------------------------------------
constexpr uint32_t kSsdSegmentQuantum = 4 * kBlock;  // keeps every segment 16-byte aligned
constexpr uint32_t kSsdMinSegment = 4 * kSsdSegmentQuantum;
constexpr uint32_t kSsdMaxParts = 64;  // one lane of a wave per part (ssd_row_finish_kernel)
static_assert(kSsdMaxParts <= static_cast<uint32_t>(kWave), "one lane per part");
constexpr uint32_t kSsdGroupsWanted = 1024;

struct SsdRowPlan {
  uint32_t parts, segment;
};

static SsdRowPlan plan_ssd_rows(uint32_t batch, uint32_t num) {
  uint32_t parts = std::min(kSsdMaxParts, (kSsdGroupsWanted + batch - 1) / std::max(batch, 1u));
  parts = std::max(1u, std::min(parts, num / kSsdMinSegment));
  uint32_t segment = (num + parts - 1) / parts;
  segment = (segment + kSsdSegmentQuantum - 1) / kSsdSegmentQuantum * kSsdSegmentQuantum;
  SsdRowPlan plan;
  plan.segment = segment;
  plan.parts = std::max(1u, (num + segment - 1) / segment);
  return plan;
}

// Workgroup b * parts + k folds segment k of item b.
template <bool VEC>
__global__ __launch_bounds__(kBlock) void ssd_row_partials_kernel(const float* x, double* partials,
                                                                   uint32_t num, uint32_t segment,
                                                                   FastDiv f_parts) {
  __shared__ double slots[kBlock / kWave];
  uint32_t item, part;
  fd_divmod(blockIdx.x, f_parts, item, part);
  const uint32_t begin = part * segment;
  const uint32_t end = min(num, begin + segment);
  const float* xr = x + static_cast<uint64_t>(item) * num;
  double acc = 0;
  if (VEC) {
    // eight loads under way per lane; the squares are added in the order of t
    constexpr int kAhead = 8;
    uint32_t t = begin / 4 + threadIdx.x;
    const uint32_t stop = end / 4;
    for (; t + (kAhead - 1) * kBlock < stop; t += kAhead * kBlock) {
      v4f q[kAhead];
#pragma unroll
      for (int u = 0; u < kAhead; ++u) q[u] = load4_stream(xr + 4ull * (t + u * kBlock));
#pragma unroll
      for (int u = 0; u < kAhead; ++u) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float sq = q[u][j] * q[u][j];
          acc += static_cast<double>(sq);
        }
      }
    }
    for (; t < stop; t += kBlock) {
      const v4f q = load4_stream(xr + 4ull * t);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float sq = q[j] * q[j];
        acc += static_cast<double>(sq);
      }
    }
  } else {
    for (uint32_t t = begin + threadIdx.x; t < end; t += kBlock) {
      const float sq = xr[t] * xr[t];
      acc += static_cast<double>(sq);
    }
  }
  const double total = row_sum<kBlock>(acc, slots);
  if (threadIdx.x == 0) partials[blockIdx.x] = total;
}

// One wave per item: lane k fetches partial k (at most 64 of them, one round
// trip for all), the sum walks the lanes in index order, and
// 1 / sqrt((float)sum + eps) goes to the item's first slot (a float, widened
// exactly).  In the scaling kernel itself this chain ran once per wave behind
// dependent loads and set its pace: 75 us for [64,512,38,38] where the same pass
// with the factor ready takes 57.
__global__ __launch_bounds__(kWave) void ssd_row_finish_kernel(double* partials, uint32_t parts, float eps) {
  double* mine = partials + blockIdx.x * parts;
  const double part = threadIdx.x < parts ? mine[threadIdx.x] : 0.0;
  double sum = 0;
  for (uint32_t k = 0; k < parts; ++k) {  // k is uniform: two v_readlane_b32 per step
    const int lo = __builtin_amdgcn_readlane(__double2loint(part), static_cast<int>(k));
    const int hi = __builtin_amdgcn_readlane(__double2hiint(part), static_cast<int>(k));
    sum += __hiloint2double(hi, lo);
  }
  const float sum_f = static_cast<float>(sum);
  const float se = sum_f + eps;
  const float factor = 1.f / __builtin_sqrtf(se);
  if (threadIdx.x == 0) mine[0] = static_cast<double>(factor);
}

// SM: 0 no scale, 1 one shared factor (Sscal), 2 one factor per channel.
template <bool VEC, int SM>
__global__ __launch_bounds__(kStream) void ssd_row_scale_kernel(const float* x, float* y,
                                                                const double* partials, uint32_t parts,
                                                                uint32_t num, const float* scale,
                                                                FastDiv f_spatial,
                                                                FastDiv f_groups) {
  uint32_t item, group;  // wave `group` of the item's stream_grid(steps) waves
  fd_divmod(blockIdx.x, f_groups, item, group);
  const uint32_t i = group * kStream + threadIdx.x;
  const uint64_t base = static_cast<uint64_t>(item) * num;
  const bool mine_valid = i < (VEC ? num / 4 : num);
  v4f q = {0.f, 0.f, 0.f, 0.f};
  if (mine_valid) {
    if (VEC) q = load4_stream(x + base + 4ull * i);
    else q[0] = x[base + i];
  }
  const float factor = static_cast<float>(partials[item * parts]);  // uniform: one scalar load
  if (!mine_valid) return;
  if (VEC) {
    v4f r;
    if (SM == 2 && f_spatial.d >= 4) {
      // four neighbours lie in one channel or in two: one division and two factors
      // per lane (a gather per element keeps the address unit busier than the
      // streamed load and store together)
      const uint32_t c0 = fd_div(4 * i, f_spatial);
      const uint32_t edge = (c0 + 1) * f_spatial.d;  // first element of the next channel
      const float s0 = scale[c0], s1 = scale[edge < num ? c0 + 1 : c0];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        r[j] = q[j] * factor;
        r[j] = r[j] * (4 * i + j < edge ? s0 : s1);
      }
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        r[j] = q[j] * factor;
        if (SM == 1) r[j] = r[j] * scale[0];
        if (SM == 2) r[j] = r[j] * scale[fd_div(4 * i + j, f_spatial)];
      }
    }
    store4_stream(y + base + 4ull * i, r);
  } else {
    float r = q[0] * factor;
    if (SM == 1) r = r * scale[0];
    if (SM == 2) r = r * scale[fd_div(i, f_spatial)];
    y[base + i] = r;
  }
}

template <bool VEC>
static void launch_ssd_rows(uint32_t batch, uint32_t num, uint32_t spatial, float eps, const float* x,
                            const float* scale, int channel_shared, float* y, double* partials,
                            hipStream_t st) {
  const SsdRowPlan plan = plan_ssd_rows(batch, num);
  ssd_row_partials_kernel<VEC><<<batch * plan.parts, kBlock, 0, st>>>(x, partials, num, plan.segment,
                                                                    make_fastdiv(plan.parts));
  ssd_row_finish_kernel<<<batch, kWave, 0, st>>>(partials, plan.parts, eps);
  const uint32_t groups = stream_grid(VEC ? num / 4 : num);  // single waves: batch * groups <= count / 64 + batch
  const uint32_t grid = batch * groups;
  const FastDiv fs = make_fastdiv(std::max(spatial, 1u)), fg = make_fastdiv(groups);
  if (!scale)
    ssd_row_scale_kernel<VEC, 0><<<grid, kStream, 0, st>>>(x, y, partials, plan.parts, num, scale, fs, fg);
  else if (channel_shared)
    ssd_row_scale_kernel<VEC, 1><<<grid, kStream, 0, st>>>(x, y, partials, plan.parts, num, scale, fs, fg);
  else
    ssd_row_scale_kernel<VEC, 2><<<grid, kStream, 0, st>>>(x, y, partials, plan.parts, num, scale, fs, fg);
}

// softmax.hip: the per-position form shares the Normalize column kernels.
int ssd_normalize_columns(int outer_num, int dim, int inner_num, float eps, const float* x,
                          const float* scale, int channel_shared, float* y, hipStream_t st);

}  // namespace shdw

using namespace shdw;

extern "C" {

size_t shdw_hip_group_norm_workspace_bytes(int outer_num, int inner_num) {
  if (outer_num <= 0 || inner_num <= 0) return 0;
  const uint32_t splits = norm_row_splits(outer_num, inner_num);
  return splits > 1 ? static_cast<size_t>(2) * outer_num * splits * sizeof(double) : 0;
}

int shdw_hip_group_norm(int outer_num, int inner_num, float eps, const float* x,
                        const float* scale, const float* bias, int scale_num, int scale_inner,
                        float* y, void* stream) {
  return shdw_hip_group_norm_ws(outer_num, inner_num, eps, x, scale, bias, scale_num, scale_inner, y, nullptr, 0,
                                stream);
}

int shdw_hip_group_norm_ws(int outer_num, int inner_num, float eps, const float* x,
                           const float* scale, const float* bias, int scale_num, int scale_inner,
                           float* y, void* workspace, size_t workspace_bytes, void* stream) {
  if (outer_num < 0 || inner_num < 0) return SHDW_E_INVALID_ARGUMENT;
  const int64_t count = static_cast<int64_t>(outer_num) * inner_num;
  if (count > INT32_MAX) return SHDW_E_INVALID_ARGUMENT;
  if (count == 0) return SHDW_OK;
  if (!x || !y || (scale == nullptr) != (bias == nullptr)) return SHDW_E_INVALID_ARGUMENT;
  if (scale && (scale_num < 1 || scale_inner < 1)) return SHDW_E_INVALID_ARGUMENT;
  NormArgs p;
  p.outer = static_cast<uint32_t>(outer_num);
  p.inner = static_cast<uint32_t>(inner_num);
  p.alpha = 1.f / inner_num;
  p.eps = eps;
  p.scale = scale;
  p.bias = bias;
  p.f_scale_inner = make_fastdiv(static_cast<uint32_t>(scale ? scale_inner : 1));
  p.f_scale_num = make_fastdiv(static_cast<uint32_t>(scale ? scale_num : 1));
  const bool vec = inner_num % 4 == 0 && aligned16(x) && aligned16(y);
  if (!scale)
    p.affine = kAffineNone;
  else if (scale_inner % inner_num == 0 && inner_num <= 1024)  // rows that up to 64 lanes hold
    p.affine = kAffineRow;
  else if (vec && scale_inner == 1 && scale_num == inner_num && aligned16(scale) && aligned16(bias))
    p.affine = kAffineRowPos;
  else if (vec && scale_inner % 4 == 0)
    p.affine = kAffineVector;
  else
    p.affine = kAffineElement;

  hipStream_t st = static_cast<hipStream_t>(stream);
  const uint32_t rows = p.outer;
  const uint32_t nvec = p.inner / 4;
  const uint32_t splits = norm_row_splits(outer_num, inner_num);
  if (splits > 1 && workspace && workspace_bytes >= shdw_hip_group_norm_workspace_bytes(outer_num, inner_num)) {
    if (reinterpret_cast<uintptr_t>(workspace) & 7u) return SHDW_E_INVALID_ARGUMENT;
    double* sums = static_cast<double*>(workspace);
    double* squares = sums + static_cast<size_t>(rows) * splits;
    uint32_t chunk = (p.inner + splits - 1) / splits;
    chunk = (chunk + 3) & ~3u;  // slices start on whole vectors
    const dim3 grid(rows, splits);
#define SHDW_SPLIT(PASS)                                                                                       \
  do {                                                                                                         \
    if (vec) norm_rows_split_kernel<PASS, true><<<grid, kBlock, 0, st>>>(x, y, p, splits, chunk, sums, squares);  \
    else norm_rows_split_kernel<PASS, false><<<grid, kBlock, 0, st>>>(x, y, p, splits, chunk, sums, squares);  \
  } while (0)
    SHDW_SPLIT(1);
    SHDW_SPLIT(2);
    SHDW_SPLIT(3);
#undef SHDW_SPLIT
    return launch_status();
  }
  // workgroups of 256 lanes holding 256 / lanes rows each
  auto groups = [rows](uint32_t lanes) { return (rows + kBlock / lanes - 1) / (kBlock / lanes); };
  if (p.inner <= kNormLdsMaxInner && rows >= 1024) {
    // short rows through LDS, L lanes per row (any row length, any dword address)
    if (!scale)
      p.affine = kAffineNone;
    else if (scale_inner % inner_num == 0)
      p.affine = kAffineRow;
    else if (scale_inner == 1 && scale_num == inner_num)
      p.affine = kAffineRowPos;  // scalar lookups by row position: no alignment asked of the parameters
    else
      p.affine = kAffineElement;
    const uint32_t want = (p.inner + 15) / 16;  // lanes for pieces of at most 16 elements
    const uint32_t lanes = want <= 1 ? 1 : (want <= 2 ? 2 : (want <= 4 ? 4 : (want <= 8 ? 8 : 16)));
    const uint32_t seg = ((p.inner + lanes - 1) / lanes) | 1u;  // an odd number of elements per lane
    const uint32_t grid = (rows + kBlock / lanes - 1) / (kBlock / lanes);
    const FastDiv f4 = make_fastdiv(std::max<uint32_t>(1, p.inner / 4));
#define SHDW_LDS(LANES)                                                                        \
  do {                                                                                         \
    if (p.inner % 4 == 0) norm_rows_lds_kernel<LANES, true><<<grid, kBlock, 0, st>>>(x, y, p, seg, f4);  \
    else norm_rows_lds_kernel<LANES, false><<<grid, kBlock, 0, st>>>(x, y, p, seg, f4);        \
  } while (0)
    switch (lanes) {
      case 1: SHDW_LDS(1); break;
      case 2: SHDW_LDS(2); break;
      case 4: SHDW_LDS(4); break;
      case 8: SHDW_LDS(8); break;
      default: SHDW_LDS(16); break;
    }
#undef SHDW_LDS
    return launch_status();
  }
  if (!vec) {
    // any row length, any dword address: whole vectors plus a partial one per row
    const uint32_t units = (p.inner + 3) / 4;
    if (units <= 16) {
      norm_rows_reg_kernel<1, 16, true><<<groups(16), kBlock, 0, st>>>(x, y, p);
    } else if (units <= 32) {
      norm_rows_reg_kernel<1, 32, true><<<groups(32), kBlock, 0, st>>>(x, y, p);
    } else if (units <= 1 * kWave) {
      norm_rows_reg_kernel<1, kWave, true><<<groups(kWave), kBlock, 0, st>>>(x, y, p);
    } else if (units <= 2 * kWave) {
      norm_rows_reg_kernel<2, kWave, true><<<groups(kWave), kBlock, 0, st>>>(x, y, p);
    } else if (units <= 4 * kWave) {
      norm_rows_reg_kernel<4, kWave, true><<<groups(kWave), kBlock, 0, st>>>(x, y, p);
    } else if (units <= 8 * kWave) {
      norm_rows_reg_kernel<8, kWave, true><<<groups(kWave), kBlock, 0, st>>>(x, y, p);
    } else if (units <= 8 * kBlock) {
      norm_rows_reg_kernel<8, kBlock, true><<<rows, kBlock, 0, st>>>(x, y, p);
    } else {
      norm_rows_stream_kernel<false><<<rows, kBlock, 0, st>>>(x, y, p);
    }
  } else if (nvec <= 16) {
    norm_rows_reg_kernel<1, 16, false><<<groups(16), kBlock, 0, st>>>(x, y, p);
  } else if (nvec <= 32) {
    norm_rows_reg_kernel<1, 32, false><<<groups(32), kBlock, 0, st>>>(x, y, p);
  } else if (nvec <= 1 * kWave) {
    norm_rows_reg_kernel<1, kWave, false><<<groups(kWave), kBlock, 0, st>>>(x, y, p);
  } else if (nvec <= 2 * kWave) {
    norm_rows_reg_kernel<2, kWave, false><<<groups(kWave), kBlock, 0, st>>>(x, y, p);
  } else if (nvec <= 4 * kWave) {
    norm_rows_reg_kernel<4, kWave, false><<<groups(kWave), kBlock, 0, st>>>(x, y, p);
  } else if (nvec <= 8 * kWave && rows >= 2048) {
    norm_rows_reg_kernel<8, kWave, false><<<groups(kWave), kBlock, 0, st>>>(x, y, p);
  } else if (nvec <= 2 * kBlock) {
    norm_rows_reg_kernel<2, kBlock, false><<<rows, kBlock, 0, st>>>(x, y, p);
  } else if (nvec <= 4 * kBlock) {
    norm_rows_reg_kernel<4, kBlock, false><<<rows, kBlock, 0, st>>>(x, y, p);
  } else if (nvec <= 8 * kBlock) {
    norm_rows_reg_kernel<8, kBlock, false><<<rows, kBlock, 0, st>>>(x, y, p);
  } else if (nvec <= 4 * kBigBlock) {
    norm_rows_reg_kernel<4, kBigBlock, false><<<rows, kBigBlock, 0, st>>>(x, y, p);
  } else if (nvec <= 8 * kBigBlock) {
    norm_rows_reg_kernel<8, kBigBlock, false><<<rows, kBigBlock, 0, st>>>(x, y, p);
  } else {
    norm_rows_stream_kernel<true><<<rows, kBlock, 0, st>>>(x, y, p);
  }
  return launch_status();
}

size_t shdw_hip_ssd_normalize_workspace_bytes(int batch, int channels, int spatial_dim,
                                              int across_spatial) {
  if (!across_spatial || batch <= 0 || channels <= 0 || spatial_dim <= 0) return 0;
  const int64_t num = static_cast<int64_t>(channels) * spatial_dim;
  if (num * batch > INT32_MAX) return 0;
  const SsdRowPlan plan = plan_ssd_rows(static_cast<uint32_t>(batch), static_cast<uint32_t>(num));
  return static_cast<size_t>(batch) * plan.parts * sizeof(double);
}

int shdw_hip_ssd_normalize(int batch, int channels, int spatial_dim, int across_spatial, float eps,
                           const float* x, const float* scale, int channel_shared, float* y,
                           void* workspace, void* stream) {
  if (batch < 0 || channels < 0 || spatial_dim < 0) return SHDW_E_INVALID_ARGUMENT;
  const int64_t num = static_cast<int64_t>(channels) * spatial_dim;
  if (num > INT32_MAX || num * batch > INT32_MAX) return SHDW_E_INVALID_ARGUMENT;
  if (num * batch == 0) return SHDW_OK;
  if (!x || !y) return SHDW_E_INVALID_ARGUMENT;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (!across_spatial)
    return ssd_normalize_columns(batch, channels, spatial_dim, eps, x, scale, channel_shared, y, st);
  if (!workspace || (reinterpret_cast<uintptr_t>(workspace) & 7u)) return SHDW_E_INVALID_ARGUMENT;
  double* partials = static_cast<double*>(workspace);
  const bool vec = num % 4 == 0 && aligned16(x) && aligned16(y);
  if (vec)
    launch_ssd_rows<true>(batch, static_cast<uint32_t>(num), spatial_dim, eps, x, scale, channel_shared, y,
                          partials, st);
  else
    launch_ssd_rows<false>(batch, static_cast<uint32_t>(num), spatial_dim, eps, x, scale, channel_shared, y,
                           partials, st);
  return launch_status();
}

}  // extern "C"
