// Kernels whose second operand is indexed, not streamed:
//   * per-row parameters (Scale / Bias / ScaleBias with an optional ReLU
//     epilogue, PRelu): x is rows of `inner` contiguous elements and the
//     parameter index is row % num;
//   * numpy-style broadcast Binary on host-collapsed dims.
// Index arithmetic is done once per 128-bit vector with multiply-high division
// by launch-time constants; there is no per-element div/mod and no device-side
// shape table.
#include <hip/hip_runtime.h>

#include "../../include/shadow_hip.h"
#include "device_common.h"
#include "functors.h"
#include "launch.h"
#include "plan.h"

#pragma clang fp contract(off)

namespace shdw {

enum RowMode { kScaleBias = 0, kScaleOnly = 1, kBiasOnly = 2, kPRelu = 3 };

template <int MODE, bool RELU>
SHDW_DEVICE float row_apply(float x, float s, float b) {
  float r;
  if (MODE == kScaleBias) {
    const float t = x * s;
    r = t + b;
  } else if (MODE == kScaleOnly) {
    r = x * s;
  } else if (MODE == kBiasOnly) {
    r = x + b;
  } else {
    r = x > 0 ? x : x * s;
  }
  if (RELU) r = r > 0 ? r : 0;
  return r;
}

template <int MODE, bool RELU>
SHDW_DEVICE float row_element(uint32_t e, float x, const float* s, const float* b,
                              const FastDiv& inner, const FastDiv& num) {
  const uint32_t row = fd_div(e, inner);
  const uint32_t c = row - fd_div(row, num) * num.d;
  const float sv = (MODE != kBiasOnly) ? s[c] : 0.f;
  const float bv = (MODE == kScaleBias || MODE == kBiasOnly) ? b[c] : 0.f;
  return row_apply<MODE, RELU>(x, sv, bv);
}

// One 128-bit vector per lane.  ROWS says how a vector meets the parameters:
//   kRowShared: inner % 4 == 0, the four elements share one row and the
//               parameters are fetched once per vector;
//   kRowEach:   inner == 1 and num % 4 == 0 (a bias per output of Connected, an
//               affine pair per position of a normalised row): the four
//               parameters are neighbours and never wrap inside a vector, one
//               128-bit fetch each (eight 4-byte fetches per lane ran at the
//               address rate: 28 us against 17 us per 51 MB with 64 and more
//               parameters);
//   kRowPair:   any other inner >= 2: a vector starts in one row and may end in
//               the next, never further, so it needs the parameters of two rows
//               (a lookup per element: 24 us against 17 us with inner = 2 or 3);
//   kRowAny:    a lookup per element (inner == 1, any num).
enum RowVectors { kRowAny = 0, kRowShared = 1, kRowEach = 2, kRowPair = 3 };

// Where the vector that starts at element e0 sits: the parameter index of its
// first row and of the row after it, and how many of its elements the first row
// still holds (4 and more: the vector does not reach the second row).
SHDW_DEVICE void row_pair(uint32_t e0, const FastDiv& inner, const FastDiv& num, uint32_t& c0, uint32_t& c1,
                          uint32_t& left) {
  const uint32_t row = fd_div(e0, inner);
  left = inner.d - (e0 - row * inner.d);
  c0 = row - fd_div(row, num) * num.d;
  c1 = c0 + 1 == num.d ? 0 : c0 + 1;
}

template <int MODE, bool RELU, int ROWS>
__global__ __launch_bounds__(kStream) void rowparam_vec_kernel(const float* x, const float* s,
                                                               const float* b, float* y,
                                                               uint32_t n4, uint32_t n,
                                                               FastDiv inner, FastDiv num) {
  constexpr bool ROWVEC = ROWS == kRowShared;
  const uint32_t i = blockIdx.x * kStream + threadIdx.x;
  if (i < n4) {
    const v4f vx = load4_stream_any(x + 4ull * i);  // any float pointer
    v4f r;
    if (ROWS == kRowEach) {
      const uint32_t c = 4 * i - fd_div(4 * i, num) * num.d;
      const v4f zero = {0.f, 0.f, 0.f, 0.f};
      const v4f sv = (MODE != kBiasOnly) ? load4_any(s + c) : zero;
      const v4f bv = (MODE == kScaleBias || MODE == kBiasOnly) ? load4_any(b + c) : zero;
#pragma unroll
      for (int j = 0; j < 4; ++j) r[j] = row_apply<MODE, RELU>(vx[j], sv[j], bv[j]);
    } else if (ROWVEC) {
      const uint32_t row = fd_div(4 * i, inner);
      const uint32_t c = row - fd_div(row, num) * num.d;
      const float sv = (MODE != kBiasOnly) ? s[c] : 0.f;
      const float bv = (MODE == kScaleBias || MODE == kBiasOnly) ? b[c] : 0.f;
#pragma unroll
      for (int j = 0; j < 4; ++j) r[j] = row_apply<MODE, RELU>(vx[j], sv, bv);
    } else if (ROWS == kRowPair) {
      uint32_t c0, c1, left;
      row_pair(4 * i, inner, num, c0, c1, left);
      const float s0 = (MODE != kBiasOnly) ? s[c0] : 0.f, s1 = (MODE != kBiasOnly) ? s[c1] : 0.f;
      const bool biased = MODE == kScaleBias || MODE == kBiasOnly;
      const float b0 = biased ? b[c0] : 0.f, b1 = biased ? b[c1] : 0.f;
#pragma unroll
      for (int j = 0; j < 4; ++j)
        r[j] = row_apply<MODE, RELU>(vx[j], static_cast<uint32_t>(j) < left ? s0 : s1,
                                     static_cast<uint32_t>(j) < left ? b0 : b1);
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) r[j] = row_element<MODE, RELU>(4 * i + j, vx[j], s, b, inner, num);
    }
    store4_stream_any(y + 4ull * i, r);
  } else if (i == n4) {
    for (uint32_t t = 4 * n4; t < n; ++t) y[t] = row_element<MODE, RELU>(t, x[t], s, b, inner, num);
  }
}

template <int MODE, bool RELU>
static int launch_rowparam(int n, int num, int inner, const float* x, const float* s,
                           const float* b, float* y, hipStream_t st) {
  const FastDiv fi = make_fastdiv(static_cast<uint32_t>(inner));
  const FastDiv fn = make_fastdiv(static_cast<uint32_t>(num));
  const uint32_t n4 = static_cast<uint32_t>(n) / 4;
  const uint32_t grid = stream_grid(n4 + 1);
  if (inner % 4 == 0)
    rowparam_vec_kernel<MODE, RELU, kRowShared><<<grid, kStream, 0, st>>>(x, s, b, y, n4, n, fi, fn);
  else if (inner == 1 && num % 4 == 0)
    rowparam_vec_kernel<MODE, RELU, kRowEach><<<grid, kStream, 0, st>>>(x, s, b, y, n4, n, fi, fn);
  else if (inner >= 2)
    rowparam_vec_kernel<MODE, RELU, kRowPair><<<grid, kStream, 0, st>>>(x, s, b, y, n4, n, fi, fn);
  else
    rowparam_vec_kernel<MODE, RELU, kRowAny><<<grid, kStream, 0, st>>>(x, s, b, y, n4, n, fi, fn);
  return launch_status();
}

// Binary with a parameter per row: a[outer][num][inner] op b[num], the channel
// broadcast of a bias add or a per-channel scale written as a Binary operator.
// Same shape as the kernel above (one quotient chain per vector instead of the
// stride walk of the general kernel: [8,64,112,112] + [1,64,1,1] 10.2 -> 9.1 us).
// Any float pointers, any inner >= 1; the operand order f(a, b) is kept.
template <class F, bool ROWVEC>
__global__ __launch_bounds__(kStream) void rowbinary_vec_kernel(F f, const float* a, const float* b,
                                                                float* y, uint32_t n4, uint32_t n,
                                                                FastDiv inner, FastDiv num) {
  const uint64_t* tab = uses_exp_table<F>::value ? libm::kExp2fTab : nullptr;
  auto param = [&](uint32_t e) {
    const uint32_t row = fd_div(e, inner);
    return b[row - fd_div(row, num) * num.d];
  };
  const uint32_t i = blockIdx.x * kStream + threadIdx.x;
  if (i < n4) {
    const v4f va = load4_stream_any(a + 4ull * i);
    v4f r;
    if (ROWVEC) {
      const float bv = param(4 * i);
#pragma unroll
      for (int j = 0; j < 4; ++j) r[j] = f(va[j], bv, tab);
    } else if (inner.d >= 2) {  // two rows at the most: see kRowPair
      uint32_t c0, c1, left;
      row_pair(4 * i, inner, num, c0, c1, left);
      const float b0 = b[c0], b1 = b[c1];
#pragma unroll
      for (int j = 0; j < 4; ++j) r[j] = f(va[j], static_cast<uint32_t>(j) < left ? b0 : b1, tab);
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) r[j] = f(va[j], param(4 * i + j), tab);
    }
    store4_stream_any(y + 4ull * i, r);
  } else if (i == n4) {
    for (uint32_t t = 4 * n4; t < n; ++t) y[t] = f(a[t], param(t), tab);
  }
}

// ---------------------------------------------------------------------------
// Broadcast binary on collapsed dims.
// ---------------------------------------------------------------------------
struct BcastArgs {
  FastDiv fd[kMaxDims];  // divisors for dims 1..NDIM-1 are used (dim 0 is the quotient)
  int sa[kMaxDims];
  int sb[kMaxDims];
  int a_full;  // a is not broadcast anywhere: stream it
  int b_full;
};

// Each lane owns 4 consecutive outputs of the innermost collapsed dim, whose
// extent is a multiple of 4.  AVEC/BVEC: the operand's innermost stride is 1
// (128-bit load) rather than 0 (one scalar, replicated).
template <class F, int NDIM, bool AVEC, bool BVEC>
__global__ __launch_bounds__(kBlock) void bcast_vec_kernel(F f, BcastArgs p, const float* a,
                                                            const float* b, float* y,
                                                            uint32_t n4) {
  const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;  // 64 or 256 lanes, see the launch
  // Pow reads the 2^(i/32) table; broadcast Pow is not a throughput case, the
  // table stays in global memory here.
  const uint64_t* tab = uses_exp_table<F>::value ? libm::kExp2fTab : nullptr;
  if (i < n4) {
    uint32_t e = 4 * i;
    uint32_t oa = 0, ob = 0;
#pragma unroll
    for (int k = NDIM - 1; k >= 1; --k) {
      uint32_t q, r;
      fd_divmod(e, p.fd[k], q, r);
      oa += r * static_cast<uint32_t>(p.sa[k]);
      ob += r * static_cast<uint32_t>(p.sb[k]);
      e = q;
    }
    oa += e * static_cast<uint32_t>(p.sa[0]);
    ob += e * static_cast<uint32_t>(p.sb[0]);
    v4f va, vb;
    if (AVEC) {
      va = p.a_full ? load4_stream(a + oa) : load4(a + oa);
    } else {
      const float t = a[oa];
      va = {t, t, t, t};
    }
    if (BVEC) {
      vb = p.b_full ? load4_stream(b + ob) : load4(b + ob);
    } else {
      const float t = b[ob];
      vb = {t, t, t, t};
    }
    v4f r;
#pragma unroll
    for (int j = 0; j < 4; ++j) r[j] = f(va[j], vb[j], tab);
    store4_stream(y + 4ull * i, r);
  }
}

// The same for an innermost extent that is not a multiple of 4 (7 x 7, 13 x 13
// maps) or operands on odd dwords: a lane still owns 4 consecutive outputs and
// one 128-bit store, but they may lie in two or more innermost rows.  Lanes whose
// four outputs share a row take one vector (or one replicated scalar) per
// operand; the others decode each output on its own.  One output per lane ran
// at 2.0-2.8 TB/s on such shapes against 5.7 TB/s for their aligned cousins.
template <class F, int NDIM>
SHDW_DEVICE void bcast_offsets(const BcastArgs& p, uint32_t e, uint32_t& oa, uint32_t& ob, uint32_t& col) {
  oa = 0, ob = 0, col = e;
#pragma unroll
  for (int k = NDIM - 1; k >= 1; --k) {
    uint32_t q, r;
    fd_divmod(e, p.fd[k], q, r);
    if (k == NDIM - 1) col = r;
    oa += r * static_cast<uint32_t>(p.sa[k]);
    ob += r * static_cast<uint32_t>(p.sb[k]);
    e = q;
  }
  oa += e * static_cast<uint32_t>(p.sa[0]);
  ob += e * static_cast<uint32_t>(p.sb[0]);
}

template <class F, int NDIM>
__global__ __launch_bounds__(kBlock) void bcast_flat_kernel(F f, BcastArgs p, const float* a,
                                                             const float* b, float* y, uint32_t n4,
                                                             uint32_t n) {
  const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;  // 64 or 256 lanes, see the launch
  const uint64_t* tab = uses_exp_table<F>::value ? libm::kExp2fTab : nullptr;
  const uint32_t last = p.fd[NDIM - 1].d;
  const int sa = p.sa[NDIM - 1], sb = p.sb[NDIM - 1];  // 0 or 1
  if (i < n4) {
    uint32_t oa, ob, col;
    bcast_offsets<F, NDIM>(p, 4 * i, oa, ob, col);
    v4f va, vb;
    if (col + 4 <= last) {
      if (sa) {  // a re-used (broadcast) operand stays cacheable
        va = p.a_full ? load4_stream_any(a + oa) : load4_any(a + oa);
      } else {
        const float t = a[oa];
        va = {t, t, t, t};
      }
      if (sb) {
        vb = p.b_full ? load4_stream_any(b + ob) : load4_any(b + ob);
      } else {
        const float t = b[ob];
        vb = {t, t, t, t};
      }
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        uint32_t pa, pb, unused;
        bcast_offsets<F, NDIM>(p, 4 * i + j, pa, pb, unused);
        va[j] = a[pa], vb[j] = b[pb];
      }
    }
    v4f r;
#pragma unroll
    for (int j = 0; j < 4; ++j) r[j] = f(va[j], vb[j], tab);
    store4_stream_any(y + 4ull * i, r);
  } else if (i == n4) {
    for (uint32_t t = 4 * n4; t < n; ++t) {
      uint32_t pa, pb, unused;
      bcast_offsets<F, NDIM>(p, t, pa, pb, unused);
      y[t] = f(a[pa], b[pb], tab);
    }
  }
}

template <class F, int NDIM>
static void launch_bcast_vec(F f, const BcastArgs& p, bool avec, bool bvec, const float* a,
                             const float* b, float* y, uint32_t n4, hipStream_t st) {
  // An operand as large as the output makes this a read-and-write stream, which
  // runs best as single-wave workgroups; when both operands are broadcast the
  // kernel mostly writes, and 256-lane workgroups are 1.5x faster than single
  // waves there (11.3 us against 16.5 us for [16,1,128,256] x [1,32,128,1]).
  const uint32_t lanes = (p.a_full || p.b_full) ? kStream : kBlock;
  const uint32_t grid = (n4 + lanes - 1) / lanes;
  if (avec && bvec)
    bcast_vec_kernel<F, NDIM, true, true><<<grid, lanes, 0, st>>>(f, p, a, b, y, n4);
  else if (avec)
    bcast_vec_kernel<F, NDIM, true, false><<<grid, lanes, 0, st>>>(f, p, a, b, y, n4);
  else if (bvec)
    bcast_vec_kernel<F, NDIM, false, true><<<grid, lanes, 0, st>>>(f, p, a, b, y, n4);
  else
    bcast_vec_kernel<F, NDIM, false, false><<<grid, lanes, 0, st>>>(f, p, a, b, y, n4);
}

template <class F>
static int launch_bcast(F f, const BroadcastPlan& plan, const float* a, const float* b, float* y,
                        hipStream_t st) {
  BroadcastPlan pl = plan;
  if (pl.ndim == 0) {  // one output element
    pl.ndim = 1;
    pl.dims[0] = 1;
    pl.sa[0] = pl.sb[0] = 0;
  }
  const int nd = pl.ndim;
  const int last = nd - 1;
  const uint32_t n = static_cast<uint32_t>(pl.count);
  // a whole, b one value per row of `inner` elements: [outer][num][inner] op [num], outer possibly 1
  int num = 0, inner = 0;
  if (nd == 3 && pl.sb[0] == 0 && pl.sb[1] == 1 && pl.sb[2] == 0 && pl.sa[2] == 1 && pl.sa[1] == pl.dims[2] &&
      pl.sa[0] == pl.dims[1] * pl.dims[2])
    num = pl.dims[1], inner = pl.dims[2];
  else if (nd == 2 && pl.sb[0] == 1 && pl.sb[1] == 0 && pl.sa[1] == 1 && pl.sa[0] == pl.dims[1])
    num = pl.dims[0], inner = pl.dims[1];
  if (inner >= 4) {
    const FastDiv fi = make_fastdiv(static_cast<uint32_t>(inner)), fn = make_fastdiv(static_cast<uint32_t>(num));
    const uint32_t n4 = n / 4, grid = stream_grid(n4 + 1);
    if (inner % 4 == 0)
      rowbinary_vec_kernel<F, true><<<grid, kStream, 0, st>>>(f, a, b, y, n4, n, fi, fn);
    else
      rowbinary_vec_kernel<F, false><<<grid, kStream, 0, st>>>(f, a, b, y, n4, n, fi, fn);
    return launch_status();
  }
  const bool vec_ok = nd <= 4 && pl.dims[last] % 4 == 0 && aligned16(y) &&
                      (pl.sa[last] == 0 || aligned16(a)) && (pl.sb[last] == 0 || aligned16(b));
  if (vec_ok) {
    BcastArgs p;
    p.a_full = p.b_full = 1;
    for (int k = 0; k < 4; ++k) {
      p.fd[k] = make_fastdiv(k < nd ? static_cast<uint32_t>(pl.dims[k]) : 1u);
      p.sa[k] = k < nd ? pl.sa[k] : 0;
      p.sb[k] = k < nd ? pl.sb[k] : 0;
      if (k < nd && pl.sa[k] == 0) p.a_full = 0;
      if (k < nd && pl.sb[k] == 0) p.b_full = 0;
    }
    const bool avec = pl.sa[last] == 1, bvec = pl.sb[last] == 1;
    const uint32_t n4 = n / 4;
    switch (nd) {
      case 1: launch_bcast_vec<F, 1>(f, p, avec, bvec, a, b, y, n4, st); break;
      case 2: launch_bcast_vec<F, 2>(f, p, avec, bvec, a, b, y, n4, st); break;
      case 3: launch_bcast_vec<F, 3>(f, p, avec, bvec, a, b, y, n4, st); break;
      default: launch_bcast_vec<F, 4>(f, p, avec, bvec, a, b, y, n4, st); break;
    }
  } else {
    // any innermost extent, any pointers, up to kMaxDims collapsed dims (more than four: operands
    // that alternate between broadcast and full extents dim by dim)
    BcastArgs p;
    p.a_full = p.b_full = 1;
    for (int k = 0; k < kMaxDims; ++k) {
      p.fd[k] = make_fastdiv(k < nd ? static_cast<uint32_t>(pl.dims[k]) : 1u);
      p.sa[k] = k < nd ? pl.sa[k] : 0;
      p.sb[k] = k < nd ? pl.sb[k] : 0;
      if (k < nd && pl.sa[k] == 0) p.a_full = 0;
      if (k < nd && pl.sb[k] == 0) p.b_full = 0;
    }
    const uint32_t n4 = n / 4;
    const uint32_t lanes = (p.a_full || p.b_full) ? kStream : kBlock;  // as in launch_bcast_vec
    const uint32_t grid = (n4 + 1 + lanes - 1) / lanes;
    switch (nd) {
      case 1: bcast_flat_kernel<F, 1><<<grid, lanes, 0, st>>>(f, p, a, b, y, n4, n); break;
      case 2: bcast_flat_kernel<F, 2><<<grid, lanes, 0, st>>>(f, p, a, b, y, n4, n); break;
      case 3: bcast_flat_kernel<F, 3><<<grid, lanes, 0, st>>>(f, p, a, b, y, n4, n); break;
      case 4: bcast_flat_kernel<F, 4><<<grid, lanes, 0, st>>>(f, p, a, b, y, n4, n); break;
      case 5: bcast_flat_kernel<F, 5><<<grid, lanes, 0, st>>>(f, p, a, b, y, n4, n); break;
      case 6: bcast_flat_kernel<F, 6><<<grid, lanes, 0, st>>>(f, p, a, b, y, n4, n); break;
      case 7: bcast_flat_kernel<F, 7><<<grid, lanes, 0, st>>>(f, p, a, b, y, n4, n); break;
      default: bcast_flat_kernel<F, 8><<<grid, lanes, 0, st>>>(f, p, a, b, y, n4, n); break;
    }
  }
  return launch_status();
}

}  // namespace shdw

using namespace shdw;

extern "C" {

int shdw_hip_scale_bias(int n, int scale_num, int inner_num, const float* x, const float* scale,
                        const float* bias, int relu, float* y, void* stream) {
  if (n < 0 || scale_num < 1 || inner_num < 1 || !x || !y || (!scale && !bias))
    return SHDW_E_INVALID_ARGUMENT;
  if (n == 0) return SHDW_OK;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (scale && bias) {
    return relu ? launch_rowparam<kScaleBias, true>(n, scale_num, inner_num, x, scale, bias, y, st)
                : launch_rowparam<kScaleBias, false>(n, scale_num, inner_num, x, scale, bias, y, st);
  } else if (scale) {
    return relu ? launch_rowparam<kScaleOnly, true>(n, scale_num, inner_num, x, scale, bias, y, st)
                : launch_rowparam<kScaleOnly, false>(n, scale_num, inner_num, x, scale, bias, y, st);
  }
  return relu ? launch_rowparam<kBiasOnly, true>(n, scale_num, inner_num, x, scale, bias, y, st)
              : launch_rowparam<kBiasOnly, false>(n, scale_num, inner_num, x, scale, bias, y, st);
}

int shdw_hip_prelu(int n, int channels, int dim, int channel_shared, const float* x,
                   const float* slope, float* y, void* stream) {
  if (n < 0 || channels < 1 || dim < 1 || !x || !slope || !y) return SHDW_E_INVALID_ARGUMENT;
  if (n == 0) return SHDW_OK;
  // c = (i / dim) % channels / div_factor with div_factor = channels when the
  // slope is shared: that is always 0, i.e. one parameter row.
  const int num = channel_shared ? 1 : channels;
  return launch_rowparam<kPRelu, false>(n, num, dim, x, slope, nullptr, y,
                                        static_cast<hipStream_t>(stream));
}

int shdw_hip_broadcast_binary(int operation, int num_axes, const int* a_shape,
                              const int* b_shape, const int* out_shape, const float* a,
                              const float* b, float* y, void* stream) {
  if (!a || !b || !y) return SHDW_E_INVALID_ARGUMENT;
  BroadcastPlan plan;
  const int rc = plan_broadcast(num_axes, a_shape, b_shape, out_shape, &plan);
  if (rc != SHDW_OK) return rc;
  hipStream_t st = static_cast<hipStream_t>(stream);
  switch (operation) {
    case SHDW_BINARY_ADD: return launch_bcast(BAdd(), plan, a, b, y, st);
    case SHDW_BINARY_SUB: return launch_bcast(BSub(), plan, a, b, y, st);
    case SHDW_BINARY_MUL: return launch_bcast(BMul(), plan, a, b, y, st);
    case SHDW_BINARY_DIV: return launch_bcast(BDiv(), plan, a, b, y, st);
    case SHDW_BINARY_POW: return launch_bcast(BPow(), plan, a, b, y, st);
    case SHDW_BINARY_MAX: return launch_bcast(BMax(), plan, a, b, y, st);
    case SHDW_BINARY_MIN: return launch_bcast(BMin(), plan, a, b, y, st);
    default: return SHDW_E_INVALID_ARGUMENT;
  }
}

}  // extern "C"
