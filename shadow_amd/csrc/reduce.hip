// Reduce kernels.  Shadow's kernel walks an index list serially per output
// (shadow/operators/kernels/reduce.cpp:9-76); here the reduced extent is spread
// over lanes, waves and, when there are few outputs, workgroups:
//
//   rows     x[outer][reduce]           reduced axis contiguous.  A group of 16,
//                                       32 or 64 lanes per row for short rows; a
//                                       workgroup per (row, slice) for long ones.
//   strided  x[outer][reduce][inner]    lanes run along `inner` (coalesced); the
//                                       lane groups or waves of a workgroup and
//                                       optional grid.y slices split `reduce`.
//   generic  any axis set               one wave per output, index lists
//                                       replaced by division by constants.
//   stage 2  combines the per-slice partials of a split first stage.
//   A reduced dim in front of the rows or strided view (the statistics of a
//   channel over batch and plane: x[lead][kept][reduce]) is treated as kept by
//   the first stage, which leaves one partial per leading index for stage 2.
//
// The accumulators (fp64 sums, or an fp32 extremum with the position of its
// first zero) are in reduce_acc.h.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cfloat>
#include <mutex>

#include "../../include/shadow_hip.h"
#include "device_common.h"
#include "launch.h"
#include "plan.h"
#include "reduce_acc.h"

#pragma clang fp contract(off)

namespace shdw {

constexpr int kBatch = 8;  // vectors a lane requests before it consumes the first

// A reduced dim in front of a kernel's own view (ReducePlan::lead).  The kernels
// run over lead * (kept outer) outer indices; where a result goes, and which list
// positions its elements have, follows from the leading index of the outer index.
struct Lead {
  uint32_t count = 1;  // extent of the leading reduced dim; 1: there is none; 0: there is none, and the
                       // strided kernel leaves partials even where it does not slice (a nested second stage)
  uint32_t step = 0;   // list positions per leading index: the extent the kernel reduces itself
  FastDiv f_inner, f_count;  // outer index = (a * count + lead) * inner + b
  SHDW_DEVICE void place(uint32_t o, uint32_t& out_outer, uint32_t& lead) const {
    uint32_t q, b, a;
    fd_divmod(o, f_inner, q, b);
    fd_divmod(q, f_count, a, lead);
    out_outer = a * f_inner.d + b;
  }
};

// The result of (row, slice) of a rows kernel: the output itself, or a partial
// in the layout [output][slot] that stage 2 reads.
template <class A>
SHDW_DEVICE void emit_row(const Lead& ld, A acc, uint32_t row, uint32_t split, uint32_t splits, uint32_t reduce,
                          float* y, Partial* part) {
  if (ld.count == 1) {
    if (splits == 1) y[row] = acc.finalize(reduce);
    else part[static_cast<size_t>(row) * splits + split] = acc.pack();
    return;
  }
  uint32_t out, lead;
  ld.place(row, out, lead);
  acc.shift_positions(lead * ld.step);
  part[(static_cast<size_t>(out) * ld.count + lead) * splits + split] = acc.pack();
}

// The result of (outer index, column, slice) of a strided kernel; partials in
// the layout [slot][output].
template <class A>
SHDW_DEVICE void emit_column(const Lead& ld, A acc, uint32_t o, uint32_t col, uint32_t inner, uint32_t split,
                             uint32_t splits, uint32_t outputs, uint32_t reduce, float* y, Partial* part) {
  if (ld.count <= 1) {
    const size_t out = static_cast<size_t>(o) * inner + col;
    if (splits == 1 && ld.count == 1) y[out] = acc.finalize(reduce);
    else part[static_cast<size_t>(split) * outputs + out] = acc.pack();
    return;
  }
  uint32_t oo, lead;
  ld.place(o, oo, lead);
  acc.shift_positions(lead * ld.step);
  const size_t out = static_cast<size_t>(oo) * inner + col;
  part[(static_cast<size_t>(lead) * splits + split) * outputs + out] = acc.pack();
}

// ---------------------------------------------------------------------------
// rows, G lanes per row (G = 16, 32, 64): short rows share a wave so that no
// lane idles and the combine stays inside DPP rows where possible.
// ---------------------------------------------------------------------------
template <int OP, bool VEC, int G>
__global__ __launch_bounds__(kBlock) void reduce_rows_group_kernel(const float* x, float* y,
                                                                    uint32_t rows,
                                                                    uint32_t reduce, Partial* part, Lead ld) {
  const uint32_t lane = threadIdx.x & (G - 1);
  const uint32_t row_raw = blockIdx.x * (kBlock / G) + (threadIdx.x / G);
  // Groups past the end recompute the last row (and do not store) so that all
  // 64 lanes stay active for the cross-lane exchange.
  const uint32_t row = row_raw < rows ? row_raw : rows - 1;
  const float* p = x + static_cast<size_t>(row) * reduce;
  Acc<OP> acc;
  acc.init();
  if (VEC) {
    const uint32_t nv = reduce / 4;
    for (uint32_t base = 0; base < nv; base += kBatch * G) {
      v4f v[kBatch];
      bool valid[kBatch];
      // all loads of the trip are issued before the first value is consumed
#pragma unroll
      for (int u = 0; u < kBatch; ++u) {
        const uint32_t i = base + u * G + lane;
        valid[u] = i < nv;
        if (valid[u]) v[u] = load4_stream_any(p + 4ull * i);  // rows start on any dword
      }
      fold_batch<kBatch, true>(&acc, v, valid, [&](int u, int j) { return 4 * (base + u * G + lane) + j; });
    }
    const uint32_t t = 4 * nv + lane;  // the reduce % 4 elements past the last whole vector
    if (t < reduce) acc.add(p[t], t);
  } else {
    for (uint32_t i = lane; i < reduce; i += G) acc.add(p[i], i);
  }
  acc = group_allreduce<Acc<OP>, G>(acc);
  if (lane == 0 && row_raw < rows) emit_row(ld, acc, row, 0, 1, reduce, y, part);
}

// ---------------------------------------------------------------------------
// rows, one workgroup per (slice, row)
// ---------------------------------------------------------------------------
template <int OP, bool VEC>
__global__ __launch_bounds__(kBlock) void reduce_rows_block_kernel(const float* x, float* y,
                                                                    Partial* part,
                                                                    uint32_t reduce,
                                                                    uint32_t chunk,
                                                                    uint32_t splits, Lead ld) {
  __shared__ Partial lds[kBlock / kWave];
  const uint32_t row = blockIdx.x, split = blockIdx.y;  // rows can exceed the 65535 limit of grid.y
  const float* p = x + static_cast<size_t>(row) * reduce;
  const uint32_t begin = split * chunk;  // chunk is a multiple of 4
  uint32_t end = begin + chunk;
  if (end > reduce || split == splits - 1) end = reduce;
  Acc<OP> acc;
  acc.init();
  if (begin < end) {
    if (VEC) {
      const uint32_t vb = begin / 4, ve = end / 4;
      // a slice is 1024 vectors unless the row is shorter: one batch of four per lane
      uint32_t base = vb;
      for (; base + 4 * kBlock <= ve; base += 4 * kBlock) {  // whole batches: no per-load tests
        v4f v[4];
        const bool valid[4] = {true, true, true, true};
#pragma unroll
        for (int u = 0; u < 4; ++u) v[u] = load4_stream_any(p + 4ull * (base + u * kBlock + threadIdx.x));
        fold_batch<4, true>(&acc, v, valid, [&](int u, int j) { return 4 * (base + u * kBlock + threadIdx.x) + j; });
      }
      if (base < ve) {
        v4f v[4];
        bool valid[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const uint32_t i = base + u * kBlock + threadIdx.x;
          valid[u] = i < ve;
          if (valid[u]) v[u] = load4_stream_any(p + 4ull * i);
        }
        fold_batch<4, true>(&acc, v, valid, [&](int u, int j) { return 4 * (base + u * kBlock + threadIdx.x) + j; });
      }
      // elements past the last whole vector (only the final slice has any)
      const uint32_t t = 4 * ve + threadIdx.x;
      if (t < end) acc.add(p[t], t);
    } else {
      for (uint32_t i = begin + threadIdx.x; i < end; i += kBlock) acc.add(p[i], i);
    }
  }
  acc = wave_allreduce(acc);
  const uint32_t lane = threadIdx.x & (kWave - 1), w = threadIdx.x / kWave;
  if (lane == 0) lds[w] = acc.pack();
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int k = 1; k < kBlock / kWave; ++k) {
      Acc<OP> o;
      o.unpack(lds[k]);
      acc.merge(o);
    }
    emit_row(ld, acc, row, split, splits, reduce, y, part);
  }
}

// ---------------------------------------------------------------------------
// rows of up to 255 floats (7x7 and 5x5 planes, 3x3 and 4x4 windows): a group of
// 16 lanes per row leaves lanes idle (a row of 49 uses 13 of 16, a row of 16
// four) and, where the length is no multiple of four, needs a second, 4-byte
// load for the row ends.  Here a workgroup's 256 / L rows, one contiguous span
// of x, pass through LDS (128-bit copies on whatever dword address the span
// starts), and L = 1, 2, 4, 8 or 16 lanes share a row, each folding its own piece of
// at most 17 elements (an odd number, so that the lanes of a row start on
// different banks); the L partial results meet by DPP.  PADDED (length a
// multiple of four): such rows would start on the same few banks, so their pitch
// is the next odd number of 128-bit pieces (rows of 12 at a pitch of 16 floats:
// 15.4 us per 51 MB, at 20 floats: see below), which the 128-bit copies never
// straddle; other lengths are copied as they lie.  Per 51 MB: mean over 7x7 planes 18.4 us with
// 16 lanes per row from global memory, 12.8 us with one lane per row from 49 KB
// tiles, 9.4 us here; max over 4x4 windows 56 us with 16 lanes per row.
// ---------------------------------------------------------------------------
constexpr int kShortRowMaxFloats = 5120;  // 256 / L rows of at most 16 L (+ 4) floats
constexpr uint32_t kShortRowMaxLen = 256;  // rows up to 255 floats: 16 lanes each

template <int OP, int L, bool PADDED>
__global__ __launch_bounds__(kBlock) void reduce_rows_lds_kernel(const float* x, float* y, uint32_t rows,
                                                                  uint32_t reduce, uint32_t seg,
                                                                  FastDiv f_reduce4, Partial* part, Lead ld) {
  constexpr uint32_t kRows = kBlock / L;
  __shared__ __align__(16) float tile[kShortRowMaxFloats];
  const uint32_t pitch = PADDED ? 4 * ((reduce / 4 + 1) | 1u) : reduce;  // an odd number of 128-bit pieces
  const uint32_t row0 = blockIdx.x * kRows;
  const uint32_t nrows = min(kRows, rows - row0);
  const float* base = x + static_cast<uint64_t>(row0) * reduce;
  const uint32_t cells = nrows * reduce, nvec = cells / 4;
  for (uint32_t v0 = 0; v0 < nvec; v0 += 4 * kBlock) {  // nvec may be 0: a last workgroup with under four elements
    v4f reg[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const uint32_t v = min(v0 + k * kBlock + threadIdx.x, nvec - 1);  // past the end: the last piece again
      reg[k] = load4_stream_any(base + 4ull * v);
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const uint32_t v = v0 + k * kBlock + threadIdx.x;
      if (v < nvec) {
        const uint32_t slot = PADDED ? 4 * v + (pitch - reduce) * fd_div(v, f_reduce4) : 4 * v;  // reduce / 4 vectors per row
        *reinterpret_cast<v4f*>(tile + slot) = reg[k];
      }
    }
  }
  if (!PADDED && threadIdx.x < (cells & 3u)) tile[4 * nvec + threadIdx.x] = base[4 * nvec + threadIdx.x];
  __syncthreads();
  // rows past the end fold whatever the tile holds and store nothing: the lanes
  // of a wave stay together for the exchanges
  const uint32_t r = threadIdx.x / L, h = threadIdx.x % L;
  const uint32_t c_begin = min(h * seg, reduce), c_end = min(c_begin + seg, reduce);
  const float* mine = tile + (r < nrows ? r : 0) * pitch;
  Acc<OP> acc;
  acc.init();
  uint32_t c = c_begin;
  for (; c + 4 <= c_end; c += 4) {
    float v[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) v[k] = mine[c + k];
#pragma unroll
    for (int k = 0; k < 4; ++k) acc.add(v[k], c + k);
  }
  for (; c < c_end; ++c) acc.add(mine[c], c);
  if (L > 1) acc = group_allreduce<Acc<OP>, (L > 1 ? L : 2)>(acc);
  if (h == 0 && r < nrows) emit_row(ld, acc, row0 + r, 0, 1, reduce, y, part);
}

// ---------------------------------------------------------------------------
// rows of D = 2 .. 7 floats (pairs, 2x2 windows): with a lane per row
// a workgroup of the kernel above has 2 KB to work on and its barrier to pay
// (sum over [6.4M][2]: 24 us per 51 MB, 13 us here).  Here a lane owns four whole rows, 4 D
// consecutive floats.  The wave's span moves from memory into the wave's own
// LDS tile as it lies, 128 bits per lane and access, and a lane reads its rows
// back at a pitch of an odd number of 128-bit pieces; no workgroup barrier.
// ---------------------------------------------------------------------------
constexpr uint32_t kTinyRowMaxLen = 7;  // rows of 8: 10.9 us here, 10.3 us with a lane per row from LDS

template <int OP, int D>
__global__ __launch_bounds__(kBlock) void reduce_rows_tiny_kernel(const float* x, float* y, uint32_t rows,
                                                                   Partial* part, Lead ld) {
  constexpr uint32_t kMine = 4 * D;                          // floats of a lane
  constexpr uint32_t kPitch = kMine + (D % 2 == 0 ? 4 : 0);  // of the lanes in the tile
  constexpr uint32_t kSpan = kWave * kMine;                  // floats of a wave
  __shared__ __align__(16) float tiles[kBlock / kWave][kWave * kPitch];
  const uint32_t lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const uint64_t total = static_cast<uint64_t>(rows) * D;
  const uint64_t wave_index = static_cast<uint64_t>(blockIdx.x) * (kBlock / kWave) + wave;
  const uint64_t first = wave_index * kSpan;
  if (first >= total) return;  // the whole wave
  const uint32_t cells = static_cast<uint32_t>(min(static_cast<uint64_t>(kSpan), total - first));
  const float* xs = x + first;
  float* tile = tiles[wave];
  auto place = [](uint32_t t) { return (t / kMine) * kPitch + t % kMine; };  // element t of the span in the tile
  v4f reg[D];
  // no branch around a load: vectors past the end re-read the tensor's first (rows * D >= 4 here)
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
  const float* mine = tile + lane * kPitch;
#pragma unroll
  for (int k = 0; k < D; ++k) reg[k] = *reinterpret_cast<const v4f*>(mine + 4 * k);
  const uint64_t row0 = wave_index * (4 * kWave) + 4 * lane;
  Acc<OP> acc[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    acc[r].init();
#pragma unroll
    for (int c = 0; c < D; ++c) acc[r].add(reg[(r * D + c) / 4][(r * D + c) % 4], c);
  }
  if (ld.count == 1 && row0 + 4 <= rows) {  // the lane's four results as one 128-bit store
    store4_stream_any(y + row0, v4f{acc[0].finalize(D), acc[1].finalize(D), acc[2].finalize(D), acc[3].finalize(D)});
  } else {
#pragma unroll
    for (int r = 0; r < 4; ++r)
      if (row0 + r < rows) emit_row(ld, acc[r], static_cast<uint32_t>(row0 + r), 0, 1, D, y, part);
  }
}

// ---------------------------------------------------------------------------
// strided over a short reduced extent (a sum over a batch of 8, a max over 4
// maps): the column-tile kernels below give a tile 16 or more row groups and an
// LDS fold, which rows this few leave idle ([4][3.2M]: sum 32 us, max 71 us per
// 51 MB).  Here a lane owns four neighbouring columns (the last lane of a row
// the one to three that are left; one column where there are fewer than four),
// 128-bit loads on whatever dword address the rows start, and walks the rows
// itself, eight loads in flight; nothing is exchanged.
// ---------------------------------------------------------------------------
constexpr uint32_t kShortStridedMaxReduce = 32;

template <int OP, bool VEC>
__global__ __launch_bounds__(kBlock) void reduce_strided_short_kernel(const float* x, float* y, uint32_t reduce,
                                                                       uint32_t inner, uint32_t units,
                                                                       FastDiv f_units_per_outer, Partial* part,
                                                                       uint32_t outputs, Lead ld) {
  constexpr int W = VEC ? 4 : 1;
  const uint32_t u = blockIdx.x * kBlock + threadIdx.x;
  if (u >= units) return;
  uint32_t o, c;
  fd_divmod(u, f_units_per_outer, o, c);
  const float* p = x + static_cast<uint64_t>(o) * reduce * inner + static_cast<uint64_t>(c) * W;
  Acc<OP> acc[W];
#pragma unroll
  for (int j = 0; j < W; ++j) acc[j].init();
  // columns of the lane that exist: four, or fewer in the last unit of a row that is no multiple of four long
  const uint32_t n = VEC ? min(4u, inner - 4 * c) : 1u;
  auto fetch = [&](uint32_t r) -> v4f {
    const float* src = p + static_cast<uint64_t>(r) * inner;
    if (!VEC) return v4f{__builtin_nontemporal_load(src), 0.f, 0.f, 0.f};
    if (n == 4) return load4_stream_any(src);  // any dword address: rows need not be whole vectors
    v4f v = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < 3; ++j)
      if (static_cast<uint32_t>(j) < n) v[j] = __builtin_nontemporal_load(src + j);
    return v;
  };
  uint32_t r = 0;
  for (; r + 8 <= reduce; r += 8) {
    v4f v[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) v[k] = fetch(r + k);
#pragma unroll
    for (int k = 0; k < 8; ++k)
#pragma unroll
      for (int j = 0; j < W; ++j) acc[j].add(v[k][j], r + k);
  }
  if (r < reduce) {
    v4f v[8];
#pragma unroll
    for (int k = 0; k < 8; ++k)
      if (r + k < reduce) v[k] = fetch(r + k);
#pragma unroll
    for (int k = 0; k < 8; ++k)
      if (r + k < reduce)
#pragma unroll
        for (int j = 0; j < W; ++j) acc[j].add(v[k][j], r + k);
  }
  if (ld.count != 1) {
#pragma unroll
    for (int j = 0; j < W; ++j)
      if (static_cast<uint32_t>(j) < n) emit_column(ld, acc[j], o, c * W + j, inner, 0, 1, outputs, reduce, y, part);
    return;
  }
  float* dst = y + static_cast<uint64_t>(o) * inner + static_cast<uint64_t>(c) * W;
  if (VEC) {
    v4f out;
#pragma unroll
    for (int j = 0; j < W; ++j) out[j] = acc[j].finalize(reduce);
    if (n == 4) {
      *reinterpret_cast<v4f_unaligned*>(dst) = out;
    } else {
#pragma unroll
      for (int j = 0; j < 3; ++j)
        if (static_cast<uint32_t>(j) < n) dst[j] = out[j];
    }
  } else {
    dst[0] = acc[0].finalize(reduce);
  }
}

// ---------------------------------------------------------------------------
// strided with few columns (8 <= inner < 128): the slab [reduce][inner] of one
// outer index is contiguous, and a workgroup walks its share of it flat.  Lane
// t takes elements 4t .. 4t+3 of every step of `period` elements; period is a
// multiple of inner (and of 4), so the lane meets the same four columns at every
// step and keeps one accumulator for each, and its rows advance by period /
// inner per step.  The loads are 128-bit on whatever dword address the slab has.
// At the end the accumulators go to LDS by position inside the period and lane
// c < inner combines positions c, c + inner, c + 2 inner, ...
// ---------------------------------------------------------------------------
template <int OP>
__global__ __launch_bounds__(kBlock) void reduce_strided_flat_kernel(
    const float* x, float* y, Partial* part, uint32_t reduce, uint32_t inner, uint32_t rows_per_split,
    uint32_t splits, uint32_t outputs, uint32_t period, FastDiv f_inner, Lead ld) {
  __shared__ Partial lds[4 * kBlock];
  const uint32_t o = blockIdx.x, split = blockIdx.y;
  const uint32_t r_begin = min(split * rows_per_split, reduce);
  const uint32_t r_end = min(r_begin + rows_per_split, reduce);
  const uint32_t t4 = 4 * threadIdx.x;
  const bool active = t4 < period;  // period % 4 == 0: a lane has four positions or none
  const uint32_t rows_per_step = period / inner;

  Acc<OP> acc[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) acc[j].init();

  if (active) {
    uint32_t drow[4];  // row of position t4 + j inside a step
#pragma unroll
    for (int j = 0; j < 4; ++j) drow[j] = fd_div(t4 + j, f_inner);
    const float* slab = x + static_cast<size_t>(o) * reduce * inner;
    const uint32_t end = r_end * inner;  // < 2^31: the tensor has at most INT32_MAX elements
    uint32_t f = r_begin * inner + t4, row = r_begin;
    for (; f + 3 * period + 3 < end; f += 4 * period, row += 4 * rows_per_step) {
      v4f v[4];
      const bool valid[4] = {true, true, true, true};
#pragma unroll
      for (int u = 0; u < 4; ++u) v[u] = load4_stream_any(slab + f + u * period);
      fold_batch<4, false>(acc, v, valid, [&](int u, int j) { return row + u * rows_per_step + drow[j]; });
    }
    for (; f < end; f += period, row += rows_per_step) {
      if (f + 3 < end) {
        const v4f v = load4_stream_any(slab + f);
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[j].add(v[j], row + drow[j]);
      } else {  // the share ends inside this lane's four elements
#pragma unroll
        for (int j = 0; j < 3; ++j)
          if (f + j < end) acc[j].add(slab[f + j], row + drow[j]);
      }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) lds[t4 + j] = acc[j].pack();
  }
  __syncthreads();
  if (threadIdx.x < inner) {  // inner < 128
    Acc<OP> total;
    total.init();
    for (uint32_t s = threadIdx.x; s < period; s += inner) {
      Acc<OP> t;
      t.unpack(lds[s]);
      total.merge(t);
    }
    emit_column(ld, total, o, threadIdx.x, inner, split, splits, outputs, reduce, y, part);
  }
}

// ---------------------------------------------------------------------------
// strided, one column per lane (inner % 4 != 0): x[outer][reduce][inner] ->
// y[outer][inner].  WAVES wave64 per workgroup (4 or 16) share one tile of 64
// columns and interleave over the rows of their slice; with 16 waves a few
// hundred tiles already fill the GPU and no second stage is needed.
// ---------------------------------------------------------------------------
template <int OP, int WAVES>
__global__ __launch_bounds__(kWave * WAVES) void reduce_strided_kernel(
    const float* x, float* y, Partial* part, uint32_t reduce, uint32_t inner,
    uint32_t rows_per_split, uint32_t splits, uint32_t outputs, FastDiv f_tiles, Lead ld) {
  constexpr int kWaves = WAVES;
  __shared__ Partial lds[kWaves - 1][kWave];
  const uint32_t lane = threadIdx.x & (kWave - 1), w = threadIdx.x / kWave;
  // grid.x = outer * tiles (either can exceed the 65535 limit of grid.y), grid.y = slices
  uint32_t o, tile;
  fd_divmod(xcd_contiguous(blockIdx.x, gridDim.x), f_tiles, o, tile);
  const uint32_t col = tile * kWave + lane;
  const uint32_t split = blockIdx.y;
  const bool col_ok = col < inner;
  const uint32_t r_begin = split * rows_per_split;
  uint32_t r_end = r_begin + rows_per_split;
  if (r_end > reduce) r_end = reduce;

  Acc<OP> acc;
  acc.init();
  if (col_ok) {
    const float* p = x + static_cast<size_t>(o) * reduce * inner + col;
    uint32_t r = r_begin + w;
    for (; r + 3 * kWaves < r_end; r += 4 * kWaves) {
      float v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) v[u] = __builtin_nontemporal_load(p + static_cast<size_t>(r + u * kWaves) * inner);
#pragma unroll
      for (int u = 0; u < 4; ++u) acc.add(v[u], r + u * kWaves);
    }
    for (; r < r_end; r += kWaves) acc.add(__builtin_nontemporal_load(p + static_cast<size_t>(r) * inner), r);
  }
  if (w > 0) lds[w - 1][lane] = acc.pack();
  __syncthreads();
  if (w == 0 && col_ok) {
    for (int k = 0; k < kWaves - 1; ++k) {
      Acc<OP> t;
      t.unpack(lds[k][lane]);
      acc.merge(t);
    }
    emit_column(ld, acc, o, col, inner, split, splits, outputs, reduce, y, part);
  }
}

// ---------------------------------------------------------------------------
// strided with whole 128-bit vectors per row (inner % 4 == 0, inner >= 128): a
// workgroup of 512 lanes owns a tile of 4 L columns; L lanes cover one row piece
// of the tile with one 128-bit load each and the 512 / L lane groups take rows
// r, r + 512/L, ...  All loads of a batch of eight rows per lane are requested
// before the first is used.  The accumulators meet in LDS and lane c < 4 L
// folds column c over the lane groups in group order.  Measured on max over the
// 512 channels of [32,512,28,28] (rows of 3136 bytes): 512-byte pieces (L = 32)
// 9.9 us, 256-byte pieces 10.6 us, 128-byte pieces 11.2 us, one column per lane
// with 8 / 16 waves per tile 10.1 / 11.2 us; workgroups of 256 or 1024 lanes and
// batches of 16 were level or slower.
// ---------------------------------------------------------------------------
constexpr int kTileThreads = 512;

template <int OP, int L>
__global__ __launch_bounds__(kTileThreads) void reduce_strided_tile_kernel(
    const float* x, float* y, Partial* part, uint32_t reduce, uint32_t inner, uint32_t rows_per_split,
    uint32_t splits, uint32_t outputs, FastDiv f_tiles, Lead ld) {
  constexpr uint32_t kGroups = kTileThreads / L;
  __shared__ Partial lds[kTileThreads * 4];
  uint32_t o, tile;
  fd_divmod(xcd_contiguous(blockIdx.x, gridDim.x), f_tiles, o, tile);
  const uint32_t pl = threadIdx.x % L, rg = threadIdx.x / L;
  const uint32_t col = (tile * L + pl) * 4;
  const uint32_t split = blockIdx.y;
  const uint32_t r_begin = min(split * rows_per_split, reduce);
  const uint32_t r_end = min(r_begin + rows_per_split, reduce);

  Acc<OP> acc[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) acc[j].init();

  if (col < inner) {
    const float* p = x + static_cast<size_t>(o) * reduce * inner + col;
    uint32_t base = r_begin + rg;
    // whole batches run without per-load tests: a tested load is a branch of its
    // own and the loads of a batch then no longer issue back to back
    for (; base + (kBatch - 1) * kGroups < r_end; base += kBatch * kGroups) {
      v4f v[kBatch];
      const bool valid[kBatch] = {true, true, true, true, true, true, true, true};
#pragma unroll
      for (int u = 0; u < kBatch; ++u) v[u] = load4_stream_any(p + static_cast<size_t>(base + u * kGroups) * inner);
      fold_batch<kBatch, false>(acc, v, valid, [&](int u, int) { return base + u * kGroups; });
    }
    if (base < r_end) {
      v4f v[kBatch];
      bool valid[kBatch];
#pragma unroll
      for (int u = 0; u < kBatch; ++u) {
        const uint32_t r = base + u * kGroups;
        valid[u] = r < r_end;
        if (valid[u]) v[u] = load4_stream_any(p + static_cast<size_t>(r) * inner);
      }
      fold_batch<kBatch, false>(acc, v, valid, [&](int u, int) { return base + u * kGroups; });
    }
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) lds[threadIdx.x * 4 + j] = acc[j].pack();  // [group][column of the tile]
  __syncthreads();
  if (threadIdx.x < 4 * L) {
    const uint32_t c = tile * 4 * L + threadIdx.x;
    Acc<OP> total;
    total.init();
    for (uint32_t g = 0; g < kGroups; ++g) {
      Acc<OP> t;
      t.unpack(lds[g * 4 * L + threadIdx.x]);
      total.merge(t);
    }
    if (c < inner) emit_column(ld, total, o, c, inner, split, splits, outputs, reduce, y, part);
  }
}

// ---------------------------------------------------------------------------
// generic: one wave per output, kept/reduced dims decoded by constant division
// ---------------------------------------------------------------------------
struct GenericArgs {
  int nk, nr;
  FastDiv kfd[kMaxDims], rfd[kMaxDims];
  int kstride[kMaxDims], rstride[kMaxDims];
};

template <int OP>
__global__ __launch_bounds__(kBlock) void reduce_generic_kernel(GenericArgs g, const float* x,
                                                                 float* y, uint32_t outputs,
                                                                 uint32_t window) {
  const uint32_t lane = threadIdx.x & (kWave - 1);
  const uint32_t o = blockIdx.x * (kBlock / kWave) + threadIdx.x / kWave;
  if (o >= outputs) return;  // wave-uniform
  uint32_t base = 0, e = o;
  for (int k = g.nk - 1; k >= 0; --k) {
    uint32_t q, r;
    fd_divmod(e, g.kfd[k], q, r);
    base += r * static_cast<uint32_t>(g.kstride[k]);
    e = q;
  }
  Acc<OP> acc;
  acc.init();
  for (uint32_t pos = lane; pos < window; pos += kWave) {
    uint32_t off = base, t = pos;
    for (int k = g.nr - 1; k >= 0; --k) {
      uint32_t q, r;
      fd_divmod(t, g.rfd[k], q, r);
      off += r * static_cast<uint32_t>(g.rstride[k]);
      t = q;
    }
    acc.add(x[off], pos);
  }
  acc = wave_allreduce(acc);
  if (lane == 0) y[o] = acc.finalize(window);
}

// ---------------------------------------------------------------------------
// stage 2: y[o] = finalize(merge_s part[o*stride_o + s*stride_s])
//   _lane : one lane per output, slices walked serially (few slices, many
//           outputs; coalesced when stride_o == 1)
//   _block: one workgroup per output (many slices, few outputs).  The full sum
//           of 12.8 M elements leaves 3136 partials for one output: 1024 lanes
//           fold them in 2.3 us including the launch, 256 lanes in 4 us.
// ---------------------------------------------------------------------------
template <int OP>
__global__ __launch_bounds__(kBlock) void reduce_stage2_lane_kernel(const Partial* part, float* y,
                                                                     uint32_t outputs,
                                                                     uint32_t splits,
                                                                     size_t stride_o,
                                                                     size_t stride_s,
                                                                     uint32_t window) {
  const uint32_t o = blockIdx.x * kBlock + threadIdx.x;
  if (o >= outputs) return;
  Acc<OP> acc;
  acc.init();
  // eight partials requested together, merged in slice order: one lane walks up
  // to 64 of them, and a request per turn of the loop would cost a memory
  // latency each (64 rows of 200 000: 9 us of the 20 us the two launches took)
  const Partial* mine = part + o * stride_o;
  uint32_t s = 0;
  for (; s + 8 <= splits; s += 8) {
    Partial p[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) p[k] = mine[(s + k) * stride_s];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      Acc<OP> t;
      t.unpack(p[k]);
      acc.merge(t);
    }
  }
  for (; s < splits; ++s) {
    Acc<OP> t;
    t.unpack(mine[s * stride_s]);
    acc.merge(t);
  }
  y[o] = acc.finalize(window);
}

template <int OP, int THREADS>
__global__ __launch_bounds__(THREADS) void reduce_stage2_block_kernel(const Partial* part, float* y,
                                                                       uint32_t splits,
                                                                       size_t stride_o,
                                                                       size_t stride_s,
                                                                       uint32_t window) {
  __shared__ Partial lds[THREADS / kWave];
  const uint32_t o = blockIdx.x;
  Acc<OP> acc;
  acc.init();
  for (uint32_t s = threadIdx.x; s < splits; s += THREADS) {
    Acc<OP> t;
    t.unpack(part[o * stride_o + s * stride_s]);
    acc.merge(t);
  }
  acc = wave_allreduce(acc);
  const uint32_t lane = threadIdx.x & (kWave - 1), w = threadIdx.x / kWave;
  if (lane == 0) lds[w] = acc.pack();
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int k = 1; k < THREADS / kWave; ++k) {
      Acc<OP> t;
      t.unpack(lds[k]);
      acc.merge(t);
    }
    y[o] = acc.finalize(window);
  }
}

template <int OP>
static int run_stage2(const Partial* part, float* y, uint32_t outputs, uint32_t splits,
                      size_t stride_o, size_t stride_s, uint32_t window, hipStream_t st) {
  // a lane per output where the outputs fill the chip or the slices are a handful; else a workgroup per output
  if (splits <= 8 || (splits <= 64 && outputs >= 4096)) {
    reduce_stage2_lane_kernel<OP><<<grid_for(outputs), kBlock, 0, st>>>(part, y, outputs, splits,
                                                                        stride_o, stride_s, window);
  } else if (splits <= 256) {
    reduce_stage2_block_kernel<OP, kBlock><<<outputs, kBlock, 0, st>>>(part, y, splits, stride_o, stride_s,
                                                                       window);
  } else {
    reduce_stage2_block_kernel<OP, 1024><<<outputs, 1024, 0, st>>>(part, y, splits, stride_o, stride_s,
                                                                   window);
  }
  return launch_status();
}

// ---------------------------------------------------------------------------
// stage 2 after a first stage that reduced the leading dim of [lead][..][nest]
// (ReducePlan::nest): an output folds the partials of `slices` slices times
// `nest` columns of the first stage's view.  The first stage counted list
// positions in leading indices; the element (leading index p, nest index j) has
// list position p * nest + j.
// ---------------------------------------------------------------------------
struct Nest {
  uint32_t nest, stride, ohi_stride;
  FastDiv f_nest, f_olo;
  size_t view;  // partials per slice
  SHDW_DEVICE size_t first_column(uint32_t o) const {
    uint32_t hi, lo;
    fd_divmod(o, f_olo, hi, lo);
    return static_cast<size_t>(hi) * ohi_stride + lo;
  }
};

template <int OP>
SHDW_DEVICE Acc<OP> nested_partial(const Partial* part, const Nest& n, size_t column0, uint32_t s) {
  uint32_t slice, j;
  fd_divmod(s, n.f_nest, slice, j);
  Acc<OP> t;
  t.unpack(part[slice * n.view + column0 + static_cast<size_t>(j) * n.stride]);
  t.nest_positions(n.nest, j);
  return t;
}

template <int OP>
__global__ __launch_bounds__(kBlock) void reduce_stage2_nested_lane_kernel(const Partial* part, float* y,
                                                                            uint32_t outputs, uint32_t slices,
                                                                            Nest n, uint32_t window) {
  const uint32_t o = blockIdx.x * kBlock + threadIdx.x;
  if (o >= outputs) return;
  const size_t column0 = n.first_column(o);
  Acc<OP> acc;
  acc.init();
  const uint32_t total = slices * n.nest;
  uint32_t s = 0;
  for (; s + 8 <= total; s += 8) {  // eight requests in flight, as in reduce_stage2_lane_kernel
    Acc<OP> t[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) t[k] = nested_partial<OP>(part, n, column0, s + k);
#pragma unroll
    for (int k = 0; k < 8; ++k) acc.merge(t[k]);
  }
  for (; s < total; ++s) acc.merge(nested_partial<OP>(part, n, column0, s));
  y[o] = acc.finalize(window);
}

template <int OP>
__global__ __launch_bounds__(kBlock) void reduce_stage2_nested_block_kernel(const Partial* part, float* y,
                                                                             uint32_t slices, Nest n,
                                                                             uint32_t window) {
  __shared__ Partial lds[kBlock / kWave];
  const uint32_t o = blockIdx.x;
  const size_t column0 = n.first_column(o);
  Acc<OP> acc;
  acc.init();
  const uint32_t total = slices * n.nest;
  for (uint32_t s = threadIdx.x; s < total; s += kBlock) acc.merge(nested_partial<OP>(part, n, column0, s));
  acc = wave_allreduce(acc);
  const uint32_t lane = threadIdx.x & (kWave - 1), w = threadIdx.x / kWave;
  if (lane == 0) lds[w] = acc.pack();
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int k = 1; k < kBlock / kWave; ++k) {
      Acc<OP> t;
      t.unpack(lds[k]);
      acc.merge(t);
    }
    y[o] = acc.finalize(window);
  }
}

template <int OP>
static int run_stage2_nested(const Partial* part, float* y, const ReducePlan& pl, uint32_t window, hipStream_t st) {
  Nest n;
  n.nest = static_cast<uint32_t>(pl.nest), n.stride = static_cast<uint32_t>(pl.nest_stride);
  n.ohi_stride = static_cast<uint32_t>(pl.nest_ohi_stride);
  n.f_nest = make_fastdiv(n.nest), n.f_olo = make_fastdiv(static_cast<uint32_t>(pl.nest_olo));
  n.view = static_cast<size_t>(pl.outer * pl.inner);
  const uint32_t outputs = static_cast<uint32_t>(pl.outputs), slices = static_cast<uint32_t>(pl.splits);
  // a lane per output where the outputs fill the chip or the walk is a few partials, else a workgroup per output
  if (static_cast<uint64_t>(slices) * n.nest <= 8 || outputs >= 16384)
    reduce_stage2_nested_lane_kernel<OP><<<grid_for(outputs), kBlock, 0, st>>>(part, y, outputs, slices, n, window);
  else
    reduce_stage2_nested_block_kernel<OP><<<outputs, kBlock, 0, st>>>(part, y, slices, n, window);
  return launch_status();
}

// ---------------------------------------------------------------------------
// Partial results of shdw_hip_reduce_static: device memory of the library
// itself, one copy on every GPU the library runs on.  Host code uses the address
// that hipGetSymbolAddress returns for the current device (static_scratch), never
// this name.
// ---------------------------------------------------------------------------
constexpr size_t kStaticScratchBytes = static_cast<size_t>(1) << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mutex;
static void* g_scratch_ptr[kMaxDevices];  // device address of `scratch`, per device

static int static_scratch(void** ptr) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return static_cast<int>(e);
  if (dev < 0 || dev >= kMaxDevices) return SHDW_E_UNSUPPORTED;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return static_cast<int>(e);
    g_scratch_ptr[dev] = p;
  }
  *ptr = g_scratch_ptr[dev];
  return SHDW_OK;
}

int library_scratch_prepare() {
  void* p = nullptr;
  return static_scratch(&p);
}

template <int OP>
static int run_reduce(const ReducePlan& pl, const float* x, float* y, void* workspace,
                      size_t workspace_bytes, hipStream_t st) {
  const size_t need = reduce_workspace_bytes(pl);
  if (need > 0 && (!workspace || workspace_bytes < need)) return SHDW_E_WORKSPACE;
  Partial* part = static_cast<Partial*>(workspace);
  const uint32_t outputs = static_cast<uint32_t>(pl.outputs);
  const uint32_t window = static_cast<uint32_t>(pl.window);
  constexpr int kWaves = kBlock / kWave;

  if (pl.kind == kGeneric) {
    GenericArgs g;
    g.nk = pl.nk;
    g.nr = pl.nr;
    for (int k = 0; k < kMaxDims; ++k) {
      g.kfd[k] = make_fastdiv(k < pl.nk ? pl.kdim[k] : 1);
      g.rfd[k] = make_fastdiv(k < pl.nr ? pl.rdim[k] : 1);
      g.kstride[k] = k < pl.nk ? pl.kstride[k] : 0;
      g.rstride[k] = k < pl.nr ? pl.rstride[k] : 0;
    }
    const uint32_t grid = (outputs + kWaves - 1) / kWaves;
    reduce_generic_kernel<OP><<<grid, kBlock, 0, st>>>(g, x, y, outputs, window);
    return launch_status();
  }

  Lead ld;
  ld.count = static_cast<uint32_t>(pl.lead);
  ld.step = static_cast<uint32_t>(pl.reduce);
  ld.f_inner = make_fastdiv(static_cast<uint32_t>(pl.lead_inner));
  ld.f_count = make_fastdiv(ld.count);
  const uint32_t slots = static_cast<uint32_t>(reduce_slots(pl));  // partials per output; 1: the first stage finishes

  if (pl.kind == kRows) {
    const uint32_t rows = static_cast<uint32_t>(pl.outer);
    const uint32_t reduce = static_cast<uint32_t>(pl.reduce);
    // 128-bit loads on any dword address: rows need not start 16-byte aligned.
    const bool vec = reduce >= 4;
    if (pl.wave_per_row && reduce >= 2 && reduce <= kTinyRowMaxLen && rows >= 4096) {
      const uint32_t grid = static_cast<uint32_t>((static_cast<uint64_t>(rows) + 4 * kBlock - 1) / (4 * kBlock));
      switch (reduce) {
#define SHDW_TINY(DV) case DV: reduce_rows_tiny_kernel<OP, DV><<<grid, kBlock, 0, st>>>(x, y, rows, part, ld); break;
        SHDW_TINY(2) SHDW_TINY(3) SHDW_TINY(4) SHDW_TINY(5) SHDW_TINY(6) SHDW_TINY(7)
#undef SHDW_TINY
      }
      const int rc = launch_status();
      if (rc != SHDW_OK || slots == 1) return rc;
      return run_stage2<OP>(part, y, outputs, slots, slots, 1, window, st);
    }
    if (pl.wave_per_row && reduce < kShortRowMaxLen) {
      const uint32_t want = (reduce + 15) / 16;  // lanes for pieces of at most 16 elements (17 where that is even)
      const uint32_t lanes = want <= 1 ? 1 : (want <= 2 ? 2 : (want <= 4 ? 4 : (want <= 8 ? 8 : 16)));
      const uint32_t seg = ((reduce + lanes - 1) / lanes) | 1u;
      const uint32_t grid = (rows + kBlock / lanes - 1) / (kBlock / lanes);
      const FastDiv f4 = make_fastdiv(std::max<uint32_t>(1, reduce / 4));
#define SHDW_SHORT(LANES)                                                                                  \
  do {                                                                                                     \
    if (reduce % 4 == 0) reduce_rows_lds_kernel<OP, LANES, true><<<grid, kBlock, 0, st>>>(x, y, rows, reduce, seg, f4, part, ld);  \
    else reduce_rows_lds_kernel<OP, LANES, false><<<grid, kBlock, 0, st>>>(x, y, rows, reduce, seg, f4, part, ld);   \
  } while (0)
      if (lanes == 1) SHDW_SHORT(1);
      else if (lanes == 2) SHDW_SHORT(2);
      else if (lanes == 4) SHDW_SHORT(4);
      else if (lanes == 8) SHDW_SHORT(8);
      else SHDW_SHORT(16);
#undef SHDW_SHORT
      const int rc = launch_status();
      if (rc != SHDW_OK || slots == 1) return rc;
      return run_stage2<OP>(part, y, outputs, slots, slots, 1, window, st);
    }
    if (pl.wave_per_row) {
      // lanes per row: a lane fetches up to 8 vectors, all requested before the
      // first is consumed (measured on 784-float rows: 16 lanes 9.4 us, 32 lanes
      // 9.0 us, 64 lanes 10.4 us; with 4 requests in flight 9.9 us)
      const uint32_t units = vec ? (reduce + 3) / 4 : reduce;
      const int g = units <= 128 ? 16 : (units <= 256 ? 32 : 64);
      const uint32_t grid = (rows + kBlock / g - 1) / (kBlock / g);
#define SHDW_ROWS(V, G) reduce_rows_group_kernel<OP, V, G><<<grid, kBlock, 0, st>>>(x, y, rows, reduce, part, ld)
      if (vec) {
        if (g == 16) SHDW_ROWS(true, 16); else if (g == 32) SHDW_ROWS(true, 32); else SHDW_ROWS(true, 64);
      } else {
        if (g == 16) SHDW_ROWS(false, 16); else if (g == 32) SHDW_ROWS(false, 32); else SHDW_ROWS(false, 64);
      }
#undef SHDW_ROWS
      const int rc = launch_status();
      if (rc != SHDW_OK || slots == 1) return rc;
      return run_stage2<OP>(part, y, outputs, slots, slots, 1, window, st);
    }
    const uint32_t splits = static_cast<uint32_t>(pl.splits);
    uint32_t chunk = (reduce + splits - 1) / splits;
    chunk = (chunk + 3) & ~3u;
    const dim3 grid(rows, splits);
    if (vec)
      reduce_rows_block_kernel<OP, true><<<grid, kBlock, 0, st>>>(x, y, part, reduce, chunk, splits, ld);
    else
      reduce_rows_block_kernel<OP, false><<<grid, kBlock, 0, st>>>(x, y, part, reduce, chunk, splits, ld);
    int rc = launch_status();
    if (rc != SHDW_OK || slots == 1) return rc;
    return run_stage2<OP>(part, y, outputs, slots, slots, 1, window, st);
  }

  // strided
  const uint32_t outer = static_cast<uint32_t>(pl.outer);
  const uint32_t reduce = static_cast<uint32_t>(pl.reduce);
  const uint32_t inner = static_cast<uint32_t>(pl.inner);
  const uint32_t splits = static_cast<uint32_t>(pl.splits);
  const bool nested = pl.nest > 1;  // the kernels below then leave partials per column of their own view
  const uint32_t view = nested ? outer * inner : outputs;
  if (nested) ld.count = 0;
  const uint32_t rows_per_split = (reduce + splits - 1) / splits;
  if (pl.flat_period == 0 && splits == 1 && reduce <= kShortStridedMaxReduce) {
    // rows that are no whole vectors long: four columns per lane where a column per lane would have under
    // eight loads in flight (sum over 3 of [3][4.3M]: 17.5 -> 13.2 us per 51 MB; over 12 or 17 rows the
    // 128-bit loads off their alignment cost more than they bring, 11.5 -> 13.6 and 15.4 us) and the rows
    // are 64 columns and more (below, the lanes of a row's cut end scatter: max over 7 of [262144][7][7]
    // 24 us with a column per lane, 78 us with four)
    const bool vec = inner % 4 == 0 || (inner >= 64 && reduce < 8);
    const uint32_t per_outer = vec ? (inner + 3) / 4 : inner;
    const uint32_t units = outer * per_outer;  // <= outputs
    const FastDiv f = make_fastdiv(per_outer);
    if (vec) reduce_strided_short_kernel<OP, true><<<grid_for(units), kBlock, 0, st>>>(x, y, reduce, inner, units, f, part, view, ld);
    else reduce_strided_short_kernel<OP, false><<<grid_for(units), kBlock, 0, st>>>(x, y, reduce, inner, units, f, part, view, ld);
    const int rc = launch_status();
    if (rc != SHDW_OK) return rc;
    if (nested) return run_stage2_nested<OP>(part, y, pl, window, st);
    if (slots == 1) return rc;
    return run_stage2<OP>(part, y, outputs, slots, 1, outputs, window, st);
  }
  if (pl.flat_period > 0) {
    // grid.x carries outer (at most INT32_MAX, as the element count), grid.y the slices (<= 1024)
    reduce_strided_flat_kernel<OP><<<dim3(outer, splits), kBlock, 0, st>>>(
        x, y, part, reduce, inner, rows_per_split, splits, view, static_cast<uint32_t>(pl.flat_period),
        make_fastdiv(inner), ld);
  } else if (pl.strided_lanes > 0) {  // inner % 4 == 0: tiles of 4 * lanes columns, 128-bit loads
    const uint32_t l = static_cast<uint32_t>(pl.strided_lanes);
    const uint32_t tiles = (inner / 4 + l - 1) / l;
    const dim3 grid(tiles * outer, splits);  // tiles * outer <= outputs; splits <= 1024
    const FastDiv f_tiles = make_fastdiv(tiles);
#define SHDW_TILE(LANES)                                                                                   \
  reduce_strided_tile_kernel<OP, LANES><<<grid, kTileThreads, 0, st>>>(x, y, part, reduce, inner, rows_per_split, \
                                                                       splits, view, f_tiles, ld)
    if (l == 8) SHDW_TILE(8); else if (l == 16) SHDW_TILE(16); else if (l == 32) SHDW_TILE(32); else SHDW_TILE(64);
#undef SHDW_TILE
  } else {
    const uint32_t tiles = (inner + kWave - 1) / kWave;  // one column per lane
    const dim3 grid(tiles * outer, splits);
    const FastDiv f_tiles = make_fastdiv(tiles);
    if (pl.strided_waves == 16)
      reduce_strided_kernel<OP, 16><<<grid, kWave * 16, 0, st>>>(x, y, part, reduce, inner, rows_per_split, splits,
                                                                 view, f_tiles, ld);
    else
      reduce_strided_kernel<OP, 4><<<grid, kWave * 4, 0, st>>>(x, y, part, reduce, inner, rows_per_split, splits,
                                                               view, f_tiles, ld);
  }
  int rc = launch_status();
  if (rc != SHDW_OK) return rc;
  if (nested) return run_stage2_nested<OP>(part, y, pl, window, st);
  if (slots == 1) return rc;
  return run_stage2<OP>(part, y, outputs, slots, 1, outputs, window, st);
}

static int dispatch_reduce(int operation, const ReducePlan& pl, const float* x, float* y,
                           void* workspace, size_t workspace_bytes, hipStream_t st) {
  switch (operation) {
    case SHDW_REDUCE_PROD: return run_reduce<SHDW_REDUCE_PROD>(pl, x, y, workspace, workspace_bytes, st);
    case SHDW_REDUCE_SUM: return run_reduce<SHDW_REDUCE_SUM>(pl, x, y, workspace, workspace_bytes, st);
    case SHDW_REDUCE_MAX: return run_reduce<SHDW_REDUCE_MAX>(pl, x, y, workspace, workspace_bytes, st);
    case SHDW_REDUCE_MIN: return run_reduce<SHDW_REDUCE_MIN>(pl, x, y, workspace, workspace_bytes, st);
    case SHDW_REDUCE_AVG: return run_reduce<SHDW_REDUCE_AVG>(pl, x, y, workspace, workspace_bytes, st);
    case SHDW_REDUCE_L1: return run_reduce<SHDW_REDUCE_L1>(pl, x, y, workspace, workspace_bytes, st);
    case SHDW_REDUCE_L2: return run_reduce<SHDW_REDUCE_L2>(pl, x, y, workspace, workspace_bytes, st);
    default: return SHDW_E_INVALID_ARGUMENT;
  }
}

}  // namespace shdw

using namespace shdw;

// Max over every row of x [rows][len] when that needs no workspace (enough rows
// for a single stage): for the whole-plane max pooling, whose walk is the same.
static bool rows_max_plan(uint32_t rows, uint32_t len, ReducePlan* pl) {
  const int shape[2] = {static_cast<int>(rows), static_cast<int>(len)}, axes[1] = {1};
  return plan_reduce(2, shape, 1, axes, pl) == SHDW_OK && reduce_workspace_bytes(*pl) == 0;
}

bool shdw::reduce_rows_max_applies(uint32_t rows, uint32_t len) {
  ReducePlan pl;
  return rows_max_plan(rows, len, &pl);
}

bool shdw::reduce_rows_max(uint32_t rows, uint32_t len, const float* x, float* y, hipStream_t st, int* rc) {
  ReducePlan pl;
  if (!rows_max_plan(rows, len, &pl)) return false;
  *rc = dispatch_reduce(SHDW_REDUCE_MAX, pl, x, y, nullptr, 0, st);
  return true;
}

extern "C" {

int shdw_hip_reduce(int operation, int num_axes, const int* in_shape, int num_reduce,
                    const int* axes, const float* x, float* y, void* workspace,
                    size_t workspace_bytes, void* stream) {
  if (!x || !y) return SHDW_E_INVALID_ARGUMENT;
  ReducePlan pl;
  const int rc = plan_reduce(num_axes, in_shape, num_reduce, axes, &pl);
  if (rc != SHDW_OK) return rc;
  return dispatch_reduce(operation, pl, x, y, workspace, workspace_bytes,
                         static_cast<hipStream_t>(stream));
}

int shdw_hip_reduce_static(int operation, int num_axes, const int* in_shape, int num_reduce,
                           const int* axes, const float* x, float* y, void* stream) {
  if (!x || !y) return SHDW_E_INVALID_ARGUMENT;
  ReducePlan pl;
  int rc = plan_reduce(num_axes, in_shape, num_reduce, axes, &pl);
  if (rc != SHDW_OK) return rc;
  if (reduce_workspace_bytes(pl) > kStaticScratchBytes) return SHDW_E_STATIC_SCRATCH;
  void* ptr = nullptr;
  rc = static_scratch(&ptr);
  if (rc != SHDW_OK) return rc;
  return dispatch_reduce(operation, pl, x, y, ptr, kStaticScratchBytes, static_cast<hipStream_t>(stream));
}

size_t shdw_hip_reduce_static_max_workspace_bytes(void) { return kStaticScratchBytes; }

int shdw_hip_asum(int n, const float* x, float* result_host, void* workspace,
                  size_t workspace_bytes, void* stream) {
  if (n < 1 || !x || !result_host) return SHDW_E_INVALID_ARGUMENT;
  const int shape[1] = {n}, axes[1] = {0};
  ReducePlan pl;
  int rc = plan_reduce(1, shape, 1, axes, &pl);
  if (rc != SHDW_OK) return rc;
  // The device-side result lives in the 16 bytes after the partials.
  const size_t need = reduce_workspace_bytes(pl);
  if (!workspace || workspace_bytes < need + 16) return SHDW_E_WORKSPACE;
  float* y = reinterpret_cast<float*>(static_cast<char*>(workspace) + need);
  hipStream_t st = static_cast<hipStream_t>(stream);
  rc = dispatch_reduce(SHDW_REDUCE_L1, pl, x, y, workspace, need, st);
  if (rc != SHDW_OK) return rc;
  hipError_t e = hipMemcpyAsync(result_host, y, sizeof(float), hipMemcpyDeviceToHost, st);
  if (e != hipSuccess) return static_cast<int>(e);
  return static_cast<int>(hipStreamSynchronize(st));
}

}  // extern "C"
