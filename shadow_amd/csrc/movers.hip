// Data movers: Concat / Slice / Stack (pitched chunk copies), Gather,
// ShuffleChannel, Pad, Permute, Reorg, Resize.  No arithmetic except Resize's
// interpolation weights; everything is bound by HBM traffic (4 bytes read and 4
// written per output element).  The contiguous copies (chunks, picked rows) run
// as single-wave workgroups like the elementwise kernels (+3 %); the kernels
// that scatter or gather (Reorg, Permute, Resize) were measured slower that way
// (Reorg 72 -> 91 us) and keep 256 lanes.  Lanes are laid along the OUTPUT so stores are
// always coalesced; where the input is contiguous in the same direction both
// sides move as 128-bit vectors, and a transposing Permute goes through an LDS
// tile so that both sides stay coalesced.
#include <hip/hip_runtime.h>

#include <algorithm>

#include "../../include/shadow_hip.h"
#include "device_common.h"
#include "launch.h"
#include "plan.h"

#pragma clang fp contract(off)

namespace shdw {

// ---------------------------------------------------------------------------
// dst[n * dst_pitch + dst_off + p] = src[n * src_pitch + src_off + p], p < chunk
// ---------------------------------------------------------------------------
template <bool VEC>
__global__ __launch_bounds__(kStream) void copy_chunks_kernel(const float* src, float* dst,
                                                              uint32_t work, FastDiv f_chunk,
                                                              uint32_t src_pitch, uint32_t src_off,
                                                              uint32_t dst_pitch, uint32_t dst_off) {
  const uint32_t i = blockIdx.x * kStream + threadIdx.x;  // element, or vector when VEC
  if (i >= work) return;
  uint32_t n, p;
  fd_divmod(i, f_chunk, n, p);  // VEC: chunk, pitches and offsets are counted in vectors
  const uint64_t s = static_cast<uint64_t>(n) * src_pitch + src_off + p;
  const uint64_t d = static_cast<uint64_t>(n) * dst_pitch + dst_off + p;
  if (VEC)
    store4_stream(dst + 4 * d, load4_stream(src + 4 * s));
  else
    dst[d] = src[s];
}

// Chunks, pitches or offsets that are no whole vectors (rows of 49, a pitch of 12545): a lane still
// moves four floats of its chunk with 128-bit accesses, on whatever dword address they lie, and the
// last lane of a chunk the chunk % 4 floats that remain (one float per lane: 46 us per 51 MB for chunks
// of 12544 at a pitch of 12545, 24 us for chunks of 49).
__global__ __launch_bounds__(kStream) void copy_chunks_any_kernel(const float* src, float* dst, uint32_t work,
                                                                  uint32_t chunk, FastDiv f_units,
                                                                  uint32_t src_pitch, uint32_t src_off,
                                                                  uint32_t dst_pitch, uint32_t dst_off) {
  const uint32_t i = blockIdx.x * kStream + threadIdx.x;
  if (i >= work) return;
  uint32_t n, p;
  fd_divmod(i, f_units, n, p);
  const uint32_t first = 4 * p;
  const float* s = src + static_cast<uint64_t>(n) * src_pitch + src_off + first;
  float* d = dst + static_cast<uint64_t>(n) * dst_pitch + dst_off + first;
  if (first + 4 <= chunk) {
    store4_stream_any(d, load4_stream_any(s));
  } else {
    for (uint32_t j = 0; first + j < chunk; ++j) d[j] = s[j];
  }
}

// ---------------------------------------------------------------------------
// Rows of `inner` elements picked by a table: Gather (device index table) and
// ShuffleChannel (closed-form source row).
// ---------------------------------------------------------------------------
struct GatherRows {
  static constexpr bool kFlat = false;
  const int* indexes;
  FastDiv f_num;  // rows per outer slice on the output side
  uint32_t gather_dim;
  // source row of output row r, or -1 when the index is outside the input
  SHDW_DEVICE int64_t source(uint32_t r) const {
    uint32_t o, k;
    fd_divmod(r, f_num, o, k);
    const int g = indexes[k];
    if (g < 0 || static_cast<uint32_t>(g) >= gather_dim) return -1;
    return static_cast<int64_t>(o) * gather_dim + g;
  }
};

struct ShuffleRows {
  static constexpr bool kFlat = true;
  FastDiv f_channel, f_group;
  uint32_t group_column;
  SHDW_DEVICE int64_t source(uint32_t r) const {
    uint32_t b, c_out;
    fd_divmod(r, f_channel, b, c_out);
    uint32_t q, m;
    fd_divmod(c_out, f_group, q, m);  // c_out = q * group + m  <=>  c = m * group_column + q
    return static_cast<int64_t>(b) * f_channel.d + m * group_column + q;
  }
};

// inner % 4 == 0 and 16-byte aligned pointers: lane i moves vector i.
template <class MAP>
__global__ __launch_bounds__(kStream) void rows_pick_kernel(MAP map, const float* x, float* y,
                                                            uint32_t work, FastDiv f_inner) {
  const uint32_t i = blockIdx.x * kStream + threadIdx.x;
  if (i >= work) return;
  uint32_t r, p;
  fd_divmod(i, f_inner, r, p);  // inner counted in vectors
  const int64_t s = map.source(r);
  const v4f zero = {0.f, 0.f, 0.f, 0.f};
  store4_stream(y + 4ull * i, s < 0 ? zero : load4(x + 4 * (s * f_inner.d + p)));
}

// Rows of any length on any dword address: a lane moves the vector at floats
// 4p .. 4p + 3 of its row with 128-bit accesses, the last lane of a row the
// inner % 4 floats that remain (rows of 49 ran 2.2x slower with one float per lane).
// Gather keeps this form: its source rows come from a table in memory, and a lane
// that looks up a row per element (below) waits for one dependent load after the
// other (rows of 1: 17 us against 30 us per 17 MB gathered).
template <class MAP>
__global__ __launch_bounds__(kStream) void rows_pick_any_kernel(MAP map, const float* x, float* y,
                                                                uint32_t work, uint32_t inner,
                                                                FastDiv f_units) {
  const uint32_t i = blockIdx.x * kStream + threadIdx.x;
  if (i >= work) return;
  uint32_t r, p;
  fd_divmod(i, f_units, r, p);
  const int64_t s = map.source(r);
  const uint32_t first = 4 * p;
  float* dst = y + static_cast<uint64_t>(r) * inner + first;
  const float* src = x + s * inner + first;
  if (first + 4 <= inner) {
    const v4f zero = {0.f, 0.f, 0.f, 0.f};
    store4_stream_any(dst, s < 0 ? zero : load4_stream_any(src));
  } else {
    for (uint32_t j = 0; first + j < inner; ++j) dst[j] = s < 0 ? 0.f : src[j];
  }
}

// Rows of any length on any dword address: a lane owns four consecutive floats of the
// OUTPUT, one 128-bit store.  Where they lie in one output row (most do, from rows of a
// dozen floats on) they are four consecutive floats of one source row as well, one
// 128-bit load; a vector that runs over the end of its row takes its floats one by
// one, each from the row it belongs to.  For maps that are arithmetic only
// (ShuffleChannel; with four floats of a row per lane, above, rows of 49 ran at 1.8 x,
// rows of 7 at 3.1 x and rows of 1 at 2.7 x the time of a copy; here 1.4, 2.0, 1.1).
template <class MAP>
__global__ __launch_bounds__(kStream) void rows_pick_flat_kernel(MAP map, const float* x, float* y,
                                                                 uint32_t n4, uint32_t n, FastDiv f_inner) {
  const uint32_t i = blockIdx.x * kStream + threadIdx.x;
  const uint32_t inner = f_inner.d;
  if (i < n4) {
    uint32_t r, p;
    fd_divmod(4 * i, f_inner, r, p);
    int64_t s = map.source(r);
    v4f v;
    if (p + 4 <= inner) {
      v = s < 0 ? v4f{0.f, 0.f, 0.f, 0.f} : load4_stream_any(x + s * inner + p);
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        v[j] = s < 0 ? 0.f : __builtin_nontemporal_load(x + s * inner + p);
        if (++p == inner) p = 0, s = map.source(++r);  // never past the last row: 4 i + 3 < n
      }
    }
    store4_stream_any(y + 4ull * i, v);
  } else if (i == n4) {
    for (uint32_t t = 4 * n4; t < n; ++t) {
      uint32_t r, p;
      fd_divmod(t, f_inner, r, p);
      const int64_t s = map.source(r);
      y[t] = s < 0 ? 0.f : x[s * inner + p];
    }
  }
}

template <class MAP>
static int launch_rows_pick(const MAP& map, int64_t rows, int inner, const float* x, float* y,
                            hipStream_t st) {
  if (inner % 4 == 0 && aligned16(x) && aligned16(y)) {
    const uint32_t work = static_cast<uint32_t>(rows * (inner / 4));
    rows_pick_kernel<MAP><<<stream_grid(work), kStream, 0, st>>>(map, x, y, work, make_fastdiv(inner / 4));
  } else if (MAP::kFlat) {
    const uint32_t n = static_cast<uint32_t>(rows * inner), n4 = n / 4;
    rows_pick_flat_kernel<MAP><<<stream_grid(n4 + 1), kStream, 0, st>>>(map, x, y, n4, n,
                                                                       make_fastdiv(static_cast<uint32_t>(inner)));
  } else {
    const uint32_t units = (static_cast<uint32_t>(inner) + 3) / 4;
    const uint32_t work = static_cast<uint32_t>(rows * units);
    rows_pick_any_kernel<MAP><<<stream_grid(work), kStream, 0, st>>>(map, x, y, work, static_cast<uint32_t>(inner),
                                                                  make_fastdiv(units));
  }
  return launch_status();
}

// ---------------------------------------------------------------------------
// Pad / crop of the two trailing axes; cells outside the input take `value`.
// ---------------------------------------------------------------------------
struct PadArgs {
  int in_h, in_w, top, left;
  FastDiv f_out_w, f_out_h;
};

// Four consecutive outputs and one 128-bit store per lane.  ROWQUAD: out_w % 4
// == 0, so the four share an output row; otherwise the lane steps over row and
// plane ends (rows of 230 after padding 224 by 3 ran 2.1x slower with one
// output per lane).  Lane n4 owns the n % 4 trailing outputs.
template <bool ROWQUAD>
__global__ __launch_bounds__(kBlock) void pad_kernel(const float* x, float* y, uint32_t n4, uint32_t n,
                                                      PadArgs p, float value) {
  const uint32_t i = blockIdx.x * kBlock + threadIdx.x;
  if (i > n4) return;
  const uint32_t count = i < n4 ? 4u : n - 4 * n4;
  uint32_t rest, wo, plane, ho;
  fd_divmod(4 * i, p.f_out_w, rest, wo);
  fd_divmod(rest, p.f_out_h, plane, ho);
  float r[4];
  if (ROWQUAD) {  // one input row serves the four outputs
    const int hi = static_cast<int>(ho) - p.top, wi = static_cast<int>(wo) - p.left;
    const bool row_inside = hi >= 0 && hi < p.in_h && count == 4;
    const float* row = x + (static_cast<uint64_t>(plane) * p.in_h + (row_inside ? hi : 0)) * p.in_w;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const bool inside = row_inside && wi + j >= 0 && wi + j < p.in_w;
      r[j] = inside ? row[wi + j] : value;
    }
  } else {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int hi = static_cast<int>(ho) - p.top, wi = static_cast<int>(wo) - p.left;
      const bool inside = hi >= 0 && hi < p.in_h && wi >= 0 && wi < p.in_w && static_cast<uint32_t>(j) < count;
      r[j] = inside ? x[(static_cast<uint64_t>(plane) * p.in_h + hi) * p.in_w + wi] : value;
      if (++wo == p.f_out_w.d) {
        wo = 0;
        if (++ho == p.f_out_h.d) ho = 0, ++plane;
      }
    }
  }
  if (count == 4) {
    store4_stream_any(y + 4ull * i, v4f{r[0], r[1], r[2], r[3]});
  } else {
    for (uint32_t j = 0; j < count; ++j) y[4ull * i + j] = r[j];
  }
}

// ---------------------------------------------------------------------------
// Permute.  Generic: one output element per lane, source offset from the
// collapsed dims.  Transposing form: dims collapsed to [batch][rows][cols] ->
// [batch][cols][rows], 64 x 64 tiles through LDS.
// ---------------------------------------------------------------------------
struct PermuteArgs {
  int ndim;
  FastDiv f_out[kMaxDims];        // output extents, outermost first
  uint32_t src_stride[kMaxDims];  // input stride of the axis each output dim walks
};

template <int Q>
__global__ __launch_bounds__(kBlock) void permute_generic_kernel(const float* x, float* y, uint32_t work,
                                                                  PermuteArgs p) {
  const uint32_t i = blockIdx.x * kBlock + threadIdx.x;
  if (i >= work) return;
  uint32_t e = Q * i, src = 0;
  for (int k = p.ndim - 1; k >= 1; --k) {
    uint32_t q, r;
    fd_divmod(e, p.f_out[k], q, r);
    src += r * p.src_stride[k];
    e = q;
  }
  src += e * p.src_stride[0];
  if (Q == 4) {
    // the innermost output extent is a multiple of 4: four steps along it
    const uint32_t step = p.src_stride[p.ndim - 1];
    store4_stream(y + 4ull * i, v4f{x[src], x[src + step], x[src + 2 * step], x[src + 3 * step]});
  } else {
    y[i] = x[src];
  }
}

// Transposition with one thin side (interleaved <-> planar images: [H*W][3] <->
// [3][H*W]): the 64 x 64 tiles below would be 3 wide, nine tenths of every
// workgroup idle ([4.3M][3] -> [3][4.3M]: 229 us per 51 MB).  Here a tile takes the
// whole thin side and `span` elements of the long one; the side that is
// contiguous in memory moves with 128-bit accesses as it lies, the element
// shuffle happens in LDS.
constexpr uint32_t kThinMax = 127;         // thin side up to this many elements: the tile keeps 64 and more of the long side
constexpr uint32_t kThinNarrow = 16;       // ... and sides of 17 to 64 stay with the 64 x 64 tiles
constexpr uint32_t kThinTileFloats = 8192;  // 32 KB

// COLS_THIN: x[batch][big][thin] -> y[batch][thin][big]; else x[batch][thin][big] -> y[batch][big][thin].
// PAD: thin is a multiple of 8.  The planar side walks the tile with a stride of
// 4 * thin floats, one bank for all lanes then (thin = 8: 30 us per 51 MB against
// 22 us for thin = 17); the tile rows get a pitch of thin + 1 instead (21 us), and
// the contiguous side, whose vectors no longer sit on 16 bytes in LDS, moves its
// four floats one by one there.
template <bool COLS_THIN, bool PAD>
__global__ __launch_bounds__(kBlock) void transpose_thin_kernel(const float* x, float* y, uint32_t big,
                                                                 FastDiv f_thin, uint32_t span,
                                                                 FastDiv f_tiles) {
  __shared__ __align__(16) float tile[kThinTileFloats];  // [span][pitch], the interleaved side's order
  const uint32_t thin = f_thin.d, pitch = PAD ? thin + 1 : thin;
  uint32_t b, t;
  fd_divmod(blockIdx.x, f_tiles, b, t);
  const uint32_t first = t * span, n = min(span, big - first);  // elements of the long side in this tile
  const uint64_t image = static_cast<uint64_t>(b) * big * thin;
  const uint32_t cells = n * thin;
  const float* inter = (COLS_THIN ? x : y) + image + static_cast<uint64_t>(first) * thin;  // contiguous, cells long
  const float* planar_src = x + image + first;  // row i at + i * big (not COLS_THIN)
  float* planar_dst = y + image + first;        // row j at + j * big (COLS_THIN)
  const uint32_t quads = n / 4;                 // whole vectors per planar row
  // where vector v of the contiguous side starts in the padded tile (its four floats share a row: thin % 4 == 0)
  auto padded = [&](uint32_t v) {
    const uint32_t c = fd_div(4 * v, f_thin);
    return c * pitch + (4 * v - c * thin);
  };
  if (COLS_THIN) {
    if (PAD) {
      for (uint32_t v = threadIdx.x; v < cells / 4; v += kBlock) {
        const v4f r = load4_stream_any(inter + 4ull * v);
        float* at = tile + padded(v);
#pragma unroll
        for (int k = 0; k < 4; ++k) at[k] = r[k];
      }
    } else {
      for (uint32_t v = threadIdx.x; v < cells / 4; v += kBlock)
        *reinterpret_cast<v4f*>(tile + 4 * v) = load4_stream_any(inter + 4ull * v);
      for (uint32_t e = (cells & ~3u) + threadIdx.x; e < cells; e += kBlock) tile[e] = inter[e];
    }
    __syncthreads();
    for (uint32_t u = threadIdx.x; u < thin * quads; u += kBlock) {
      const uint32_t j = u / quads, q = u - j * quads;
      v4f r;
#pragma unroll
      for (int k = 0; k < 4; ++k) r[k] = tile[(4 * q + k) * pitch + j];
      store4_stream_any(planar_dst + static_cast<uint64_t>(j) * big + 4 * q, r);
    }
    const uint32_t rest = n - 4 * quads;
    for (uint32_t u = threadIdx.x; u < thin * rest; u += kBlock) {
      const uint32_t j = u / rest, r = 4 * quads + (u - j * rest);
      planar_dst[static_cast<uint64_t>(j) * big + r] = tile[r * pitch + j];
    }
  } else {
    for (uint32_t u = threadIdx.x; u < thin * quads; u += kBlock) {
      const uint32_t i = u / quads, q = u - i * quads;
      const v4f r = load4_stream_any(planar_src + static_cast<uint64_t>(i) * big + 4 * q);
#pragma unroll
      for (int k = 0; k < 4; ++k) tile[(4 * q + k) * pitch + i] = r[k];
    }
    const uint32_t rest = n - 4 * quads;
    for (uint32_t u = threadIdx.x; u < thin * rest; u += kBlock) {
      const uint32_t i = u / rest, c = 4 * quads + (u - i * rest);
      tile[c * pitch + i] = planar_src[static_cast<uint64_t>(i) * big + c];
    }
    __syncthreads();
    float* out = const_cast<float*>(inter);
    if (PAD) {
      for (uint32_t v = threadIdx.x; v < cells / 4; v += kBlock) {
        const float* at = tile + padded(v);
        store4_stream_any(out + 4ull * v, v4f{at[0], at[1], at[2], at[3]});
      }
    } else {
      for (uint32_t v = threadIdx.x; v < cells / 4; v += kBlock)
        store4_stream_any(out + 4ull * v, *reinterpret_cast<const v4f*>(tile + 4 * v));
      for (uint32_t e = (cells & ~3u) + threadIdx.x; e < cells; e += kBlock) out[e] = tile[e];
    }
  }
}

constexpr int kTile = 64;

// 128-bit loads along the input's fast axis and 128-bit stores along the
// output's, on whatever dword address a row starts (extents that are not
// multiples of four, odd pointers); the last vector of a row that is not whole
// moves float by float.  One float per lane instead ran at 2.2 to 2.7 times a
// copy ([24][129][4148] -> [24][4148][129]: 38 us per 51 MB).
__global__ __launch_bounds__(kBlock) void transpose_kernel(const float* x, float* y, uint32_t rows,
                                                            uint32_t cols, uint32_t tiles_c,
                                                            FastDiv f_tiles) {
  __shared__ float tile[kTile][kTile + 1];
  uint32_t batch, t, tr, tc;
  fd_divmod(blockIdx.x, f_tiles, batch, t);
  tr = t / tiles_c, tc = t - tr * tiles_c;
  const uint64_t plane = static_cast<uint64_t>(batch) * rows * cols;
  const uint32_t r0 = tr * kTile, c0 = tc * kTile;
  const uint32_t q = threadIdx.x & 15u, line = threadIdx.x >> 4;  // 16 vectors x 16 lines
#pragma unroll
  for (uint32_t k = line; k < kTile; k += kBlock / 16) {
    const uint32_t r = r0 + k, c = c0 + 4 * q;
    if (r < rows && c < cols) {
      const float* src = x + plane + static_cast<uint64_t>(r) * cols + c;
      if (c + 4 <= cols) {
        const v4f v = load4_stream_any(src);
#pragma unroll
        for (int j = 0; j < 4; ++j) tile[k][4 * q + j] = v[j];
      } else {
        for (uint32_t j = 0; c + j < cols; ++j) tile[k][4 * q + j] = __builtin_nontemporal_load(src + j);
      }
    }
  }
  __syncthreads();
#pragma unroll
  for (uint32_t k = line; k < kTile; k += kBlock / 16) {
    const uint32_t c = c0 + k, r = r0 + 4 * q;
    if (r < rows && c < cols) {
      float* dst = y + plane + static_cast<uint64_t>(c) * rows + r;
      if (r + 4 <= rows) {
        v4f v;
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = tile[4 * q + j][k];
        store4_stream_any(dst, v);
      } else {
        for (uint32_t j = 0; r + j < rows; ++j) dst[j] = tile[4 * q + j][k];
      }
    }
  }
}

// ---------------------------------------------------------------------------
// Reorg: a fixed index permutation between [B][C][H][W] and
// [B][C*s*s][H/s][W/s] (natural) or Darknet's variant of it.
// ---------------------------------------------------------------------------
struct ReorgArgs {
  int in_c, in_h, in_w, stride;
  FastDiv f_w, f_h, f_c;  // extents of the index space the lanes walk
  FastDiv f_stride, f_out_c;
};

template <bool DARKNET, int Q>
__global__ __launch_bounds__(kBlock) void reorg_kernel(const float* x, float* y, uint32_t work, ReorgArgs p) {
  const uint32_t i = blockIdx.x * kBlock + threadIdx.x;
  if (i >= work) return;
  uint32_t rest, w, h, b, c;
  fd_divmod(Q * i, p.f_w, rest, w);
  fd_divmod(rest, p.f_h, rest, h);
  fd_divmod(rest, p.f_c, b, c);
  const uint32_t s = p.stride;
  uint32_t src;  // source of the lane's first element; the next ones are `s` further
  if (DARKNET) {
    // lanes walk the input index space; the value comes from the "output" index
    uint32_t offset, c2, oh, ow;
    fd_divmod(c, p.f_out_c, offset, c2);
    fd_divmod(offset, p.f_stride, oh, ow);
    const uint32_t h2 = h * s + oh, w2 = w * s + ow;
    src = ((b * p.f_out_c.d + c2) * p.in_h * s + h2) * p.in_w * s + w2;
  } else {
    uint32_t offset, cw, c2, oh;
    fd_divmod(c, p.f_stride, offset, cw);
    fd_divmod(offset, p.f_stride, c2, oh);
    const uint32_t h2 = h * s + oh, w2 = w * s + cw;
    src = ((b * p.in_c + c2) * p.in_h + h2) * p.in_w + w2;
  }
  if (Q == 4)
    store4_stream(y + 4ull * i, v4f{x[src], x[src + s], x[src + 2 * s], x[src + 3 * s]});
  else
    y[i] = x[src];
}

// The same two maps walked from the SOURCE side: a lane reads one 128-bit vector
// (every input byte is fetched once; walking the destination reads with stride
// `s` and fetched each 32-byte sector s times over, 2.3x the traffic at s = 2)
// and scatters its four elements.  Neighbouring lanes fill the same
// destination lines, so the stores still leave L2 as whole lines.
struct ReorgScatterArgs {
  uint32_t s, src_c, dst_c, dst_h, dst_w;  // source channels; destination [.][dst_c][dst_h][dst_w]
  FastDiv f_src_w, f_src_h, f_src_c, f_s;
};

typedef float v2f __attribute__((ext_vector_type(2)));

// S2: stride 2.  Elements 0,2 of the vector are neighbours in one destination
// channel and 1,3 in the next, so they leave as two 64-bit stores that are
// contiguous across lanes.
template <bool DARKNET, bool S2>
__global__ __launch_bounds__(kBlock) void reorg_scatter_kernel(const float* x, float* y, uint32_t n4,
                                                                ReorgScatterArgs p) {
  // The natural order writes neighbouring source rows into the same destination
  // lines: XCD-contiguous workgroups let those halves meet in one L2 (72 -> 69 us);
  // the Darknet order does not share lines and is 3 us slower that way.
  const uint32_t block = DARKNET ? blockIdx.x : xcd_contiguous(blockIdx.x, gridDim.x);
  const uint32_t i = block * kBlock + threadIdx.x;
  if (i >= n4) return;
  const v4f v = load4_stream(x + 4ull * i);
  uint32_t rest, ws, hs, b, cs, h, oh;
  fd_divmod(4 * i, p.f_src_w, rest, ws);
  fd_divmod(rest, p.f_src_h, rest, hs);
  fd_divmod(rest, p.f_src_c, b, cs);
  fd_divmod(hs, p.f_s, h, oh);
  if (S2) {
    const uint32_t w = ws >> 1;  // ws is a multiple of 4: w is even, the pair is 8-byte aligned
#pragma unroll
    for (uint32_t ow = 0; ow < 2; ++ow) {
      const uint32_t c = DARKNET ? (oh * 2 + ow) * p.src_c + cs : (cs * 2 + oh) * 2 + ow;
      float* dst = y + ((static_cast<uint64_t>(b) * p.dst_c + c) * p.dst_h + h) * p.dst_w + w;
      __builtin_nontemporal_store(v2f{v[ow], v[ow + 2]}, reinterpret_cast<v2f*>(dst));
    }
    return;
  }
  // any row length: the vector may run over the end of its source row (rows of 38 or 26 floats), then the
  // next element starts the next row, channel or image
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    uint32_t w, ow;
    fd_divmod(ws, p.f_s, w, ow);
    const uint32_t c = DARKNET ? (oh * p.s + ow) * p.src_c + cs : (cs * p.s + oh) * p.s + ow;
    y[((static_cast<uint64_t>(b) * p.dst_c + c) * p.dst_h + h) * p.dst_w + w] = v[j];
    if (++ws == p.f_src_w.d) {
      ws = 0;
      if (++hs == p.f_src_h.d) {
        hs = 0;
        if (++cs == p.f_src_c.d) cs = 0, ++b;
      }
      fd_divmod(hs, p.f_s, h, oh);
    }
  }
}

// ---------------------------------------------------------------------------
// Resize of the two trailing axes.
// ---------------------------------------------------------------------------
struct ResizeArgs {
  int in_h, in_w;
  float fh, fw;
  FastDiv f_out_w, f_out_h;
};

// Nearest resize by gathers, for rows too wide for the staged kernel further
// down: four consecutive outputs and one 128-bit store per lane.
// FLAT = false: output rows of a multiple of four positions on a 16-byte
// aligned y, the four lie in one row.  FLAT = true: any output width on any
// dword address; the output is one contiguous array, the four may lie in two
// rows (or more, for rows shorter than four), so each element carries its own
// row and column (one output per lane with 4-byte stores: 228 us for x2 of
// [64,64,75,75] against 144 us).
// From HBM this kernel runs x2 of [64,64,56,56] in 64-68 us, and four times as
// many gathers in flight per lane did not change that; it reached 38 us only
// while the 51 MB input stayed in the Infinity Cache between launches.  The
// staged kernel, which reads the input rows as contiguous 128-bit spans, takes
// 48 us from HBM.
template <bool FLAT>
__global__ __launch_bounds__(kBlock) void resize_nearest_kernel(const float* x, float* y, uint32_t n,
                                                                 ResizeArgs p) {
  // neighbouring workgroups read the same input rows
  const uint32_t first = 4 * (xcd_contiguous(blockIdx.x, gridDim.x) * kBlock + threadIdx.x);
  if (first >= n) return;
  uint32_t rest, w, plane, h;
  fd_divmod(first, p.f_out_w, rest, w);
  fd_divmod(rest, p.f_out_h, plane, h);
  v4f r = {0.f, 0.f, 0.f, 0.f};
  if (!FLAT) {
    const float hf = static_cast<float>(static_cast<int>(h)) * p.fh;
    // h * (in / out) < in for every extent below 2^24; the clamps only guard larger ones
    const int src_h = min(static_cast<int>(hf), p.in_h - 1);
    const float* row = x + (static_cast<uint64_t>(plane) * p.in_h + src_h) * p.in_w;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float wf = static_cast<float>(static_cast<int>(w) + j) * p.fw;
      r[j] = row[min(static_cast<int>(wf), p.in_w - 1)];
    }
    store4_stream(y + first, r);
    return;
  }
  const uint32_t count = min(4u, n - first);
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    if (j < count) {
      const float hf = static_cast<float>(static_cast<int>(h)) * p.fh;
      const float wf = static_cast<float>(static_cast<int>(w)) * p.fw;
      const int src_h = min(static_cast<int>(hf), p.in_h - 1), src_w = min(static_cast<int>(wf), p.in_w - 1);
      r[j] = x[(static_cast<uint64_t>(plane) * p.in_h + src_h) * p.in_w + src_w];
      if (++w == p.f_out_w.d) {
        w = 0;
        if (++h == p.f_out_h.d) h = 0, ++plane;
      }
    }
  }
  if (count == 4) {
    store4_stream_any(y + first, r);
  } else {
#pragma unroll
    for (int j = 0; j < 3; ++j)
      if (j < count) y[first + j] = r[j];
  }
}

// Source coordinate, its two neighbours and the weight of the upper one.
template <bool ALIGN>
__host__ __device__ __forceinline__ void bilinear_axis(uint32_t o, float f, int extent, int& lo, int& hi,
                                                       float& frac) {
  float src;
  if (ALIGN) {
    src = static_cast<float>(static_cast<int>(o)) * f;
  } else {
    const float centre = static_cast<float>(static_cast<int>(o)) + 0.5f;
    const float scaled = centre * f;
    src = scaled - 0.5f;
    src = src < 0 ? 0 : src;
  }
  lo = static_cast<int>(src);
  hi = lo + 1;
  if (lo >= extent - 1) hi = lo = extent - 1;
  frac = src - static_cast<float>(lo);
}

template <bool ALIGN, int Q>
__global__ __launch_bounds__(kBlock) void resize_bilinear_kernel(const float* x, float* y, uint32_t work,
                                                                  ResizeArgs p) {
  const uint32_t i = blockIdx.x * kBlock + threadIdx.x;
  if (i >= work) return;
  uint32_t rest, w, plane, h;
  fd_divmod(Q * i, p.f_out_w, rest, w);
  fd_divmod(rest, p.f_out_h, plane, h);
  int h_l, h_h;
  float sh;
  bilinear_axis<ALIGN>(h, p.fh, p.in_h, h_l, h_h, sh);
  const float* img = x + static_cast<uint64_t>(plane) * p.in_h * p.in_w;
  const float* row_l = img + h_l * p.in_w;
  const float* row_h = img + h_h * p.in_w;
  const float ih = 1 - sh;
  float r[Q];
#pragma unroll
  for (int j = 0; j < Q; ++j) {
    int w_l, w_h;
    float sw;
    bilinear_axis<ALIGN>(w + j, p.fw, p.in_w, w_l, w_h, sw);
    const float v0 = row_l[w_l], v1 = row_h[w_l], v2 = row_l[w_h], v3 = row_h[w_h];
    // ((1-sh)(1-sw) v0 + sh(1-sw) v1) + (1-sh) sw v2) + sh sw v3, each product
    // formed left to right and rounded, no fused operations
    const float iw = 1 - sw;
    const float a0 = ih * iw, a1 = sh * iw, a2 = ih * sw, a3 = sh * sw;
    const float t0 = a0 * v0, t1 = a1 * v1, t2 = a2 * v2, t3 = a3 * v3;
    const float s01 = t0 + t1;
    const float s012 = s01 + t2;
    r[j] = s012 + t3;
  }
  if (Q == 4)
    store4_stream(y + 4ull * i, v4f{r[0], r[Q > 1 ? 1 : 0], r[Q > 2 ? 2 : 0], r[Q > 3 ? 3 : 0]});
  else
    y[i] = r[0];
}

// Which input index an output index reads along one axis: the bilinear pair
// and weight, or for kResizeNearest the one source position (lo == hi).
enum ResizeMode { kResizeBilinear = 0, kResizeBilinearAligned = 1, kResizeNearest = 2 };

template <int MODE>
__host__ __device__ __forceinline__ void resize_axis(uint32_t o, float f, int extent, int& lo, int& hi,
                                                     float& frac) {
  if (MODE == kResizeNearest) {
    const float src = static_cast<float>(static_cast<int>(o)) * f;
    lo = hi = min(static_cast<int>(src), extent - 1);
    frac = 0.f;
  } else {
    bilinear_axis<MODE == kResizeBilinearAligned>(o, f, extent, lo, hi, frac);
  }
}

// Resize staged through LDS, bilinear and nearest.  The bilinear kernel above
// issues sixteen 4-byte gathers per lane, and a gather occupies the address
// unit for a full wave whatever its width, so it runs at the gather rate and
// not at the HBM rate; the nearest gathers are fewer but run well only on input
// that is still in the Infinity Cache.
// Here one workgroup owns a band of `rows` output rows of one plane: it
//   1. evaluates the column axis once (neighbour offsets and weight per output
//      column) into LDS,
//   2. copies the input rows the band touches, one contiguous span of the plane,
//      into LDS with 128-bit loads,
//   3. forms each output from four LDS reads with the same operations, in the
//      same order, as the gather kernel.
// The arithmetic is unchanged, so the results are bit-identical.
struct ResizeBandArgs {
  int in_h, in_w, out_h, out_w;
  float fh, fw;
  int rows;       // output rows per band
  int tile_rows;  // input rows the LDS tile holds (the widest band's span)
  FastDiv f_bands;  // bands per plane
  FastDiv f_cols;   // lane-tasks per output row: out_w / Q
  // Small planes: a band is `group` whole planes (rows == out_h, one band per
  // plane in f_bands' sense), so that a workgroup still has a few thousand
  // outputs; their input planes are one contiguous span as well.
  int group, planes;
  FastDiv f_out_h;
};

constexpr int kResizeBandOutputs = 4096;    // outputs per workgroup aimed at
constexpr int kResizeBandLdsBytes = 20480;  // 8 workgroups per CU keep their tiles resident
constexpr int kResizeBandMaxLdsBytes = 65536;
constexpr int kResizeBandGroups = 2048;     // keep at least this many workgroups when shrinking bands

template <int MODE, int Q>
__global__ __launch_bounds__(kBlock) void resize_band_kernel(const float* x, float* y,
                                                                       ResizeBandArgs p) {
  extern __shared__ __align__(16) float band_lds[];
  const uint32_t cols_pad = (static_cast<uint32_t>(p.out_w) + 3u) & ~3u;
  float* frac = band_lds;
  uint32_t* lo_b = reinterpret_cast<uint32_t*>(band_lds + cols_pad);
  uint32_t* hi_b = lo_b + cols_pad;
  float* tile = band_lds + 3 * cols_pad;

  uint32_t plane, band;
  int h0, nrows, nplanes = 1;
  if (p.group > 1) {
    plane = blockIdx.x * static_cast<uint32_t>(p.group);
    nplanes = min(p.group, p.planes - static_cast<int>(plane));
    h0 = 0, nrows = nplanes * p.out_h;
  } else {
    fd_divmod(blockIdx.x, p.f_bands, plane, band);
    h0 = static_cast<int>(band) * p.rows;
    nrows = min(p.rows, p.out_h - h0);
  }

  for (uint32_t c = threadIdx.x; c < static_cast<uint32_t>(p.out_w); c += kBlock) {
    int w_l, w_h;
    float sw;
    resize_axis<MODE>(c, p.fw, p.in_w, w_l, w_h, sw);
    frac[c] = sw;
    lo_b[c] = static_cast<uint32_t>(w_l) * 4u;  // byte offsets inside a tile row
    hi_b[c] = static_cast<uint32_t>(w_h) * 4u;
  }

  int first = 0, last = nplanes * p.in_h - 1, unused;  // whole planes
  float unused_f;
  if (p.group <= 1) {
    resize_axis<MODE>(static_cast<uint32_t>(h0), p.fh, p.in_h, first, unused, unused_f);
    resize_axis<MODE>(static_cast<uint32_t>(h0 + nrows - 1), p.fh, p.in_h, unused, last, unused_f);
  }
  // The host sized the tile from these same expressions; the clamp only keeps a
  // disagreement from writing past the tile.
  const uint32_t span_rows = static_cast<uint32_t>(min(last - first + 1, p.tile_rows));
  const uint32_t count = span_rows * static_cast<uint32_t>(p.in_w);
  const float* src = x + (static_cast<uint64_t>(plane) * p.in_h + first) * p.in_w;
  // one contiguous span on whatever dword address the band's first row has
  for (uint32_t i = threadIdx.x; i < count / 4; i += kBlock)
    *reinterpret_cast<v4f*>(tile + 4 * i) = load4_any(src + 4 * i);
  if (threadIdx.x < (count & 3u)) tile[(count & ~3u) + threadIdx.x] = src[(count & ~3u) + threadIdx.x];
  __syncthreads();

  const char* tile_b = reinterpret_cast<const char*>(tile);
  const uint32_t row_bytes = static_cast<uint32_t>(p.in_w) * 4u;
  float* out = y + (static_cast<uint64_t>(plane) * p.out_h + h0) * p.out_w;
  if (Q == 1) {
    // Any output width: the band is one contiguous piece of y, and a lane writes
    // four consecutive elements of it with one 128-bit store on whatever dword
    // address they have; the four may lie in two rows (more, for rows shorter
    // than four), so each carries its own row and column.  f_cols divides by
    // out_w here.  Plain stores: a band ends inside a sector that the next
    // band's workgroup completes, and the halves merge in L2.
    const uint32_t total = static_cast<uint32_t>(nrows) * static_cast<uint32_t>(p.out_w);
    for (uint32_t t = threadIdx.x; 4 * t < total; t += kBlock) {
      uint32_t r, c;
      fd_divmod(4 * t, p.f_cols, r, c);
      const uint32_t valid = min(4u, total - 4 * t);
      v4f res = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (j < valid) {
          int h_l, h_h;
          float sh;
          uint32_t pl = 0, h = static_cast<uint32_t>(h0) + r;
          if (p.group > 1) fd_divmod(r, p.f_out_h, pl, h);
          resize_axis<MODE>(h, p.fh, p.in_h, h_l, h_h, sh);
          const uint32_t row0 = pl * static_cast<uint32_t>(p.in_h) - static_cast<uint32_t>(first);
          const char* row_l = tile_b + (row0 + static_cast<uint32_t>(h_l)) * row_bytes;
          const char* row_h = tile_b + (row0 + static_cast<uint32_t>(h_h)) * row_bytes;
          const float ih = 1 - sh, sw = frac[c];
          const uint32_t lo = lo_b[c], hi = hi_b[c];
          const float v0 = *reinterpret_cast<const float*>(row_l + lo);
          if (MODE == kResizeNearest) {
            res[j] = v0;
            if (++c == static_cast<uint32_t>(p.out_w)) c = 0, ++r;
            continue;
          }
          const float v1 = *reinterpret_cast<const float*>(row_h + lo);
          const float v2 = *reinterpret_cast<const float*>(row_l + hi);
          const float v3 = *reinterpret_cast<const float*>(row_h + hi);
          const float iw = 1 - sw;
          const float a0 = ih * iw, a1 = sh * iw, a2 = ih * sw, a3 = sh * sw;
          const float t0 = a0 * v0, t1 = a1 * v1, t2 = a2 * v2, t3 = a3 * v3;
          const float s01 = t0 + t1;
          const float s012 = s01 + t2;
          res[j] = s012 + t3;
          if (++c == static_cast<uint32_t>(p.out_w)) c = 0, ++r;
        }
      }
      float* dst = out + 4 * t;
      if (valid == 4) {
        *reinterpret_cast<v4f_unaligned*>(dst) = res;
      } else {
#pragma unroll
        for (int j = 0; j < 3; ++j)
          if (j < valid) dst[j] = res[j];
      }
    }
    return;
  }
  const uint32_t tasks = static_cast<uint32_t>(nrows) * p.f_cols.d;
  for (uint32_t t = threadIdx.x; t < tasks; t += kBlock) {
    uint32_t r, cq;
    fd_divmod(t, p.f_cols, r, cq);
    int h_l, h_h;
    float sh;
    uint32_t pl = 0, h = static_cast<uint32_t>(h0) + r;
    if (p.group > 1) fd_divmod(r, p.f_out_h, pl, h);
    resize_axis<MODE>(h, p.fh, p.in_h, h_l, h_h, sh);
    const uint32_t row0 = pl * static_cast<uint32_t>(p.in_h) - static_cast<uint32_t>(first);
    const char* row_l = tile_b + (row0 + static_cast<uint32_t>(h_l)) * row_bytes;
    const char* row_h = tile_b + (row0 + static_cast<uint32_t>(h_h)) * row_bytes;
    const float ih = 1 - sh;
    // Q == 4 from here on: rows of a multiple of four positions on an aligned y
    const v4f sw = *reinterpret_cast<const v4f*>(frac + 4 * cq);
    const v4u lo = *reinterpret_cast<const v4u*>(lo_b + 4 * cq);
    const v4u hi = *reinterpret_cast<const v4u*>(hi_b + 4 * cq);
    v4f res;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float v0 = *reinterpret_cast<const float*>(row_l + lo[j]);
      if (MODE == kResizeNearest) {
        res[j] = v0;
        continue;
      }
      const float v1 = *reinterpret_cast<const float*>(row_h + lo[j]);
      const float v2 = *reinterpret_cast<const float*>(row_l + hi[j]);
      const float v3 = *reinterpret_cast<const float*>(row_h + hi[j]);
      const float iw = 1 - sw[j];
      const float a0 = ih * iw, a1 = sh * iw, a2 = ih * sw[j], a3 = sh * sw[j];
      const float t0 = a0 * v0, t1 = a1 * v1, t2 = a2 * v2, t3 = a3 * v3;
      const float s01 = t0 + t1;
      const float s012 = s01 + t2;
      res[j] = s012 + t3;
    }
    store4_stream(out + static_cast<uint64_t>(r) * p.out_w + 4 * cq, res);
  }
}

// Band height and tile size for the kernel above; false when even a one-row
// band does not fit (very wide rows or a strong vertical reduction).
template <int MODE>
static bool plan_resize_band(int planes, int in_h, int in_w, int out_h, int out_w, float fh,
                             ResizeBandArgs* p, size_t* lds_bytes) {
  const size_t table_bytes = 3 * static_cast<size_t>((out_w + 3) & ~3) * 4;
  p->group = 1, p->planes = planes, p->f_out_h = make_fastdiv(out_h);
  const int64_t plane_outputs = static_cast<int64_t>(out_h) * out_w;
  if (2 * plane_outputs <= kResizeBandOutputs) {
    // x2 of 13x13 maps: 676 outputs per plane; one plane per workgroup ran at 25 us
    // per 56 MB where the gather kernel took 12
    int group = static_cast<int>(std::min<int64_t>(planes, kResizeBandOutputs / plane_outputs));
    while (group > 1 && (planes + group - 1) / group < kResizeBandGroups) group = (group + 1) / 2;
    while (group > 1 && table_bytes + static_cast<size_t>(group) * in_h * in_w * 4 > kResizeBandLdsBytes)
      group = (group + 1) / 2;
    if (group > 1) {
      p->group = group;
      p->rows = out_h, p->tile_rows = group * in_h;
      p->f_bands = make_fastdiv(1);
      *lds_bytes = table_bytes + static_cast<size_t>(group) * in_h * in_w * 4;
      return true;
    }
  }
  int rows = std::max(1, std::min(out_h, kResizeBandOutputs / out_w));
  while (rows > 1 && static_cast<int64_t>(planes) * ((out_h + rows - 1) / rows) < kResizeBandGroups)
    rows = (rows + 1) / 2;
  for (;; rows = (rows + 1) / 2) {
    int tile_rows = 1;
    for (int h0 = 0; h0 < out_h; h0 += rows) {
      int first, last, unused;
      float unused_f;
      resize_axis<MODE>(static_cast<uint32_t>(h0), fh, in_h, first, unused, unused_f);
      resize_axis<MODE>(static_cast<uint32_t>(std::min(h0 + rows, out_h) - 1), fh, in_h, unused, last,
                           unused_f);
      tile_rows = std::max(tile_rows, last - first + 1);
    }
    const size_t bytes = table_bytes + static_cast<size_t>(tile_rows) * in_w * 4;
    if (bytes <= static_cast<size_t>(kResizeBandLdsBytes) || (rows == 1 && bytes <= kResizeBandMaxLdsBytes)) {
      p->rows = rows, p->tile_rows = tile_rows;
      p->f_bands = make_fastdiv((out_h + rows - 1) / rows);
      *lds_bytes = bytes;
      return true;
    }
    if (rows == 1) return false;
  }
}

template <int MODE>
static bool launch_resize_band(int planes, int in_h, int in_w, int out_h, int out_w, float fh, float fw,
                               bool quad, const float* x, float* y, hipStream_t st) {
  ResizeBandArgs p;
  size_t lds_bytes;
  if (!plan_resize_band<MODE>(planes, in_h, in_w, out_h, out_w, fh, &p, &lds_bytes)) return false;
  p.in_h = in_h, p.in_w = in_w, p.out_h = out_h, p.out_w = out_w, p.fh = fh, p.fw = fw;
  const uint32_t grid = p.group > 1 ? static_cast<uint32_t>((planes + p.group - 1) / p.group)
                                    : static_cast<uint32_t>(planes) * p.f_bands.d;
  if (quad) {
    p.f_cols = make_fastdiv(out_w / 4);
    resize_band_kernel<MODE, 4><<<grid, kBlock, lds_bytes, st>>>(x, y, p);
  } else {
    p.f_cols = make_fastdiv(out_w);
    resize_band_kernel<MODE, 1><<<grid, kBlock, lds_bytes, st>>>(x, y, p);
  }
  return true;
}

// ---------------------------------------------------------------------------
// Resize by exactly two along both axes (decoder and pyramid upsampling), rows
// of an even number (>= 4) of positions: no staging.  fh = fw = 0.5 exactly, so
// every output vector of four columns 4o ... 4o+3 reads the input columns
// 2o-1 ... 2o+2 (bilinear) or 2o, 2o+1 (nearest) of one or two rows: one or two
// 128-bit loads per lane on whatever dword address, neighbours overlapping in the
// caches, and one 128-bit store per output row.  Source indices and weights
// still come from resize_axis / bilinear_axis and the sums are formed in the
// same order as everywhere else, so the results are the same bits.
// ---------------------------------------------------------------------------
struct ResizeDoubleArgs {
  int in_h, in_w;
  uint32_t out_w;
  FastDiv f_vecs;   // output vectors per row: out_w / 4 = in_w / 2
  FastDiv f_pairs;  // bilinear: row pairs per plane, in_h + 1
};

// Nearest: lane t owns the input pair x[2t], x[2t + 1] (the input is one flat
// array of such pairs) and writes it, doubled, to two output rows: 43 us for
// [64,64,56,56] where the staged kernel takes 48.  Two pairs per lane (a
// 128-bit load, two stores side by side per row) took 93 us: a store instruction
// then covers every other 16 bytes.  Workgroups of 256 lanes and plain instead of
// streaming stores: 44 to 46 us.
__global__ __launch_bounds__(kStream) void resize_double_nearest_kernel(const float* x, float* y, uint32_t tasks,
                                                                        ResizeDoubleArgs p) {
  const uint32_t t = blockIdx.x * kStream + threadIdx.x;
  if (t >= tasks) return;
  typedef float v2f __attribute__((ext_vector_type(2)));
  const v2f v = __builtin_nontemporal_load(reinterpret_cast<const v2f*>(x) + t);
  uint32_t row, o;  // row counts input rows over all planes; o the lane's place in the row
  fd_divmod(t, p.f_vecs, row, o);
  float* dst = y + 2 * row * p.out_w + 4 * o;
  const v4f r = {v[0], v[0], v[1], v[1]};
  store4_stream(dst, r);
  store4_stream(dst + p.out_w, r);
}

// Bilinear: output rows 2q - 1 and 2q (q = 0 ... in_h; the first pair has only
// its second row, the last only its first) have the same two source rows.
// With f = 0.5 the axis rule (bilinear_axis) gives, for output index i:
//   i = 0: neighbours 0, 1, weight 0 (the coordinate -0.25 is clamped to 0);
//   i = 2m - 1: neighbours m-1, m, weight 0.25;   i = 2m: m-1, m, weight 0.75;
// an upper neighbour beyond the extent is the lower one again.  All of these
// weights and their products are exact, so forming them here from constants
// gives the bits of the general kernels, which take them from bilinear_axis; the
// host checks the rule against bilinear_axis before it launches this kernel.
__global__ __launch_bounds__(kBlock) void resize_double_bilinear_kernel(const float* x, float* y, uint32_t tasks,
                                                                        ResizeDoubleArgs p) {
  // runs of eight workgroups (about 70 row pairs) on one XCD: neighbouring pairs share a source row
  // and the ends of their output rows share lines (42.0 -> 40.8 us on [64,64,56,56]; each XCD on one
  // contiguous eighth of the pairs: no change)
  const uint32_t t = xcd_runs(blockIdx.x, gridDim.x, 3) * kBlock + threadIdx.x;
  if (t >= tasks) return;
  uint32_t rest, o, plane, q;
  fd_divmod(t, p.f_vecs, rest, o);
  fd_divmod(rest, p.f_pairs, plane, q);
  const uint32_t in_h = static_cast<uint32_t>(p.in_h), in_w = static_cast<uint32_t>(p.in_w);
  const bool top = q == 0, has_b = q < in_h;
  const uint32_t h_l = top ? 0u : q - 1;
  const uint32_t h_h = min(top ? 1u : q, in_h - 1);
  const float sh_b = top ? 0.f : 0.75f, ih_b = top ? 1.f : 0.25f;  // row 2q; row 2q - 1: 0.25, 0.75

  // columns 2o-1 ... 2o+2, of which the first lane of a row lacks the first and
  // the last lane the last: the window moves inside the row and e[] repeats the
  // edge column, which is what the clamped neighbours read there
  const int want = 2 * static_cast<int>(o) - 1;
  const int base = min(max(want, 0), p.in_w - 4);
  const bool first = want < 0, last = want > base;
  const uint32_t plane_at = plane * in_h * in_w + static_cast<uint32_t>(base);
  const v4f wl = load4_any(x + (plane_at + h_l * in_w)), wh = load4_any(x + (plane_at + h_h * in_w));
  float el[4], eh[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int down = k > 0 ? k - 1 : 0, up = k < 3 ? k + 1 : 3;
    el[k] = first ? wl[down] : (last ? wl[up] : wl[k]);
    eh[k] = first ? wh[down] : (last ? wh[up] : wh[k]);
  }
  v4f res_a, res_b;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    // neighbours e[kl], e[kl + 1] with kl = 0, 1, 1, 2; column 0 of the row has
    // e[1], e[2] (columns 0 and 1) and weight 0
    const int kl = j == 0 ? 0 : (j == 3 ? 2 : 1);
    const bool col0 = j == 0 && first;
    const float v0 = col0 ? el[1] : el[kl], v1 = col0 ? eh[1] : eh[kl];
    const float v2 = col0 ? el[2] : el[kl + 1], v3 = col0 ? eh[2] : eh[kl + 1];
    const float sw = (j & 1) ? 0.25f : (col0 ? 0.f : 0.75f);
    const float iw = (j & 1) ? 0.75f : (col0 ? 1.f : 0.25f);
    {
      const float ih = 0.75f, sh = 0.25f;
      const float a0 = ih * iw, a1 = sh * iw, a2 = ih * sw, a3 = sh * sw;
      const float t0 = a0 * v0, t1 = a1 * v1, t2 = a2 * v2, t3 = a3 * v3;
      const float s01 = t0 + t1;
      const float s012 = s01 + t2;
      res_a[j] = s012 + t3;
    }
    {
      const float a0 = ih_b * iw, a1 = sh_b * iw, a2 = ih_b * sw, a3 = sh_b * sw;
      const float t0 = a0 * v0, t1 = a1 * v1, t2 = a2 * v2, t3 = a3 * v3;
      const float s01 = t0 + t1;
      const float s012 = s01 + t2;
      res_b[j] = s012 + t3;
    }
  }
  float* dst = y + ((plane * (2 * in_h) + 2 * q) * p.out_w + 4 * o);  // row 2q
  if (!top) store4_stream(dst - p.out_w, res_a);
  if (has_b) store4_stream(dst, res_b);
}

// The rule the bilinear kernel above is written from, against bilinear_axis.
static bool double_rule_holds(int extent) {
  for (int i = 0; i < std::min(2 * extent, 64); ++i) {
    int lo, hi;
    float frac;
    bilinear_axis<false>(static_cast<uint32_t>(i), 0.5f, extent, lo, hi, frac);
    const int m = (i + 1) / 2;
    const int want_lo = i == 0 ? 0 : m - 1, want_hi = std::min(i == 0 ? 1 : m, extent - 1);
    const float want_frac = i == 0 ? 0.f : ((i & 1) ? 0.25f : 0.75f);
    if (lo != want_lo || hi != want_hi || frac != want_frac) return false;
  }
  return true;
}

// True when the kernels above apply (and then they have been launched).
static bool launch_resize_double(int type, int planes, int in_h, int in_w, int out_h, int out_w, const float* x,
                                 float* y, hipStream_t st) {
  if (out_h != 2 * in_h || out_w != 2 * in_w || in_w % 2 != 0 || in_w < 4 || !aligned16(y)) return false;
  ResizeDoubleArgs p;
  p.in_h = in_h, p.in_w = in_w, p.out_w = static_cast<uint32_t>(out_w);
  // the factors as shdw_hip_resize forms them: exactly one half
  if (static_cast<float>(in_h) / out_h != 0.5f || static_cast<float>(in_w) / out_w != 0.5f) return false;
  p.f_vecs = make_fastdiv(in_w / 2), p.f_pairs = make_fastdiv(in_h + 1);
  if (type == 0) {
    const uintptr_t at = reinterpret_cast<uintptr_t>(x);
    const uint32_t pairs = static_cast<uint32_t>(planes) * in_h * (in_w / 2);
    if ((at & 7u) != 0) return false;
    resize_double_nearest_kernel<<<stream_grid(pairs), kStream, 0, st>>>(x, y, pairs, p);
    return true;
  }
  const int64_t tasks = static_cast<int64_t>(planes) * (in_h + 1) * (in_w / 2);
  if (tasks > INT32_MAX || !double_rule_holds(in_h) || !double_rule_holds(in_w)) return false;
  // 256 lanes per workgroup: 47 to 48 us for [64,64,56,56] against 50 for single waves (staged kernel: 56)
  resize_double_bilinear_kernel<<<grid_for(static_cast<uint32_t>(tasks)), kBlock, 0, st>>>(
      x, y, static_cast<uint32_t>(tasks), p);
  return true;
}

static bool count_fits(const int* shape, int n, int64_t* count) {
  int64_t c = 1;
  for (int k = 0; k < n; ++k) {
    if (shape[k] < 0) return false;
    c *= shape[k];
    if (c > INT32_MAX) return false;
  }
  *count = c;
  return true;
}

}  // namespace shdw

using namespace shdw;

extern "C" {

int shdw_hip_copy_chunks(int outer, int chunk, const float* src, int src_pitch, int src_offset,
                         float* dst, int dst_pitch, int dst_offset, void* stream) {
  if (outer < 0 || chunk < 0 || src_offset < 0 || dst_offset < 0) return SHDW_E_INVALID_ARGUMENT;
  if (static_cast<int64_t>(src_offset) + chunk > src_pitch ||
      static_cast<int64_t>(dst_offset) + chunk > dst_pitch)
    return SHDW_E_INVALID_ARGUMENT;  // a chunk must stay inside its row
  if (static_cast<int64_t>(outer) * src_pitch > INT32_MAX ||
      static_cast<int64_t>(outer) * dst_pitch > INT32_MAX)
    return SHDW_E_INVALID_ARGUMENT;
  if (outer == 0 || chunk == 0) return SHDW_OK;
  if (!src || !dst) return SHDW_E_INVALID_ARGUMENT;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool vec = ((chunk | src_pitch | src_offset | dst_pitch | dst_offset) & 3) == 0 &&
                   aligned16(src) && aligned16(dst);
  if (vec) {
    const uint32_t work = static_cast<uint32_t>(outer) * (chunk / 4);
    copy_chunks_kernel<true><<<stream_grid(work), kStream, 0, st>>>(
        src, dst, work, make_fastdiv(chunk / 4), src_pitch / 4, src_offset / 4, dst_pitch / 4,
        dst_offset / 4);
  } else if (chunk >= 4) {
    const uint32_t units = (static_cast<uint32_t>(chunk) + 3) / 4;
    const uint32_t work = static_cast<uint32_t>(outer) * units;  // <= outer * chunk
    copy_chunks_any_kernel<<<stream_grid(work), kStream, 0, st>>>(src, dst, work, static_cast<uint32_t>(chunk),
                                                                 make_fastdiv(units), src_pitch, src_offset,
                                                                 dst_pitch, dst_offset);
  } else {
    const uint32_t work = static_cast<uint32_t>(outer) * chunk;
    copy_chunks_kernel<false><<<stream_grid(work), kStream, 0, st>>>(
        src, dst, work, make_fastdiv(chunk), src_pitch, src_offset, dst_pitch, dst_offset);
  }
  return launch_status();
}

int shdw_hip_gather(int outer_num, int gather_dim, int inner_num, int num_indexes,
                    const int* indexes, const float* x, float* y, void* stream) {
  if (outer_num < 0 || gather_dim < 1 || inner_num < 0 || num_indexes < 1)
    return SHDW_E_INVALID_ARGUMENT;
  const int64_t rows = static_cast<int64_t>(outer_num) * num_indexes;
  if (rows * inner_num > INT32_MAX || static_cast<int64_t>(outer_num) * gather_dim * inner_num > INT32_MAX)
    return SHDW_E_INVALID_ARGUMENT;
  if (rows * inner_num == 0) return SHDW_OK;
  if (!indexes || !x || !y) return SHDW_E_INVALID_ARGUMENT;
  GatherRows map{indexes, make_fastdiv(num_indexes), static_cast<uint32_t>(gather_dim)};
  return launch_rows_pick(map, rows, inner_num, x, y, static_cast<hipStream_t>(stream));
}

int shdw_hip_shuffle_channel(int batch, int channel, int spatial_dim, int group, const float* x,
                             float* y, void* stream) {
  if (batch < 0 || channel < 1 || spatial_dim < 0 || group < 1 || channel % group != 0)
    return SHDW_E_INVALID_ARGUMENT;
  const int64_t rows = static_cast<int64_t>(batch) * channel;
  if (rows * spatial_dim > INT32_MAX) return SHDW_E_INVALID_ARGUMENT;
  if (rows * spatial_dim == 0) return SHDW_OK;
  if (!x || !y) return SHDW_E_INVALID_ARGUMENT;
  ShuffleRows map{make_fastdiv(channel), make_fastdiv(group), static_cast<uint32_t>(channel / group)};
  return launch_rows_pick(map, rows, spatial_dim, x, y, static_cast<hipStream_t>(stream));
}

int shdw_hip_pad(const int* in_shape, const int* paddings, float value, const float* x, float* y,
                 void* stream) {
  if (!in_shape || !paddings) return SHDW_E_INVALID_ARGUMENT;
  int out_shape[4] = {in_shape[0], in_shape[1], in_shape[2] + paddings[0] + paddings[1],
                      in_shape[3] + paddings[2] + paddings[3]};
  int64_t in_count, out_count;
  if (!count_fits(in_shape, 4, &in_count) || !count_fits(out_shape, 4, &out_count))
    return SHDW_E_INVALID_ARGUMENT;
  if (out_count == 0) return SHDW_OK;
  if (!y || (in_count > 0 && !x)) return SHDW_E_INVALID_ARGUMENT;
  PadArgs p{in_shape[2], in_shape[3], paddings[0], paddings[2], make_fastdiv(out_shape[3]),
            make_fastdiv(out_shape[2])};
  const uint32_t n = static_cast<uint32_t>(out_count);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (out_shape[3] % 4 == 0)
    pad_kernel<true><<<grid_for(n / 4 + 1), kBlock, 0, st>>>(x, y, n / 4, n, p, value);
  else
    pad_kernel<false><<<grid_for(n / 4 + 1), kBlock, 0, st>>>(x, y, n / 4, n, p, value);
  return launch_status();
}

int shdw_hip_permute(int num_axes, const int* in_shape, const int* order, const float* x, float* y,
                     void* stream) {
  if (num_axes < 1 || num_axes > kMaxDims || !in_shape || !order) return SHDW_E_INVALID_ARGUMENT;
  int64_t count;
  if (!count_fits(in_shape, num_axes, &count)) return SHDW_E_INVALID_ARGUMENT;
  bool seen[kMaxDims] = {false};
  for (int k = 0; k < num_axes; ++k) {
    if (order[k] < 0 || order[k] >= num_axes || seen[order[k]]) return SHDW_E_INVALID_ARGUMENT;
    seen[order[k]] = true;
  }
  if (count == 0) return SHDW_OK;
  if (!x || !y) return SHDW_E_INVALID_ARGUMENT;
  hipStream_t st = static_cast<hipStream_t>(stream);

  // Input strides; then output dims (extent, input stride), dropping extent-1
  // dims and merging neighbours that are also neighbours in the input.
  int64_t in_stride[kMaxDims];
  in_stride[num_axes - 1] = 1;
  for (int d = num_axes - 2; d >= 0; --d) in_stride[d] = in_stride[d + 1] * in_shape[d + 1];
  int nd = 0;
  int64_t ext[kMaxDims], str[kMaxDims];
  for (int k = 0; k < num_axes; ++k) {
    const int64_t e = in_shape[order[k]], s = in_stride[order[k]];
    if (e == 1) continue;
    if (nd > 0 && str[nd - 1] == s * e) {
      ext[nd - 1] *= e;
      str[nd - 1] = s;
    } else {
      ext[nd] = e, str[nd] = s, ++nd;
    }
  }
  const uint32_t n = static_cast<uint32_t>(count);
  if (nd <= 1) {  // the order keeps memory as it is
    return shdw_hip_copy(static_cast<int>(count), x, y, stream);
  }
  // [batch][rows][cols] -> [batch][cols][rows]
  const bool plain2 = nd == 2 && str[0] == 1 && str[1] == ext[0];
  const bool batch3 = nd == 3 && str[1] == 1 && str[2] == ext[1] && str[0] == ext[1] * ext[2];
  if (plain2 || batch3) {
    const uint32_t batch = plain2 ? 1u : static_cast<uint32_t>(ext[0]);
    const uint32_t cols = static_cast<uint32_t>(plain2 ? ext[0] : ext[1]);  // input's fast axis
    const uint32_t rows = static_cast<uint32_t>(plain2 ? ext[1] : ext[2]);
    // sides of 17 to 64 fill a 64 x 64 tile well enough: measured level with the thin kernel or ahead of it
    const uint32_t side = std::min(rows, cols);
    if ((side <= kThinNarrow || (side > static_cast<uint32_t>(kTile) && side <= kThinMax)) && std::max(rows, cols) >= 256) {
      const bool cols_thin = cols <= rows;
      const uint32_t thin = cols_thin ? cols : rows, big = cols_thin ? rows : cols;
      const bool pad = thin % 8 == 0;
      const uint32_t span = (kThinTileFloats / (thin + (pad ? 1 : 0))) & ~63u;
      const uint32_t tiles = span ? (big + span - 1) / span : 0;  // span 0: a padded side of 128 does not fit
      const int64_t groups = static_cast<int64_t>(batch) * tiles;
      if (span && groups <= INT32_MAX) {
        const FastDiv ft = make_fastdiv(tiles), fthin = make_fastdiv(thin);
        const uint32_t g = static_cast<uint32_t>(groups);
        if (cols_thin && pad)
          transpose_thin_kernel<true, true><<<g, kBlock, 0, st>>>(x, y, big, fthin, span, ft);
        else if (cols_thin)
          transpose_thin_kernel<true, false><<<g, kBlock, 0, st>>>(x, y, big, fthin, span, ft);
        else if (pad)
          transpose_thin_kernel<false, true><<<g, kBlock, 0, st>>>(x, y, big, fthin, span, ft);
        else
          transpose_thin_kernel<false, false><<<g, kBlock, 0, st>>>(x, y, big, fthin, span, ft);
        return launch_status();
      }
    }
    const uint32_t tiles_r = (rows + kTile - 1) / kTile, tiles_c = (cols + kTile - 1) / kTile;
    const int64_t groups = static_cast<int64_t>(batch) * tiles_r * tiles_c;
    if (groups <= INT32_MAX) {
      const FastDiv ft = make_fastdiv(tiles_r * tiles_c);
      const uint32_t g = static_cast<uint32_t>(groups);
      transpose_kernel<<<g, kBlock, 0, st>>>(x, y, rows, cols, tiles_c, ft);
      return launch_status();
    }
  }
  PermuteArgs p;
  p.ndim = nd;
  for (int k = 0; k < nd; ++k) {
    p.f_out[k] = make_fastdiv(static_cast<uint32_t>(ext[k]));
    p.src_stride[k] = static_cast<uint32_t>(str[k]);
  }
  if (ext[nd - 1] % 4 == 0 && aligned16(y))
    permute_generic_kernel<4><<<grid_for(n / 4), kBlock, 0, st>>>(x, y, n / 4, p);
  else
    permute_generic_kernel<1><<<grid_for(n), kBlock, 0, st>>>(x, y, n, p);
  return launch_status();
}

int shdw_hip_reorg(const int* in_shape, int type, int stride, const float* x, float* y,
                   void* stream) {
  if (!in_shape || stride < 1 || type < 0 || type > 1) return SHDW_E_INVALID_ARGUMENT;
  int64_t count;
  if (!count_fits(in_shape, 4, &count)) return SHDW_E_INVALID_ARGUMENT;
  const int in_c = in_shape[1], in_h = in_shape[2], in_w = in_shape[3];
  if (in_h % stride != 0 || in_w % stride != 0) return SHDW_E_INVALID_ARGUMENT;
  if (type == 0 && in_c % (stride * stride) != 0) return SHDW_E_INVALID_ARGUMENT;
  if (count == 0) return SHDW_OK;
  if (!x || !y) return SHDW_E_INVALID_ARGUMENT;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const uint32_t n = static_cast<uint32_t>(count);
  const int ss = stride * stride;
  // source-side walk whenever the tensor is whole vectors (one float per lane from the destination side ran
  // the natural order on 38x38 maps at 39 us per 51 MB against 20 us)
  const int src_w = type == 0 ? in_w * stride : in_w;
  if (n % 4 == 0 && aligned16(x)) {
    ReorgScatterArgs a;
    a.s = stride;
    if (type == 0) {  // source = the [B][C/ss][H*s][W*s] view, destination = [B][C][H][W]
      a.src_c = in_c / ss, a.dst_c = in_c, a.dst_h = in_h, a.dst_w = in_w;
      a.f_src_w = make_fastdiv(in_w * stride), a.f_src_h = make_fastdiv(in_h * stride);
    } else {  // source = [B][C][H][W], destination = [B][C*ss][H/s][W/s]
      a.src_c = in_c, a.dst_c = in_c * ss, a.dst_h = in_h / stride, a.dst_w = in_w / stride;
      a.f_src_w = make_fastdiv(in_w), a.f_src_h = make_fastdiv(in_h);
    }
    a.f_src_c = make_fastdiv(a.src_c);
    a.f_s = make_fastdiv(stride);
    // 64-bit stores need an even destination row length and an 8-byte aligned base
    const bool s2 = stride == 2 && src_w % 4 == 0 && a.dst_w % 2 == 0 && (reinterpret_cast<uintptr_t>(y) & 7u) == 0;
    const uint32_t g = grid_for(n / 4);
    if (type == 0) {
      if (s2)
        reorg_scatter_kernel<true, true><<<g, kBlock, 0, st>>>(x, y, n / 4, a);
      else
        reorg_scatter_kernel<true, false><<<g, kBlock, 0, st>>>(x, y, n / 4, a);
    } else {
      if (s2)
        reorg_scatter_kernel<false, true><<<g, kBlock, 0, st>>>(x, y, n / 4, a);
      else
        reorg_scatter_kernel<false, false><<<g, kBlock, 0, st>>>(x, y, n / 4, a);
    }
    return launch_status();
  }
  ReorgArgs p;
  p.in_c = in_c, p.in_h = in_h, p.in_w = in_w, p.stride = stride;
  p.f_stride = make_fastdiv(stride);
  if (type == 0) {
    p.f_w = make_fastdiv(in_w), p.f_h = make_fastdiv(in_h), p.f_c = make_fastdiv(in_c);
    p.f_out_c = make_fastdiv(in_c / (stride * stride));
    if (in_w % 4 == 0 && aligned16(y))
      reorg_kernel<true, 4><<<grid_for(n / 4), kBlock, 0, st>>>(x, y, n / 4, p);
    else
      reorg_kernel<true, 1><<<grid_for(n), kBlock, 0, st>>>(x, y, n, p);
  } else {
    p.f_w = make_fastdiv(in_w / stride), p.f_h = make_fastdiv(in_h / stride);
    p.f_c = make_fastdiv(in_c * stride * stride);
    p.f_out_c = make_fastdiv(1);
    if ((in_w / stride) % 4 == 0 && aligned16(y))
      reorg_kernel<false, 4><<<grid_for(n / 4), kBlock, 0, st>>>(x, y, n / 4, p);
    else
      reorg_kernel<false, 1><<<grid_for(n), kBlock, 0, st>>>(x, y, n, p);
  }
  return launch_status();
}

int shdw_hip_resize(const int* in_shape, const int* out_shape, int type, int align_corners,
                    const float* x, float* y, void* stream) {
  if (!in_shape || !out_shape || type < 0 || type > 1) return SHDW_E_INVALID_ARGUMENT;
  int64_t in_count, out_count;
  if (!count_fits(in_shape, 4, &in_count) || !count_fits(out_shape, 4, &out_count))
    return SHDW_E_INVALID_ARGUMENT;
  if (in_shape[0] != out_shape[0] || in_shape[1] != out_shape[1]) return SHDW_E_INVALID_ARGUMENT;
  if (out_count == 0) return SHDW_OK;
  if (in_count == 0 || !x || !y) return SHDW_E_INVALID_ARGUMENT;
  const int in_h = in_shape[2], in_w = in_shape[3], out_h = out_shape[2], out_w = out_shape[3];
  // align_corners divides by (out - 1): a single output row or column has no
  // defined source coordinate (the reference computes 0 * inf there).
  if (type == 1 && align_corners && (out_h < 2 || out_w < 2)) return SHDW_E_UNSUPPORTED;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const uint32_t n = static_cast<uint32_t>(out_count);
  ResizeArgs p;
  p.in_h = in_h, p.in_w = in_w;
  p.f_out_w = make_fastdiv(out_w), p.f_out_h = make_fastdiv(out_h);
  const bool quad = out_w % 4 == 0 && aligned16(y);
  const uint32_t work = quad ? n / 4 : n;
  const uint32_t grid = grid_for(work);
  const int planes = in_shape[0] * in_shape[1];
  if (type == 1 && align_corners) {
    p.fh = static_cast<float>(in_h - 1) / (out_h - 1);
    p.fw = static_cast<float>(in_w - 1) / (out_w - 1);
    if (launch_resize_band<kResizeBilinearAligned>(planes, in_h, in_w, out_h, out_w, p.fh, p.fw, quad, x, y, st))
      return launch_status();
    if (quad)
      resize_bilinear_kernel<true, 4><<<grid, kBlock, 0, st>>>(x, y, work, p);
    else
      resize_bilinear_kernel<true, 1><<<grid, kBlock, 0, st>>>(x, y, work, p);
  } else {
    p.fh = static_cast<float>(in_h) / out_h;
    p.fw = static_cast<float>(in_w) / out_w;
    if (launch_resize_double(type, planes, in_h, in_w, out_h, out_w, x, y, st)) return launch_status();
    if (type == 0) {
      // Maps of a few hundred positions keep the gathers: their tensors are small
      // enough to come from cache (x2 of [64,256,13,13]: 12 us, staged 17 us).
      if (2 * static_cast<int64_t>(out_h) * out_w > kResizeBandOutputs &&
          launch_resize_band<kResizeNearest>(planes, in_h, in_w, out_h, out_w, p.fh, p.fw, quad, x, y, st))
        return launch_status();
      const uint32_t groups = grid_for((n + 3) / 4);
      if (quad)
        resize_nearest_kernel<false><<<groups, kBlock, 0, st>>>(x, y, n, p);
      else
        resize_nearest_kernel<true><<<groups, kBlock, 0, st>>>(x, y, n, p);
    } else if (launch_resize_band<kResizeBilinear>(planes, in_h, in_w, out_h, out_w, p.fh, p.fw, quad, x, y, st)) {
      return launch_status();
    } else if (quad) {
      resize_bilinear_kernel<false, 4><<<grid, kBlock, 0, st>>>(x, y, work, p);
    } else {
      resize_bilinear_kernel<false, 1><<<grid, kBlock, 0, st>>>(x, y, work, p);
    }
  }
  return launch_status();
}

}  // extern "C"
