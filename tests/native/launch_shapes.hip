// Measurement of the launch shapes the kernels were given, on the device it runs on.
// Prints one table per question; tests/test_gpu_launch_shapes.py runs it and
// checks that the shapes the library uses are still the fast ones.
//
//   stream  : a plain copy, a read-only and a write-only pass over 51 MB and
//             411 MB (rotating through 1.2 GB so that the 256 MB Infinity Cache
//             cannot serve repeats), as workgroups of 64, 256 or 1024 lanes with
//             1, 2 or 4 vectors per lane that cover the tensor, and as a
//             2048-workgroup grid-stride loop with 4 vectors in flight per lane.
//   strided : max over the 512 channels of [32,512,28,28] with the library's
//             column-tile kernel shape, workgroups numbered round-robin over the
//             8 XCDs (as dispatched) or XCD-contiguously, for three tile widths.
//   tile    : a plain copy of [64,256,56,56] and [64,512,38,38] in the access
//             pattern of the channel-tile kernels (Normalize, SSDNormalize, Softmax
//             over 65..512 channels): a workgroup owns 32 neighbouring positions
//             with all their channels, i.e. one 128-byte piece of every row of
//             an image, holds them in registers and writes them back, as 256
//             lanes with room for 16 vectors each (the library's shape) or 1024
//             lanes with 4, with streaming or plain stores, and with the tile also
//             parked in LDS between two barriers as the kernels do; for the
//             256-channel shape also with room for 8 vectors, which lets eight
//             instead of five workgroups share a CU.  The same
//             bytes as a flat copy give the yardstick: what the pattern costs
//             before any arithmetic.
//
//   full sum: one value from 12.8 M floats, as two launches (slices, then a
//             fold) and as one launch whose last workgroup to draw a ticket
//             from a device-scope counter folds the slices: with one counter
//             and with two levels of counters.  No workgroup waits for
//             another; the partials and the tickets are relaxed device-scope
//             atomics, ordered by a data dependency (the ticket's increment
//             is computed from what the exchange that stores the partial
//             returns).
//
// Usage: launch_shapes            (all tables)
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <vector>

#include "../../shadow_amd/csrc/device_common.h"
#include "../../shadow_amd/csrc/reduce_acc.h"

using namespace shdw;

#define CK(x)                                                                      \
  do {                                                                             \
    hipError_t err_ = (x);                                                         \
    if (err_ != hipSuccess) {                                                      \
      printf("error: %s at line %d\n", hipGetErrorString(err_), __LINE__);         \
      return 1;                                                                    \
    }                                                                              \
  } while (0)

enum { kCopy = 0, kRead = 1, kWrite = 2 };

// A workgroup covers T * V consecutive vectors; vector u of lane t is first + u * T.
// STRIDE: the grid is fixed and every workgroup walks the tensor in steps of grid * T * V.
template <int KIND, int T, int V, bool STRIDE>
__global__ __launch_bounds__(T) void stream_kernel(const float* a, float* y, uint32_t n4, float val) {
  const uint32_t step = STRIDE ? gridDim.x * (T * V) : 0xffffffffu;
  for (uint32_t first = blockIdx.x * (T * V) + threadIdx.x; first < n4; first += step) {
    v4f v[V];
    if (KIND != kWrite) {
#pragma unroll
      for (int u = 0; u < V; ++u)
        if (first + u * T < n4) v[u] = load4_stream(a + 4ull * (first + u * T));
    }
    if (KIND == kRead) {
      float s = 0;
#pragma unroll
      for (int u = 0; u < V; ++u)
        if (first + u * T < n4) s += (v[u][0] + v[u][1]) + (v[u][2] + v[u][3]);
      if (s == val) *y = s;
    } else {
#pragma unroll
      for (int u = 0; u < V; ++u)
        if (first + u * T < n4) {
          v4f w;
          if (KIND == kWrite) w = v4f{val, val, val, val}; else w = v[u];
          store4_stream(y + 4ull * (first + u * T), w);
        }
    }
    if (!STRIDE) break;
  }
}

// The shape of the library's reduce_strided_tile_kernel (reduce.hip), with the
// workgroup numbering as a template switch.
template <int OP, int L, bool XCD>
__global__ __launch_bounds__(512) void tile_kernel(const float* x, float* y, uint32_t reduce, uint32_t inner,
                                                    FastDiv f_tiles) {
  constexpr uint32_t kGroups = 512 / L;
  constexpr int kBatch = 8;
  __shared__ Partial lds[512 * 4];
  uint32_t o, tile;
  fd_divmod(XCD ? xcd_contiguous(blockIdx.x, gridDim.x) : blockIdx.x, f_tiles, o, tile);
  const uint32_t pl = threadIdx.x % L, rg = threadIdx.x / L;
  const uint32_t col = (tile * L + pl) * 4;
  Acc<OP> acc[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) acc[j].init();
  if (col < inner) {
    const float* p = x + static_cast<size_t>(o) * reduce * inner + col;
    uint32_t base = rg;
    for (; base + (kBatch - 1) * kGroups < reduce; base += kBatch * kGroups) {
      v4f v[kBatch];
      const bool valid[kBatch] = {true, true, true, true, true, true, true, true};
#pragma unroll
      for (int u = 0; u < kBatch; ++u) v[u] = load4_stream_any(p + static_cast<size_t>(base + u * kGroups) * inner);
      fold_batch<kBatch, false>(acc, v, valid, [&](int u, int) { return base + u * kGroups; });
    }
    for (; base < reduce; base += kGroups) {
      const v4f v = load4_stream_any(p + static_cast<size_t>(base) * inner);
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[j].add(v[j], base);
    }
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) lds[threadIdx.x * 4 + j] = acc[j].pack();
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
    if (c < inner) y[static_cast<size_t>(o) * inner + c] = total.finalize(reduce);
  }
}

// The tile of the channel-tile kernels (softmax.hip), as a copy.  PARK: the tile
// also passes through LDS between two barriers, and the stores depend on it.
typedef float v4f_any __attribute__((ext_vector_type(4), aligned(4)));
template <int T, int PER, bool NT, bool PARK>
__global__ __launch_bounds__(T) void tile_copy_kernel(const float* x, float* y, uint32_t dim, uint32_t inner,
                                                       FastDiv f_tiles) {
  extern __shared__ __align__(16) float tile_lds[];
  constexpr uint32_t TS = 32, LPR = TS / 4, STEP = T / LPR;
  uint32_t n, tile;
  fd_divmod(xcd_contiguous(blockIdx.x, gridDim.x), f_tiles, n, tile);
  const uint32_t p0 = tile * TS;
  const uint32_t width = min(TS, inner - p0);
  const uint64_t base = static_cast<uint64_t>(n) * dim * inner + p0;
  const uint32_t j = (threadIdx.x & (LPR - 1)) * 4, c0 = threadIdx.x / LPR;
  const bool valid = j + 4 <= width;  // inner is a multiple of 4 here
  v4f r[PER];
  if (valid) {
#pragma unroll
    for (int u = 0; u < PER; ++u) {
      const uint32_t c = c0 + u * STEP;
      if (c < dim)
        r[u] = __builtin_nontemporal_load(reinterpret_cast<const v4f_any*>(x + base + static_cast<uint64_t>(c) * inner + j));
    }
  }
  float m = 1.f;
  if (PARK) {
    if (valid) {
#pragma unroll
      for (int u = 0; u < PER; ++u) {
        const uint32_t c = c0 + u * STEP;
        if (c < dim) *reinterpret_cast<v4f*>(tile_lds + c * TS + j) = r[u];
      }
    }
    __syncthreads();
    if (threadIdx.x < width) {
      float a = 0.f;
      for (int c = 0; c < 16; ++c) a += tile_lds[c * TS + threadIdx.x];
      tile_lds[threadIdx.x] = a;
    }
    __syncthreads();
    m = tile_lds[j] == 12345.f ? 2.f : 1.f;
  }
  if (!valid) return;
#pragma unroll
  for (int u = 0; u < PER; ++u) {
    const uint32_t c = c0 + u * STEP;
    if (c >= dim) continue;
    const v4f q = r[u] * m;
    float* dst = y + base + static_cast<uint64_t>(c) * inner + j;
    if (NT)
      __builtin_nontemporal_store(q, reinterpret_cast<v4f_any*>(dst));
    else
      *reinterpret_cast<v4f_any*>(dst) = q;
  }
}

// ---- full sum ----
template <int T>
__device__ double block_sum(double v, double* lds) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m, 64);
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  __syncthreads();  // lds may still be read from an earlier call
  if (lane == 0) lds[w] = v;
  __syncthreads();
  double t = 0;
  for (int k = 0; k < T / 64; ++k) t += lds[k];
  return t;
}

// Slice blockIdx.x of x (per = vectors per lane) summed in fp64.
template <int T>
__device__ double slice_sum(const float* x, uint32_t n4, uint32_t per, double* lds) {
  double acc = 0;
  const uint32_t first = blockIdx.x * (T * per) + threadIdx.x;
  for (uint32_t u0 = 0; u0 < per; u0 += 4) {
    v4f v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const uint32_t i = first + (u0 + u) * T;
      v[u] = (u0 + u < per && i < n4) ? load4_stream(x + 4ull * i) : v4f{0.f, 0.f, 0.f, 0.f};
    }
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc += static_cast<double>(v[u][j]);
  }
  return block_sum<T>(acc, lds);
}

template <int T>
__global__ __launch_bounds__(T) void sum_slices_kernel(const float* x, uint32_t n4, uint32_t per, double* part) {
  __shared__ double lds[T / 64];
  const double s = slice_sum<T>(x, n4, per, lds);
  if (threadIdx.x == 0) part[blockIdx.x] = s;
}

__global__ __launch_bounds__(1024) void sum_fold_kernel(const double* part, uint32_t count, float* out) {
  __shared__ double lds[16];
  double acc = 0;
  for (uint32_t i = threadIdx.x; i < count; i += 1024) acc += part[i];
  const double s = block_sum<1024>(acc, lds);
  if (threadIdx.x == 0) *out = static_cast<float>(s);
}

__device__ unsigned long long dbits(double d) { return __builtin_bit_cast(unsigned long long, d); }
__device__ double bitsd(unsigned long long u) { return __builtin_bit_cast(double, u); }

// One launch.  GROUP = 0: one counter; otherwise workgroups draw from the counter of their group of
// GROUP and the last of a group from the top counter (counters 256 bytes apart).  The workgroup that
// draws the last ticket folds all partials and puts the counters back to zero.
template <int T, int GROUP>
__global__ __launch_bounds__(T) void sum_ticket_kernel(const float* x, uint32_t n4, uint32_t per,
                                                        unsigned long long* part, unsigned* counters, float* out) {
  __shared__ double lds[T / 64];
  __shared__ bool last;
  const double s = slice_sum<T>(x, n4, per, lds);
  if (threadIdx.x == 0) {
    // the exchange has been performed when its result is here, and the ticket depends on that result
    const unsigned long long old =
        __hip_atomic_exchange(part + blockIdx.x, dbits(s), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const unsigned one = 1u + static_cast<unsigned>(old & 0);
    bool mine;
    if (GROUP == 0) {
      mine = __hip_atomic_fetch_add(counters, one, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == gridDim.x - 1;
    } else {
      const unsigned g = blockIdx.x / GROUP, groups = (gridDim.x + GROUP - 1) / GROUP;
      const unsigned members = min(static_cast<unsigned>(GROUP), gridDim.x - g * GROUP);
      const unsigned t = __hip_atomic_fetch_add(counters + 64 * (1 + g), one, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      mine = false;
      if (t == members - 1) {
        const unsigned up = 1u + (t & 0);
        mine = __hip_atomic_fetch_add(counters, up, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == groups - 1;
      }
    }
    last = mine;
  }
  __syncthreads();
  if (!last) return;
  double acc = 0;
  for (uint32_t i = threadIdx.x; i < gridDim.x; i += T)
    acc += bitsd(__hip_atomic_load(part + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
  const double total = block_sum<T>(acc, lds);
  if (threadIdx.x == 0) *out = static_cast<float>(total);
  const unsigned groups = GROUP ? (gridDim.x + GROUP - 1) / GROUP : 0;
  for (unsigned c = threadIdx.x; c <= groups; c += T)
    __hip_atomic_store(counters + 64 * c, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

static hipEvent_t e0, e1;

// Average time of one launch in us: best of three batches of `reps` back-to-back launches.
template <class F>
static int time_us(F launch, int reps, float* us) {
  for (int i = 0; i < 5; ++i) launch(i);
  float best = 1e30f;
  for (int rep = 0; rep < 3; ++rep) {
    CK(hipEventRecord(e0));
    for (int i = 0; i < reps; ++i) launch(i);
    CK(hipEventRecord(e1));
    CK(hipEventSynchronize(e1));
    float ms;
    CK(hipEventElapsedTime(&ms, e0, e1));
    best = std::min(best, ms);
  }
  CK(hipGetLastError());
  *us = best / reps * 1e3f;
  return 0;
}

// A chain of dependent fp32 additions, as the in-order sums of Pooling, Softmax and Normalize are one per
// row or column: CHAINS independent chains per wave, all lanes alike.  The asm statement keeps the
// compiler from reassociating or hoisting the chain.  Workgroups of four waves: one wave to each SIMD of a CU
// (single-wave workgroups may share a SIMD while others idle).
template <int CHAINS>
__global__ __launch_bounds__(256) void add_chain_kernel(const float* in, float* out, int n) {
  float s[CHAINS];
#pragma unroll
  for (int c = 0; c < CHAINS; ++c) s[c] = in[threadIdx.x + c];
  const float a = in[256 + threadIdx.x], b = in[512 + threadIdx.x];
  for (int i = 0; i < n; i += 8) {
#pragma unroll
    for (int k = 0; k < 4; ++k) {
#pragma unroll
      for (int c = 0; c < CHAINS; ++c) s[c] += a;
#pragma unroll
      for (int c = 0; c < CHAINS; ++c) s[c] += b;
    }
#pragma unroll
    for (int c = 0; c < CHAINS; ++c) asm volatile("" : "+v"(s[c]));
  }
  float t = 0.f;
#pragma unroll
  for (int c = 0; c < CHAINS; ++c) t += s[c];
  out[blockIdx.x * 256 + threadIdx.x] = t;
}

// Both renumberings of the workgroups must visit every work item exactly once, whatever the grid.
static bool numberings_are_bijections() {
  std::vector<uint8_t> seen;
  for (uint32_t grid = 1; grid <= 3000; grid += (grid < 300 ? 1 : 7)) {
    for (int k = -1; k <= 5; ++k) {  // -1: xcd_contiguous
      seen.assign(grid, 0);
      for (uint32_t b = 0; b < grid; ++b) {
        const uint32_t w = k < 0 ? xcd_contiguous(b, grid) : xcd_runs(b, grid, static_cast<uint32_t>(k));
        if (w >= grid || seen[w]++) return false;
      }
    }
  }
  return true;
}

int main() {
  printf("numberings %s\n", numberings_are_bijections() ? "same" : "DIFFERENT");
  const size_t kPool = 6ull * 205520896;
  float *rp, *wp;
  CK(hipMalloc(&rp, kPool));
  CK(hipMalloc(&wp, kPool));
  CK(hipMemset(rp, 0x3c, kPool));
  CK(hipEventCreate(&e0));
  CK(hipEventCreate(&e1));

  printf("# stream: us per launch; total bytes moved = the size given (copy: half read, half written)\n");
  const size_t sizes[] = {51380224, 411041792};
  const char* kinds[] = {"copy", "read", "write"};
  for (size_t total : sizes) {
    for (int kind = 0; kind < 3; ++kind) {
      const size_t side = kind == kCopy ? total / 2 : total;
      const uint32_t n4 = static_cast<uint32_t>(side / 16);
      const int m = static_cast<int>(std::max<size_t>(1, std::min<size_t>(64, kPool / side)));
      printf("stream %-5s %3zu MB:", kinds[kind], total / 1000000);
#define RUN(KIND, T, V, STRIDE)                                                                        \
  if (kind == KIND) {                                                                                  \
    const uint32_t grid = STRIDE ? 2048u : (n4 + T * V - 1) / (T * V);                                 \
    float us;                                                                                          \
    if (time_us([&](int i) {                                                                           \
          const size_t off = (i % m) * (side / 4);                                                     \
          stream_kernel<KIND, T, V, STRIDE><<<grid, T>>>(rp + off, wp + off, n4, 1e30f);               \
        }, 40, &us)) return 1;                                                                         \
    printf("  %s%dx%d %.2f", STRIDE ? "stride" : "T", T, V, us);                                       \
    fflush(stdout);                                                                                    \
  }
#define ALLV(KIND, T) RUN(KIND, T, 1, false) RUN(KIND, T, 2, false) RUN(KIND, T, 4, false)
#define ALL(KIND) ALLV(KIND, 64) ALLV(KIND, 256) ALLV(KIND, 1024) RUN(KIND, 256, 4, true)
      ALL(kCopy) ALL(kRead) ALL(kWrite)
      printf("\n");
    }
  }

  // strided reduce: [32][512][784], max over the middle extent
  {
    const uint32_t outer = 32, reduce = 512, inner = 784;
    const size_t n = static_cast<size_t>(outer) * reduce * inner;
    const int sets = 6;
    std::vector<float> h(n);
    for (size_t i = 0; i < n; ++i) h[i] = static_cast<float>((i * 2654435761u) >> 8 & 0xffff) / 65536.f - 0.5f;
    for (int k = 0; k < sets; ++k) CK(hipMemcpy(rp + k * n, h.data(), 4 * n, hipMemcpyHostToDevice));
    printf("# strided: max over 512 channels of [32,512,28,28], us per launch; L = lanes per row piece (4 L columns per tile)\n");
    std::vector<float> ref, got(outer * inner);
#define TILE(L, XCD)                                                                                   \
  {                                                                                                    \
    const uint32_t tiles = (inner / 4 + L - 1) / L;                                                    \
    const FastDiv f = make_fastdiv(tiles);                                                             \
    float us;                                                                                          \
    if (time_us([&](int i) {                                                                           \
          tile_kernel<SHDW_REDUCE_MAX, L, XCD><<<tiles * outer, 512>>>(rp + (i % sets) * n, wp + (i % sets) * n, reduce, inner, f); \
        }, 40, &us)) return 1;                                                                         \
    CK(hipMemcpy(got.data(), wp, 4 * outer * inner, hipMemcpyDeviceToHost));                           \
    if (ref.empty()) ref = got;                                                                        \
    printf("strided L%-2d %-14s %.2f %s\n", L, XCD ? "xcd-contiguous" : "round-robin", us,             \
           memcmp(ref.data(), got.data(), 4 * outer * inner) == 0 ? "same" : "DIFFERENT");             \
  }
    TILE(32, true) TILE(32, false) TILE(16, true) TILE(16, false) TILE(8, true) TILE(8, false)
  }

  // channel tiles as a copy: [64][256][3136] (rows start on 64-byte boundaries) and [64][512][1444] (they do not)
  {
    printf("# tile: copy of [outer,dim,inner] in the channel-tile pattern, us per launch; flat = the same bytes as a flat copy\n");
    const uint32_t shapes[2][3] = {{64, 256, 3136}, {64, 512, 1444}};
    for (const auto& sh : shapes) {
      const uint32_t outer = sh[0], dim = sh[1], inner = sh[2];
      const size_t n = static_cast<size_t>(outer) * dim * inner;
      const int sets = static_cast<int>(kPool / (4 * n));
      std::vector<float> h(n), got(n);
      for (size_t i = 0; i < n; ++i) h[i] = static_cast<float>((i * 2654435761u) >> 8 & 0xffff) / 65536.f - 0.5f;
      for (int k = 0; k < sets; ++k) CK(hipMemcpy(rp + k * n, h.data(), 4 * n, hipMemcpyHostToDevice));
      const uint32_t n4 = static_cast<uint32_t>(n / 4);
      float us;
      if (time_us([&](int i) { stream_kernel<kCopy, 64, 1, false><<<(n4 + 63) / 64, 64>>>(rp + (i % sets) * n, wp + (i % sets) * n, n4, 0.f); }, 20, &us)) return 1;
      printf("tile [%u,%u,%u] flat %.2f\n", outer, dim, inner, us);
      const uint32_t tiles = (inner + 31) / 32;
      const FastDiv f = make_fastdiv(tiles);
      const size_t lds = static_cast<size_t>(dim) * 32 * sizeof(float);
#define TILECOPY(T, PER, NT, PARK)                                                                     \
  {                                                                                                    \
    CK(hipMemset(wp, 0, 4 * n));                                                                       \
    if (time_us([&](int i) {                                                                           \
          tile_copy_kernel<T, PER, NT, PARK><<<tiles * outer, T, PARK ? lds : 0>>>(rp + (i % sets) * n, wp + (i % sets) * n, dim, inner, f); \
        }, 20, &us)) return 1;                                                                         \
    CK(hipMemcpy(got.data(), wp, 4 * n, hipMemcpyDeviceToHost));                                       \
    printf("tile [%u,%u,%u] T%dx%d %-9s %-6s %.2f %s\n", outer, dim, inner, T, PER, NT ? "streaming" : "plain", \
           PARK ? "parked" : "direct", us, memcmp(h.data(), got.data(), 4 * n) == 0 ? "same" : "DIFFERENT"); \
  }
      TILECOPY(256, 16, true, false) TILECOPY(256, 16, false, false) TILECOPY(256, 16, true, true) TILECOPY(256, 16, false, true)
      TILECOPY(1024, 4, true, false) TILECOPY(1024, 4, false, true)
      // half the registers per lane: eight instead of five workgroups fit a CU, and the copy gets slower
      if (dim <= 256) TILECOPY(256, 8, true, false)
    }
  }
  // ordered sums: what one dependent fp32 addition costs a chain, by the waves that share a SIMD
  {
    printf("# add chain: ns per addition of one chain / of the SIMD, 2^18 dependent fp32 additions per chain; "
           "waves = per SIMD (workgroups of four waves, one to a SIMD, 256 workgroups per wave wanted), chains = independent "
           "chains per wave\n");
    const int n = 1 << 18;
#define CHAIN(WAVES, CHAINS)                                                                           \
  {                                                                                                    \
    float us;                                                                                          \
    if (time_us([&](int) { add_chain_kernel<CHAINS><<<256 * WAVES, 256>>>(rp, wp, n); }, 3, &us)) return 1; \
    printf("add chain waves %d chains %d: %.2f %.2f\n", WAVES, CHAINS, us * 1e3f / n, us * 1e3f / n / (WAVES * CHAINS)); \
  }
    CHAIN(1, 1) CHAIN(1, 2) CHAIN(1, 4) CHAIN(2, 1) CHAIN(4, 1) CHAIN(8, 1) CHAIN(8, 2)
  }
  // full sum of [32,512,28,28]
  {
    const size_t n = 12845056;
    const uint32_t n4 = static_cast<uint32_t>(n / 4);
    const int sets = 6;
    std::vector<float> h(n);
    double exact = 0;
    for (size_t i = 0; i < n; ++i) {
      h[i] = static_cast<float>((i * 2654435761u) >> 8 & 0xffff) / 65536.f - 0.25f;
      exact += h[i];
    }
    for (int k = 0; k < sets; ++k) CK(hipMemcpy(rp + k * n, h.data(), 4 * n, hipMemcpyHostToDevice));
    double* part = reinterpret_cast<double*>(wp);
    unsigned* counters = reinterpret_cast<unsigned*>(wp + (1 << 20));
    float* out = wp + (2 << 20);
    CK(hipMemset(counters, 0, 64 * 4 * 128));
    printf("# full sum: one value from 12.8 M floats (51 MB), us per call; two launches = slices then a fold; ticket = one "
           "launch, the last workgroup to draw from a device-scope counter folds\n");
    const float want = static_cast<float>(exact);
    float got, us;
#define CHECK(label)                                                                                   \
  CK(hipMemcpy(&got, out, 4, hipMemcpyDeviceToHost));                                                  \
  printf("full sum %-44s %.2f %s\n", label, us, std::fabs(got - want) <= 1e-6f * std::fabs(want) ? "same" : "DIFFERENT");                   \
  fflush(stdout);
    if (time_us([&](int i) {
          sum_slices_kernel<256><<<3136, 256>>>(rp + (i % sets) * n, n4, 4, part);
          sum_fold_kernel<<<1, 1024>>>(part, 3136, out);
        }, 40, &us)) return 1;
    CHECK("two launches, 3136 x 256 lanes")
    if (time_us([&](int i) {
          sum_slices_kernel<1024><<<392, 1024>>>(rp + (i % sets) * n, n4, 8, part);
          sum_fold_kernel<<<1, 1024>>>(part, 392, out);
        }, 40, &us)) return 1;
    CHECK("two launches, 392 x 1024 lanes")
    if (time_us([&](int i) {
          sum_ticket_kernel<256, 0><<<3136, 256>>>(rp + (i % sets) * n, n4, 4, reinterpret_cast<unsigned long long*>(part), counters, out);
        }, 40, &us)) return 1;
    CHECK("ticket, 3136 x 256 lanes, one counter")
    if (time_us([&](int i) {
          sum_ticket_kernel<1024, 0><<<392, 1024>>>(rp + (i % sets) * n, n4, 8, reinterpret_cast<unsigned long long*>(part), counters, out);
        }, 40, &us)) return 1;
    CHECK("ticket, 392 x 1024 lanes, one counter")
    if (time_us([&](int i) {
          sum_ticket_kernel<256, 56><<<3136, 256>>>(rp + (i % sets) * n, n4, 4, reinterpret_cast<unsigned long long*>(part), counters, out);
        }, 40, &us)) return 1;
    CHECK("ticket, 3136 x 256 lanes, counters of 56 + 1")
    if (time_us([&](int i) {
          sum_slices_kernel<256><<<3136, 256>>>(rp + (i % sets) * n, n4, 4, part);
        }, 40, &us)) return 1;
    printf("full sum %-44s %.2f\n", "slices alone (first of the two launches)", us);
  }
  return 0;
}
