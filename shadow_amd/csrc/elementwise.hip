// Contiguous elementwise kernels: Blas::Set, the 15 unary ops, the 7 binary ops
// in tensor and scalar form, Scal/Copy/Axpy, Activate, and the K-ary Eltwise.
//
// One kernel family: every lane moves exactly one 128-bit vector per operand and
// the grid covers the tensor (no grid-stride loop).  Measured on MI355X with
// operands rotating through more memory than the 256 MB Infinity Cache, one
// vector per lane with tens of thousands of short workgroups streams at
// ~6.5 TB/s, against ~5.9 TB/s for a 2048-workgroup grid-stride loop with four
// vectors in flight per lane: the hardware dispatcher keeps more independent
// wavefronts (and so more outstanding HBM requests) in flight than unrolling
// does.  All of these are HBM bound (8 or 12 bytes per element).
#include <hip/hip_runtime.h>

#include "../../include/shadow_hip.h"
#include "device_common.h"
#include "functors.h"
#include "launch.h"

#pragma clang fp contract(off)

namespace shdw {

// NIN = 0: y = f(alpha, alpha)     (fill)
// NIN = 1: y = f(a, alpha)
// NIN = 2: y = f(a, b)
// A lane owns V vectors (V = 1 except where the functor asks for more), kStream
// vectors apart so that every load instruction of the wave is contiguous; the
// lane whose vector index is n4 (one past the last whole vector) owns the
// n % 4 trailing elements.
// The workgroup is a single wave64 where something is read (T = kStream); a fill
// (NIN = 0) takes 256 lanes: a wave that only stores 1 KB is gone so quickly that
// single-wave workgroups are bounded by the rate at which workgroups can be
// started (4.2 per ns: 4.3 TB/s of stores, measured 12.1 us for 51 MB against
// 8.4 us with 256 lanes; a copy moves 2 KB per wave and is not bounded by it).
template <int NIN, class F, int V, int T>
__global__ __launch_bounds__(T) void ew_vec_kernel(F f, const float* a, const float* b,
                                                    float* y, uint32_t n4, uint32_t n,
                                                    float alpha) {
  const uint32_t first = blockIdx.x * (T * V) + threadIdx.x;
  // The tanh table's piece is requested first: it comes from the caches and is in
  // LDS long before the streamed vector arrives.
  constexpr int kPieces = libm::kTanhSteps * sizeof(libm::TanhStep) / sizeof(v4f);
  static_assert(!uses_tanh_table<F>::value || kPieces <= T, "one piece per lane");
  v4f piece;
  if (uses_tanh_table<F>::value && (kPieces == T || threadIdx.x < kPieces))
    piece = reinterpret_cast<const v4f*>(libm::kTanhStepTab)[threadIdx.x];
  v4f va[V], vb[V];
#pragma unroll
  for (int u = 0; u < V; ++u) {  // issue the streaming loads before anything else
    const uint32_t i = first + u * T;
    if (i < n4) {
      if (NIN >= 1) va[u] = load4_stream_any(a + 4ull * i);
      if (NIN >= 2) vb[u] = load4_stream_any(b + 4ull * i);
    }
  }
  const uint64_t* tab = nullptr;
  if (uses_exp_table<F>::value) {
    __shared__ uint64_t lds_tab[32];
    if (threadIdx.x < 32) lds_tab[threadIdx.x] = libm::kExp2fTab[threadIdx.x];
    __syncthreads();
    tab = lds_tab;
  }
  if (uses_tanh_table<F>::value) {
    __shared__ __align__(32) v4f lds_steps[kPieces];
    if (kPieces == T || threadIdx.x < kPieces) lds_steps[threadIdx.x] = piece;
    __syncthreads();
    tab = reinterpret_cast<const uint64_t*>(lds_steps);
  }
#pragma unroll
  for (int u = 0; u < V; ++u) {
    const uint32_t i = first + u * T;
    if (i < n4) {
      v4f r;
      if constexpr (NIN == 1 && has_four<F>::value) {
        r = f.four(va[u], tab);
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float x = NIN >= 1 ? va[u][j] : alpha;
          const float w = NIN >= 2 ? vb[u][j] : alpha;
          r[j] = f(x, w, tab);
        }
      }
      store4_stream_any(y + 4ull * i, r);
    } else if (i == n4) {
      for (uint32_t t = 4 * n4; t < n; ++t) {
        const float x = NIN >= 1 ? a[t] : alpha;
        const float w = NIN >= 2 ? b[t] : alpha;
        y[t] = f(x, w, tab);
      }
    }
  }
}

template <int NIN, class F>
static int launch_ew(F f, int n, const float* a, const float* b, float alpha, float* y,
                     void* stream) {
  if (n < 0 || !y || (NIN >= 1 && !a) || (NIN >= 2 && !b)) return SHDW_E_INVALID_ARGUMENT;
  if (n == 0) return SHDW_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  // Any float pointers: the 128-bit accesses need dword alignment only.
  const uint32_t n4 = static_cast<uint32_t>(n) / 4;
  constexpr int V = vectors_per_lane<F>::value;
  constexpr int T = NIN == 0 ? kBlock : kStream;
  const uint32_t slots = (n4 + V) / V;  // n4 + 1 vector slots, V per lane
  ew_vec_kernel<NIN, F, V, T><<<(slots + T - 1) / T, T, 0, s>>>(f, a, b, y, n4, static_cast<uint32_t>(n), alpha);
  return launch_status();
}

// Adapters onto the (x, w) functor shape used by the kernels.
template <class U>
struct Unary2 {
  U u;
  static constexpr bool kExpTable = uses_exp_table<U>::value;
  SHDW_DEVICE float operator()(float a, float, const uint64_t* tab) const { return u(a, tab); }
};
struct Fill {
  SHDW_DEVICE float operator()(float v, float, const uint64_t*) const { return v; }
};
struct ScalOp {  // x *= alpha
  SHDW_DEVICE float operator()(float x, float alpha, const uint64_t*) const { return x * alpha; }
};
struct AxpyOp {  // y += alpha * x, multiply then add
  float alpha;
  SHDW_DEVICE float operator()(float x, float y, const uint64_t*) const {
    const float t = alpha * x;
    return y + t;
  }
};

// Read-only pass: every lane requests one vector and stores nothing unless its
// four values add up to `sentinel`.  It exists for the measurement harness (the
// read ceiling of a tensor size).  1024-lane workgroups: of the shapes measured
// (64, 256, 1024 lanes x 1, 2, 4, 8 vectors per lane) the fastest or level with
// it at every size from 25 to 411 MB (411 MB: 55.8 us, 256 lanes 59.5 us, single
// waves 86.5 us).
constexpr int kReadProbeThreads = 1024;
__global__ __launch_bounds__(kReadProbeThreads) void read_probe_kernel(const float* a, float* sink, uint32_t n4,
                                                                        float sentinel) {
  const uint32_t i = blockIdx.x * kReadProbeThreads + threadIdx.x;
  if (i < n4) {
    const v4f v = load4_stream_any(a + 4ull * i);
    if ((v[0] + v[1]) + (v[2] + v[3]) == sentinel) *sink = sentinel;
  }
}

// ---------------------------------------------------------------------------
// K-ary Eltwise in one pass.
// ---------------------------------------------------------------------------
constexpr int kEltwiseMaxK = 8;

struct EltwiseArgs {
  const float* x[kEltwiseMaxK];
  float coeff[kEltwiseMaxK];
  int k;
  // bit j set: input j aliases the output and Shadow's pass-by-pass evaluation
  // would have read something else than its original contents (see header).
  unsigned alias_mask;
  int has_seed;  // continuation call: the accumulator starts from y
};

template <int OP, int KMAX>
SHDW_DEVICE float eltwise_fold(const EltwiseArgs& p, const float (&v)[KMAX], float seed) {
  // SUM starts from +0 (or the stored accumulator); the others start from the
  // first input unless continuing.
  float acc = (OP == SHDW_ELTWISE_SUM) ? (p.has_seed ? seed : 0.0f) : (p.has_seed ? seed : v[0]);
  const int first = (OP == SHDW_ELTWISE_SUM || p.has_seed) ? 0 : 1;
#pragma unroll
  for (int j = 0; j < KMAX; ++j) {
    if (j >= first && j < p.k) {
      float x = v[j];
      const bool aliased = (p.alias_mask >> j) & 1u;
      if (OP == SHDW_ELTWISE_SUM) {
        if (aliased) x = acc;  // y += c*y: the pass reads its own running sum
        const float t = p.coeff[j] * x;
        acc = acc + t;
      } else {
        if (aliased) x = acc;
        if (OP == SHDW_ELTWISE_PROD) acc = acc * x;
        if (OP == SHDW_ELTWISE_MAX) acc = sel_max(acc, x);
        if (OP == SHDW_ELTWISE_MIN) acc = sel_min(acc, x);
      }
    }
  }
  return acc;
}

// KMAX is the compile-time bound on p.k (2, 3, 4 or 8) so that the per-input
// registers are never indexed dynamically.
// RELU: Activate(relu) on the folded value, the Eltwise -> Activate pair in one pass.
template <int OP, int KMAX, bool RELU = false>
__global__ __launch_bounds__(kStream) void eltwise_kernel(EltwiseArgs p, float* y, uint32_t n) {
  const uint32_t i = blockIdx.x * kStream + threadIdx.x;
  const uint32_t n4 = n / 4;
  if (i < n4) {
    v4f v[KMAX];
    v4f seed = {0, 0, 0, 0};
#pragma unroll
    for (int j = 0; j < KMAX; ++j)
      if (j < p.k) v[j] = load4_stream_any(p.x[j] + 4ull * i);
    if (p.has_seed) seed = load4_stream_any(y + 4ull * i);
    v4f r;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      float col[KMAX];
#pragma unroll
      for (int j = 0; j < KMAX; ++j) col[j] = (j < p.k) ? v[j][c] : 0.0f;
      r[c] = eltwise_fold<OP, KMAX>(p, col, seed[c]);
      if (RELU) r[c] = r[c] > 0 ? r[c] : 0;
    }
    store4_stream_any(y + 4ull * i, r);
  } else if (i == n4) {
    for (uint32_t t = 4 * n4; t < n; ++t) {
      float col[KMAX];
#pragma unroll
      for (int j = 0; j < KMAX; ++j) col[j] = (j < p.k) ? p.x[j][t] : 0.0f;
      float r = eltwise_fold<OP, KMAX>(p, col, p.has_seed ? y[t] : 0.0f);
      if (RELU) r = r > 0 ? r : 0;
      y[t] = r;
    }
  }
}

template <int OP, int KMAX>
static int launch_eltwise_k(const EltwiseArgs& p, int n, float* y, bool relu, hipStream_t s) {
  const uint32_t grid = stream_grid(static_cast<uint32_t>(n) / 4 + 1);
  if (relu) eltwise_kernel<OP, KMAX, true><<<grid, kStream, 0, s>>>(p, y, static_cast<uint32_t>(n));
  else eltwise_kernel<OP, KMAX><<<grid, kStream, 0, s>>>(p, y, static_cast<uint32_t>(n));
  return launch_status();
}

template <int OP>
static int launch_eltwise_chunk(const EltwiseArgs& p, int n, float* y, bool relu, hipStream_t s) {
  if (p.k <= 2) return launch_eltwise_k<OP, 2>(p, n, y, relu, s);
  if (p.k == 3) return launch_eltwise_k<OP, 3>(p, n, y, relu, s);
  if (p.k == 4) return launch_eltwise_k<OP, 4>(p, n, y, relu, s);
  return launch_eltwise_k<OP, kEltwiseMaxK>(p, n, y, relu, s);
}

}  // namespace shdw

using namespace shdw;

extern "C" {

int shdw_hip_set(int n, float val, float* y, void* stream) {
  return launch_ew<0>(Fill(), n, nullptr, nullptr, val, y, stream);
}

int shdw_hip_unary(int operation, int n, const float* a, float* y, void* stream) {
#define SHDW_CASE(code, functor) \
  case code:                     \
    return launch_ew<1>(Unary2<functor>(), n, a, nullptr, 0.f, y, stream)
  switch (operation) {
    SHDW_CASE(SHDW_UNARY_ABS, UAbs);
    SHDW_CASE(SHDW_UNARY_SQUARE, USquare);
    SHDW_CASE(SHDW_UNARY_SQRT, USqrt);
    SHDW_CASE(SHDW_UNARY_LOG, ULog);
    SHDW_CASE(SHDW_UNARY_EXP, UExp);
    SHDW_CASE(SHDW_UNARY_SIN, USin);
    SHDW_CASE(SHDW_UNARY_COS, UCos);
    SHDW_CASE(SHDW_UNARY_TAN, UTan);
    SHDW_CASE(SHDW_UNARY_ASIN, UAsin);
    SHDW_CASE(SHDW_UNARY_ACOS, UAcos);
    SHDW_CASE(SHDW_UNARY_ATAN, UAtan);
    SHDW_CASE(SHDW_UNARY_FLOOR, UFloor);
    SHDW_CASE(SHDW_UNARY_CEIL, UCeil);
    SHDW_CASE(SHDW_UNARY_NEG, UNeg);
    SHDW_CASE(SHDW_UNARY_RECIPROCAL, UReciprocal);
    default:
      return SHDW_E_INVALID_ARGUMENT;
  }
#undef SHDW_CASE
}

int shdw_hip_binary(int operation, int n, const float* a, const float* b, float* y,
                    void* stream) {
#define SHDW_CASE(code, functor) \
  case code:                     \
    return launch_ew<2>(functor(), n, a, b, 0.f, y, stream)
  switch (operation) {
    SHDW_CASE(SHDW_BINARY_ADD, BAdd);
    SHDW_CASE(SHDW_BINARY_SUB, BSub);
    SHDW_CASE(SHDW_BINARY_MUL, BMul);
    SHDW_CASE(SHDW_BINARY_DIV, BDiv);
    SHDW_CASE(SHDW_BINARY_POW, BPow);
    SHDW_CASE(SHDW_BINARY_MAX, BMax);
    SHDW_CASE(SHDW_BINARY_MIN, BMin);
    default:
      return SHDW_E_INVALID_ARGUMENT;
  }
#undef SHDW_CASE
}

int shdw_hip_binary_scalar(int operation, int n, const float* a, float alpha, float* y,
                           void* stream) {
#define SHDW_CASE(code, functor) \
  case code:                     \
    return launch_ew<1>(functor(), n, a, nullptr, alpha, y, stream)
  switch (operation) {
    SHDW_CASE(SHDW_BINARY_ADD, BAdd);
    SHDW_CASE(SHDW_BINARY_SUB, BSub);
    SHDW_CASE(SHDW_BINARY_MUL, BMul);
    SHDW_CASE(SHDW_BINARY_DIV, BDiv);
    SHDW_CASE(SHDW_BINARY_POW, BPow);
    SHDW_CASE(SHDW_BINARY_MAX, BMax);
    SHDW_CASE(SHDW_BINARY_MIN, BMin);
    default:
      return SHDW_E_INVALID_ARGUMENT;
  }
#undef SHDW_CASE
}

int shdw_hip_scal(int n, float alpha, float* x, void* stream) {
  return launch_ew<1>(ScalOp(), n, x, nullptr, alpha, x, stream);
}

int shdw_hip_copy(int n, const float* x, float* y, void* stream) {
  return launch_ew<1>(Unary2<UCopy>(), n, x, nullptr, 0.f, y, stream);
}

int shdw_hip_probe_read(int n, const float* x, float sentinel, float* sink, void* stream) {
  if (n < 0 || !x || !sink) return SHDW_E_INVALID_ARGUMENT;
  const uint32_t n4 = static_cast<uint32_t>(n) / 4;
  if (n4 == 0) return SHDW_OK;
  const uint32_t grid = (n4 + kReadProbeThreads - 1) / kReadProbeThreads;
  read_probe_kernel<<<grid, kReadProbeThreads, 0, static_cast<hipStream_t>(stream)>>>(x, sink, n4, sentinel);
  return launch_status();
}

int shdw_hip_axpy(int n, float alpha, const float* x, float* y, void* stream) {
  AxpyOp op;
  op.alpha = alpha;
  return launch_ew<2>(op, n, x, y, 0.f, y, stream);
}

int shdw_hip_activate(int type, float slope, int n, const float* x, float* y, void* stream) {
#define SHDW_CASE(code, functor) \
  case code:                     \
    return launch_ew<1>(functor(), n, x, nullptr, slope, y, stream)
  switch (type) {
    SHDW_CASE(SHDW_ACT_RELU, ARelu);
    SHDW_CASE(SHDW_ACT_LEAKY, ALeaky);
    SHDW_CASE(SHDW_ACT_SIGMOID, ASigmoid);
    SHDW_CASE(SHDW_ACT_SOFTPLUS, ASoftPlus);
    SHDW_CASE(SHDW_ACT_TANH, ATanh);
    SHDW_CASE(SHDW_ACT_RELU6, ARelu6);
    SHDW_CASE(SHDW_ACT_HARDSWISH, AHardSwish);
    SHDW_CASE(SHDW_ACT_GELU, AGelu);
    default:
      return SHDW_E_INVALID_ARGUMENT;
  }
#undef SHDW_CASE
}

static int run_eltwise(int operation, int k, const float* const* xs, const float* coeff, int n, float* y, bool relu,
                       void* stream) {
  if (k < 2 || !xs || !y || n < 0) return SHDW_E_INVALID_ARGUMENT;
  if (operation < SHDW_ELTWISE_PROD || operation > SHDW_ELTWISE_MIN) return SHDW_E_INVALID_ARGUMENT;
  for (int j = 0; j < k; ++j)
    if (!xs[j]) return SHDW_E_INVALID_ARGUMENT;
  if (n == 0) return SHDW_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  // Inputs are consumed kEltwiseMaxK at a time; later chunks continue from the
  // accumulator already stored in y, which is exactly Shadow's chaining.
  int done = 0;
  while (done < k) {
    EltwiseArgs p;
    p.k = (k - done > kEltwiseMaxK) ? kEltwiseMaxK : (k - done);
    p.alias_mask = 0;
    p.has_seed = done > 0;
    for (int j = 0; j < kEltwiseMaxK; ++j) {
      p.x[j] = nullptr;
      p.coeff[j] = 1.f;
    }
    for (int j = 0; j < p.k; ++j) {
      const int g = done + j;
      p.x[j] = xs[g];
      p.coeff[j] = coeff ? coeff[g] : 1.f;
      if (xs[g] == y) {
        if (operation == SHDW_ELTWISE_SUM) {
          p.alias_mask |= 1u << j;  // Set(out, 0) overwrote it; it now reads as the running sum
        } else if (g >= 2) {
          p.alias_mask |= 1u << j;  // it already holds the running result
        }
      }
    }
    int rc;
    const bool last = relu && done + p.k == k;  // the activation belongs to the last chunk
    switch (operation) {
      case SHDW_ELTWISE_PROD: rc = launch_eltwise_chunk<SHDW_ELTWISE_PROD>(p, n, y, last, s); break;
      case SHDW_ELTWISE_SUM: rc = launch_eltwise_chunk<SHDW_ELTWISE_SUM>(p, n, y, last, s); break;
      case SHDW_ELTWISE_MAX: rc = launch_eltwise_chunk<SHDW_ELTWISE_MAX>(p, n, y, last, s); break;
      default: rc = launch_eltwise_chunk<SHDW_ELTWISE_MIN>(p, n, y, last, s); break;
    }
    if (rc != SHDW_OK) return rc;
    done += p.k;
  }
  return SHDW_OK;
}

int shdw_hip_eltwise(int operation, int k, const float* const* xs, const float* coeff, int n,
                     float* y, void* stream) {
  return run_eltwise(operation, k, xs, coeff, n, y, false, stream);
}

int shdw_hip_eltwise_relu(int operation, int k, const float* const* xs, const float* coeff, int n,
                          float* y, void* stream) {
  return run_eltwise(operation, k, xs, coeff, n, y, true, stream);
}

}  // extern "C"
