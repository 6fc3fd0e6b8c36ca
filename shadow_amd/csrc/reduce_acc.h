// Accumulators of the reduce kernels and their wave64 combine.
//
// PROD/SUM/AVG/L1/L2 accumulate in fp64 exactly as the reference does
// (shadow/operators/kernels/reduce.cpp:19-60), so the only difference is
// association order.  MAX/MIN must be bit-exact although the reference's "first
// element attaining the extremum wins" depends on order when the extremum is a
// zero (+0 and -0 compare equal): every accumulator therefore also tracks the
// smallest list position of a zero together with its sign, and the sign of a
// zero result is taken from there.
#ifndef SHADOW_AMD_CSRC_REDUCE_ACC_H_
#define SHADOW_AMD_CSRC_REDUCE_ACC_H_

#include <hip/hip_runtime.h>

#include <cfloat>

#include "../../include/shadow_hip.h"
#include "device_common.h"
#include "plan.h"

#pragma clang fp contract(off)

namespace shdw {

// What a first stage hands to the second, 8 bytes per (output, slice): the fp64
// accumulator, or {fp32 extremum, zero key} for MAX/MIN.
struct Partial {
  uint64_t bits;
};
static_assert(sizeof(Partial) == kReducePartialBytes, "partial layout");

constexpr bool is_select(int op) { return op == SHDW_REDUCE_MAX || op == SHDW_REDUCE_MIN; }

// ---- fp64 accumulating ops ----
template <int OP, bool SELECT = is_select(OP)>
struct Acc {
  static constexpr bool kSelect = false;
  double v;
  SHDW_DEVICE void init() { v = (OP == SHDW_REDUCE_PROD) ? 1.0 : 0.0; }
  SHDW_DEVICE void add_value(float x) { add(x, 0u); }
  SHDW_DEVICE void add_key(float, uint32_t) {}
  SHDW_DEVICE void add(float x, uint32_t) {
    if (OP == SHDW_REDUCE_PROD) {
      v *= static_cast<double>(x);
    } else if (OP == SHDW_REDUCE_L1) {
      v += static_cast<double>(__builtin_fabsf(x));
    } else if (OP == SHDW_REDUCE_L2) {
      const float ax = __builtin_fabsf(x);
      const float sq = ax * ax;  // fp32 product, then widened
      v += static_cast<double>(sq);
    } else {
      v += static_cast<double>(x);
    }
  }
  SHDW_DEVICE void merge(const Acc& o) {
    if (OP == SHDW_REDUCE_PROD) v *= o.v; else v += o.v;
  }
  template <int CTRL>
  SHDW_DEVICE Acc dpp() const {
    Acc r;
    r.v = dpp_f64<CTRL>(v);
    return r;
  }
  SHDW_DEVICE Acc shfl_xor(int m) const {
    Acc r;
    r.v = __shfl_xor(v, m, kWave);
    return r;
  }
  SHDW_DEVICE float finalize(uint32_t window) const {
    if (OP == SHDW_REDUCE_AVG) return static_cast<float>(v / static_cast<double>(static_cast<int>(window)));
    if (OP == SHDW_REDUCE_L2) return __builtin_sqrtf(static_cast<float>(v));
    return static_cast<float>(v);
  }
  SHDW_DEVICE void shift_positions(uint32_t) {}
  SHDW_DEVICE void nest_positions(uint32_t, uint32_t) {}
  SHDW_DEVICE Partial pack() const { return Partial{static_cast<uint64_t>(__double_as_longlong(v))}; }
  SHDW_DEVICE void unpack(const Partial& p) { v = __longlong_as_double(static_cast<long long>(p.bits)); }
};

// ---- MAX / MIN ----
template <int OP>
struct Acc<OP, true> {
  static constexpr bool kSelect = true;
  float v;
  uint32_t key;  // min over zeros seen of (list position << 1 | sign bit)
  SHDW_DEVICE void init() {
    v = (OP == SHDW_REDUCE_MAX) ? -FLT_MAX : FLT_MAX;
    key = 0xffffffffu;
  }
  // add(x, pos) == add_value(x) followed by add_key(x, pos).  Zeros are rare in
  // real data: the streaming loops take the values of a whole batch first, test
  // once whether any lane of the wave met a zero in it (fold_batch below), and
  // only then walk the batch again for the keys.
  SHDW_DEVICE void add_value(float x) {
    if (OP == SHDW_REDUCE_MAX) v = (v < x) ? x : v; else v = (x < v) ? x : v;
  }
  // the hardware's maximum / minimum; x must not be a signalling NaN (see fold_batch)
  SHDW_DEVICE void take(float x) {
    if (OP == SHDW_REDUCE_MAX) v = __builtin_fmaxf(v, x); else v = __builtin_fminf(v, x);
  }
  SHDW_DEVICE void add_key(float x, uint32_t pos) {
    if (x == 0.0f) {
      const uint32_t k = (pos << 1) | (__float_as_uint(x) >> 31);
      key = k < key ? k : key;
    }
  }
  SHDW_DEVICE void add(float x, uint32_t pos) {
    add_value(x);
    add_key(x, pos);
  }
  SHDW_DEVICE void merge(const Acc& o) {
    if (OP == SHDW_REDUCE_MAX) v = (v < o.v) ? o.v : v; else v = (o.v < v) ? o.v : v;
    key = o.key < key ? o.key : key;
  }
  template <int CTRL>
  SHDW_DEVICE Acc dpp() const {
    Acc r;
    r.v = dpp_f32<CTRL>(v);
    r.key = dpp_u32<CTRL>(key);
    return r;
  }
  SHDW_DEVICE Acc shfl_xor(int m) const {
    Acc r;
    r.v = __shfl_xor(v, m, kWave);
    r.key = __shfl_xor(key, m, kWave);
    return r;
  }
  SHDW_DEVICE float finalize(uint32_t) const {
    if (v == 0.0f) return (key & 1u) ? -0.0f : 0.0f;
    return v;
  }
  // the positions given to add() were relative to `by`
  SHDW_DEVICE void shift_positions(uint32_t by) {
    if (key != 0xffffffffu) key += by << 1;
  }
  // the positions given to add() were leading indices p of elements (p, j) whose
  // list position is p * nest + j
  SHDW_DEVICE void nest_positions(uint32_t nest, uint32_t j) {
    if (key != 0xffffffffu) key = (((key >> 1) * nest + j) << 1) | (key & 1u);
  }
  SHDW_DEVICE Partial pack() const {
    return Partial{(static_cast<uint64_t>(key) << 32) | __float_as_uint(v)};
  }
  SHDW_DEVICE void unpack(const Partial& p) {
    v = __uint_as_float(static_cast<uint32_t>(p.bits));
    key = static_cast<uint32_t>(p.bits >> 32);
  }
};

// Folds a batch of N vectors into the four column accumulators of a lane (or,
// with ONE, into a single accumulator): element j of vector u has list position
// pos(u, j); vectors with valid[u] false are skipped.  The votes are over the
// lanes that are active here, which then all take the same branch.
//
// MAX / MIN take the batch with v_max3_f32 / v_min3_f32 (two elements per
// instruction, where compare-and-select is two instructions and a wait per
// element).  Those give the reference's `(v < x) ? x : v` for every pair of
// numbers (up to the sign of a zero, which the key decides) and skip a quiet NaN
// as the comparison does; a signalling NaN they would hand on as a NaN, so every
// element is made quiet first (v_max_f32 x, x), which leaves numbers as they
// are.  Zeros: the smallest magnitude of the batch is zero exactly when it
// holds one (a NaN never is the minimum), so the keys cost one v_min3_f32 per
// two elements and one comparison per batch unless a zero is there.
template <int N, bool ONE, class A, class POS>
SHDW_DEVICE void fold_batch(A* acc, const v4f (&v)[N], const bool (&valid)[N], POS pos) {
  if constexpr (A::kSelect) {
    float smallest = FLT_MAX;
#pragma unroll
    for (int u = 0; u < N; ++u)
      if (valid[u]) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float q = __builtin_canonicalizef(v[u][j]);
          acc[ONE ? 0 : j].take(q);
          smallest = __builtin_fminf(smallest, __builtin_fabsf(q));
        }
      }
    if (__builtin_amdgcn_ballot_w64(smallest == 0.0f) != 0) {
#pragma unroll
      for (int u = 0; u < N; ++u)
        if (valid[u]) {
#pragma unroll
          for (int j = 0; j < 4; ++j) acc[ONE ? 0 : j].add_key(v[u][j], pos(u, j));
        }
    }
  } else {
#pragma unroll
    for (int u = 0; u < N; ++u)
      if (valid[u]) {
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[ONE ? 0 : j].add_value(v[u][j]);
      }
  }
}

// All 64 lanes must be active.  Every lane ends with the same combined value:
// each exchange pairs two lanes that both compute merge(own, other), and every
// merge used here is commutative bit-for-bit.
template <class A, int G = kWave>
SHDW_DEVICE A group_allreduce(A a) {  // G = 2, 4, 8, 16, 32 or 64 consecutive lanes
  a.merge(a.template dpp<kDppXor1>());
  if (G >= 4) a.merge(a.template dpp<kDppXor2>());
  if (G >= 8) a.merge(a.template dpp<kDppHalfMirror>());
  if (G >= 16) a.merge(a.template dpp<kDppMirror>());
  if (G >= 32) a.merge(a.shfl_xor(16));
  if (G >= 64) a.merge(a.shfl_xor(32));
  return a;
}
template <class A>
SHDW_DEVICE A wave_allreduce(A a) {
  return group_allreduce<A, kWave>(a);
}

}  // namespace shdw

#endif  // SHADOW_AMD_CSRC_REDUCE_ACC_H_
