// Per-element arithmetic of Shadow's CPU kernels, as device functors.
// Selection ops are written in the std::max / std::min / ternary forms the
// reference uses so that NaN and signed-zero behaviour is identical:
//   std::max(a, b) == (a < b) ? b : a      std::min(a, b) == (b < a) ? b : a
#ifndef SHADOW_AMD_CSRC_FUNCTORS_H_
#define SHADOW_AMD_CSRC_FUNCTORS_H_

#include "device_common.h"
#include "libm_exact.h"

#pragma clang fp contract(off)

namespace shdw {

// Functors that evaluate exact_expf declare `static constexpr bool kExpTable =
// true`; the kernels then stage the 32-entry 2^(i/32) table in LDS and pass it
// as `tab` (nullptr otherwise).  ATanh declares `kTanhTable` instead and gets the
// 32 TanhStep entries the same way, behind the same pointer.
template <class F, class = void>
struct uses_exp_table { static constexpr bool value = false; };
template <class F>
struct uses_exp_table<F, decltype((void)F::kExpTable)> { static constexpr bool value = F::kExpTable; };

template <class F, class = void>
struct uses_tanh_table { static constexpr bool value = false; };
template <class F>
struct uses_tanh_table<F, decltype((void)F::kTanhTable)> { static constexpr bool value = F::kTanhTable; };

// Functors with a long dependent chain per element declare
// `static constexpr int kVectorsPerLane = 2`: a lane then owns two vectors and
// has the second one's load in flight while it works on the first.
template <class F, class = void>
struct vectors_per_lane { static constexpr int value = 1; };
template <class F>
struct vectors_per_lane<F, decltype((void)F::kVectorsPerLane)> { static constexpr int value = F::kVectorsPerLane; };

// Functors whose arithmetic has a short form for ordinary arguments and a long
// one for the rest define `four(x)`: the four elements of a lane's vector at once,
// with one wave-wide choice for all of them, so that the four evaluations stay
// interleaved instead of each sitting behind a branch of its own.
template <class F, class = void>
struct has_four { static constexpr bool value = false; };
template <class F>
struct has_four<F, decltype((void)&F::four)> { static constexpr bool value = true; };

// Both forms are pure arithmetic, which the compiler is free to evaluate side by
// side and select from; an empty statement it may not move keeps the rare form
// behind its wave-wide branch.
SHDW_DEVICE void keep_branch() { asm volatile("" ::: "memory"); }

SHDW_DEVICE float sel_max(float a, float b) { return (a < b) ? b : a; }
SHDW_DEVICE float sel_min(float a, float b) { return (b < a) ? b : a; }

// ---- unary: shadow/core/blas.cpp:151-165 ----
struct UAbs { SHDW_DEVICE float operator()(float a, const uint64_t* tab) const { return __builtin_fabsf(a); } };
struct USquare { SHDW_DEVICE float operator()(float a, const uint64_t* tab) const { return a * a; } };
struct USqrt { SHDW_DEVICE float operator()(float a, const uint64_t* tab) const { return __builtin_sqrtf(a); } };
struct ULog { SHDW_DEVICE float operator()(float a, const uint64_t* tab) const { return libm::exact_logf(a); } };
struct UExp { static constexpr bool kExpTable = true; SHDW_DEVICE float operator()(float a, const uint64_t* tab) const { return libm::exact_expf(a, tab); } };
struct USin { SHDW_DEVICE float operator()(float a, const uint64_t* tab) const { return libm::exact_sinf(a); } };
struct UCos { SHDW_DEVICE float operator()(float a, const uint64_t* tab) const { return libm::exact_cosf(a); } };
struct UTan { SHDW_DEVICE float operator()(float a, const uint64_t* tab) const { return libm::exact_tanf(a); } };
struct UAsin { SHDW_DEVICE float operator()(float a, const uint64_t* tab) const { return libm::exact_asinf(a); } };
struct UAcos { SHDW_DEVICE float operator()(float a, const uint64_t* tab) const { return libm::exact_acosf(a); } };
struct UAtan { SHDW_DEVICE float operator()(float a, const uint64_t* tab) const { return libm::exact_atanf(a); } };
struct UFloor { SHDW_DEVICE float operator()(float a, const uint64_t* tab) const { return __builtin_floorf(a); } };
struct UCeil { SHDW_DEVICE float operator()(float a, const uint64_t* tab) const { return __builtin_ceilf(a); } };
struct UNeg { SHDW_DEVICE float operator()(float a, const uint64_t* tab) const { return -a; } };
struct UReciprocal { SHDW_DEVICE float operator()(float a, const uint64_t* tab) const { return 1 / a; } };
struct UCopy { SHDW_DEVICE float operator()(float a, const uint64_t* tab) const { return a; } };

// ---- binary: shadow/core/blas.cpp:114-120, kernels/binary.cpp:9-28 ----
struct BAdd { SHDW_DEVICE float operator()(float a, float b, const uint64_t* tab) const { return a + b; } };
struct BSub { SHDW_DEVICE float operator()(float a, float b, const uint64_t* tab) const { return a - b; } };
struct BMul { SHDW_DEVICE float operator()(float a, float b, const uint64_t* tab) const { return a * b; } };
struct BDiv { SHDW_DEVICE float operator()(float a, float b, const uint64_t* tab) const { return a / b; } };
struct BPow { static constexpr bool kExpTable = true; SHDW_DEVICE float operator()(float a, float b, const uint64_t* tab) const { return libm::exact_powf(a, b, tab); } };
struct BMax { SHDW_DEVICE float operator()(float a, float b, const uint64_t* tab) const { return sel_max(a, b); } };
struct BMin { SHDW_DEVICE float operator()(float a, float b, const uint64_t* tab) const { return sel_min(a, b); } };

// ---- activations: shadow/operators/kernels/activate.cpp:9-31 ----
struct ARelu { SHDW_DEVICE float operator()(float x, float, const uint64_t* tab) const { return x > 0 ? x : 0; } };
struct ALeaky { SHDW_DEVICE float operator()(float x, float s, const uint64_t* tab) const { return x > 0 ? x : s * x; } };
struct ASigmoid {
  static constexpr bool kExpTable = true;
  SHDW_DEVICE float operator()(float x, float, const uint64_t* tab) const { return libm::exact_sigmoidf(x, tab); }
  SHDW_DEVICE v4f four(v4f x, const uint64_t* tab) const {
    bool ok = true;
#pragma unroll
    for (int j = 0; j < 4; ++j) ok &= libm::sigmoidf_short_ok(x[j]);
    v4f r;
    if (__builtin_amdgcn_ballot_w64(!ok) == 0) {
#pragma unroll
      for (int j = 0; j < 4; ++j) r[j] = libm::sigmoidf_short(x[j], tab);
    } else {
      keep_branch();
#pragma unroll
      for (int j = 0; j < 4; ++j) r[j] = libm::sigmoidf_any(x[j], tab);
    }
    return r;
  }
};
struct ASoftPlus { static constexpr bool kExpTable = true; SHDW_DEVICE float operator()(float x, float, const uint64_t* tab) const { return libm::exact_softplusf(x, tab); } };
struct ATanh {
  static constexpr bool kTanhTable = true;
  static constexpr int kVectorsPerLane = 2;
  static SHDW_DEVICE const libm::TanhStep* steps(const uint64_t* tab) {
    return reinterpret_cast<const libm::TanhStep*>(tab);
  }
  SHDW_DEVICE float operator()(float x, float, const uint64_t* tab) const { return libm::exact_tanhf(x, steps(tab)); }
  SHDW_DEVICE v4f four(v4f x, const uint64_t* tab) const {
    bool ok = true;
#pragma unroll
    for (int j = 0; j < 4; ++j) ok &= libm::tanhf_short_ok(x[j]);
    v4f r;
    if (__builtin_amdgcn_ballot_w64(!ok) == 0) {
#pragma unroll
      for (int j = 0; j < 4; ++j) r[j] = libm::tanhf_short(x[j], steps(tab));
    } else {
      keep_branch();
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        // A copy the compiler cannot relate to x[j]: the integer |x| that this form
        // needs is then computed here and not ahead of the branch, where the short
        // form (which takes |x| as an operand modifier) would pay for it too.
        float xj = x[j];
        asm("" : "+v"(xj));
        r[j] = libm::tanhf_any(xj, steps(tab));
      }
    }
    return r;
  }
};
struct ARelu6 { SHDW_DEVICE float operator()(float x, float, const uint64_t* tab) const { return x < 0 ? 0 : (x > 6 ? 6 : x); } };
struct AHardSwish {
  SHDW_DEVICE float operator()(float x, float, const uint64_t* tab) const {
    return x < -3 ? 0 : (x > 3 ? x : (x * (x + 3) / 6.f));
  }
};
struct AGelu {
  static constexpr bool kExpTable = true;
  SHDW_DEVICE float operator()(float x, float, const uint64_t* tab) const {
    return libm::exact_geluf(x, tab);
  }
};

}  // namespace shdw

#endif  // SHADOW_AMD_CSRC_FUNCTORS_H_
