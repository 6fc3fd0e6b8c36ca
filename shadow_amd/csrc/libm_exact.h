// Bit-exact restatements of the glibc 2.35 (x86-64) single-precision libm
// routines that Shadow's CPU kernels call through std::exp / std::tanh
// (shadow/core/blas.cpp:153, shadow/operators/kernels/activate.cpp:16,20).
//
// Each routine is written with IEEE-754 fp32/fp64 operations and integer bit
// manipulation only, so gfx950 and the host evaluate it identically as long as
// the compiler neither contracts a*b+c nor reassociates.  fma() appears only
// where the host library's selected variant fuses.  The same text is compiled
// by the host C++ compiler for exhaustive comparison against the host's libm.
//
//   exact_expf  : ARM optimized-routines expf as shipped in glibc
//                 (sysdeps/ieee754/flt-32/e_expf.c), FMA multiarch variant:
//                 the reduction r = InvLn2N*x - k is one fused operation.
//   exact_expm1f: fdlibm s_expm1f.c (glibc sysdeps/ieee754/flt-32/s_expm1f.c).
//   exact_tanhf : fdlibm s_tanhf.c  (glibc sysdeps/ieee754/flt-32/s_tanhf.c).
//   exact_logf, exact_sinf, exact_cosf, exact_powf: ARM optimized routines as
//                 shipped in glibc, FMA multiarch variants.
//   exact_tanf, exact_asinf, exact_acosf, exact_atanf, exact_log1pf, exact_erff:
//                 fdlibm lineage, fp32 arithmetic without fused operations.
// Every function here was compared with glibc 2.35's libm on all 2^32 inputs
// (powf: on 5.6e10 pairs) with zero mismatches.
#ifndef SHADOW_AMD_CSRC_LIBM_EXACT_H_
#define SHADOW_AMD_CSRC_LIBM_EXACT_H_

#include <stdint.h>

#if defined(__HIPCC__)
#define SHDW_LIBM_FN __device__ __forceinline__
#define SHDW_LIBM_TABLE static __device__ const
#pragma clang fp contract(off)
#else
#define SHDW_LIBM_FN static inline
#define SHDW_LIBM_TABLE static const
#endif

// The divisions that are a hardware reciprocal plus one correction (div_normal,
// sigmoidf_short) return the library's bits on gfx950's v_rcp_f32, which is what
// the exhaustive device tests establish; another architecture's reciprocal would
// have to be swept again before this header is compiled for it.
#if defined(__HIP_DEVICE_COMPILE__) && !defined(__gfx950__)
#error "libm_exact.h: the reciprocal-based divisions are verified for gfx950 only"
#endif

namespace shdw {
namespace libm {

SHDW_LIBM_FN uint32_t f2u(float f) { return __builtin_bit_cast(uint32_t, f); }
SHDW_LIBM_FN float u2f(uint32_t u) { return __builtin_bit_cast(float, u); }
SHDW_LIBM_FN uint64_t d2u(double d) { return __builtin_bit_cast(uint64_t, d); }
SHDW_LIBM_FN double u2d(uint64_t u) { return __builtin_bit_cast(double, u); }

// a / b for the two quotients of exact_tanhf, whose operands and result are
// well inside the normal range.  On the device: the hardware reciprocal (1 ulp),
// a * r, and one correction from the exact remainder a - b * q.  That is shorter
// than a division that is correctly rounded for every operand pair (no second
// correction, no refinement of r); it is used only here because exact_tanhf on
// the device returns the library's result for every one of the 2^32 inputs with
// it, which the exhaustive device test checks.  On the host it is `/`.
SHDW_LIBM_FN float div_normal(float a, float b) {
#if defined(__HIP_DEVICE_COMPILE__)
  const float r = __builtin_amdgcn_rcpf(b);
  const float q = a * r;
  const float e = __builtin_fmaf(-b, q, a);
  return __builtin_fmaf(e, r, q);
#else
  return a / b;
#endif
}

// T[i] = bits(2^(i/32)) - (i << 47)
SHDW_LIBM_TABLE uint64_t kExp2fTab[32] = {
    0x3ff0000000000000ull, 0x3fefd9b0d3158574ull, 0x3fefb5586cf9890full, 0x3fef9301d0125b51ull,
    0x3fef72b83c7d517bull, 0x3fef54873168b9aaull, 0x3fef387a6e756238ull, 0x3fef1e9df51fdee1ull,
    0x3fef06fe0a31b715ull, 0x3feef1a7373aa9cbull, 0x3feedea64c123422ull, 0x3feece086061892dull,
    0x3feebfdad5362a27ull, 0x3feeb42b569d4f82ull, 0x3feeab07dd485429ull, 0x3feea47eb03a5585ull,
    0x3feea09e667f3bcdull, 0x3fee9f75e8ec5f74ull, 0x3feea11473eb0187ull, 0x3feea589994cce13ull,
    0x3feeace5422aa0dbull, 0x3feeb737b0cdc5e5ull, 0x3feec49182a3f090ull, 0x3feed503b23e255dull,
    0x3feee89f995ad3adull, 0x3feeff76f2fb5e47ull, 0x3fef199bdd85529cull, 0x3fef3720dcef9069ull,
    0x3fef5818dcfba487ull, 0x3fef7c97337b9b5full, 0x3fefa4afa2a490daull, 0x3fefd0765b6e4540ull};

// `tab` is kExp2fTab or a copy of it in faster memory (the kernels stage it in
// LDS so that the lookup does not queue behind the streaming HBM traffic).
//
// The library's main path.  By itself it is the whole function for
// -0x1.9fe368p6 <= x <= 0x1.62e42ep6 (where the conversion at the end rounds to
// a subnormal or to 2^-149 exactly as the library's own cases do) and for NaN;
// outside, the table scale may wrap, so the result must be replaced.  Nothing in
// it can trap and the table index is masked.
SHDW_LIBM_FN float expf_main(float x, const uint64_t* tab) {
  const double InvLn2N = 0x1.71547652b82fep+5;  // 32 / ln 2
  const double Shift = 0x1.8p+52;
  const double xd = static_cast<double>(x);
  const double z = InvLn2N * xd;
  double kd = z + Shift;
  const uint64_t ki = d2u(kd);
  kd -= Shift;
  const double r = __builtin_fma(InvLn2N, xd, -kd);
  const double s = u2d(tab[ki & 31] + (ki << 47));
  const double c0 = 0x1.c6af84b912394p-20, c1 = 0x1.ebfce50fac4f3p-13,
               c2 = 0x1.62e42ff0c52d6p-6;
  const double p = __builtin_fma(c0, r, c1);
  const double r2 = r * r;
  double y = __builtin_fma(c2, r, 1.0);
  y = __builtin_fma(p, r2, y);
  y = y * s;
  return static_cast<float>(y);
}

SHDW_LIBM_FN float exact_expf(float x, const uint64_t* tab) {
  float res = expf_main(x, tab);
  // Out of range: both comparisons are false for NaN, which the main path has
  // already propagated.
  res = (x > 0x1.62e42ep6f) ? __builtin_inff() : res;  // overflow (and +inf)
  res = (x < -0x1.9fe368p6f) ? 0.0f : res;             // underflow to zero (and -inf)
  return res;
}

SHDW_LIBM_FN float exact_expm1f(float x) {
  const float one = 1.0f, huge = 1.0e+30f, tiny = 1.0e-30f;
  const float o_threshold = 8.8721679688e+01f;
  const float ln2_hi = 6.9313812256e-01f, ln2_lo = 9.0580006145e-06f;
  const float invln2 = 1.4426950216e+00f;
  const float Q1 = -3.3333335072e-02f, Q2 = 1.5873016091e-03f, Q3 = -7.9365076090e-05f,
              Q4 = 4.0082177293e-06f, Q5 = -2.0109921195e-07f;
  float y, hi, lo, c = 0.0f, t, e, hxs, hfx, r1;
  int32_t k;
  uint32_t hx = f2u(x);
  const uint32_t xsb = hx & 0x80000000u;
  hx &= 0x7fffffffu;

  if (hx >= 0x4195b844u) {    // |x| >= 27 ln2
    if (hx >= 0x42b17218u) {  // |x| >= 88.72
      if (hx > 0x7f800000u) return x + x;
      if (hx == 0x7f800000u) return xsb == 0 ? x : -1.0f;
      if (x > o_threshold) return huge * huge;
    }
    if (xsb != 0) return tiny - one;
  }

  if (hx > 0x3eb17218u) {    // |x| > 0.5 ln2
    if (hx < 0x3F851592u) {  // |x| < 1.5 ln2
      if (xsb == 0) {
        hi = x - ln2_hi;
        lo = ln2_lo;
        k = 1;
      } else {
        hi = x + ln2_hi;
        lo = -ln2_lo;
        k = -1;
      }
    } else {
      k = static_cast<int32_t>(invln2 * x + (xsb == 0 ? 0.5f : -0.5f));
      t = static_cast<float>(k);
      hi = x - t * ln2_hi;
      lo = t * ln2_lo;
    }
    x = hi - lo;
    c = (hi - x) - lo;
  } else if (hx < 0x33000000u) {  // |x| < 2^-25
    t = huge + x;
    return x - (t - (huge + x));
  } else {
    k = 0;
  }

  hfx = 0.5f * x;
  hxs = x * hfx;
  r1 = one + hxs * (Q1 + hxs * (Q2 + hxs * (Q3 + hxs * (Q4 + hxs * Q5))));
  t = 3.0f - r1 * hfx;
  e = hxs * ((r1 - t) / (6.0f - x * t));
  if (k == 0) return x - (x * e - hxs);
  e = (x * (e - c) - c);
  e -= hxs;
  if (k == -1) return 0.5f * (x - e) - 0.5f;
  if (k == 1) {
    if (x < -0.25f) return -2.0f * (e - (x + 0.5f));
    return one + 2.0f * (x - e);
  }
  if (k <= -2 || k > 56) {
    y = one - (e - x);
    y = u2f(f2u(y) + (static_cast<uint32_t>(k) << 23));
    return y - one;
  }
  if (k < 23) {
    t = u2f(0x3f800000u - (0x1000000u >> k));  // 1 - 2^-k
    y = t - (e - x);
    y = u2f(f2u(y) + (static_cast<uint32_t>(k) << 23));
  } else {
    t = u2f(static_cast<uint32_t>(0x7f - k) << 23);  // 2^-k
    y = x - (e + t);
    y += one;
    y = u2f(f2u(y) + (static_cast<uint32_t>(k) << 23));
  }
  return y;
}

// tanhf without divergent control flow.  s_tanhf.c calls expm1f only with
// a = 2|x| in [2, 44) or a = -2|x| in (-2, -2^-54], so of expm1f's cases only
// k = 0, k = -1, k <= -2 (a < 0) and k >= 3 (a > 0) can occur.  They differ in
// constants only, which a table indexed by k holds (TanhStep), so every lane runs
// the same operations whatever its k, in the library's order.  Where a cheaper
// form gives the same bits on every input it replaces the library's.  Exact
// rewrites (they change no rounding):
//   * hxs = x * (0.5 x) is half of s = x * x, and a halving commutes with every
//     rounding here, so 0.5 * round(s * p) stands for the library's round(hxs * p)
//     and "v - hxs" is one fused -0.5 * s + v; hfx and hxs are never formed;
//   * a = 2 h is never formed either: invln2 * a is (2 invln2) * h, and
//     a - k * ln2_hi is one fused 2 h - khi, the product k * ln2_hi being exact;
//   * k = 0 has lo = 0 and therefore c = 0, which makes the library's special
//     form x - (x * e - hxs) equal to x - e with the general e = x * (e - c) - c
//     - hxs.  With d = x - e, the library's results are
//         k = 0:   d                     k = -1:  0.5 d - 0.5
//         k <= -2: 2^k (1 + d) - 1       k >= 3:  2^k ((1 - 2^-k) + d)
//     which are all fma(2^k, T + d, off) with T = 0, 0, 1, 1 - 2^-k and
//     off = 0, -0.5, -1, 0: T + d is exact where T = 0, the scaling by 2^k is exact
//     everywhere, so each is rounded where the library rounds it;
//   * |x| >= 1 returns 1 - q and |x| < 1 the magnitude of q: base - q with base = 1
//     or 0, which the table holds as well since k >= 3 exactly when |x| >= 1.
// Rewrites that do change intermediate roundings, kept because the function
// still returns the library's bits for all 2^32 inputs with them (compared on
// the host and on the device; none of it is argued from error bounds):
//   * k = rint(a / ln2), taken from one fused multiply-add with 1.5 * 2^23,
//     instead of the truncation of a / ln2 -+ 0.5 and of the separate
//     |a| < 0.5 ln2 and |a| < 1.5 ln2 cases (k = 0, k = +-1 there too);
//   * the four innermost steps of the degree-5 polynomial are fused
//     multiply-adds (their rounding differences are attenuated by the steps that
//     follow; fusing the outermost one as well differs on 70 inputs, fusing the
//     products of t3, of the divisor or of e on thousands);
//   * y = (1 - 2^-k) + d also for 23 <= k, where the library switches to
//     (x - (e + 2^-k)) + 1: the two differ far below what 1 - 2 / (t + 2) keeps;
//   * |x| >= 9.75 is evaluated at 9.75 (the result is already exactly 1 there;
//     the library's own cut is at 22), which also bounds k by 28;
//   * the |x| < 2^-55 and |a| < 2^-25 early returns are left to the general
//     path, which returns x there as well.
struct alignas(32) TanhStep {
  float khi, klo;  // k * ln2_hi (exact), k * ln2_lo (rounded as the library's product is)
  float T, off;    // expm1f(a) = fma(scale, T + d, off)
  float scale;     // 2^k
  float base;      // 1 where k >= 1 (|x| >= 1), else 0
  float pad[2];
};
constexpr int kTanhStepLog2Bytes = 5;
constexpr int kTanhSteps = 32;            // k = -3 ... 28
constexpr float kTanhCut = 9.75f;         // 2 * 9.75 / ln2 = 28.13
SHDW_LIBM_TABLE TanhStep kTanhStepTab[kTanhSteps] = {
    {-0x1.0a2a4p+1f, -0x1.c7e774p-16f, 0x1.0p+0f, -0x1.0p+0f, 0x1.0p-3f, 0.0f, 0.0f, 0.0f},  // k = -3
    {-0x1.62e3p+0f, -0x1.2fefa2p-16f, 0x1.0p+0f, -0x1.0p+0f, 0x1.0p-2f, 0.0f, 0.0f, 0.0f},  // k = -2
    {-0x1.62e3p-1f, -0x1.2fefa2p-17f, 0.0f, -0x1.0p-1f, 0x1.0p-1f, 0.0f, 0.0f, 0.0f},  // k = -1
    {0.0f, 0.0f, 0.0f, 0.0f, 0x1.0p+0f, 0.0f, 0.0f, 0.0f},  // k = 0
    {0x1.62e3p-1f, 0x1.2fefa2p-17f, 0x1.0p-1f, 0.0f, 0x1.0p+1f, 0x1.0p+0f, 0.0f, 0.0f},  // k = 1
    {0x1.62e3p+0f, 0x1.2fefa2p-16f, 0x1.8p-1f, 0.0f, 0x1.0p+2f, 0x1.0p+0f, 0.0f, 0.0f},  // k = 2
    {0x1.0a2a4p+1f, 0x1.c7e774p-16f, 0x1.cp-1f, 0.0f, 0x1.0p+3f, 0x1.0p+0f, 0.0f, 0.0f},  // k = 3
    {0x1.62e3p+1f, 0x1.2fefa2p-15f, 0x1.ep-1f, 0.0f, 0x1.0p+4f, 0x1.0p+0f, 0.0f, 0.0f},  // k = 4
    {0x1.bb9bcp+1f, 0x1.7beb8ap-15f, 0x1.fp-1f, 0.0f, 0x1.0p+5f, 0x1.0p+0f, 0.0f, 0.0f},  // k = 5
    {0x1.0a2a4p+2f, 0x1.c7e774p-15f, 0x1.f8p-1f, 0.0f, 0x1.0p+6f, 0x1.0p+0f, 0.0f, 0.0f},  // k = 6
    {0x1.3686ap+2f, 0x1.09f1aep-14f, 0x1.fcp-1f, 0.0f, 0x1.0p+7f, 0x1.0p+0f, 0.0f, 0.0f},  // k = 7
    {0x1.62e3p+2f, 0x1.2fefa2p-14f, 0x1.fep-1f, 0.0f, 0x1.0p+8f, 0x1.0p+0f, 0.0f, 0.0f},  // k = 8
    {0x1.8f3f6p+2f, 0x1.55ed96p-14f, 0x1.ffp-1f, 0.0f, 0x1.0p+9f, 0x1.0p+0f, 0.0f, 0.0f},  // k = 9
    {0x1.bb9bcp+2f, 0x1.7beb8ap-14f, 0x1.ff8p-1f, 0.0f, 0x1.0p+10f, 0x1.0p+0f, 0.0f, 0.0f},  // k = 10
    {0x1.e7f82p+2f, 0x1.a1e97ep-14f, 0x1.ffcp-1f, 0.0f, 0x1.0p+11f, 0x1.0p+0f, 0.0f, 0.0f},  // k = 11
    {0x1.0a2a4p+3f, 0x1.c7e774p-14f, 0x1.ffep-1f, 0.0f, 0x1.0p+12f, 0x1.0p+0f, 0.0f, 0.0f},  // k = 12
    {0x1.20587p+3f, 0x1.ede568p-14f, 0x1.fffp-1f, 0.0f, 0x1.0p+13f, 0x1.0p+0f, 0.0f, 0.0f},  // k = 13
    {0x1.3686ap+3f, 0x1.09f1aep-13f, 0x1.fff8p-1f, 0.0f, 0x1.0p+14f, 0x1.0p+0f, 0.0f, 0.0f},  // k = 14
    {0x1.4cb4dp+3f, 0x1.1cf0a8p-13f, 0x1.fffcp-1f, 0.0f, 0x1.0p+15f, 0x1.0p+0f, 0.0f, 0.0f},  // k = 15
    {0x1.62e3p+3f, 0x1.2fefa2p-13f, 0x1.fffep-1f, 0.0f, 0x1.0p+16f, 0x1.0p+0f, 0.0f, 0.0f},  // k = 16
    {0x1.79113p+3f, 0x1.42ee9cp-13f, 0x1.ffffp-1f, 0.0f, 0x1.0p+17f, 0x1.0p+0f, 0.0f, 0.0f},  // k = 17
    {0x1.8f3f6p+3f, 0x1.55ed96p-13f, 0x1.ffff8p-1f, 0.0f, 0x1.0p+18f, 0x1.0p+0f, 0.0f, 0.0f},  // k = 18
    {0x1.a56d9p+3f, 0x1.68ec9p-13f, 0x1.ffffcp-1f, 0.0f, 0x1.0p+19f, 0x1.0p+0f, 0.0f, 0.0f},  // k = 19
    {0x1.bb9bcp+3f, 0x1.7beb8ap-13f, 0x1.ffffep-1f, 0.0f, 0x1.0p+20f, 0x1.0p+0f, 0.0f, 0.0f},  // k = 20
    {0x1.d1c9fp+3f, 0x1.8eea84p-13f, 0x1.fffffp-1f, 0.0f, 0x1.0p+21f, 0x1.0p+0f, 0.0f, 0.0f},  // k = 21
    {0x1.e7f82p+3f, 0x1.a1e97ep-13f, 0x1.fffff8p-1f, 0.0f, 0x1.0p+22f, 0x1.0p+0f, 0.0f, 0.0f},  // k = 22
    {0x1.fe265p+3f, 0x1.b4e878p-13f, 0x1.fffffcp-1f, 0.0f, 0x1.0p+23f, 0x1.0p+0f, 0.0f, 0.0f},  // k = 23
    {0x1.0a2a4p+4f, 0x1.c7e774p-13f, 0x1.fffffep-1f, 0.0f, 0x1.0p+24f, 0x1.0p+0f, 0.0f, 0.0f},  // k = 24
    {0x1.154158p+4f, 0x1.dae66ep-13f, 0x1.0p+0f, 0.0f, 0x1.0p+25f, 0x1.0p+0f, 0.0f, 0.0f},  // k = 25
    {0x1.20587p+4f, 0x1.ede568p-13f, 0x1.0p+0f, 0.0f, 0x1.0p+26f, 0x1.0p+0f, 0.0f, 0.0f},  // k = 26
    {0x1.2b6f88p+4f, 0x1.00723p-12f, 0x1.0p+0f, 0.0f, 0x1.0p+27f, 0x1.0p+0f, 0.0f, 0.0f},  // k = 27
    {0x1.3686ap+4f, 0x1.09f1aep-12f, 0x1.0p+0f, 0.0f, 0x1.0p+28f, 0x1.0p+0f, 0.0f, 0.0f},  // k = 28
};

// tanhf_magnitude is |tanhf(x)| from h = |x| where |x| >= 1 (`big`) and -|x|
// otherwise, |x| <= 9.75; exact_tanhf puts the sign back.  `steps` is
// kTanhStepTab or a copy of it in faster memory.  On the device a wave whose
// lanes all have |x| < 9.75 (no NaN among them) needs neither the cut nor the NaN
// case; any other wave goes the long way.  Both ways run the same
// tanhf_magnitude on the same h.
SHDW_LIBM_FN float tanhf_magnitude(float h, bool big, const TanhStep* steps) {
  const float one = 1.0f, two = 2.0f, half = 0.5f;
  const float invln2 = 1.4426950216e+00f;
  const float Q1 = -3.3333335072e-02f, Q2 = 1.5873016091e-03f, Q3 = -7.9365076090e-05f,
              Q4 = 4.0082177293e-06f, Q5 = -2.0109921195e-07f;

  // --- expm1f(a), a = 2 h: argument reduction ---
  // k = rint(a / ln2) by the 1.5 * 2^23 trick, three added so that the sum's low
  // mantissa bits are the table index k + 3 (0 ... 31 for the h allowed here).
  const float magic = 12582912.0f;
  const float tsum = __builtin_fmaf(two * invln2, h, magic + 3.0f);
  uint32_t byte_offset = (f2u(tsum) << kTanhStepLog2Bytes) - (f2u(magic) << kTanhStepLog2Bytes);
#if defined(__HIP_DEVICE_COMPILE__)
  // One shift-and-add.  Opaque to the compiler from here on, so that the fields
  // of the entry are fixed offsets from one address and not a sum each.
  asm("" : "+v"(byte_offset));
#endif
  const TanhStep& st = *static_cast<const TanhStep*>(
      __builtin_assume_aligned(reinterpret_cast<const char*>(steps) + byte_offset, sizeof(TanhStep)));
  const float hi = __builtin_fmaf(two, h, -st.khi);
  const float xr = hi - st.klo;
  const float c = (hi - xr) - st.klo;

  // --- primary range ---
  const float s = xr * xr;  // 2 hxs
  // r1 = 1 + hxs (Q1 + hxs (Q2 + hxs (Q3 + hxs (Q4 + hxs Q5)))).  Step i of the
  // fused part works on its value divided by 2^(i-1): hxs * v = s * (v / 2), and a
  // power of two passes through every rounding here, so the halvings sit in the
  // constants and each step is one fused multiply-add on s.
  float p = __builtin_fmaf(s, Q5 * 0.0625f, Q4 * 0.125f);
  p = __builtin_fmaf(s, p, Q3 * 0.25f);
  p = __builtin_fmaf(s, p, Q2 * half);
  p = __builtin_fmaf(s, p, Q1);
  const float r1 = __builtin_fmaf(half, s * p, one);
  const float t3 = __builtin_fmaf(-half, r1 * xr, 3.0f);  // 3 - r1 * hfx
  // numerator ~ -2, denominator in [4.9, 7.1]; twice the library's e = hxs * (...)
  const float e2x = s * div_normal(r1 - t3, 6.0f - xr * t3);
  float e = xr * __builtin_fmaf(half, e2x, -c) - c;  // x * (e - c) - c
  e = __builtin_fmaf(-half, s, e);                   // - hxs
  const float d = xr - e;
  const float t = __builtin_fmaf(st.scale, st.T + d, st.off);

  // --- tanhf ---
  // |x| >= 1: 1 - 2 / (t + 2); else -t / (t + 2), whose magnitude is |q|.
  const float q = div_normal(big ? two : t, t + two);
  return st.base - q;
}

// The long way: any x.
SHDW_LIBM_FN float tanhf_any(float x, const TanhStep* steps) {
  const uint32_t jx = f2u(x);
  const uint32_t ix = jx & 0x7fffffffu;
  // from |x| = 9.75 on 2 / (t + 2) < 2^-25 and 1 - q rounds to 1: evaluate there
  const uint32_t cut = f2u(kTanhCut);
  const float ac = u2f(ix < cut ? ix : cut);
  const bool big = ix >= 0x3f800000u;
  const float z = tanhf_magnitude(big ? ac : -ac, big, steps);
  // The result takes x's sign; a NaN keeps all of its bits.
  const uint32_t keep = (ix > 0x7f800000u) ? 0u : 0x7fffffffu;
  return u2f((f2u(z) & keep) | (jx & ~keep));
}

// The short way: |x| < 9.75 (tanhf_short_ok), and so no NaN.
SHDW_LIBM_FN bool tanhf_short_ok(float x) { return __builtin_fabsf(x) < kTanhCut; }
SHDW_LIBM_FN float tanhf_short(float x, const TanhStep* steps) {
  const float ax = __builtin_fabsf(x);
  const bool big = ax >= 1.0f;
  return __builtin_copysignf(tanhf_magnitude(big ? ax : -ax, big, steps), x);
}

SHDW_LIBM_FN float exact_tanhf(float x, const TanhStep* steps) {
#if defined(__HIP_DEVICE_COMPILE__)
  if (__builtin_amdgcn_ballot_w64(!tanhf_short_ok(x)) == 0) return tanhf_short(x, steps);
#endif
  return tanhf_any(x, steps);
}

// 1 / (1 + exp(-x)) in fp32, the way shadow/operators/kernels/activate.cpp:16
// writes it.
SHDW_LIBM_FN float sigmoidf_any(float x, const uint64_t* tab) {
  return 1.0f / (1.0f + exact_expf(-x, tab));
}
#if defined(__HIPCC__)
// |x| < 87: exp(-x) lies in (2^-126, 2^126), so expf's main path is the whole
// function, d = 1 + exp(-x) is in [1, 2^126) and the quotient is a normal
// number; the hardware reciprocal of gfx950 plus one correction from the exact
// remainder 1 - d * r is then the correctly rounded 1 / d for every d this
// function can produce (all 2^32 inputs compared with the full form on that
// device; nothing here is argued for another architecture's reciprocal).  From
// 2^126 on, x < -87.3, the quotient is subnormal and only the full division is
// right.
SHDW_LIBM_FN bool sigmoidf_short_ok(float x) { return __builtin_fabsf(x) < 87.0f; }
SHDW_LIBM_FN float sigmoidf_short(float x, const uint64_t* tab) {
#if defined(__HIP_DEVICE_COMPILE__)
  const float d = 1.0f + expf_main(-x, tab);
  const float r = __builtin_amdgcn_rcpf(d);
  const float e = __builtin_fmaf(-d, r, 1.0f);
  return __builtin_fmaf(e, r, r);
#else
  return sigmoidf_any(x, tab);  // the compiler's host pass over device code; never called
#endif
}
#endif
SHDW_LIBM_FN float exact_sigmoidf(float x, const uint64_t* tab) {
#if defined(__HIP_DEVICE_COMPILE__)
  // The wave takes the short form when all of its lanes may; a NaN, an infinity
  // or a large |x| anywhere in the wave sends it through the full form.
  if (__builtin_amdgcn_ballot_w64(!sigmoidf_short_ok(x)) == 0) return sigmoidf_short(x, tab);
#endif
  return sigmoidf_any(x, tab);
}
#if !defined(__HIPCC__)
SHDW_LIBM_FN float exact_expf(float x) { return exact_expf(x, kExp2fTab); }
SHDW_LIBM_FN float exact_sigmoidf(float x) { return exact_sigmoidf(x, kExp2fTab); }
SHDW_LIBM_FN float exact_tanhf(float x) { return exact_tanhf(x, kTanhStepTab); }
#endif


// ===========================================================================
// logf: glibc sysdeps/ieee754/flt-32/e_logf.c (ARM optimized routines), FMA
// multiarch variant: every a*b+c below is one fused operation.
// ===========================================================================
struct LogfEntry {
  double invc, logc;
};
SHDW_LIBM_TABLE LogfEntry kLogfTab[16] = {
    {0x1.661ec79f8f3bep+0, -0x1.57bf7808caadep-2}, {0x1.571ed4aaf883dp+0, -0x1.2bef0a7c06ddbp-2},
    {0x1.49539f0f010bp+0, -0x1.01eae7f513a67p-2},  {0x1.3c995b0b80385p+0, -0x1.b31d8a68224e9p-3},
    {0x1.30d190c8864a5p+0, -0x1.6574f0ac07758p-3}, {0x1.25e227b0b8eap+0, -0x1.1aa2bc79c81p-3},
    {0x1.1bb4a4a1a343fp+0, -0x1.a4e76ce8c0e5ep-4}, {0x1.12358f08ae5bap+0, -0x1.1973c5a611cccp-4},
    {0x1.0953f419900a7p+0, -0x1.252f438e10c1ep-5}, {0x1p+0, 0x0p+0},
    {0x1.e608cfd9a47acp-1, 0x1.aa5aa5df25984p-5},  {0x1.ca4b31f026aap-1, 0x1.c5e53aa362eb4p-4},
    {0x1.b2036576afce6p-1, 0x1.526e57720db08p-3},  {0x1.9c2d163a1aa2dp-1, 0x1.bc2860d22477p-3},
    {0x1.886e6037841edp-1, 0x1.1058bc8a07ee1p-2},  {0x1.767dcf5534862p-1, 0x1.4043057b6ee09p-2}};

SHDW_LIBM_FN float exact_logf(float x) {
  const double Ln2 = 0x1.62e42fefa39efp-1;
  const double A0 = -0x1.00ea348b88334p-2, A1 = 0x1.5575b0be00b6ap-2, A2 = -0x1.ffffef20a4123p-2;
  uint32_t ix = f2u(x);
  if (ix == 0x3f800000u) return 0.0f;
  if (ix - 0x00800000u >= 0x7f800000u - 0x00800000u) {
    // x < 0x1p-126, inf or NaN
    if (ix * 2 == 0) return -__builtin_inff();
    if (ix == 0x7f800000u) return x;
    if ((ix & 0x80000000u) || ix * 2 >= 0xff000000u) return __builtin_nanf("");
    ix = f2u(x * 0x1p23f);  // subnormal: normalise
    ix -= 23u << 23;
  }
  const uint32_t tmp = ix - 0x3f330000u;
  const int i = (tmp >> 19) & 15;
  const int k = static_cast<int32_t>(tmp) >> 23;
  const uint32_t iz = ix - (tmp & (0x1ffu << 23));
  const double invc = kLogfTab[i].invc, logc = kLogfTab[i].logc;
  const double z = static_cast<double>(u2f(iz));
  const double r = __builtin_fma(z, invc, -1.0);
  const double y0 = __builtin_fma(static_cast<double>(k), Ln2, logc);
  const double r2 = r * r;
  double y = __builtin_fma(A1, r, A2);
  y = __builtin_fma(A0, r2, y);
  y = __builtin_fma(y, r2, y0 + r);
  return static_cast<float>(y);
}

// ===========================================================================
// sinf / cosf: glibc sysdeps/ieee754/flt-32/s_sinf.c, s_cosf.c, sincosf.h (ARM
// optimized routines), FMA multiarch variant.
// ===========================================================================
// 2/pi in 32-bit windows that slide by 8 bits
SHDW_LIBM_TABLE uint32_t kInvPio4[24] = {
    0xa2,       0xa2f9,     0xa2f983,   0xa2f9836e, 0xf9836e4e, 0x836e4e44, 0x6e4e4415, 0x4e441529,
    0x441529fc, 0x1529fc27, 0x29fc2757, 0xfc2757d1, 0x2757d1f5, 0x57d1f534, 0xd1f534dd, 0xf534ddc0,
    0x34ddc0db, 0xddc0db62, 0xc0db6295, 0xdb629599, 0x6295993c, 0x95993c43, 0x993c4390, 0x3c439041};

// Polynomial of sincosf.h: n even -> sine of x, n odd -> cosine; `flip` negates
// the cosine coefficients (the library's second coefficient table).
SHDW_LIBM_FN float sincosf_poly(double x, double x2, bool flip, int n) {
  const double S1 = -0x1.555545995a603p-3, S2 = 0x1.1107605230bc4p-7, S3 = -0x1.994eb3774cf24p-13;
  const double sg = flip ? -1.0 : 1.0;
  const double C0 = sg * 0x1p0, C1 = sg * -0x1.ffffffd0c621cp-2, C2 = sg * 0x1.55553e1068f19p-5,
               C3 = sg * -0x1.6c087e89a359dp-10, C4 = sg * 0x1.99343027bf8c3p-16;
  if ((n & 1) == 0) {
    const double x3 = x * x2;
    const double s1 = __builtin_fma(x2, S3, S2);
    const double x7 = x3 * x2;
    const double s = __builtin_fma(x3, S1, x);
    return static_cast<float>(__builtin_fma(x7, s1, s));
  }
  const double x4 = x2 * x2;
  const double c2 = __builtin_fma(x2, C4, C3);
  const double c1 = __builtin_fma(x2, C2, C1);
  const double x6 = x4 * x2;
  const double c = __builtin_fma(x2, c1, C0);
  return static_cast<float>(__builtin_fma(x6, c2, c));
}

SHDW_LIBM_FN double sincosf_reduce_fast(double x, int* np) {
  const double hpi_inv = 0x1.45F306DC9C883p+23, hpi = 0x1.921FB54442D18p0;
  const double r = x * hpi_inv;
  const int n = (static_cast<int32_t>(r) + 0x800000) >> 24;
  *np = n;
  return __builtin_fma(-static_cast<double>(n), hpi, x);
}

SHDW_LIBM_FN double sincosf_reduce_large(uint32_t xi, int* np) {
  const uint32_t* arr = &kInvPio4[(xi >> 26) & 15];
  const int shift = (xi >> 23) & 7;
  xi = (xi & 0xffffff) | 0x800000;
  xi <<= shift;
  uint64_t res0 = static_cast<uint32_t>(xi * arr[0]);
  const uint64_t res1 = static_cast<uint64_t>(xi) * arr[4];
  const uint64_t res2 = static_cast<uint64_t>(xi) * arr[8];
  res0 = (res2 >> 32) | (res0 << 32);
  res0 += res1;
  const uint64_t n = (res0 + (1ULL << 61)) >> 62;
  res0 -= n << 62;
  const double x = static_cast<double>(static_cast<int64_t>(res0));
  *np = static_cast<int>(n);
  return x * 0x1.921FB54442D18p-62;
}

// which = 0: sinf, 1: cosf
SHDW_LIBM_FN float exact_sincosf(float y, int which) {
  const uint32_t top = (f2u(y) >> 20) & 0x7ff;
  double x = static_cast<double>(y);
  int n;
  if (top < 0x3f4) {  // |y| < pi/4
    const double x2 = x * x;
    if (top < 0x398) return which ? 1.0f : y;  // |y| < 2^-12
    return sincosf_poly(x, x2, false, which);
  }
  if (top < 0x42f) {  // |y| < 120
    x = sincosf_reduce_fast(x, &n);
    const double s = ((n & 3) == 1 || (n & 3) == 2) ? -1.0 : 1.0;
    return sincosf_poly(x * s, x * x, (n & 2) != 0, n ^ which);
  }
  if (top < 0x7f8) {
    const uint32_t xi = f2u(y);
    const int sign = xi >> 31;
    x = sincosf_reduce_large(xi, &n);
    const int q = (n + sign) & 3;
    const double s = (q == 1 || q == 2) ? -1.0 : 1.0;
    return sincosf_poly(x * s, x * x, (q & 2) != 0, n ^ which);
  }
  return __builtin_nanf("");
}
SHDW_LIBM_FN float exact_sinf(float y) { return exact_sincosf(y, 0); }
SHDW_LIBM_FN float exact_cosf(float y) { return exact_sincosf(y, 1); }


// ===========================================================================
// atanf / asinf / acosf: glibc sysdeps/ieee754/flt-32/{s_atanf,e_asinf,e_acosf}.c
// (fdlibm lineage, all-fp32, no fused operations on x86-64).
// ===========================================================================
SHDW_LIBM_FN float exact_atanf(float x) {
  // The library's decimal literals; they, not the hex values in its comments,
  // are what gets compiled (aT[0] is 0x3eaaaaab, its comment says ...aa).
  const float atanhi[4] = {4.6364760399e-01f, 7.8539812565e-01f, 9.8279368877e-01f,
                           1.5707962513e+00f};
  const float atanlo[4] = {5.0121582440e-09f, 3.7748947079e-08f, 3.4473217170e-08f,
                           7.5497894159e-08f};
  const float aT0 = 3.3333334327e-01f, aT1 = -2.0000000298e-01f, aT2 = 1.4285714924e-01f,
              aT3 = -1.1111110449e-01f, aT4 = 9.0908870101e-02f, aT5 = -7.6918758452e-02f,
              aT6 = 6.6610731184e-02f, aT7 = -5.8335702866e-02f, aT8 = 4.9768779427e-02f,
              aT9 = -3.6531571299e-02f, aT10 = 1.6285819933e-02f;
  const float one = 1.0f;
  const uint32_t hx = f2u(x);
  const uint32_t ix = hx & 0x7fffffffu;
  const bool neg = (hx >> 31) != 0;
  int id;
  if (ix >= 0x4c000000u) {  // |x| >= 2^25
    if (ix > 0x7f800000u) return x + x;
    return neg ? -atanhi[3] - atanlo[3] : atanhi[3] + atanlo[3];
  }
  if (ix < 0x3ee00000u) {  // |x| < 0.4375
    if (ix < 0x31000000u) return x;  // |x| < 2^-29
    id = -1;
  } else {
    x = u2f(ix);
    if (ix < 0x3f980000u) {    // |x| < 1.1875
      if (ix < 0x3f300000u) {  // 7/16 <= |x| < 11/16
        id = 0;
        x = (2.0f * x - one) / (2.0f + x);
      } else {
        id = 1;
        x = (x - one) / (x + one);
      }
    } else if (ix < 0x401c0000u) {  // |x| < 2.4375
      id = 2;
      x = (x - 1.5f) / (one + 1.5f * x);
    } else {
      id = 3;
      x = -1.0f / x;
    }
  }
  const float z = x * x;
  const float w = z * z;
  const float s1 = z * (aT0 + w * (aT2 + w * (aT4 + w * (aT6 + w * (aT8 + w * aT10)))));
  const float s2 = w * (aT1 + w * (aT3 + w * (aT5 + w * (aT7 + w * aT9))));
  if (id < 0) return x - x * (s1 + s2);
  const float r = atanhi[id] - ((x * (s1 + s2) - atanlo[id]) - x);
  return neg ? -r : r;
}

SHDW_LIBM_FN float exact_asinf(float x) {
  const float one = 1.0f;
  const float pio2_hi = 1.57079637050628662109375f, pio2_lo = -4.37113900018624283e-8f,
              pio4_hi = 0.785398185253143310546875f;
  const float p0 = 1.666675248e-1f, p1 = 7.495297643e-2f, p2 = 4.547037598e-2f,
              p3 = 2.417951451e-2f, p4 = 4.216630880e-2f;
  const uint32_t hx = f2u(x);
  const uint32_t ix = hx & 0x7fffffffu;
  float t, w, p, q, c, r, s;
  if (ix == 0x3f800000u) return x * pio2_hi + x * pio2_lo;
  if (ix > 0x3f800000u) return (x - x) / (x - x);
  if (ix < 0x3f000000u) {            // |x| < 0.5
    if (ix < 0x32000000u) return x;  // |x| < 2^-27
    t = x * x;
    w = t * (p0 + t * (p1 + t * (p2 + t * (p3 + t * p4))));
    return x + x * w;
  }
  w = one - u2f(ix);
  t = w * 0.5f;
  p = t * (p0 + t * (p1 + t * (p2 + t * (p3 + t * p4))));
  s = __builtin_sqrtf(t);
  if (ix >= 0x3F79999Au) {  // |x| > 0.975
    t = pio2_hi - (2.0f * (s + s * p) - pio2_lo);
  } else {
    w = u2f(f2u(s) & 0xfffff000u);
    c = (t - w * w) / (s + w);
    r = p;
    p = 2.0f * s * r - (pio2_lo - 2.0f * c);
    q = pio4_hi - 2.0f * w;
    t = pio4_hi - (p - q);
  }
  return (hx >> 31) ? -t : t;
}

SHDW_LIBM_FN float exact_acosf(float x) {
  const float one = 1.0f;
  const float pi = u2f(0x40490fdau), pio2_hi = u2f(0x3fc90fdau), pio2_lo = u2f(0x33a22168u);
  const float pS0 = u2f(0x3e2aaaabu), pS1 = u2f(0xbea6b090u), pS2 = u2f(0x3e4e0aa8u),
              pS3 = u2f(0xbd241146u), pS4 = u2f(0x3a4f7f04u), pS5 = u2f(0x3811ef08u);
  const float qS1 = u2f(0xc019d139u), qS2 = u2f(0x4001572du), qS3 = u2f(0xbf303361u),
              qS4 = u2f(0x3d9dc62eu);
  const uint32_t hx = f2u(x);
  const uint32_t ix = hx & 0x7fffffffu;
  const bool neg = (hx >> 31) != 0;
  float z, p, q, r, w, s, c, df;
  if (ix == 0x3f800000u) return neg ? pi + 2.0f * pio2_lo : 0.0f;
  if (ix > 0x3f800000u) return (x - x) / (x - x);
  if (ix < 0x3f000000u) {  // |x| < 0.5
    if (ix <= 0x32800000u) return pio2_hi + pio2_lo;
    z = x * x;
    p = z * (pS0 + z * (pS1 + z * (pS2 + z * (pS3 + z * (pS4 + z * pS5)))));
    q = one + z * (qS1 + z * (qS2 + z * (qS3 + z * qS4)));
    r = p / q;
    return pio2_hi - (x - (pio2_lo - x * r));
  }
  if (neg) {  // x < -0.5
    z = (one + x) * 0.5f;
    p = z * (pS0 + z * (pS1 + z * (pS2 + z * (pS3 + z * (pS4 + z * pS5)))));
    q = one + z * (qS1 + z * (qS2 + z * (qS3 + z * qS4)));
    s = __builtin_sqrtf(z);
    r = p / q;
    w = r * s - pio2_lo;
    return pi - 2.0f * (s + w);
  }
  z = (one - x) * 0.5f;  // x > 0.5
  s = __builtin_sqrtf(z);
  df = u2f(f2u(s) & 0xfffff000u);
  c = (z - df * df) / (s + df);
  p = z * (pS0 + z * (pS1 + z * (pS2 + z * (pS3 + z * (pS4 + z * pS5)))));
  q = one + z * (qS1 + z * (qS2 + z * (qS3 + z * qS4)));
  r = p / q;
  w = r * s + c;
  return 2.0f * (df + w);
}


// ===========================================================================
// log1pf: glibc sysdeps/ieee754/flt-32/s_log1pf.c (fdlibm), used by SoftPlus.
// ===========================================================================
SHDW_LIBM_FN float exact_log1pf(float x) {
  const float ln2_hi = 6.9313812256e-01f, ln2_lo = 9.0580006145e-06f, two25 = 3.355443200e+07f;
  const float Lp1 = 6.6666668653e-01f, Lp2 = 4.0000000596e-01f, Lp3 = 2.8571429849e-01f,
              Lp4 = 2.2222198546e-01f, Lp5 = 1.8183572590e-01f, Lp6 = 1.5313838422e-01f,
              Lp7 = 1.4798198640e-01f;
  const float zero = 0.0f;
  float hfsq, f = 0.0f, c = 0.0f, s, z, R, u;
  const int32_t hx = static_cast<int32_t>(f2u(x));
  const int32_t ax = hx & 0x7fffffff;
  int32_t k = 1, hu = 0;
  if (hx < 0x3ed413d7) {      // x < 0.41422
    if (ax >= 0x3f800000) {   // x <= -1
      if (x == -1.0f) return -two25 / zero;
      return (x - x) / (x - x);
    }
    if (ax < 0x31000000) {    // |x| < 2^-29
      if (ax < 0x24800000) return x;
      return x - x * x * 0.5f;
    }
    if (hx > 0 || hx <= static_cast<int32_t>(0xbe95f61fu)) {  // -0.2929 < x < 0.41422
      k = 0;
      f = x;
      hu = 1;
    }
  }
  if (hx >= 0x7f800000) return x + x;
  if (k != 0) {
    if (hx < 0x5a000000) {
      u = 1.0f + x;
      hu = static_cast<int32_t>(f2u(u));
      k = (hu >> 23) - 127;
      c = (k > 0) ? 1.0f - (u - x) : x - (u - 1.0f);
      c /= u;
    } else {
      u = x;
      hu = static_cast<int32_t>(f2u(u));
      k = (hu >> 23) - 127;
      c = 0;
    }
    hu &= 0x007fffff;
    if (hu < 0x3504f7) {
      u = u2f(static_cast<uint32_t>(hu) | 0x3f800000u);
    } else {
      k += 1;
      u = u2f(static_cast<uint32_t>(hu) | 0x3f000000u);
      hu = (0x00800000 - hu) >> 2;
    }
    f = u - 1.0f;
  }
  hfsq = 0.5f * f * f;
  const float fk = static_cast<float>(k);
  if (hu == 0) {  // |f| < 2^-20
    if (f == zero) {
      if (k == 0) return zero;
      c += fk * ln2_lo;
      return fk * ln2_hi + c;
    }
    R = hfsq * (1.0f - 0.66666666666666666f * f);
    if (k == 0) return f - R;
    return fk * ln2_hi - ((R - (fk * ln2_lo + c)) - f);
  }
  s = f / (2.0f + f);
  z = s * s;
  R = z * (Lp1 + z * (Lp2 + z * (Lp3 + z * (Lp4 + z * (Lp5 + z * (Lp6 + z * Lp7))))));
  if (k == 0) return f - (hfsq - s * (hfsq + R));
  return fk * ln2_hi - ((hfsq - (s * (hfsq + R) + (fk * ln2_lo + c))) - f);
}

SHDW_LIBM_FN float exact_softplusf(float x, const uint64_t* tab) {
  return exact_log1pf(exact_expf(x, tab));
}

// ===========================================================================
// erff: glibc sysdeps/ieee754/flt-32/s_erff.c (fdlibm), used by Gelu.  The
// coefficients are fdlibm's double-precision ones rounded to fp32.
// ===========================================================================
SHDW_LIBM_FN float exact_erff(float x, const uint64_t* tab) {
  const float tiny = 1e-30f, one = 1.0f;
  const float erx = 8.45062911510467529297e-01f, efx = 1.28379167095512586316e-01f;
  const float pp0 = 1.28379167095512558561e-01f, pp1 = -3.25042107247001499370e-01f,
              pp2 = -2.84817495755985104766e-02f, pp3 = -5.77027029648944159157e-03f,
              pp4 = -2.37630166566501626084e-05f;
  const float qq1 = 3.97917223959155352819e-01f, qq2 = 6.50222499887672944485e-02f,
              qq3 = 5.08130628187576562776e-03f, qq4 = 1.32494738004321644526e-04f,
              qq5 = -3.96022827877536812320e-06f;
  const float pa0 = -2.36211856075265944077e-03f, pa1 = 4.14856118683748331666e-01f,
              pa2 = -3.72207876035701323847e-01f, pa3 = 3.18346619901161753674e-01f,
              pa4 = -1.10894694282396677476e-01f, pa5 = 3.54783043256182359371e-02f,
              pa6 = -2.16637559486879084300e-03f;
  const float qa1 = 1.06420880400844228286e-01f, qa2 = 5.40397917702171048937e-01f,
              qa3 = 7.18286544141962662868e-02f, qa4 = 1.26171219808761642112e-01f,
              qa5 = 1.36370839120290507362e-02f, qa6 = 1.19844998467991074170e-02f;
  const float ra0 = -9.86494403484714822705e-03f, ra1 = -6.93858572707181764372e-01f,
              ra2 = -1.05586262253232909814e+01f, ra3 = -6.23753324503260060396e+01f,
              ra4 = -1.62396669462573470355e+02f, ra5 = -1.84605092906711035994e+02f,
              ra6 = -8.12874355063065934246e+01f, ra7 = -9.81432934416914548592e+00f;
  const float sa1 = 1.96512716674392571292e+01f, sa2 = 1.37657754143519042600e+02f,
              sa3 = 4.34565877475229228821e+02f, sa4 = 6.45387271733267880336e+02f,
              sa5 = 4.29008140027567833386e+02f, sa6 = 1.08635005541779435134e+02f,
              sa7 = 6.57024977031928170135e+00f, sa8 = -6.04244152148580987438e-02f;
  const float rb0 = -9.86494292470009928597e-03f, rb1 = -7.99283237680523006574e-01f,
              rb2 = -1.77579549177547519889e+01f, rb3 = -1.60636384855821916062e+02f,
              rb4 = -6.37566443368389627722e+02f, rb5 = -1.02509513161107724954e+03f,
              rb6 = -4.83519191608651397019e+02f;
  const float sb1 = 3.03380607434824582924e+01f, sb2 = 3.25792512996573918826e+02f,
              sb3 = 1.53672958608443695994e+03f, sb4 = 3.19985821950859553908e+03f,
              sb5 = 2.55305040643316442583e+03f, sb6 = 4.74528541206955367215e+02f,
              sb7 = -2.24409524465858183362e+01f;
  const uint32_t hxu = f2u(x);
  const bool neg = (hxu >> 31) != 0;
  uint32_t ix = hxu & 0x7fffffffu;
  float R, S, P, Q, s, y, z, r;
  if (ix >= 0x7f800000u) {
    const int i = static_cast<int>(hxu >> 31) << 1;
    return static_cast<float>(1 - i) + one / x;
  }
  if (ix < 0x3f580000u) {    // |x| < 0.84375
    if (ix < 0x31800000u) {  // |x| < 2^-28
      if (ix < 0x04000000u) return 0.0625f * (16.0f * x + (16.0f * efx) * x);
      return x + efx * x;
    }
    z = x * x;
    r = pp0 + z * (pp1 + z * (pp2 + z * (pp3 + z * pp4)));
    s = one + z * (qq1 + z * (qq2 + z * (qq3 + z * (qq4 + z * qq5))));
    y = r / s;
    return x + x * y;
  }
  if (ix < 0x3fa00000u) {  // 0.84375 <= |x| < 1.25
    s = u2f(ix) - one;
    P = pa0 + s * (pa1 + s * (pa2 + s * (pa3 + s * (pa4 + s * (pa5 + s * pa6)))));
    Q = one + s * (qa1 + s * (qa2 + s * (qa3 + s * (qa4 + s * (qa5 + s * qa6)))));
    return neg ? -erx - P / Q : erx + P / Q;
  }
  if (ix >= 0x40c00000u) return neg ? tiny - one : one - tiny;  // |x| >= 6
  x = u2f(ix);
  s = one / (x * x);
  if (ix < 0x4036DB6Eu) {  // |x| < 1/0.35
    R = ra0 + s * (ra1 + s * (ra2 + s * (ra3 + s * (ra4 + s * (ra5 + s * (ra6 + s * ra7))))));
    S = one + s * (sa1 + s * (sa2 + s * (sa3 + s * (sa4 + s * (sa5 + s * (sa6 + s * (sa7 + s * sa8)))))));
  } else {
    R = rb0 + s * (rb1 + s * (rb2 + s * (rb3 + s * (rb4 + s * (rb5 + s * rb6)))));
    S = one + s * (sb1 + s * (sb2 + s * (sb3 + s * (sb4 + s * (sb5 + s * (sb6 + s * sb7))))));
  }
  z = u2f(ix & 0xfffff000u);
  r = exact_expf(-z * z - 0.5625f, tab) * exact_expf((z - x) * (z + x) + R / S, tab);
  return neg ? r / x - one : one - r / x;
}

// 0.5f * x * (1 + erff(0.707107f * x)), shadow/operators/kernels/activate.cpp:26
SHDW_LIBM_FN float exact_geluf(float x, const uint64_t* tab) {
  return 0.5f * x * (1 + exact_erff(0.707107f * x, tab));
}

// ===========================================================================
// powf: glibc sysdeps/ieee754/flt-32/e_powf.c (ARM optimized routines), FMA
// multiarch variant.
// ===========================================================================
struct PowfLog2Entry {
  double invc, logc;
};
SHDW_LIBM_TABLE PowfLog2Entry kPowfLog2Tab[16] = {
    {0x1.661ec79f8f3bep+0, -0x1.efec65b963019p-2}, {0x1.571ed4aaf883dp+0, -0x1.b0b6832d4fca4p-2},
    {0x1.49539f0f010bp+0, -0x1.7418b0a1fb77bp-2},  {0x1.3c995b0b80385p+0, -0x1.39de91a6dcf7bp-2},
    {0x1.30d190c8864a5p+0, -0x1.01d9bf3f2b631p-2}, {0x1.25e227b0b8eap+0, -0x1.97c1d1b3b7afp-3},
    {0x1.1bb4a4a1a343fp+0, -0x1.2f9e393af3c9fp-3}, {0x1.12358f08ae5bap+0, -0x1.960cbbf788d5cp-4},
    {0x1.0953f419900a7p+0, -0x1.a6f9db6475fcep-5}, {0x1p+0, 0x0p+0},
    {0x1.e608cfd9a47acp-1, 0x1.338ca9f24f53dp-4},  {0x1.ca4b31f026aap-1, 0x1.476a9543891bap-3},
    {0x1.b2036576afce6p-1, 0x1.e840b4ac4e4d2p-3},  {0x1.9c2d163a1aa2dp-1, 0x1.40645f0c6651cp-2},
    {0x1.886e6037841edp-1, 0x1.88e9c2c1b9ff8p-2},  {0x1.767dcf5534862p-1, 0x1.ce0a44eb17bccp-2}};

// 0: y is not an integer, 1: odd integer, 2: even integer
SHDW_LIBM_FN int powf_checkint(uint32_t iy) {
  const int e = iy >> 23 & 0xff;
  if (e < 0x7f) return 0;
  if (e > 0x7f + 23) return 2;
  if (iy & ((1u << (0x7f + 23 - e)) - 1)) return 0;
  if (iy & (1u << (0x7f + 23 - e))) return 1;
  return 2;
}
SHDW_LIBM_FN bool powf_zeroinfnan(uint32_t ix) { return 2 * ix - 1 >= 2u * 0x7f800000u - 1; }
SHDW_LIBM_FN bool powf_issignaling(uint32_t ix) { return 2 * (ix ^ 0x00400000u) > 2u * 0x7fc00000u; }

// Whether powf(x, y) takes the straight path below: x a positive normal number,
// y finite and not zero.
SHDW_LIBM_FN bool powf_is_ordinary(uint32_t ix, uint32_t iy) {
  return !(ix - 0x00800000u >= 0x7f800000u - 0x00800000u || powf_zeroinfnan(iy));
}

// x^y for the bits ix of a positive normal x and a finite y != 0 (the caller has
// scaled a subnormal x up and moved the sign of a negative base to an odd power
// into sign_bias).  No branches: results that overflow or underflow are put in
// place at the end, so several of these can run side by side in one lane; any
// other ix and y give some number and no fault.
// log_tab is kPowfLog2Tab or a copy of it in faster memory, as tab is of kExp2fTab.
SHDW_LIBM_FN float powf_ordinary(uint32_t ix, float y, uint32_t sign_bias, const uint64_t* tab,
                                 const PowfLog2Entry* log_tab) {
  // log2(x)
  const double A0 = 0x1.27616c9496e0bp-2, A1 = -0x1.71969a075c67ap-2, A2 = 0x1.ec70a6ca7baddp-2,
               A3 = -0x1.7154748bef6c8p-1, A4 = 0x1.71547652ab82bp0;
  const uint32_t tmp = ix - 0x3f330000u;
  const int i = (tmp >> 19) & 15;
  const uint32_t top = tmp & 0xff800000u;
  const uint32_t iz = ix - top;
  const int k = static_cast<int32_t>(top) >> 23;
  const double invc = log_tab[i].invc, logc = log_tab[i].logc;
  const double z = static_cast<double>(u2f(iz));
  const double r = __builtin_fma(z, invc, -1.0);
  const double y0 = logc + static_cast<double>(k);
  const double r2 = r * r;
  double yy = __builtin_fma(A0, r, A1);
  const double p = __builtin_fma(A2, r, A3);
  const double r4 = r2 * r2;
  double q = __builtin_fma(A4, r, y0);
  q = __builtin_fma(p, r2, q);
  const double logx = __builtin_fma(yy, r4, q);
  const double ylogx = static_cast<double>(y) * logx;
  // 2^(y log2 x)
  const double C0 = 0x1.c6af84b912394p-5, C1 = 0x1.ebfce50fac4f3p-3, C2 = 0x1.62e42ff0c52d6p-1;
  const double Shift = 0x1.8p+52 / 32;
  double kd = ylogx + Shift;
  const uint64_t ki = d2u(kd);
  kd -= Shift;
  const double rr = ylogx - kd;
  uint64_t t = tab[ki & 31];
  const uint64_t ski = ki + sign_bias;
  t += ski << 47;
  const double sc = u2d(t);
  const double zz = __builtin_fma(C0, rr, C1);
  const double rr2 = rr * rr;
  double res = __builtin_fma(C2, rr, 1.0);
  res = __builtin_fma(zz, rr2, res);
  res = res * sc;
  float out = static_cast<float>(res);
  // |y log2 x| >= 126: past the largest float, below half the smallest, or the smallest itself
  const bool far = (d2u(ylogx) >> 47 & 0xffff) >= (d2u(126.0) >> 47);
  const bool over = far && ylogx > 0x1.fffffffd1d571p+6;
  const bool under = far && !over && ylogx <= -150.0;
  const bool least = far && !over && !under && ylogx < -149.0;
  out = over ? (sign_bias ? -__builtin_inff() : __builtin_inff()) : out;
  out = under ? (sign_bias ? -0.0f : 0.0f) : out;
  out = least ? (sign_bias ? -0x1p-149f : 0x1p-149f) : out;
  return out;
}

SHDW_LIBM_FN float powf_ordinary(uint32_t ix, float y, uint32_t sign_bias, const uint64_t* tab) {
  return powf_ordinary(ix, y, sign_bias, tab, kPowfLog2Tab);
}

SHDW_LIBM_FN float exact_powf(float x, float y, const uint64_t* tab) {
  const uint32_t kSignBias = 1u << (5 + 11);
  uint32_t sign_bias = 0;
  uint32_t ix = f2u(x);
  const uint32_t iy = f2u(y);
  if (!powf_is_ordinary(ix, iy)) {
    if (powf_zeroinfnan(iy)) {
      if (2 * iy == 0) return powf_issignaling(ix) ? x + y : 1.0f;
      if (ix == 0x3f800000u) return powf_issignaling(iy) ? x + y : 1.0f;
      if (2 * ix > 2u * 0x7f800000u || 2 * iy > 2u * 0x7f800000u) return x + y;
      if (2 * ix == 2 * 0x3f800000u) return 1.0f;
      if ((2 * ix < 2 * 0x3f800000u) == !(iy & 0x80000000u)) return 0.0f;
      return y * y;
    }
    if (powf_zeroinfnan(ix)) {
      float x2 = x * x;
      if ((ix & 0x80000000u) && powf_checkint(iy) == 1) {
        x2 = -x2;
        sign_bias = 1;
      }
      if (2 * ix == 0 && (iy & 0x80000000u)) return sign_bias ? -__builtin_inff() : __builtin_inff();
      return (iy & 0x80000000u) ? 1 / x2 : x2;
    }
    if (ix & 0x80000000u) {  // finite x < 0
      const int yint = powf_checkint(iy);
      if (yint == 0) return __builtin_nanf("");
      if (yint == 1) sign_bias = kSignBias;
      ix &= 0x7fffffffu;
    }
    if (ix < 0x00800000u) {  // subnormal x
      ix = f2u(x * 0x1p23f);
      ix &= 0x7fffffffu;
      ix -= 23u << 23;
    }
  }
  return powf_ordinary(ix, y, sign_bias, tab);
}
#if !defined(__HIPCC__)
SHDW_LIBM_FN float exact_softplusf(float x) { return exact_softplusf(x, kExp2fTab); }
SHDW_LIBM_FN float exact_erff(float x) { return exact_erff(x, kExp2fTab); }
SHDW_LIBM_FN float exact_geluf(float x) { return exact_geluf(x, kExp2fTab); }
SHDW_LIBM_FN float exact_powf(float x, float y) { return exact_powf(x, y, kExp2fTab); }
#endif


// ===========================================================================
// tanf: glibc sysdeps/ieee754/flt-32/{s_tanf,k_tanf,e_rem_pio2f}.c (fdlibm
// kernel in fp32 on top of the fp64 sincosf argument reduction).
// ===========================================================================
SHDW_LIBM_FN float kernel_tanf(float x, float y, int iy) {
  const float one = 1.0f, pio4 = 7.8539812565e-01f, pio4lo = 3.7748947079e-08f;
  const float T0 = 3.3333334327e-01f, T1 = 1.3333334029e-01f, T2 = 5.3968254477e-02f,
              T3 = 2.1869488060e-02f, T4 = 8.8632395491e-03f, T5 = 3.5920790397e-03f,
              T6 = 1.4562094584e-03f, T7 = 5.8804126456e-04f, T8 = 2.4646313977e-04f,
              T9 = 7.8179444245e-05f, T10 = 7.1407252108e-05f, T11 = -1.8558637748e-05f,
              T12 = 2.5907305826e-05f;
  float z, r, v, w, s;
  const int32_t hx = static_cast<int32_t>(f2u(x));
  const int32_t ix = hx & 0x7fffffff;
  if (ix < 0x39000000) {  // |x| < 2^-13
    if (static_cast<int>(x) == 0) {
      if ((ix | (iy + 1)) == 0) return one / __builtin_fabsf(x);
      if (iy == 1) return x;
      return -one / x;
    }
  }
  if (ix >= 0x3f2ca140) {  // |x| >= 0.6744
    if (hx < 0) {
      x = -x;
      y = -y;
    }
    z = pio4 - x;
    w = pio4lo - y;
    x = z + w;
    y = 0.0f;
    if (__builtin_fabsf(x) < 0x1p-13f)
      return static_cast<float>((1 - ((hx >> 30) & 2)) * iy) * (1.0f - static_cast<float>(2 * iy) * x);
  }
  z = x * x;
  w = z * z;
  r = T1 + w * (T3 + w * (T5 + w * (T7 + w * (T9 + w * T11))));
  v = z * (T2 + w * (T4 + w * (T6 + w * (T8 + w * (T10 + w * T12)))));
  s = z * x;
  r = y + z * (s * (r + v) + y);
  r += T0 * s;
  w = x + r;
  if (ix >= 0x3f2ca140) {
    v = static_cast<float>(iy);
    return static_cast<float>(1 - ((hx >> 30) & 2)) * (v - 2.0f * (x - (w * w / (w + v) - r)));
  }
  if (iy == 1) return w;
  // -1/(x+r), accurately
  float a, t;
  z = u2f(f2u(w) & 0xfffff000u);
  v = r - (z - x);
  t = a = -1.0f / w;
  t = u2f(f2u(t) & 0xfffff000u);
  s = 1.0f + t * z;
  return t + a * (s + t * v);
}

// s_tanf.c with e_rem_pio2f.c as glibc >= 2.28 has it: the reduction is the
// sincosf one (reduce_fast below 120, 64-bit fixed point above) evaluated in
// fp64 and split into the fp32 pair y0 = fp32(r), y1 = fp32(r - y0).  tanf has no
// FMA multiarch variant, so here x - n*hpi is a rounded product and a rounded
// difference.
SHDW_LIBM_FN float exact_tanf(float x) {
  const uint32_t ux = f2u(x);
  const uint32_t ix = ux & 0x7fffffffu;
  if (ix <= 0x3f490fdau) return kernel_tanf(x, 0.0f, 1);
  if (ix >= 0x7f800000u) return x - x;
  double r;
  int n;
  if (((ux >> 20) & 0x7ff) < 0x42f) {  // |x| < 120
    const double hpi_inv = 0x1.45F306DC9C883p+23, hpi = 0x1.921FB54442D18p0;
    const double xd = static_cast<double>(x);
    const double q = xd * hpi_inv;
    n = (static_cast<int32_t>(q) + 0x800000) >> 24;
    const double prod = static_cast<double>(n) * hpi;
    r = xd - prod;
  } else {
    r = sincosf_reduce_large(ux, &n);
    if (ux >> 31) r = -r;
  }
  const float y0 = static_cast<float>(r);
  const float y1 = static_cast<float>(r - static_cast<double>(y0));
  return kernel_tanf(y0, y1, 1 - ((n & 1) << 1));
}

}  // namespace libm
}  // namespace shdw

#endif  // SHADOW_AMD_CSRC_LIBM_EXACT_H_
