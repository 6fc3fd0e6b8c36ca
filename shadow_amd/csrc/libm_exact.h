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

namespace shdw {
namespace libm {

SHDW_LIBM_FN uint32_t f2u(float f) { return __builtin_bit_cast(uint32_t, f); }
SHDW_LIBM_FN float u2f(uint32_t u) { return __builtin_bit_cast(float, u); }
SHDW_LIBM_FN uint64_t d2u(double d) { return __builtin_bit_cast(uint64_t, d); }
SHDW_LIBM_FN double u2d(uint64_t u) { return __builtin_bit_cast(double, u); }

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
SHDW_LIBM_FN float exact_expf(float x, const uint64_t* tab) {
  // Main path, evaluated for every input (its result is discarded for the
  // out-of-range inputs handled below; nothing in it can trap).
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
  float res = static_cast<float>(y);

  const uint32_t ux = f2u(x);
  const uint32_t abstop = (ux >> 20) & 0x7ff;
  if (abstop >= 0x42b) {  // |x| >= 88 or x is NaN: rare, one skipped block
    if (x > 0x1.62e42ep6f) res = __builtin_inff();        // overflow
    if (x < -0x1.9d1d9ep6f) res = 0x1p-149f;              // smallest subnormal
    if (x < -0x1.9fe368p6f) res = 0.0f;                   // underflow to zero (also -inf)
    if (abstop >= 0x7f8 && ux != 0xff800000u) res = x + x;  // +inf, NaN
  }
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
// a = 2|x| in [2, 44) or a = -2|x| in (-2, -2^-54], so only these expm1f cases
// can occur: the 2^-25 early return, k = 0, k = -1, k <= -2 (a < 0) and
// 3 <= k <= 63 (a > 0).  Every case is evaluated with the same operations in the
// same order as the library and the applicable one is selected.
SHDW_LIBM_FN float exact_tanhf(float x) {
  const float one = 1.0f, two = 2.0f;
  const float ln2_hi = 6.9313812256e-01f, ln2_lo = 9.0580006145e-06f;
  const float invln2 = 1.4426950216e+00f;
  const float Q1 = -3.3333335072e-02f, Q2 = 1.5873016091e-03f, Q3 = -7.9365076090e-05f,
              Q4 = 4.0082177293e-06f, Q5 = -2.0109921195e-07f;
  const uint32_t jx = f2u(x);
  const uint32_t ix = jx & 0x7fffffffu;
  const bool big = ix >= 0x3f800000u;  // |x| >= 1: expm1f(+2|x|), else expm1f(-2|x|)
  const float ax = u2f(ix);
  const float a = big ? two * ax : -two * ax;  // argument of expm1f
  const uint32_t ha = f2u(a) & 0x7fffffffu;
  const bool aneg = !big;

  // --- expm1f(a): argument reduction ---
  const bool reduce = ha > 0x3eb17218u;   // |a| > 0.5 ln2
  const bool unit_k = ha < 0x3F851592u;   // |a| < 1.5 ln2  ->  k = +-1
  const int32_t kgen = static_cast<int32_t>(invln2 * a + (aneg ? -0.5f : 0.5f));
  int32_t k = unit_k ? (aneg ? -1 : 1) : kgen;
  k = reduce ? k : 0;
  const float tk = static_cast<float>(k);
  // k = +-1 uses hi = a -+ ln2_hi, lo = +-ln2_lo, which is what t*ln2_hi and
  // t*ln2_lo give for t = +-1 (both products exact).
  const float hi = a - tk * ln2_hi;
  const float lo = tk * ln2_lo;
  const float xr = reduce ? hi - lo : a;
  const float c = reduce ? (hi - xr) - lo : 0.0f;

  // --- primary range ---
  const float hfx = 0.5f * xr;
  const float hxs = xr * hfx;
  const float r1 = one + hxs * (Q1 + hxs * (Q2 + hxs * (Q3 + hxs * (Q4 + hxs * Q5))));
  const float t3 = 3.0f - r1 * hfx;
  float e = hxs * ((r1 - t3) / (6.0f - xr * t3));
  const float res_k0 = xr - (xr * e - hxs);
  e = (xr * (e - c) - c);
  e -= hxs;
  const float res_km1 = 0.5f * (xr - e) - 0.5f;
  // k <= -2 or k > 56: y = 1 - (e - x); 2 <= k < 23: y = (1 - 2^-k) - (e - x)
  const bool mid = (k >= 2) && (k < 23);
  const uint32_t ksh = static_cast<uint32_t>(k) & 31u;
  const float t_lo = mid ? u2f(0x3f800000u - (0x1000000u >> ksh)) : one;
  const float y_a = t_lo - (e - xr);
  // 23 <= k <= 56: y = (x - (e + 2^-k)) + 1
  const float t_hi = u2f(static_cast<uint32_t>(0x7f - k) << 23);
  float y_b = xr - (e + t_hi);
  y_b += one;
  const bool hi_k = (k >= 23) && (k <= 56);
  float yk = hi_k ? y_b : y_a;
  yk = u2f(f2u(yk) + (static_cast<uint32_t>(k) << 23));  // scale by 2^k
  const float res_gen = (mid || hi_k) ? yk : yk - one;
  float t = (k == 0) ? res_k0 : ((k == -1) ? res_km1 : res_gen);
  t = (ha < 0x33000000u) ? a : t;  // |a| < 2^-25: expm1f returns a

  // --- tanhf ---
  const float q = (big ? two : t) / (t + two);
  float z = big ? one - q : -q;
  z = (ix < 0x41b00000u) ? z : one;           // |x| >= 22 (and +-inf): 1 - tiny == 1
  float res = (jx >> 31) ? -z : z;
  res = (ix < 0x24000000u) ? x * (one + x) : res;  // |x| < 2^-55, including +-0
  res = (ix > 0x7f800000u) ? x + x : res;          // NaN
  return res;
}

// 1 / (1 + exp(-x)) in fp32, the way shadow/operators/kernels/activate.cpp:16
// writes it.
SHDW_LIBM_FN float exact_sigmoidf(float x, const uint64_t* tab) {
  return 1.0f / (1.0f + exact_expf(-x, tab));
}
#if !defined(__HIPCC__)
SHDW_LIBM_FN float exact_expf(float x) { return exact_expf(x, kExp2fTab); }
SHDW_LIBM_FN float exact_sigmoidf(float x) { return exact_sigmoidf(x, kExp2fTab); }
#endif

}  // namespace libm
}  // namespace shdw

#endif  // SHADOW_AMD_CSRC_LIBM_EXACT_H_
