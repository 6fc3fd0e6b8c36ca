// Host build of the device math restatements (shadow_amd/csrc/libm_exact.h)
// compared bit-for-bit with the libm of the machine this runs on, over any
// arithmetic progression of the 2^32 float bit patterns.  NaN results are
// compared by NaN-ness only.  Loaded through ctypes by the tests.
#include <cmath>
#include <cstdint>
#include <cstring>
#include <thread>
#include <vector>
#include <atomic>

#include "../../shadow_amd/csrc/libm_exact.h"

namespace {

typedef float (*fn1)(float);

float ref_sigmoid(float x) { return 1 / (1 + std::exp(-x)); }
float ref_exp(float x) { return std::exp(x); }
float ref_tanh(float x) { return std::tanh(x); }
float ref_expm1(float x) { return std::expm1(x); }
float ref_log(float x) { return std::log(x); }
float ref_sin(float x) { return std::sin(x); }
float ref_cos(float x) { return std::cos(x); }
float ref_atan(float x) { return std::atan(x); }
float ref_asin(float x) { return std::asin(x); }
float ref_acos(float x) { return std::acos(x); }
float ref_log1p(float x) { return std::log1p(x); }
float ref_tan(float x) { return std::tan(x); }
float ref_erf(float x) { return std::erf(x); }
float ref_softplus(float x) { return std::log1p(std::exp(x)); }
float ref_gelu(float x) { return 0.5f * x * (1 + std::erf(0.707107f * x)); }

struct Pair {
  fn1 mine, ref;
};

Pair pick(int id) {
  using namespace shdw::libm;
  switch (id) {
    case 0: return {exact_expf, ref_exp};
    case 1: return {exact_tanhf, ref_tanh};
    case 2: return {exact_sigmoidf, ref_sigmoid};
    case 3: return {exact_expm1f, ref_expm1};
    case 4: return {exact_logf, ref_log};
    case 5: return {exact_sinf, ref_sin};
    case 6: return {exact_cosf, ref_cos};
    case 7: return {exact_atanf, ref_atan};
    case 8: return {exact_asinf, ref_asin};
    case 9: return {exact_acosf, ref_acos};
    case 10: return {exact_log1pf, ref_log1p};
    case 11: return {exact_erff, ref_erf};
    case 12: return {exact_softplusf, ref_softplus};
    case 13: return {exact_geluf, ref_gelu};
    case 14: return {exact_tanf, ref_tan};
    default: return {nullptr, nullptr};
  }
}

inline uint32_t bits(float f) {
  uint32_t u;
  std::memcpy(&u, &f, 4);
  return u;
}

}  // namespace

extern "C" {

// Evaluate one value with the restatement (for spot checks from Python).
float libm_exact_eval(int func, float x) {
  Pair p = pick(func);
  return p.mine ? p.mine(x) : NAN;
}

float libm_host_eval(int func, float x) {
  Pair p = pick(func);
  return p.ref ? p.ref(x) : NAN;
}

// Entry `index` of the tanh step table as eight floats; returns the bytes of an
// entry, or the number of entries for a negative index.
int libm_tanh_step(int index, float* out) {
  using namespace shdw::libm;
  if (index < 0 || index >= kTanhSteps) return kTanhSteps;
  std::memcpy(out, &kTanhStepTab[index], sizeof(TanhStep));
  return static_cast<int>(sizeof(TanhStep));
}

// Compare on patterns start, start+stride, ... (count of them), split over
// `threads` threads.  Returns the number of mismatches and stores up to
// max_report offending input patterns.
long long libm_sweep(int func, uint32_t start, uint64_t count, uint32_t stride, int threads,
                     uint32_t* report, int max_report) {
  Pair p = pick(func);
  if (!p.mine) return -1;
  if (threads < 1) threads = 1;
  std::atomic<long long> bad(0);
  std::atomic<int> nrep(0);
  std::vector<std::thread> pool;
  const uint64_t per = (count + threads - 1) / threads;
  for (int t = 0; t < threads; ++t) {
    const uint64_t lo = per * t, hi = std::min<uint64_t>(count, lo + per);
    if (lo >= hi) break;
    pool.emplace_back([=, &bad, &nrep]() {
      long long local = 0;
      for (uint64_t i = lo; i < hi; ++i) {
        const uint32_t u = static_cast<uint32_t>(start + i * stride);
        float x;
        std::memcpy(&x, &u, 4);
        const float a = p.mine(x), b = p.ref(x);
        const bool same = (a != a && b != b) || bits(a) == bits(b);
        if (!same) {
          ++local;
          const int slot = nrep.fetch_add(1);
          if (slot < max_report && report) report[slot] = u;
        }
      }
      bad += local;
    });
  }
  for (auto& th : pool) th.join();
  return bad.load();
}

// powf(x, y) for x on an arithmetic progression of bit patterns.  mode 0: y is
// the fixed pattern `ybits`; mode 1: y is drawn per x from a splitmix64 stream
// seeded with `ybits` (uniform over all bit patterns); mode 2: like 1 but y is
// scaled into [-40, 40] where results are mostly finite.
long long libm_sweep_pow(uint32_t start, uint64_t count, uint32_t stride, uint32_t ybits, int mode,
                         int threads, uint32_t* report, int max_report) {
  if (threads < 1) threads = 1;
  std::atomic<long long> bad(0);
  std::atomic<int> nrep(0);
  std::vector<std::thread> pool;
  const uint64_t per = (count + threads - 1) / threads;
  for (int t = 0; t < threads; ++t) {
    const uint64_t lo = per * t, hi = std::min<uint64_t>(count, lo + per);
    if (lo >= hi) break;
    pool.emplace_back([=, &bad, &nrep]() {
      long long local = 0;
      for (uint64_t i = lo; i < hi; ++i) {
        const uint32_t u = static_cast<uint32_t>(start + i * stride);
        float x, y;
        std::memcpy(&x, &u, 4);
        uint32_t yb = ybits;
        if (mode != 0) {
          uint64_t zz = (static_cast<uint64_t>(ybits) << 32 | u) + 0x9e3779b97f4a7c15ull;
          zz = (zz ^ (zz >> 30)) * 0xbf58476d1ce4e5b9ull;
          zz = (zz ^ (zz >> 27)) * 0x94d049bb133111ebull;
          zz ^= zz >> 31;
          yb = static_cast<uint32_t>(zz);
          if (mode == 2) {
            const float f = (static_cast<float>(yb >> 8) * 0x1p-24f - 0.5f) * 80.0f;
            std::memcpy(&yb, &f, 4);
          }
        }
        std::memcpy(&y, &yb, 4);
        const float a = shdw::libm::exact_powf(x, y), b = std::pow(x, y);
        const bool same = (a != a && b != b) || bits(a) == bits(b);
        if (!same) {
          ++local;
          const int slot = nrep.fetch_add(2);
          if (slot + 1 < max_report && report) report[slot] = u, report[slot + 1] = yb;
        }
      }
      bad += local;
    });
  }
  for (auto& th : pool) th.join();
  return bad.load();
}

}  // extern "C"
