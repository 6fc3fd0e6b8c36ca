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

}  // extern "C"
