// Shared device-side helpers for the gfx950 kernels: 128-bit vector access,
// exact division by launch-time constants, wave64 reductions.
#ifndef SHADOW_AMD_CSRC_DEVICE_COMMON_H_
#define SHADOW_AMD_CSRC_DEVICE_COMMON_H_

#include <hip/hip_runtime.h>

#include <cstdint>

// Shadow's CPU kernels are compiled for baseline x86-64: a*b+c is always a
// rounded multiply followed by a rounded add.  Keep the device code the same.
#pragma clang fp contract(off)

namespace shdw {

typedef float v4f __attribute__((ext_vector_type(4)));
typedef uint32_t v4u __attribute__((ext_vector_type(4)));

constexpr int kWave = 64;
constexpr int kBlock = 256;  // 4 wave64 per workgroup
// Workgroup of the streaming kernels (one vector per lane, no LDS exchange, no
// barrier that matters): a single wave64.  A 256-lane workgroup is placed only
// when four wave slots of one CU are free at once; single waves fill the slots
// as they free up.  Measured on y = max(x, 0): 6.62 TB/s against 6.39 TB/s at
// 411 MB, 5.96 against 5.65 TB/s at 103 MB, 5.41 against 5.12 TB/s at 51 MB
// (128 lanes: no gain).
constexpr int kStream = 64;

#define SHDW_DEVICE __device__ __forceinline__

// 128-bit streaming accesses.  Every element of these kernels is touched once,
// so loads and stores carry the non-temporal hint and do not displace the
// small re-used operands (per-channel parameters, broadcast rows) from L2.
SHDW_DEVICE v4f load4_stream(const float* p) {
  return __builtin_nontemporal_load(reinterpret_cast<const v4f*>(p));
}
SHDW_DEVICE void store4_stream(float* p, v4f v) {
  __builtin_nontemporal_store(v, reinterpret_cast<v4f*>(p));
}
SHDW_DEVICE v4f load4(const float* p) { return *reinterpret_cast<const v4f*>(p); }

// The same for addresses that are only 4-byte aligned (Blas offsets, odd row
// lengths).  The hardware takes a 128-bit global access at any dword address
// and splits the ones that straddle a line; on aligned addresses it costs the
// same as the aligned form (61.7 us against 61.8 us for 411 MB), one dword off
// 73 us, where four 4-byte accesses per lane need 172 us.
typedef float v4f_unaligned __attribute__((ext_vector_type(4), aligned(4)));
SHDW_DEVICE v4f load4_stream_any(const float* p) {
  return __builtin_nontemporal_load(reinterpret_cast<const v4f_unaligned*>(p));
}
SHDW_DEVICE v4f load4_any(const float* p) { return *reinterpret_cast<const v4f_unaligned*>(p); }
SHDW_DEVICE void store4_stream_any(float* p, v4f v) {
  __builtin_nontemporal_store(v, reinterpret_cast<v4f_unaligned*>(p));
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
SHDW_DEVICE bool aligned16_device(const void* p) {
  return (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
}

// Workgroups are handed to the 8 XCDs (accelerator dies, each with its own L2)
// round-robin by blockIdx.x, so workgroups b and b + 1 never share an L2.  A
// kernel whose neighbouring work items touch the same cache lines (halo rows,
// rows that straddle a line) renumbers its workgroups with this map: XCD x then
// owns one contiguous range of work items and the shared lines are fetched from
// HBM once.  A bijection of [0, grid) for every grid size.
constexpr uint32_t kXcds = 8;
__host__ SHDW_DEVICE uint32_t xcd_contiguous(uint32_t block, uint32_t grid) {
  const uint32_t x = block % kXcds, slot = block / kXcds;
  const uint32_t q = grid / kXcds, r = grid % kXcds;
  return x * q + (x < r ? x : r) + slot;
}

// Between the two: XCD x gets runs of 2^log2_run consecutive work items (its
// workgroups b, b + 8, ... of one run), the runs of the eight XCDs interleaved.
// For kernels that stream and also write a few bytes per workgroup (a row's mean,
// a row's maximum): the workgroups whose small results share a cache line then
// complete that line in one L2, while the stream stays spread over all XCDs.  A
// bijection of [0, grid); the incomplete last span keeps its numbering.
__host__ SHDW_DEVICE uint32_t xcd_runs(uint32_t block, uint32_t grid, uint32_t log2_run) {
  const uint32_t span = kXcds << log2_run;
  if (block >= grid - grid % span) return block;
  const uint32_t turn = block / kXcds, xcd = block % kXcds;
  return (turn >> log2_run) * span + (xcd << log2_run) + (turn & ((1u << log2_run) - 1u));
}

// ---------------------------------------------------------------------------
// Division of a 31-bit unsigned value by a divisor fixed at launch time:
//   q = (mulhi(n, m) + n) >> s
// with s = ceil(log2 d), m = floor(2^32 (2^s - d) / d) + 1.  Exact for every
// n < 2^31 (the sum cannot wrap because mulhi(n, m) < 2^31).
// ---------------------------------------------------------------------------
struct FastDiv {
  uint32_t d = 1, m = 0, s = 0;
};

inline FastDiv make_fastdiv(uint32_t d) {
  FastDiv f;
  f.d = d;
  uint32_t s = 0;
  while ((1ull << s) < d) ++s;
  f.s = s;
  f.m = static_cast<uint32_t>(((1ull << 32) * ((1ull << s) - d)) / d + 1);
  return f;
}

SHDW_DEVICE uint32_t fd_div(uint32_t n, const FastDiv& f) {
  return (__umulhi(n, f.m) + n) >> f.s;
}
SHDW_DEVICE void fd_divmod(uint32_t n, const FastDiv& f, uint32_t& q, uint32_t& r) {
  q = fd_div(n, f);
  r = n - q * f.d;
}

// ---------------------------------------------------------------------------
// wave64 exchange.  Steps 1..8 stay inside a row of 16 lanes and use DPP
// (no LDS traffic); 16 and 32 cross rows and go through ds_bpermute.
// ---------------------------------------------------------------------------
template <int CTRL>
SHDW_DEVICE int dpp_i32(int v) {
  return __builtin_amdgcn_update_dpp(v, v, CTRL, 0xf, 0xf, false);
}
template <int CTRL>
SHDW_DEVICE float dpp_f32(float v) {
  return __int_as_float(dpp_i32<CTRL>(__float_as_int(v)));
}
template <int CTRL>
SHDW_DEVICE double dpp_f64(double v) {
  const long long b = __double_as_longlong(v);
  const int lo = dpp_i32<CTRL>(static_cast<int>(b));
  const int hi = dpp_i32<CTRL>(static_cast<int>(b >> 32));
  return __longlong_as_double((static_cast<long long>(hi) << 32) | static_cast<unsigned int>(lo));
}
template <int CTRL>
SHDW_DEVICE uint32_t dpp_u32(uint32_t v) {
  return static_cast<uint32_t>(dpp_i32<CTRL>(static_cast<int>(v)));
}

constexpr int kDppXor1 = 0xB1;        // quad_perm [1,0,3,2]
constexpr int kDppXor2 = 0x4E;        // quad_perm [2,3,0,1]
constexpr int kDppHalfMirror = 0x141;  // lane i <-> 7-i inside 8
constexpr int kDppMirror = 0x140;      // lane i <-> 15-i inside 16

}  // namespace shdw

#endif  // SHADOW_AMD_CSRC_DEVICE_COMMON_H_
