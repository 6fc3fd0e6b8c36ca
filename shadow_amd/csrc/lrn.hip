// LRN across channels (shadow/operators/kernels/lrn.cpp:9-60, lrn.cu).
//
// The reference walks the channels of one (batch, h, w) position with a running
// fp32 sum of squares -- the entering square is added, then the one that leaves
// the window is subtracted -- writes scale = k + sum * (alpha / size) into a
// scratch blob, and multiplies x by powf(scale, -beta) in a second pass.  The
// order of the additions and subtractions fixes the bits, so the walk stays: one
// lane per position, channel after channel.  What goes is the scratch blob and
// the second pass: the window's values wait in registers (windows of up to seven
// channels) or in LDS (a column of `size` floats per lane, no two lanes share a
// bank row), the centre of the window is multiplied as soon as its scale is
// known, x is read once and y written once.  Neighbouring lanes hold neighbouring
// positions, so every load and store of a wave is one run of 256 bytes.  y may be x: a lane has read every channel of a round, and all
// before it, when it writes the channels the round finishes, which lie behind them.
#include <hip/hip_runtime.h>

#include <climits>

#include "../../include/shadow_hip.h"
#include "device_common.h"
#include "launch.h"
#include "libm_exact.h"

#pragma clang fp contract(off)

namespace shdw {

// Windows of up to 63 channels: 63 KB of LDS for the 256 lanes of a workgroup, beside the tables.
constexpr int kLrnMaxSize = 63;

// Channels a lane takes per round: their loads go out together, the sum walks
// through them one by one, and only then come the powers, which do not depend on
// one another -- eight of them side by side, in their branch-free form, hide the
// latency of their table look-ups and fp64 chains, which the walk itself cannot
// (one power per step of the walk: 378 us on [64,256,56,56]; in rounds: 236 us; with the
// window in registers, the next round's loads under way and the tables in LDS: 140 us).
constexpr uint32_t kLrnRound = 8;

// The two tables of powf in LDS: read from there, the powers leave the vector
// memory counter alone, so that waiting for a table entry is not waiting for the
// next round's channels, which were asked for before it.
struct LrnTables {
  uint64_t exp2[32];
  libm::PowfLog2Entry log2[16];
};

// All lanes of the workgroup, before any of them leaves.
SHDW_DEVICE void lrn_stage_tables(LrnTables* t) {
  if (threadIdx.x < 32) t->exp2[threadIdx.x] = libm::kExp2fTab[threadIdx.x];
  if (threadIdx.x < 16) t->log2[threadIdx.x] = libm::kPowfLog2Tab[threadIdx.x];
  __syncthreads();
}

// powf(scale, y) for the scales of a round.  The straight path for all of them (any
// bits may go in, see powf_ordinary); then, if some lane holds a scale that is not a
// positive normal number, the whole function for those, one instance of its code.
SHDW_DEVICE void lrn_powers(const float (&scale)[kLrnRound], float y, const LrnTables* t,
                            float (&power)[kLrnRound]) {
  bool plain = true;
#pragma unroll
  for (uint32_t j = 0; j < kLrnRound; ++j) {
    power[j] = libm::powf_ordinary(__float_as_uint(scale[j]), y, 0u, t->exp2, t->log2);
    plain = plain && libm::powf_is_ordinary(__float_as_uint(scale[j]), __float_as_uint(y));
  }
  if (__builtin_amdgcn_ballot_w64(!plain) == 0) return;
#pragma unroll 1
  for (uint32_t pick = 0; pick < kLrnRound; ++pick) {
    float s = scale[0];
#pragma unroll
    for (uint32_t j = 1; j < kLrnRound; ++j) s = pick == j ? scale[j] : s;
    if (libm::powf_is_ordinary(__float_as_uint(s), __float_as_uint(y))) continue;
    const float r = libm::exact_powf(s, y, libm::kExp2fTab);
#pragma unroll
    for (uint32_t j = 0; j < kLrnRound; ++j) power[j] = pick == j ? r : power[j];
  }
}

// The channels of the round that starts at head0 (zeros past the last one).
SHDW_DEVICE void lrn_fetch(const float* in, uint32_t head0, uint32_t channels, uint32_t step,
                           float (&values)[kLrnRound]) {
#pragma unroll
  for (uint32_t j = 0; j < kLrnRound; ++j)
    values[j] = head0 + j < channels ? in[static_cast<size_t>(head0 + j) * step] : 0.f;
}

// ---- windows of 1, 3, 5 and 7 channels: the window lives in registers ----
// prev[t] is channel head0 - SIZE + t, the last SIZE channels of the round before.
// EDGE: the first round and those that reach past the last channel, with the tests
// of the reference's three loops; the rounds between them need none.
// `round` holds the channels of this round on entry and those of the next on
// return: they are asked for before the powers and arrive while those are worked
// out.  (The channels this round writes lie behind all of them, y may be x.)
template <int SIZE, bool EDGE>
SHDW_DEVICE void lrn_round(const float* in, float* out, uint32_t head0, uint32_t channels, uint32_t step,
                           float (&round)[kLrnRound], float (&prev)[SIZE], float& accum, float alpha_over_size,
                           float neg_beta, float k, const LrnTables* tables, bool finish) {
  static_assert(SIZE % 2 == 1 && SIZE <= static_cast<int>(kLrnRound), "the window must fit into a round");
  constexpr uint32_t post = (SIZE - 1) / 2;
  const uint32_t steps = channels + post;  // step `head` takes channel head in and finishes channel head - post
  float entering[kLrnRound], scale[kLrnRound], centre[kLrnRound], power[kLrnRound];
#pragma unroll
  for (uint32_t j = 0; j < kLrnRound; ++j) entering[j] = round[j];
  lrn_fetch(in, head0 + kLrnRound, channels, step, round);
#pragma unroll
  for (uint32_t j = 0; j < kLrnRound; ++j) {
    const uint32_t head = head0 + j;  // the same for every lane, and so is every test on it
    scale[j] = 1.f;
    centre[j] = 0.f;
    if (!EDGE || head < channels) accum += entering[j] * entering[j];
    if (!EDGE || (head >= SIZE && head < steps)) {
      const float leaving = j >= SIZE ? entering[j >= SIZE ? j - SIZE : 0] : prev[j < SIZE ? j : 0];
      accum -= leaving * leaving;
    }
    if (!EDGE || (head >= post && head < steps)) {
      scale[j] = k + accum * alpha_over_size;
      centre[j] = j >= post ? entering[j >= post ? j - post : 0] : prev[j < post ? SIZE - post + j : 0];
    }
  }
#pragma unroll
  for (int t = 0; t < SIZE; ++t) prev[t] = entering[kLrnRound - SIZE + t];
  if (!finish) return;  // a round in front of this workgroup's share: only the sum had to pass through it
  lrn_powers(scale, neg_beta, tables, power);
#pragma unroll
  for (uint32_t j = 0; j < kLrnRound; ++j) {
    const uint32_t head = head0 + j;
    if (!EDGE || (head >= post && head < steps)) out[static_cast<size_t>(head - post) * step] = centre[j] * power[j];
  }
}

template <int SIZE>
__global__ __launch_bounds__(kBlock) void lrn_window_kernel(const float* x, float* y, uint32_t positions,
                                                            uint32_t step, uint32_t channels, FastDiv f_step,
                                                            float alpha_over_size, float neg_beta, float k) {
  __shared__ LrnTables tables;
  lrn_stage_tables(&tables);
  const uint32_t p = blockIdx.x * kBlock + threadIdx.x;
  if (p >= positions) return;
  const uint32_t b = fd_div(p, f_step);
  const size_t base = static_cast<size_t>(b) * channels * step + (p - b * step);
  const float* in = x + base;
  float* out = y + base;
  float prev[SIZE], round[kLrnRound];
#pragma unroll
  for (int t = 0; t < SIZE; ++t) prev[t] = 0.f;
  float accum = 0.f;
  const uint32_t steps = channels + (SIZE - 1) / 2;
  // gridDim.y workgroups share the rounds of a position: each walks the sum from the
  // first channel on, which is cheap, and works out the powers of its own rounds only
  const uint32_t rounds = (steps + kLrnRound - 1) / kLrnRound;
  const uint32_t first = blockIdx.y * rounds / gridDim.y * kLrnRound;
  const uint32_t end = (blockIdx.y + 1) * rounds / gridDim.y * kLrnRound;
  lrn_fetch(in, 0, channels, step, round);
  for (uint32_t head0 = 0; head0 < end; head0 += kLrnRound) {
    const bool finish = head0 >= first;
    if (head0 >= SIZE && head0 + kLrnRound <= channels)
      lrn_round<SIZE, false>(in, out, head0, channels, step, round, prev, accum, alpha_over_size, neg_beta, k, &tables,
                             finish);
    else
      lrn_round<SIZE, true>(in, out, head0, channels, step, round, prev, accum, alpha_over_size, neg_beta, k, &tables,
                            finish);
  }
}

// ---- any window up to kLrnMaxSize channels: the window lives in LDS ----
__global__ __launch_bounds__(kBlock) void lrn_across_channels_kernel(
    const float* x, float* y, uint32_t positions, uint32_t step, uint32_t channels, FastDiv f_step,
    uint32_t size, float alpha_over_size, float neg_beta, float k) {
  extern __shared__ float window[];  // [size][kBlock]
  __shared__ LrnTables tables;
  lrn_stage_tables(&tables);
  const uint32_t p = blockIdx.x * kBlock + threadIdx.x;
  if (p >= positions) return;  // no barrier below: a lane only meets its own column
  const uint32_t b = fd_div(p, f_step);
  const size_t base = static_cast<size_t>(b) * channels * step + (p - b * step);
  const float* in = x + base;
  float* out = y + base;
  float* mine = window + threadIdx.x;
  const uint32_t post = (size - 1) / 2;
  const uint32_t steps = channels + post;  // step `head` takes channel head in and finishes channel head - post
  float accum = 0.f;
  uint32_t slot_head = 0, slot_mid = 0;  // head % size and (head - post) % size
  float round[kLrnRound];
  const uint32_t rounds = (steps + kLrnRound - 1) / kLrnRound;  // shared out over gridDim.y as above
  const uint32_t first = blockIdx.y * rounds / gridDim.y * kLrnRound;
  const uint32_t end = (blockIdx.y + 1) * rounds / gridDim.y * kLrnRound;
  lrn_fetch(in, 0, channels, step, round);
  for (uint32_t head0 = 0; head0 < end; head0 += kLrnRound) {
    float entering[kLrnRound], scale[kLrnRound], centre[kLrnRound], power[kLrnRound];
#pragma unroll
    for (uint32_t j = 0; j < kLrnRound; ++j) entering[j] = round[j];
    lrn_fetch(in, head0 + kLrnRound, channels, step, round);  // the next round's, on their way during the powers
#pragma unroll
    for (uint32_t j = 0; j < kLrnRound; ++j) {
      const uint32_t head = head0 + j;
      scale[j] = 1.f;
      centre[j] = 0.f;
      if (head < steps) {  // the same for every lane
        if (head < channels) accum += entering[j] * entering[j];
        if (head >= size) {  // channel head - size lives where channel head goes
          const float leaving = mine[slot_head * kBlock];
          accum -= leaving * leaving;
        }
        if (head < channels) mine[slot_head * kBlock] = entering[j];
        slot_head = slot_head + 1 == size ? 0 : slot_head + 1;
        if (head >= post) {
          scale[j] = k + accum * alpha_over_size;
          centre[j] = mine[slot_mid * kBlock];
          slot_mid = slot_mid + 1 == size ? 0 : slot_mid + 1;
        }
      }
    }
    if (head0 < first) continue;  // in front of this workgroup's share: only the sum had to pass through
    lrn_powers(scale, neg_beta, &tables, power);
#pragma unroll
    for (uint32_t j = 0; j < kLrnRound; ++j) {
      const uint32_t head = head0 + j;
      if (head >= post && head < steps) out[static_cast<size_t>(head - post) * step] = centre[j] * power[j];
    }
  }
}

}  // namespace shdw

using namespace shdw;

extern "C" int shdw_hip_lrn(const int* in_shape, int size, float alpha, float beta, float k, const float* x,
                            float* y, void* stream) {
  if (!in_shape || size < 1 || size % 2 == 0) return SHDW_E_INVALID_ARGUMENT;
  long long count = 1;
  for (int d = 0; d < 4; ++d) {
    if (in_shape[d] < 0) return SHDW_E_INVALID_ARGUMENT;
    count *= in_shape[d];
    if (count > INT_MAX) return SHDW_E_UNSUPPORTED;
  }
  const int channels = in_shape[1], post = (size - 1) / 2;
  // fewer channels than lie behind the centre of a window: the reference's last
  // loop then writes in front of its scale blob
  if (channels < post) return SHDW_E_INVALID_ARGUMENT;
  if (count == 0) return SHDW_OK;
  if (!x || !y) return SHDW_E_INVALID_ARGUMENT;
  if (size > kLrnMaxSize) return SHDW_E_UNSUPPORTED;
  const uint32_t step = static_cast<uint32_t>(in_shape[2]) * static_cast<uint32_t>(in_shape[3]);
  const uint32_t positions = static_cast<uint32_t>(in_shape[0]) * step;
  const float alpha_over_size = alpha / size;  // float / int, as the reference forms it
  hipStream_t st = static_cast<hipStream_t>(stream);
  const uint32_t grid = grid_for(positions), chan = static_cast<uint32_t>(channels);
  const FastDiv f_step = make_fastdiv(step);
  // A tensor with few positions has few waves, and each walks all the channels one round after
  // the other (82 us for 256 channels, however few the waves).  Up to eight workgroups then share
  // the rounds of a position, about 4096 waves in all and four rounds each at the least; measured
  // on 12.8 M elements: [16,256,56,56] (784 waves) 82 -> 65, 56, 60, 77 us with 2, 4, 8, 16 shares,
  // [44,96,55,55] (2080 waves) 49 -> 42, 47, 55; [64,256,56,56] (3136 waves) 141 -> 139, 149.
  // In place a workgroup would overwrite what another still has to read: one share.
  const uint32_t waves = (positions + kWave - 1) / kWave;
  const uint32_t rounds = (chan + static_cast<uint32_t>(post) + kLrnRound - 1) / kLrnRound;
  uint32_t shares = (4096 + waves / 2) / waves;
  const uint32_t most = waves <= 512 ? 8u : 4u;
  shares = shares > most ? most : shares;
  shares = shares > rounds / 4 ? rounds / 4 : shares;
  if (x == y || shares < 1) shares = 1;
#define SHDW_LRN(S) \
  lrn_window_kernel<S><<<dim3(grid, shares), kBlock, 0, st>>>(x, y, positions, step, chan, f_step, alpha_over_size, -beta, k)
  if (size == 1) {
    SHDW_LRN(1);
  } else if (size == 3) {
    SHDW_LRN(3);
  } else if (size == 5) {
    SHDW_LRN(5);
  } else if (size == 7) {
    SHDW_LRN(7);
  } else {
    const size_t lds = static_cast<size_t>(size) * kBlock * sizeof(float);
    lrn_across_channels_kernel<<<dim3(grid, shares), kBlock, lds, st>>>(x, y, positions, step, chan, f_step,
                                                          static_cast<uint32_t>(size), alpha_over_size, -beta, k);
  }
#undef SHDW_LRN
  return launch_status();
}
