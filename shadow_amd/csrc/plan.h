// Host-side launch planning for the broadcast and reduce kernels.  Pure C++ (no
// HIP types) so the same code is exercised by CPU-only tests through the
// shdw_hip_plan_* entry points.
#ifndef SHADOW_AMD_CSRC_PLAN_H_
#define SHADOW_AMD_CSRC_PLAN_H_

#include <cstddef>
#include <cstdint>

namespace shdw {

constexpr int kMaxDims = 8;  // Shadow's CUDA broadcast kernel stops at 8 axes
                             // (shadow/operators/kernels/binary.cu:34)

// ---------------------------------------------------------------------------
// Broadcast: the output is viewed as `ndim` dims (outermost first); operand
// offset = sum_k idx[k] * stride[k], stride 0 on the dims an operand broadcasts.
// Size-1 output dims are dropped and neighbouring dims with the same
// (a broadcasts?, b broadcasts?) status are merged.
// ---------------------------------------------------------------------------
struct BroadcastPlan {
  int ndim = 0;
  int dims[kMaxDims] = {0};
  int sa[kMaxDims] = {0};
  int sb[kMaxDims] = {0};
  int64_t count = 1;  // number of output elements
};

// Returns 0, or a negative SHDW_E_* code.
int plan_broadcast(int num_axes, const int* a_shape, const int* b_shape,
                   const int* out_shape, BroadcastPlan* plan);

// ---------------------------------------------------------------------------
// Reduce.
//   kRows    : x viewed as [outer][reduce], reduced axis contiguous.
//   kStrided : x viewed as [outer][reduce][inner], inner > 1 contiguous.
//   Either view may have one more reduced dim in front (ReducePlan::lead): the
//   statistics of a channel over batch and plane are [lead][outer][reduce].
//   kGeneric : any other axis pattern (several separated reduced groups, or
//              axes not listed in ascending order, where Shadow's list order is
//              not memory order).  Kept/reduced dims are passed uncollapsed.
// `splits` > 1 means a first stage writes `splits` partial results per output
// and a second stage combines them in slice order.
// ---------------------------------------------------------------------------
enum ReduceKind { kRows = 0, kStrided = 1, kGeneric = 2 };

struct ReducePlan {
  int kind = kRows;
  int64_t outer = 1, reduce = 1, inner = 1;
  int splits = 1;
  bool wave_per_row = false;  // kRows: 16/32/64 lanes per row instead of a workgroup
  int strided_lanes = 0;      // kStrided with whole 128-bit vectors per row (inner % 4 == 0, inner >= 128):
                              // lanes per row piece (8, 16, 32 or 64), a column tile is 4 * lanes wide;
                              // 0 selects one column per lane
  int strided_waves = 4;      // kStrided, one column per lane: wave64 per workgroup sharing a column tile (4 or 16)
  int flat_period = 0;        // kStrided with fewer than 128 columns: > 0 selects the flat kernel; elements
                              // the 256 lanes cover per step (a multiple of inner and of 4, <= 1024)
  int64_t lead = 1;           // > 1: one more reduced dim in front of the view above, [a][lead][b][reduce] for
                              // kRows (outer = a * lead * b) and [lead][b][reduce][inner] for kStrided
                              // (outer = lead * b); the first stage treats it as kept and leaves one partial
                              // per leading index (and slice), the second stage folds them
  int64_t lead_inner = 1;     // b
  // nest > 1: the other order for a short reduce extent behind a long leading one ([lead][kept][nest] or
  // [lead][kept][nest][kept'], nest <= 64 < lead): the view is kStrided over the leading dim with everything
  // behind it as columns (lead = 1 for the kernels), the first stage leaves partials per slice and column of the
  // view, and the second stage folds slices and the nest columns of an output: column of (output o, j) =
  // (o / nest_olo) * nest_ohi_stride + o % nest_olo + j * nest_stride
  int64_t nest = 1, nest_olo = 1, nest_ohi_stride = 1, nest_stride = 1;
  int64_t outputs = 1;        // number of output elements
  int64_t window = 1;         // elements per output (Shadow's num_list)
  // kGeneric only: kept dims (outermost first) and reduced dims in LIST order,
  // i.e. rdim[nr-1] is the fastest-varying one, as Shadow enumerates them.
  int nk = 0, nr = 0;
  int kdim[kMaxDims] = {0}, kstride[kMaxDims] = {0};
  int rdim[kMaxDims] = {0}, rstride[kMaxDims] = {0};
};

constexpr size_t kReducePartialBytes = 8;  // fp64 accumulator, or {fp32 extremum, zero key}

int plan_reduce(int num_axes, const int* in_shape, int num_reduce, const int* axes,
                ReducePlan* plan);

// Partials per output that the first stage leaves (1: it writes the results itself).
inline int64_t reduce_slots(const ReducePlan& p) { return p.lead * p.splits; }

inline size_t reduce_workspace_bytes(const ReducePlan& p) {
  if (p.nest > 1) return static_cast<size_t>(p.outer * p.inner) * p.splits * kReducePartialBytes;
  return reduce_slots(p) > 1 ? static_cast<size_t>(p.outputs) * reduce_slots(p) * kReducePartialBytes : 0;
}

}  // namespace shdw

#endif  // SHADOW_AMD_CSRC_PLAN_H_
