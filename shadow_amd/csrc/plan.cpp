#include "plan.h"

#include <algorithm>
#include <climits>

#include "../../include/shadow_hip.h"

namespace shdw {

// kStrided with kFlatMinInner <= inner < kFlatMaxInner goes through the flat
// kernel (4 * inner <= 1024 must hold for odd inner: 127 * 4 = 508); so do 2 to
// 7 columns when a slab fills at least one step of the workgroup (channels over
// a row of 7: the column kernels would use 7 lanes of 64).
constexpr int64_t kFlatMinInner = 8, kFlatMaxInner = 128, kFlatNarrowInner = 2, kFlatNarrowSlab = 1024;
// Two reduced dims around a kept one: the second stage takes the inner one when
// it is this short and the leading one at least this long (the partials then
// stay under a sixteenth of the input).
constexpr int64_t kNestMax = 64, kNestMinLead = 32;

int plan_broadcast(int num_axes, const int* a_shape, const int* b_shape,
                   const int* out_shape, BroadcastPlan* plan) {
  if (num_axes < 0 || (num_axes > 0 && (!a_shape || !b_shape || !out_shape)) || !plan)
    return SHDW_E_INVALID_ARGUMENT;
  *plan = BroadcastPlan();

  // Contiguous strides of both operands, computed over the full rank first so
  // that dropped size-1 dims cannot disturb them.
  int64_t stride_a = 1, stride_b = 1, count = 1;
  // Walk from the innermost axis outwards and build the collapsed dims in
  // reverse; flip at the end.
  int rdims[kMaxDims], rsa[kMaxDims], rsb[kMaxDims];
  int n = 0;
  bool prev_a_bc = false, prev_b_bc = false;
  for (int ax = num_axes - 1; ax >= 0; --ax) {
    const int da = a_shape[ax], db = b_shape[ax], dout = out_shape[ax];
    if (da < 1 || db < 1 || dout < 1) return SHDW_E_INVALID_ARGUMENT;
    if (dout != std::max(da, db)) return SHDW_E_INVALID_ARGUMENT;
    if ((da != dout && da != 1) || (db != dout && db != 1)) return SHDW_E_INVALID_ARGUMENT;
    if (dout > 1) {
      const bool a_bc = (da == 1), b_bc = (db == 1);
      if (n > 0 && a_bc == prev_a_bc && b_bc == prev_b_bc) {
        // Same broadcast status as the dim just inside: one longer dim.
        const int64_t merged = static_cast<int64_t>(rdims[n - 1]) * dout;
        if (merged > INT_MAX) return SHDW_E_UNSUPPORTED;
        rdims[n - 1] = static_cast<int>(merged);
      } else {
        if (n == kMaxDims) return SHDW_E_UNSUPPORTED;
        rdims[n] = dout;
        rsa[n] = a_bc ? 0 : static_cast<int>(stride_a);
        rsb[n] = b_bc ? 0 : static_cast<int>(stride_b);
        ++n;
      }
      prev_a_bc = a_bc;
      prev_b_bc = b_bc;
    }
    stride_a *= da;
    stride_b *= db;
    count *= dout;
    if (count > INT_MAX || stride_a > INT_MAX || stride_b > INT_MAX) return SHDW_E_UNSUPPORTED;
  }
  plan->ndim = n;
  for (int k = 0; k < n; ++k) {
    plan->dims[k] = rdims[n - 1 - k];
    plan->sa[k] = rsa[n - 1 - k];
    plan->sb[k] = rsb[n - 1 - k];
  }
  plan->count = count;
  return SHDW_OK;
}

static int ceil_div64(int64_t a, int64_t b) { return static_cast<int>((a + b - 1) / b); }

int plan_reduce(int num_axes, const int* in_shape, int num_reduce, const int* axes,
                ReducePlan* plan) {
  if (num_axes < 0 || num_axes > kMaxDims) return num_axes < 0 ? SHDW_E_INVALID_ARGUMENT : SHDW_E_UNSUPPORTED;
  if (num_reduce < 0 || num_reduce > num_axes) return SHDW_E_INVALID_ARGUMENT;
  if ((num_axes > 0 && !in_shape) || (num_reduce > 0 && !axes) || !plan)
    return SHDW_E_INVALID_ARGUMENT;
  *plan = ReducePlan();

  bool reduced[kMaxDims] = {false};
  bool ascending = true;
  for (int k = 0; k < num_reduce; ++k) {
    const int ax = axes[k];
    // Shadow indexes its stride table with the raw axis value
    // (shadow/operators/kernels/reduce.hpp:54-57): negative or repeated axes
    // read out of bounds there, so they are rejected here.
    if (ax < 0 || ax >= num_axes || reduced[ax]) return SHDW_E_INVALID_ARGUMENT;
    reduced[ax] = true;
    if (k > 0 && axes[k] < axes[k - 1]) ascending = false;
  }
  int64_t stride[kMaxDims];
  int64_t total = 1;
  for (int ax = num_axes - 1; ax >= 0; --ax) {
    if (in_shape[ax] < 1) return SHDW_E_INVALID_ARGUMENT;
    stride[ax] = total;
    total *= in_shape[ax];
    if (total > INT_MAX) return SHDW_E_UNSUPPORTED;
  }
  int64_t outputs = 1, window = 1;
  for (int ax = 0; ax < num_axes; ++ax) (reduced[ax] ? window : outputs) *= in_shape[ax];
  plan->outputs = outputs;
  plan->window = window;

  // Collapse: drop size-1 dims, merge neighbours with the same reduced flag.
  int64_t cdim[kMaxDims];
  bool cred[kMaxDims];
  int nc = 0;
  for (int ax = 0; ax < num_axes; ++ax) {
    if (in_shape[ax] == 1) continue;
    if (nc > 0 && cred[nc - 1] == reduced[ax]) {
      cdim[nc - 1] *= in_shape[ax];
    } else {
      cdim[nc] = in_shape[ax];
      cred[nc] = reduced[ax];
      ++nc;
    }
  }

  bool fast = ascending;
  if (fast) {
    if (nc == 0) {
      plan->kind = kStrided;  // single element, one output
      plan->outer = 1, plan->reduce = 1, plan->inner = 1;
    } else if (nc == 1 && !cred[0]) {
      plan->kind = kStrided;  // nothing to fold: every output has a 1-element window
      plan->outer = 1, plan->reduce = 1, plan->inner = cdim[0];
    } else if (nc == 1 && cred[0]) {
      plan->kind = kRows;
      plan->outer = 1, plan->reduce = cdim[0], plan->inner = 1;
    } else if (nc == 2 && !cred[0]) {
      plan->kind = kRows;
      plan->outer = cdim[0], plan->reduce = cdim[1], plan->inner = 1;
    } else if (nc == 2 && cred[0]) {
      plan->kind = kStrided;
      plan->outer = 1, plan->reduce = cdim[0], plan->inner = cdim[1];
    } else if (nc == 3 && !cred[0]) {
      plan->kind = kStrided;
      plan->outer = cdim[0], plan->reduce = cdim[1], plan->inner = cdim[2];
    } else if (nc == 3 || nc == 4) {
      // two reduced dims with a kept one between them: [k0][lead][k1][r1] (k0 = 1 for nc == 3), or
      // [lead][k0][r1][k1] where the last dim is kept
      const bool rows = cred[nc - 1];
      const int64_t k0 = rows ? (nc == 4 ? cdim[0] : 1) : cdim[1];
      const int64_t lead = rows ? cdim[nc - 3] : cdim[0];
      const int64_t k1 = rows ? cdim[nc - 2] : cdim[3];
      const int64_t r1 = rows ? cdim[nc - 1] : cdim[2];
      if (r1 <= kNestMax && lead >= kNestMinLead && r1 < lead) {
        // the long leading dim first, as a strided reduce with all that follows as columns
        plan->kind = kStrided;
        plan->nest = r1;
        if (rows) {  // columns (k1, r1): those of output (k0, k1) are neighbours
          plan->outer = k0, plan->reduce = lead, plan->inner = k1 * r1;
          plan->nest_olo = 1, plan->nest_ohi_stride = r1, plan->nest_stride = 1;
        } else {  // columns (k0, r1, k1)
          plan->outer = 1, plan->reduce = lead, plan->inner = k0 * r1 * k1;
          plan->nest_olo = k1, plan->nest_ohi_stride = r1 * k1, plan->nest_stride = k1;
        }
      } else if (rows) {
        plan->kind = kRows;
        plan->lead = lead, plan->lead_inner = k1;
        plan->outer = k0 * lead * k1, plan->reduce = r1, plan->inner = 1;
      } else {
        plan->kind = kStrided;
        plan->lead = lead, plan->lead_inner = k0;
        plan->outer = lead * k0, plan->reduce = r1, plan->inner = k1;
      }
    } else {
      fast = false;
    }
  }

  if (!fast) {
    plan->kind = kGeneric;
    plan->outer = outputs, plan->reduce = window, plan->inner = 0;
    for (int ax = 0; ax < num_axes; ++ax) {
      if (!reduced[ax] && in_shape[ax] > 1) {
        plan->kdim[plan->nk] = in_shape[ax];
        plan->kstride[plan->nk] = static_cast<int>(stride[ax]);
        ++plan->nk;
      }
    }
    for (int k = 0; k < num_reduce; ++k) {
      const int ax = axes[k];
      if (in_shape[ax] > 1) {
        plan->rdim[plan->nr] = in_shape[ax];
        plan->rstride[plan->nr] = static_cast<int>(stride[ax]);
        ++plan->nr;
      }
    }
    plan->splits = 1;
    return SHDW_OK;
  }

  // Work split.  The aim is >= ~2k workgroups of 256 lanes when the input is
  // large enough, so that all 256 CUs (8 XCDs) have several waves in flight,
  // while every slice still streams a few KiB.
  if (plan->kind == kRows) {
    if (plan->reduce <= 4096 && plan->outer >= 256) {
      plan->wave_per_row = true;
      plan->splits = 1;
    } else {
      const int by_fill = ceil_div64(4096, plan->outer);
      const int by_work = ceil_div64(plan->reduce, 4096);  // >= 4 vectors per lane
      plan->splits = std::max(1, std::min(by_fill, by_work));
    }
  } else if (plan->inner < kFlatMaxInner &&
             (plan->inner >= kFlatMinInner ||
              (plan->inner >= kFlatNarrowInner && plan->reduce * plan->inner >= kFlatNarrowSlab))) {
    // Few columns: a column tile would leave most lanes idle (56 columns use 14
    // of a wave's 64 lanes with 128-bit loads).  The [reduce][inner] slab of one
    // outer index is contiguous, so the 256 lanes of a workgroup walk it flat,
    // four consecutive elements per lane, in steps of `flat_period` elements: a
    // multiple of inner, so each lane keeps meeting the same four columns.
    const int64_t unit = (plan->inner % 4 == 0) ? plan->inner : (plan->inner % 2 == 0 ? 2 : 4) * plan->inner;
    plan->flat_period = static_cast<int>(1024 / unit * unit);
    const int by_fill = ceil_div64(1024, plan->outer);
    const int by_work = ceil_div64(plan->reduce * plan->inner, 8 * 1024);  // >= 8 steps per workgroup
    plan->splits = std::max(1, std::min(std::min(by_fill, by_work), 1024));
  } else if (plan->inner % 4 == 0) {
    // Whole 128-bit vectors per row.  A workgroup of 512 lanes owns a tile of 4 L
    // columns (L lanes per row piece, 512 / L rows per step); wider pieces are
    // longer contiguous reads, narrower ones give more workgroups.  Take the
    // widest piece up to 512 bytes that still gives 192 workgroups (6 waves per
    // CU, each with eight 128-bit loads in flight); when even 128-byte pieces do
    // not, slice the reduced axis and keep the pieces as wide as the rows allow
    // (sum over 12544 of [12544x1024]: 12.2 us with 512-byte pieces and 24
    // slices, 15.4 us with 128-byte pieces and 6).
    const int64_t inner4 = plan->inner / 4;
    const int64_t want = 192;
    int lanes = inner4 >= 32 ? 32 : (inner4 >= 16 ? 16 : 8);
    for (int l : {32, 16, 8}) {
      if (((inner4 + l - 1) / l) * plan->outer >= 192) {
        lanes = l;
        break;
      }
    }
    // 1024-byte pieces stream at the rate of a plain read where 512-byte pieces reach
    // four fifths of it (max over 512 of [128,512,784]: 35.8 -> 32.9 us), but a launch of
    // few such tiles starts and ends slowly (2.5 us more at 128 workgroups, level at 256):
    // taken from two workgroups per CU on, and only where they are mostly full.
    if (inner4 >= 64 && ((inner4 + 63) / 64) * plan->outer >= 512 && inner4 * 4 >= ((inner4 + 63) / 64) * 64 * 3)
      lanes = 64;
    plan->strided_lanes = lanes;
    const int64_t blocks = ((inner4 + lanes - 1) / lanes) * plan->outer;
    const int by_fill = ceil_div64(want, blocks);
    const int by_work = ceil_div64(plan->reduce, 8 * (512 / lanes));  // a full batch of loads per lane
    plan->splits = std::max(1, std::min(std::min(by_fill, by_work), 1024));
  } else {
    // One column per lane: 4 or 16 waves per 64-column tile, so that one launch
    // gives >= 256 workgroups (one per CU) and >= 2048 waves; only when neither
    // does, slice the reduced axis and fold the slices afterwards.
    const int64_t tiles = (plan->inner + 63) / 64;
    const int64_t base_blocks = tiles * plan->outer;
    bool single = false;
    for (int waves : {4, 16}) {
      if (base_blocks >= 256 && base_blocks * waves >= 2048 && plan->reduce >= 8 * waves) {
        plan->strided_waves = waves;
        single = true;
        break;
      }
    }
    if (single) {
      plan->splits = 1;
    } else {
      plan->strided_waves = 4;
      const int by_fill = ceil_div64(1024, base_blocks);
      const int by_work = ceil_div64(plan->reduce, 64);  // >= 16 rows per wave
      plan->splits = std::max(1, std::min(by_fill, by_work));
    }
  }
  return SHDW_OK;
}

}  // namespace shdw

extern "C" {

int shdw_hip_plan_broadcast(int num_axes, const int* a_shape, const int* b_shape,
                            const int* out_shape, int* dims, int* a_strides,
                            int* b_strides) {
  shdw::BroadcastPlan p;
  const int rc = shdw::plan_broadcast(num_axes, a_shape, b_shape, out_shape, &p);
  if (rc != SHDW_OK) return rc;
  for (int k = 0; k < p.ndim; ++k) {
    if (dims) dims[k] = p.dims[k];
    if (a_strides) a_strides[k] = p.sa[k];
    if (b_strides) b_strides[k] = p.sb[k];
  }
  return p.ndim;
}

int shdw_hip_plan_reduce(int num_axes, const int* in_shape, int num_reduce,
                         const int* axes, int* kind, int* outer, int* reduce,
                         int* inner, int* splits) {
  shdw::ReducePlan p;
  const int rc = shdw::plan_reduce(num_axes, in_shape, num_reduce, axes, &p);
  if (rc != SHDW_OK) return rc;
  if (kind) *kind = p.kind;
  if (outer) *outer = static_cast<int>(p.outer);
  if (reduce) *reduce = static_cast<int>(p.reduce);
  if (inner) *inner = static_cast<int>(p.inner);
  if (splits) *splits = p.splits;
  return SHDW_OK;
}

size_t shdw_hip_reduce_workspace_bytes(int num_axes, const int* in_shape, int num_reduce,
                                       const int* axes) {
  shdw::ReducePlan p;
  if (shdw::plan_reduce(num_axes, in_shape, num_reduce, axes, &p) != SHDW_OK) return 0;
  return shdw::reduce_workspace_bytes(p);
}

}  // extern "C"
