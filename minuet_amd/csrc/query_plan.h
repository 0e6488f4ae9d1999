// The query plan of a stride-1 kernel map worked out on the device: packing
// frame, key deltas of the offsets in ascending order and their groups, as
// make_plan() in query.hip builds them on the host from coordinate bounds
// that it had to wait for.  A chain of launches that never returns to the
// host (sort -> query -> lists) lets one wavefront of an earlier kernel write
// this block instead; the query kernel reads it from device memory.
#pragma once

#include "device_utils.h"

namespace mnt {

constexpr int kPlanGroupSpan = 4;                // key span of one offset group (kGroupSpan of the query)
constexpr int kPlanMaxOffsets = 64;              // one lane per offset
constexpr int kPlanInts = 6 * kPlanMaxOffsets;   // 4 words per group + 2 per member

// Kernel offsets as launch arguments (rows past the count are ignored), and
// what the host worked out about them for a cloud that is mapped onto itself:
// halves != 0 when the offsets come in pairs d / -d (no offset named twice, at
// least one pair); kind[o] is then 0 for the offset of a pair that is looked
// up (the one whose first non-zero coordinate is positive, i.e. whose key delta
// is), 1 for its mirror image, 2 for the zero offset, and mirror[o] the index
// of the offset's mirror image.
struct OffsetTable {
  int v[kPlanMaxOffsets][MNT_MAX_NDIM];
  int halves;
  signed char kind[kPlanMaxOffsets];
  signed char mirror[kPlanMaxOffsets];
};

// Fills halves / kind / mirror of `table` from its first num_offsets rows.
inline void classify_offset_pairs(OffsetTable &table, int num_offsets, int ndim, bool allow) {
  table.halves = 0;
  for (int o = 0; o < kPlanMaxOffsets; ++o) {
    table.kind[o] = 0;
    table.mirror[o] = -1;
  }
  if (!allow || num_offsets > kPlanMaxOffsets) return;
  bool paired = true, any_positive = false;
  for (int o = 0; o < num_offsets && paired; ++o) {
    int sign = 0;
    for (int k = 0; k < ndim && sign == 0; ++k) sign = table.v[o][k] > 0 ? 1 : table.v[o][k] < 0 ? -1 : 0;
    int mirror = -1;
    for (int p = 0; p < num_offsets; ++p) {
      bool negated = true, same = true;
      for (int k = 0; k < ndim; ++k) {
        negated = negated && table.v[p][k] == -table.v[o][k];
        same = same && table.v[p][k] == table.v[o][k];
      }
      if (negated && mirror < 0) mirror = p;
      if (same && p != o) paired = false;                     // an offset named twice
    }
    paired = paired && mirror >= 0;
    table.kind[o] = static_cast<signed char>(sign > 0 ? 0 : sign == 0 ? 2 : 1);
    table.mirror[o] = static_cast<signed char>(mirror);
    any_positive = any_positive || sign > 0;
  }
  if (paired && any_positive) {
    table.halves = 1;
    return;
  }
  for (int o = 0; o < kPlanMaxOffsets; ++o) {
    table.kind[o] = 0;
    table.mirror[o] = -1;
  }
}

struct DevicePlan {
  Frame frame;
  long long delta_min, delta_max;
  int num_groups;
  int groups_in_rows;       // every group's offsets differ in the last coordinate only
  int verdict;              // 0: go; otherwise the chain stops (sort declined, or keys beyond 63 bits)
  int num_offsets;
  int tables[kPlanInts];    // groups (first delta low / high, first member, members), then members (step, offset)
  // A cloud mapped onto itself under offsets that come in pairs d / -d: the
  // hits of -d are those of d with source and target exchanged, in the same
  // order (source positions rise with target positions), so only the offsets
  // of positive key delta are looked up.  halves != 0: kind[o] says what
  // offset o is (0 looked up, 1 the mirror image of offset mirror[o], 2 the
  // zero offset: every voxel is its own hit).
  int halves;
  int kind[kPlanMaxOffsets];
  int mirror[kPlanMaxOffsets];
  // the offsets that have rows of their own to write (all but the mirror
  // images), in offset order: offset | kind << 8 | (mirror + 1) << 16
  int rows[kPlanMaxOffsets];
  // Upper end of a tile's source window from the sort's bucket starts instead
  // of a search (a chain whose dealing launch worked by slabs; 0 buckets:
  // search).  The sort's key has coordinate 0 in its top field, so the rows
  // with coordinate 0 below x end where bucket ((x - lo) << shift) >> bucket_shift
  // starts (its next bucket when a bucket holds parts of two such planes).
  int window_buckets;
  int window_shift;               // of coordinate 0 in the sort's key
  int window_bucket_shift;        // sort key >> this = bucket
  int window_reach;               // largest offset along coordinate 0
  long long window_lo, window_hi; // range of coordinate 0 in the cloud
  const unsigned *window_starts;  // [window_buckets + 1]
};

struct PlanScratch {        // LDS of the wavefront that builds the plan
  int inverse[kPlanMaxOffsets];              // offset at each place of the ascending delta order
};

__device__ __forceinline__ int plan_bits(unsigned long long range) {
  return range == 0 ? 0 : 64 - __builtin_clzll(range);
}

// Run by ONE whole wavefront.  bounds = lo[4], hi[4] of the cloud (sources and
// targets are the same rows); the frame leaves room for every offset on both
// sides of every field, so key(q + offset) == key(q) + delta(offset).
// `declined` is the verdict of the launches before (non-zero: stop).
__device__ __forceinline__ void make_plan_on_device(const long long *__restrict__ bounds,
                                                    const OffsetTable &offsets, int num_offsets,
                                                    int ndim, unsigned declined, PlanScratch &lds,
                                                    DevicePlan *__restrict__ out,
                                                    const unsigned *__restrict__ bucket_starts = nullptr,
                                                    int msd_cap = 0) {
  const int lane = lane_id();
  // lane o takes offset o: selects on scalar operands, no indexed access to the arguments
  int d[MNT_MAX_NDIM] = {0, 0, 0, 0};
#pragma unroll
  for (int l = 0; l < kPlanMaxOffsets; ++l) {
#pragma unroll
    for (int k = 0; k < MNT_MAX_NDIM; ++k) d[k] = lane == l ? offsets.v[l][k] : d[k];
  }
  const bool live = lane < num_offsets;
  Frame f;
  int bits = 0;
  int reach_lo[MNT_MAX_NDIM], reach_hi[MNT_MAX_NDIM];
#pragma unroll
  for (int k = 0; k < MNT_MAX_NDIM; ++k) {
    int lo = live && k < ndim ? d[k] : 0, hi = lo;
    for (int off = 32; off > 0; off >>= 1) {
      const int a = __shfl_xor(lo, off), b = __shfl_xor(hi, off);
      lo = a < lo ? a : lo;
      hi = b > hi ? b : hi;
    }
    reach_lo[k] = lo < 0 ? lo : 0;
    reach_hi[k] = hi > 0 ? hi : 0;
  }
  bool fits = true;
#pragma unroll
  for (int k = MNT_MAX_NDIM - 1; k >= 0; --k) {
    f.lo[k] = 0;
    f.shift[k] = 0;
    f.width[k] = 0;
    if (k < ndim) {
      // coordinates are at most 64-bit and the reach is small: a range that wraps is caught below
      const long long lo = bounds[k] + reach_lo[k];
      const long long hi = bounds[MNT_MAX_NDIM + k] + reach_hi[k];
      const unsigned long long range = static_cast<unsigned long long>(hi) - static_cast<unsigned long long>(lo);
      fits = fits && hi >= lo && lo <= bounds[k] && hi >= bounds[MNT_MAX_NDIM + k] && range < (1ull << 63);
      f.lo[k] = lo;
      f.width[k] = plan_bits(range);
      f.shift[k] = bits < 63 ? bits : 63;
      bits += f.width[k];
    }
  }
  f.batch_width = 0;
  f.batch_shift = bits < 63 ? bits : 63;
  f.ndim = ndim;
  f.total_bits = bits;
  fits = fits && bits <= 63;

  long long delta = 0;
#pragma unroll
  for (int k = 0; k < MNT_MAX_NDIM; ++k) {
    if (k < ndim) {
      delta += static_cast<long long>(static_cast<unsigned long long>(static_cast<long long>(d[k])) << f.shift[k]);
    }
  }
  // what the host found out about the offsets: lane o takes entry o
  const bool halves = offsets.halves != 0;
  int kind = 0, mirror = -1;
#pragma unroll
  for (int l = 0; l < kPlanMaxOffsets; ++l) {
    kind = lane == l ? offsets.kind[l] : kind;
    mirror = lane == l ? offsets.mirror[l] : mirror;
  }
  // the offsets that are looked up: all of them, or those of positive key delta
  const bool kept = live && (!halves || kind == 0);
  const int num_kept = __popcll(__ballot(kept));
  // place among the kept offsets in ascending delta order (ties keep offset order)
  int place = 0;
  for (int p = 0; p < num_offsets; ++p) {
    const long long other = __shfl(delta, p);
    const bool other_kept = __shfl(kept ? 1 : 0, p) != 0;
    place += other_kept && (other < delta || (other == delta && p < lane)) ? 1 : 0;
  }
  // lane i takes over the offset of place i; from here on lanes are places
  if (kept) lds.inverse[place] = lane;
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
  const bool placed = lane < num_kept;
  const int origin = placed ? lds.inverse[lane] : lane;
  const long long mine = __shfl(delta, origin);
  int lead[MNT_MAX_NDIM];
#pragma unroll
  for (int k = 0; k < MNT_MAX_NDIM; ++k) lead[k] = __shfl(d[k], origin);
  // first place whose delta lies beyond this one's group span (num_kept if
  // none), and never more than kPlanGroupSpan + 1 members (repeated offsets)
  int next = num_kept;
  for (int p = num_kept - 1; p >= 0; --p) {
    const long long other = __shfl(mine, p);
    next = p > lane && other - mine > kPlanGroupSpan ? p : next;
  }
  next = next < lane + kPlanGroupSpan + 1 ? next : lane + kPlanGroupSpan + 1;
  // the greedy grouping follows those links from place 0
  unsigned long long starts = 0;
  int num_groups = 0;
  for (int cur = 0; cur < num_kept; cur = __shfl(next, cur)) {
    starts |= 1ull << cur;
    ++num_groups;
  }
  const unsigned long long upto = starts & ((2ull << lane) - 1ull);
  const int group = __popcll(upto) - 1;
  const int first_place = placed ? 63 - __builtin_clzll(upto) : 0;
  const long long first_delta = __shfl(mine, first_place);
  bool same_row = true;
#pragma unroll
  for (int k = 0; k < MNT_MAX_NDIM; ++k) {
    const int other = __shfl(lead[k], first_place);
    same_row = same_row && (k + 1 >= ndim || other == lead[k]);
  }
  const bool in_rows = __ballot(placed && !same_row) == 0ull;
  if (placed) {
    out->tables[4 * num_groups + 2 * lane + 0] = static_cast<int>(mine - first_delta);
    out->tables[4 * num_groups + 2 * lane + 1] = origin;
    if ((starts >> lane) & 1ull) {
      const unsigned long long first = static_cast<unsigned long long>(mine);
      out->tables[4 * group + 0] = static_cast<int>(static_cast<unsigned>(first & 0xffffffffull));
      out->tables[4 * group + 1] = static_cast<int>(static_cast<unsigned>(first >> 32));
      out->tables[4 * group + 2] = lane;
      out->tables[4 * group + 3] = next - lane;
    }
  }
  if (live) {
    out->kind[lane] = halves ? kind : 0;
    out->mirror[lane] = halves ? mirror : -1;
    const bool writes = !halves || kind != 1;
    const unsigned long long writers = __ballot(writes);
    if (writes) {
      const int y = __popcll(writers & ((1ull << lane) - 1ull));
      out->rows[y] = lane | ((halves ? kind : 0) << 8) | ((halves ? mirror + 1 : 0) << 16);
    }
  }
  // an offset that is looked up must have a positive key delta, which is what
  // the host's reading of its coordinates says; anything else stops the chain
  const bool consistent = !halves || __ballot(kept && delta <= 0) == 0ull;
  const long long delta_min = __shfl(mine, 0);
  const long long delta_max = __shfl(mine, num_kept > 0 ? num_kept - 1 : 0);
  if (lane == 0) {
    out->frame = f;
    out->delta_min = num_kept > 0 ? delta_min : 0;
    out->delta_max = num_kept > 0 ? delta_max : 0;
    out->halves = halves ? 1 : 0;
    out->num_groups = num_groups;
    out->groups_in_rows = in_rows ? 1 : 0;
    out->verdict = declined != 0 ? static_cast<int>(declined) : (fits && consistent ? 0 : 2);
    out->num_offsets = num_offsets;
    // the sort's key: fields of the cloud's own ranges, coordinate 0 on top
    int sort_bits = 0, below_top = 0;
#pragma unroll
    for (int k = MNT_MAX_NDIM - 1; k >= 0; --k) {
      if (k < ndim) {
        const int w = plan_bits(static_cast<unsigned long long>(bounds[MNT_MAX_NDIM + k]) -
                                static_cast<unsigned long long>(bounds[k]));
        if (k > 0) below_top += w;
        sort_bits += w;
      }
    }
    const int msd_bits = sort_bits < msd_cap ? sort_bits : msd_cap;
    const bool usable = bucket_starts != nullptr && sort_bits >= 1 && sort_bits <= 63 && sort_bits > below_top;
    out->window_buckets = usable ? 1 << msd_cap : 0;
    out->window_shift = below_top;
    out->window_bucket_shift = sort_bits - msd_bits;
    out->window_reach = reach_hi[0];
    out->window_lo = bounds[0];
    out->window_hi = bounds[MNT_MAX_NDIM];
    out->window_starts = bucket_starts;
  }
}

}  // namespace mnt
