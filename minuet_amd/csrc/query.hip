// Map step, part 3: kernel-map query on packed voxel keys, per-offset sizes,
// stable size order, rank tables (masks) and per-offset pair lists.
//
// The dense map has the meaning of QuerySortedIndexWithOffsets
// (csrc/minuet/cuda/kernels/query_sorted_index_with_offsets.cuh:36-77, batched:
// multi_query_sorted_index_with_offsets.cuh:38-91): M[o,t] = j iff
// sources[j] == targets[t] + offsets[o] within one batch.  Sizes and rank
// tables follow ComputeKernelMapSizes / ComputeKernelMapMasks
// (csrc/minuet/cuda/functions/scan.cu:220-365).
//
// Layout of one query workgroup: 512 consecutive sorted targets, one per lane.
// Because the targets are sorted, every shifted query of the tile lies between
// key(first)+min_delta and key(last)+max_delta, so ONE window of the sorted
// sources serves all offsets.  The window is packed to 64-bit keys and staged
// in LDS (2048 keys at a time).  Offsets are visited in ascending key order
// and split into groups of near-adjacent deltas (e.g. the three z-neighbours
// of one (dx,dy)): the first query of a group is located by a branch-free
// binary search in LDS (three groups searched in lockstep for latency
// hiding), the others by walking forward from there.  Hits are counted per
// offset with wavefront ballots.
#include <algorithm>
#include <mutex>

#include "device_utils.h"
#include "query_plan.h"
#include "sort.h"

namespace mnt {

constexpr int kQueryBlock = 256;          // emit / count kernels
constexpr int kQueryThreads = 512;        // query kernel: one target per lane
constexpr int kTargetsPerTile = 512;
constexpr int kWindowChunk = 4096;
constexpr int kWindowPad = 64;            // sentinel keys behind a full chunk
constexpr int kGroupSpan = 4;             // key span of one offset group
constexpr int kGroupsInFlight = 3;
constexpr int kDirectoryRows = 14000;     // 16-bit entries of the row directory (dynamic LDS)


template <typename CT, typename BT>
struct KeyReader {
  const CT *coords;
  const BT *batch_dims;
  int num_batches;
  long long count;
  __device__ __forceinline__ unsigned long long operator()(long long i, const Frame &f) const {
    int b = 0;
    if (f.batch_width > 0) b = batch_of<BT>(i, batch_dims, num_batches);
    return pack_row<CT>(coords + i * f.ndim, f, b);
  }
};

// Width of the last coordinate's field, the least significant one of a key
// (no indexing by a run-time value: the frame stays in registers).
__device__ __forceinline__ int last_width(const Frame &f) {
  return f.ndim == 1 ? f.width[0] : f.ndim == 2 ? f.width[1] : f.ndim == 3 ? f.width[2] : f.width[3];
}

// First index in [lo, hi) whose key is >= q (hi if none), found by one
// wavefront probing 64 equally spaced rows per step.  All lanes must call
// with the same arguments.
template <typename CT, typename BT>
__device__ __forceinline__ long long wave_lower_bound(const KeyReader<CT, BT> &src, const Frame &f,
                                                      unsigned long long q, long long lo,
                                                      long long hi) {
  const int lane = lane_id();
  while (hi > lo) {
    const long long len = hi - lo;
    const long long step = (len + kWave - 1) / kWave;
    const long long idx = lo + lane * step;
    const bool less = idx < hi && src(idx, f) < q;
    const int c = __popcll(__ballot(less));
    if (c == 0) {
      hi = lo;
    } else {
      const long long new_hi = lo + c * step;
      lo = lo + (c - 1) * step + 1;
      hi = new_hi < hi ? new_hi : hi;
    }
  }
  return lo;
}

// Where a query launch that feeds the pair lists leaves its hits (the dense
// map is not written then).  A wavefront owns 64 consecutive targets; the
// hits it finds under offset o are stored compacted, in target order, at the
// start of the wavefront's own 64 slots of stage[o, :], and the ballot that
// says which of its targets they belong to goes to masks[o, wavefront].  A
// tile whose source window takes several chunks cannot compact (a later chunk
// may answer for a lower target): it marks itself in tile_mode and writes
// every target's slot, -1 for a miss, like a row of the dense map.
struct HitSink {
  int *stage;                      // [O, T]
  unsigned long long *masks;       // [O, ceil(T / 64)]
  unsigned *row_totals;            // [total_copies][total_stride], zero before the launch; a tile adds its hits
                                   // to copy (tile % total_copies) with atomics: one copy of a few dozen words
                                   // is two cache lines that every tile's atomics would queue up behind
  unsigned *tile_mode;             // [tiles]: 0 = compacted, 1 = a slot per target
  long long num_wave_tiles;        // ceil(T / 64)
  int num_offsets;
  unsigned *repeats;               // raised when two rows of a cloud mapped onto itself are equal (nullable)
  int total_copies, total_stride;
};

// Settles the queries of one group against the candidates cand[0 .. span]
// read from window position p on: writes the map entries this workgroup's
// chunk is responsible for and counts the hits per offset.  The group and
// member tables hold the same values for every lane; they are moved to scalar
// registers, so that the loop, the row offsets of the map and the deltas are
// scalar work.  d0 = q0 - base (wraps to a huge value when q0 < base, which
// the range test then rejects like any other query outside the window).
template <typename K, typename OT, bool kWholeWindow, bool kLists>
__device__ __forceinline__ void settle_group(
    const K (&cand)[kGroupSpan + 1], int p, unsigned long long q0, unsigned long long d0,
    const int4 &group, long long c0, bool valid, unsigned long long first_key,
    unsigned long long next_first, const int2 *s_members, unsigned *s_counts, bool count_hits,
    OT *__restrict__ column, long long num_targets, const HitSink &sink, long long t) {
  constexpr unsigned long long kLimit = static_cast<unsigned long long>(static_cast<K>(~static_cast<K>(0)));
  const int first_member = __builtin_amdgcn_readfirstlane(group.z);
  const int members = __builtin_amdgcn_readfirstlane(group.w);
  const OT found_base = static_cast<OT>(c0 + p);
  for (int m = 0; m < members; ++m) {
    const int2 member = s_members[first_member + m];
    const unsigned step = static_cast<unsigned>(__builtin_amdgcn_readfirstlane(member.x));
    const int o = __builtin_amdgcn_readfirstlane(member.y);
    const unsigned long long d = d0 + step;
    bool mine = valid;
    if (!kWholeWindow) {                       // several chunks: this one answers for its own key range only
      const unsigned long long q = q0 + step;
      mine = mine && q >= first_key && q < next_first;
    }
    const K q_rel = static_cast<K>(d);
    int at = -1;
#pragma unroll
    for (int x = 0; x <= kGroupSpan; ++x) at = cand[x] == q_rel ? x : at;
    const bool hit = mine && d < kLimit && at >= 0;
    const unsigned long long votes = __ballot(hit);
    if (kLists) {
      const long long row = static_cast<long long>(o) * num_targets;
      const long long wave_t0 = t - lane_id();
      if (kWholeWindow) {
        if (hit) sink.stage[row + wave_t0 + __popcll(votes & lanes_below())] = static_cast<int>(found_base) + at;
        if (lane_id() == 0 && wave_t0 < num_targets) {
          sink.masks[static_cast<long long>(o) * sink.num_wave_tiles + (wave_t0 >> 6)] = votes;
        }
      } else {
        if (mine) sink.stage[row + t] = hit ? static_cast<int>(found_base) + at : -1;
      }
    } else {
      if (mine) column[static_cast<long long>(o) * num_targets] = hit ? found_base + static_cast<OT>(at) : static_cast<OT>(-1);
    }
    const unsigned hits = __popcll(votes);
    if (count_hits && hits != 0 && lane_id() == 0) atomicAdd(&s_counts[o], hits);
  }
}

// Resolves every (offset, target) pair of the tile against the window chunk
// staged in LDS as keys of type K relative to `base` (K = 32 bits when the
// chunk's key range allows, which halves the LDS traffic of the searches).
// A query outside [base, base + max K) cannot match and is forced to miss.
template <typename K, typename OT, bool kWholeWindow, bool kLists>
__device__ __forceinline__ void resolve_chunk(
    const K *__restrict__ win, int top, unsigned long long base, long long c0,
    unsigned long long key, bool valid, unsigned long long first_key, unsigned long long next_first,
    const int4 *s_groups, const int2 *s_members, int num_groups, unsigned *s_counts, bool count_hits,
    long long t, long long num_targets, OT *__restrict__ kernel_map, const HitSink &sink) {
  OT *column = kernel_map + t;
  constexpr unsigned long long kLimit = static_cast<unsigned long long>(static_cast<K>(~static_cast<K>(0)));
  for (int g0 = 0; g0 < num_groups; g0 += kGroupsInFlight) {
    // lower bound of the first query of up to three groups, in lockstep
    int4 group[kGroupsInFlight];
    unsigned long long q0[kGroupsInFlight];
    K q0_rel[kGroupsInFlight];
    int pos[kGroupsInFlight];
#pragma unroll
    for (int j = 0; j < kGroupsInFlight; ++j) {
      group[j] = s_groups[g0 + j < num_groups ? g0 + j : num_groups - 1];
      const unsigned long long first_delta =
          static_cast<unsigned long long>(static_cast<unsigned>(group[j].x)) |
          (static_cast<unsigned long long>(static_cast<unsigned>(group[j].y)) << 32);
      q0[j] = key + first_delta;
      const unsigned long long d = q0[j] - base;
      q0_rel[j] = q0[j] < base ? static_cast<K>(0)
                               : (d < kLimit ? static_cast<K>(d) : static_cast<K>(kLimit - 1));
      pos[j] = 0;
    }
    for (int step = top; step >= 1; step >>= 1) {
#pragma unroll
      for (int j = 0; j < kGroupsInFlight; ++j) {
        if (win[pos[j] + step - 1] < q0_rel[j]) pos[j] += step;
      }
    }
#pragma unroll
    for (int j = 0; j < kGroupsInFlight; ++j) {
      if (g0 + j >= num_groups) continue;       // uniform across the workgroup
      int p = pos[j];
      p += win[p] < q0_rel[j] ? 1 : 0;
      K cand[kGroupSpan + 1];
#pragma unroll
      for (int x = 0; x <= kGroupSpan; ++x) cand[x] = win[p + x];
      settle_group<K, OT, kWholeWindow, kLists>(cand, p, q0[j], q0[j] - base, group[j], c0, valid,
                                                first_key, next_first, s_members, s_counts, count_hits,
                                                column, num_targets, sink, t);
    }
  }
}

// The same with a row directory instead of the binary search.  Keys that
// differ only in their last coordinate (a "row": same batch, same leading
// coordinates) are neighbours in the window; dir[b] holds 1 + the window
// position of the first key of row b (0: the row is empty), b = relative key
// >> zbits.  All queries of a group lie in one row, so a group costs one
// directory read and four candidate reads; only when the row is longer than
// four keys and the queries may sit further on does a binary search inside
// the row (at most zbits steps) follow.  Needs 32-bit relative keys whose
// base is the start of a row, and at least 3 bits of last coordinate (then
// the deltas of a group, at most kGroupSpan apart, never leave the row).
// settle_group for the form the list builds spend their time in: 32-bit
// relative keys, a window of one chunk, hits going to the staging slots.  The
// member entries were read together with the candidates (a group has at most
// kGroupSpan + 1 members: unique deltas within a span of kGroupSpan), the loop
// is unrolled and compares are 32 bits wide.  With kCollect the ballot of
// offset o is not stored here but parked in lane o of `votes` (up to 64
// offsets); the caller stores all of them with one instruction at the end.
template <bool kCollect>
__device__ __forceinline__ void settle_group_staged(
    const unsigned (&cand)[kGroupSpan + 1], int p, unsigned long long d0, const int2 (&member)[kGroupSpan + 1],
    int members, long long c0, bool inside, unsigned *s_counts, long long num_targets,
    const HitSink &sink, long long wave_t0, unsigned &votes_lo, unsigned &votes_hi) {
  const unsigned q0_rel = static_cast<unsigned>(d0);
  // the largest step of a group is kGroupSpan: one test of the key range for all members
  const bool low = inside && (d0 >> 32) == 0ull && q0_rel < 0xffffffffu - kGroupSpan;
  const int found_base = static_cast<int>(c0) + p;
#pragma unroll
  for (int m = 0; m <= kGroupSpan; ++m) {
    if (m >= members) break;                    // uniform
    const unsigned step = static_cast<unsigned>(__builtin_amdgcn_readfirstlane(member[m].x));
    const int o = __builtin_amdgcn_readfirstlane(member[m].y);
    const unsigned q_rel = q0_rel + step;
    int at = -1;
#pragma unroll
    for (int x = 0; x <= kGroupSpan; ++x) at = cand[x] == q_rel ? x : at;
    const bool hit = low && at >= 0;
    const unsigned long long votes = __builtin_amdgcn_ballot_w64(hit);
    const unsigned lo = static_cast<unsigned>(votes), hi = static_cast<unsigned>(votes >> 32);
    const unsigned rank = __builtin_amdgcn_mbcnt_hi(hi, __builtin_amdgcn_mbcnt_lo(lo, 0u));
    // the row and the wavefront's first slot are the same in every lane: the
    // store takes them as its scalar base and the rank as its 32-bit offset
    int *slots = sink.stage + (static_cast<long long>(o) * num_targets + wave_t0);
    if (hit) slots[rank] = found_base + at;
    if (kCollect) {
      const bool keeper = static_cast<int>(lane_id()) == o;
      votes_lo = keeper ? lo : votes_lo;
      votes_hi = keeper ? hi : votes_hi;
    } else if (lane_id() == 0 && wave_t0 < num_targets) {
      sink.masks[static_cast<long long>(o) * sink.num_wave_tiles + (wave_t0 >> 6)] = votes;
      atomicAdd(&s_counts[o], static_cast<unsigned>(__popcll(votes)));
    }
  }
}

template <typename OT, bool kWholeWindow, bool kLists>
__device__ __forceinline__ void resolve_chunk_rows(
    const unsigned *__restrict__ win, const unsigned short *__restrict__ dir, int len, int zbits,
    unsigned num_rows, unsigned long long base, long long c0, unsigned long long key, bool valid,
    unsigned long long first_key, unsigned long long next_first, const int4 *s_groups,
    const int2 *s_members, int num_groups, unsigned *s_counts, bool count_hits, long long t,
    long long num_targets, OT *__restrict__ kernel_map, const HitSink &sink) {
  OT *column = kernel_map + t;
  constexpr bool kStaged = kWholeWindow && kLists;
  // staged form: up to 64 offsets leave their ballots in the lanes of one
  // register pair; they are stored once, after the last group
  const bool collect = kStaged && sink.num_offsets <= kWave;
  const long long wave_t0 = uniform64(t - lane_id());
  unsigned votes_lo = 0, votes_hi = 0;
  // three groups in lockstep: their directory reads, then their candidate
  // reads, are in flight together
  for (int g0 = 0; g0 < num_groups; g0 += kGroupsInFlight) {
    int4 group[kGroupsInFlight];
    unsigned long long q0[kGroupsInFlight], d0[kGroupsInFlight], row[kGroupsInFlight];
    unsigned start[kGroupsInFlight], q_last[kGroupsInFlight];
    int2 member[kGroupsInFlight][kGroupSpan + 1];
    bool inside[kGroupsInFlight];
#pragma unroll
    for (int j = 0; j < kGroupsInFlight; ++j) {
      group[j] = s_groups[g0 + j < num_groups ? g0 + j : num_groups - 1];
      const unsigned long long first_delta =
          static_cast<unsigned long long>(static_cast<unsigned>(group[j].x)) |
          (static_cast<unsigned long long>(static_cast<unsigned>(group[j].y)) << 32);
      q0[j] = key + first_delta;
      d0[j] = q0[j] - base;
      row[j] = d0[j] >> zbits;
      inside[j] = valid && q0[j] >= base && row[j] < num_rows;
      start[j] = inside[j] ? dir[row[j]] : 0u;
      // entries past the group's last member repeat the last one
#pragma unroll
      for (int m = 0; m <= kGroupSpan; ++m) {
        member[j][m] = s_members[group[j].z + (m < group[j].w ? m : group[j].w - 1)];
      }
      q_last[j] = static_cast<unsigned>(d0[j]) + static_cast<unsigned>(member[j][kGroupSpan].x);
    }
    int p[kGroupsInFlight];
    unsigned cand[kGroupsInFlight][kGroupSpan + 1];
#pragma unroll
    for (int j = 0; j < kGroupsInFlight; ++j) {
      p[j] = start[j] != 0 ? static_cast<int>(start[j]) - 1 : 0;
#pragma unroll
      for (int x = 0; x < 4; ++x) cand[j][x] = win[p[j] + x];
      cand[j][4] = 0xffffffffu;
    }
#pragma unroll
    for (int j = 0; j < kGroupsInFlight; ++j) {
      if (g0 + j >= num_groups) continue;       // uniform across the workgroup
      const unsigned q0_rel = static_cast<unsigned>(d0[j]);
      if (start[j] != 0 && cand[j][3] < q_last[j] && (cand[j][3] >> zbits) == row[j]) {
        // a long row whose first four keys do not cover the queries.  In a row
        // without holes (a wall: every height occupied) the first query sits
        // as far behind the row's first key as their last coordinates differ:
        // look there first and keep the place if its neighbours confirm that
        // it is the lower bound; search the row otherwise.
        const int last = len - 1;
        int guess = p[j] + (q0_rel > cand[j][0] ? static_cast<int>(q0_rel - cand[j][0]) : 0);
        guess = guess < last ? guess : last;
        const unsigned before = win[guess > 0 ? guess - 1 : 0];
        unsigned at[kGroupSpan + 1];
#pragma unroll
        for (int x = 0; x <= kGroupSpan; ++x) at[x] = win[guess + x];
        if ((guess == 0 || before < q0_rel) && at[0] >= q0_rel) {
          p[j] = guess;
        } else {
          int lo = p[j];
          int hi = p[j] + (1 << zbits) < len ? p[j] + (1 << zbits) : len;      // zbits <= 24 here
          while (lo < hi) {
            const int mid = (lo + hi) >> 1;
            if (win[mid] < q0_rel) {
              lo = mid + 1;
            } else {
              hi = mid;
            }
          }
          p[j] = lo;
#pragma unroll
          for (int x = 0; x <= kGroupSpan; ++x) at[x] = win[lo + x];
        }
#pragma unroll
        for (int x = 0; x <= kGroupSpan; ++x) cand[j][x] = at[x];
      }
      if (kStaged) {
        const int members = __builtin_amdgcn_readfirstlane(group[j].w);
        if (collect) {
          settle_group_staged<true>(cand[j], p[j], d0[j], member[j], members, c0, inside[j], s_counts,
                                    num_targets, sink, wave_t0, votes_lo, votes_hi);
        } else {
          settle_group_staged<false>(cand[j], p[j], d0[j], member[j], members, c0, inside[j], s_counts,
                                     num_targets, sink, wave_t0, votes_lo, votes_hi);
        }
      } else {
        settle_group<unsigned, OT, kWholeWindow, kLists>(cand[j], p[j], q0[j], d0[j], group[j], c0, valid,
                                                         first_key, next_first, s_members, s_counts,
                                                         count_hits, column, num_targets, sink, t);
      }
    }
  }
  if (collect && wave_t0 < num_targets) {
    // lane o holds the ballot of offset o
    const int o = lane_id();
    if (o < sink.num_offsets) {
      const unsigned long long votes = (static_cast<unsigned long long>(votes_hi) << 32) | votes_lo;
      sink.masks[static_cast<long long>(o) * sink.num_wave_tiles + (wave_t0 >> 6)] = votes;
      atomicAdd(&s_counts[o], static_cast<unsigned>(__popcll(votes)));
    }
  }
}

// Offsets are visited in ascending key order, in groups whose deltas lie within
// kGroupSpan of the group's first one.  `tables` holds, as 32-bit words,
//   group g : first delta (low, high), index of its first member, member count
//   member i: delta minus the group's first delta, original offset row
// (groups first, then members); the kernel copies it into LDS once.
//
// Because source keys are unique and ascending, the key at window position
// p + j is at least win[p] + j; so once p = lower_bound(first query of the
// group) is known, every query of the group can only sit in win[p .. p+span]:
// one search plus span+1 independent LDS reads resolve the whole group.
//
// Small tables (the usual 27 offsets) travel as kernel arguments (`carried`,
// tables == nullptr), which saves the launch that would upload them; the last
// wavefront copies them into LDS with uniform (scalar) reads while the first
// two look for the window.
__device__ __forceinline__ void plan_from_sizes(const unsigned *row_sizes, int num_offsets, int reorder,
                                                unsigned *__restrict__ plan,
                                                unsigned *__restrict__ plan_host,
                                                unsigned long long *flag,
                                                unsigned long long sequence);
constexpr int kMaxTotalCopies = 16;          // copies of the per-offset totals a chain's query launch adds to
constexpr int kCarriedInts = 160;
struct CarriedTables {
  int v[kCarriedInts];
};

template <typename CT, typename BT, typename OT, bool kLists>
__global__ __launch_bounds__(kQueryThreads) void query_kernel(
    KeyReader<CT, BT> src, KeyReader<CT, BT> tgt, Frame frame, const int *__restrict__ tables,
    CarriedTables carried, int num_groups, int num_offsets, long long delta_min, long long delta_max,
    OT *__restrict__ kernel_map, unsigned *__restrict__ tile_counts, int num_tiles, int dir_rows,
    HitSink sink, const DevicePlan *__restrict__ device_plan) {
  extern __shared__ __align__(16) unsigned s_dynamic[];
  // Only half of the offsets are looked up (a cloud mapped onto itself under
  // offsets that come in pairs d / -d; see DevicePlan): the totals of the other
  // half are kept here as well, and equal rows, which break the symmetry, are
  // reported.
  bool halves = false;
  if (device_plan != nullptr) {
    // a launch inside a chain that never went back to the host: the verdict of
    // the launches before it and the plan come from device memory.  The values
    // are the same in every lane; saying so keeps them in scalar registers.
    const int verdict = device_plan->verdict;
#pragma unroll
    for (int k = 0; k < MNT_MAX_NDIM; ++k) {
      frame.lo[k] = uniform64(device_plan->frame.lo[k]);
      frame.shift[k] = __builtin_amdgcn_readfirstlane(device_plan->frame.shift[k]);
      frame.width[k] = __builtin_amdgcn_readfirstlane(device_plan->frame.width[k]);
    }
    frame.batch_shift = __builtin_amdgcn_readfirstlane(device_plan->frame.batch_shift);
    frame.batch_width = 0;
    frame.total_bits = __builtin_amdgcn_readfirstlane(device_plan->frame.total_bits);
    tables = device_plan->tables;
    num_groups = __builtin_amdgcn_readfirstlane(device_plan->num_groups);
    delta_min = uniform64(device_plan->delta_min);
    delta_max = uniform64(device_plan->delta_max);
    const int in_rows = __builtin_amdgcn_readfirstlane(device_plan->groups_in_rows);
    halves = __builtin_amdgcn_readfirstlane(device_plan->halves) != 0;
    if (__builtin_amdgcn_readfirstlane(verdict) != 0) return;
    dir_rows = in_rows != 0 && last_width(frame) >= 3 ? dir_rows : 0;
  }
  __shared__ unsigned long long win[kWindowChunk + kWindowPad];
  __shared__ long long s_bounds[2];
  __shared__ unsigned long long s_wave_first[kQueryThreads / kWave + 1];
  // dynamic LDS: [group table: 4 words each][member table: 2 words each][hit counts]
  // [row directory: dir_rows 16-bit entries]
  // With gridDim.y > 1 the offset groups are dealt over the y index: every
  // workgroup of a tile finds and stages the same window and resolves its
  // share of the groups (a cloud of a few tiles fills the chip that way).
  int my_first_group = 0, my_groups = num_groups;
  if (gridDim.y > 1) {
    const int share = (num_groups + static_cast<int>(gridDim.y) - 1) / static_cast<int>(gridDim.y);
    my_first_group = static_cast<int>(blockIdx.y) * share;
    my_groups = min(num_groups, my_first_group + share) - my_first_group;
    if (my_groups <= 0) return;
  }
  const int4 *s_all_groups = reinterpret_cast<const int4 *>(s_dynamic);
  const int4 *s_groups = s_all_groups + my_first_group;
  const int2 *s_members = reinterpret_cast<const int2 *>(s_dynamic + 4 * num_groups);
  unsigned *s_counts = s_dynamic + 4 * num_groups + 2 * num_offsets;
  unsigned *s_dir_words = s_counts + num_offsets;
  unsigned short *s_dir = reinterpret_cast<unsigned short *>(s_dir_words);
  // last coordinate: the least significant field of a key
  const int zbits = last_width(frame);

  const int tid = threadIdx.x;
  const int w = tid >> 6;
  const long long num_sources = src.count;
  const long long num_targets = tgt.count;
  const long long t0 = static_cast<long long>(blockIdx.x) * kTargetsPerTile;
  const long long t_end = t0 + kTargetsPerTile < num_targets ? t0 + kTargetsPerTile : num_targets;

  if (tables != nullptr) {
    for (int i = tid; i < 4 * num_groups + 2 * num_offsets; i += kQueryThreads) s_dynamic[i] = tables[i];
  } else if (w == kQueryThreads / kWave - 1) {
    const int count = 4 * num_groups + 2 * num_offsets;
#pragma unroll
    for (int i0 = 0; i0 < kCarriedInts; i0 += kWave) {
      if (i0 < count) {                                     // uniform
        // lane l takes entry i0 + l: 64 selects on scalar operands
        int mine = 0;
#pragma unroll
        for (int l = 0; l < kWave; ++l) mine = static_cast<int>(lane_id()) == l ? carried.v[i0 + l < kCarriedInts ? i0 + l : 0] : mine;
        if (i0 + static_cast<int>(lane_id()) < count) s_dynamic[i0 + lane_id()] = static_cast<unsigned>(mine);
      }
    }
  }
  for (int o = tid; o < num_offsets; o += kQueryThreads) s_counts[o] = 0;
  // where the totals of the offsets that are not looked up go: read now, used by the
  // last lines of the kernel, which would otherwise wait for a trip to memory
  __shared__ short s_mirror[kPlanMaxOffsets];
  __shared__ int s_zero_offset;
  if (halves && w == 2) {                      // one wavefront, a lane per offset (at most 64 of them in a chain)
    const int o = lane_id();
    const bool named = o < num_offsets && o < kPlanMaxOffsets;
    if (named) s_mirror[o] = static_cast<short>(device_plan->mirror[o]);
    const unsigned long long zero = __ballot(named && device_plan->kind[o] == 2);
    if (o == 0) s_zero_offset = zero != 0ull ? __builtin_ctzll(zero) : -1;
  }

  // ---- window of sources that can match any (offset, target) pair of the tile:
  // wavefront 0 finds its lower end, wavefront 1 its upper end
  const long long t = t0 + tid;
  const bool valid = t < t_end;
  const unsigned long long key = valid ? tgt(t, frame) : 0ull;
  // A cloud mapped onto itself under offsets of positive key delta only (halves):
  // nothing below the tile's first target can match, and where the sort left
  // its bucket starts the upper end is one table entry instead of a search:
  // the end of the rows whose coordinate 0 is at most that of the last target
  // plus the reach.  The window is then a little larger than the exact one;
  // should it take more than one chunk, the searches are done after all.
  const bool by_buckets = halves && device_plan->window_buckets > 0;
  auto search_end = [&](int which) {
    const unsigned long long edge =
        which == 0 ? tgt(t0, frame) + static_cast<unsigned long long>(delta_min)
                   : tgt(t_end - 1, frame) + static_cast<unsigned long long>(delta_max) + 1ull;
    const long long pos = wave_lower_bound<CT, BT>(src, frame, edge, 0, num_sources);
    if (lane_id() == 0) s_bounds[which] = pos;
  };
  if (w < 2) {
    if (!by_buckets) {
      search_end(w);
    } else if (w == 0) {
      if (lane_id() == 0) s_bounds[0] = t0;
    } else {
      const long long x = static_cast<long long>(tgt.coords[(t_end - 1) * frame.ndim]) + device_plan->window_reach;
      long long pos = num_sources;
      if (x < device_plan->window_hi) {
        const int buckets = device_plan->window_buckets;
        const int shift = device_plan->window_shift, bucket_shift = device_plan->window_bucket_shift;
        const unsigned long long key = static_cast<unsigned long long>(x + 1 - device_plan->window_lo) << shift;
        const unsigned long long bucket = (key >> bucket_shift) + (bucket_shift > shift ? 1ull : 0ull);
        pos = device_plan->window_starts[bucket < static_cast<unsigned long long>(buckets) ? bucket : buckets];
      }
      if (lane_id() == 0) s_bounds[1] = pos;
    }
  }
  if (halves) {
    if (lane_id() == 0) s_wave_first[w] = key;
    if (tid == kQueryThreads - 1) s_wave_first[kQueryThreads / kWave] = t_end < num_targets ? tgt(t_end, frame) : ~0ull;
  }
  __syncthreads();
  if (halves) {
    // a row equal to the row behind it (the rows are sorted): no symmetry to rely on
    const unsigned long long down = __shfl_down(key, 1);
    const unsigned long long next_key = t + 1 >= t_end ? s_wave_first[kQueryThreads / kWave]
                                        : lane_id() == kWave - 1 ? s_wave_first[w + 1] : down;
    if (__ballot(valid && next_key == key) != 0ull && lane_id() == 0) sink.repeats[0] = 1u;
  }
  if (by_buckets && s_bounds[1] - s_bounds[0] > kWindowChunk) {        // the same for the whole workgroup
    __syncthreads();
    if (w < 2) search_end(w);
    __syncthreads();
  }
  const long long w_lo = s_bounds[0];
  const long long w_hi = s_bounds[1] > w_lo ? s_bounds[1] : w_lo;
  const long long span = w_hi - w_lo;
  const int num_chunks = span <= kWindowChunk ? 1 : static_cast<int>((span + kWindowChunk - 1) / kWindowChunk);

  for (int c = 0; c < num_chunks; ++c) {
    const long long c0 = w_lo + static_cast<long long>(c) * kWindowChunk;
    const long long c1 = c0 + kWindowChunk < w_hi ? c0 + kWindowChunk : w_hi;
    const int len = static_cast<int>(c1 - c0);
    if (c > 0) __syncthreads();               // everyone is done with the previous chunk
    int top = 1;
    while (top * 2 < len) top *= 2;           // highest power of two below len (>= 1)
    const int fill = 2 * top + kWindowPad < kWindowChunk + kWindowPad ? 2 * top + kWindowPad : kWindowChunk + kWindowPad;
    // first and last key of the chunk and the first key behind it: the same
    // addresses for every lane, issued together with the staging loads
    const unsigned long long first_key = len > 0 ? src(c0, frame) : ~0ull;
    const unsigned long long last_key = len > 0 ? src(c1 - 1, frame) : 0ull;
    const unsigned long long next_first = c1 < w_hi ? src(c1, frame) : ~0ull;
    // relative keys count from the start of the first key's row
    const bool rows_possible = dir_rows > 0 && zbits >= 3 && zbits <= 24;
    const unsigned long long base = rows_possible ? first_key & ~((1ull << zbits) - 1ull) : first_key;
    const bool narrow = len > 0 && last_key - base < 0xffffffffull;
    const unsigned long long num_rows = narrow && rows_possible ? ((last_key - base) >> zbits) + 1ull : 0ull;
    const bool by_rows = num_rows != 0 && num_rows <= static_cast<unsigned long long>(dir_rows);
    if (narrow) {
      unsigned *win32 = reinterpret_cast<unsigned *>(win);
      if (by_rows) {
        for (int i = tid; i < static_cast<int>((num_rows + 1) >> 1); i += kQueryThreads) s_dir_words[i] = 0u;
      }
      for (int i = tid; i < fill; i += kQueryThreads) {
        win32[i] = i < len ? static_cast<unsigned>(src(c0 + i, frame) - base) : 0xffffffffu;
      }
      if (by_rows) {
        __syncthreads();
        // the first key of every row enters the directory
        for (int i = tid; i < len; i += kQueryThreads) {
          const unsigned row = win32[i] >> zbits;
          if (i == 0 || (win32[i - 1] >> zbits) != row) s_dir[row] = static_cast<unsigned short>(i + 1);
        }
      }
    } else {
      for (int i = tid; i < fill; i += kQueryThreads) {
        win[i] = i < len ? src(c0 + i, frame) : ~0ull;
      }
    }
    __syncthreads();
    // a chunk answers for the queries between its first key and the first key
    // of the next chunk; a window of one chunk answers for all of them
    const unsigned long long answers_from = c == 0 ? 0ull : first_key;
    const unsigned long long answers_to = c == num_chunks - 1 ? ~0ull : next_first;
    const bool counting = tile_counts != nullptr;
#define MNT_RESOLVE(WHOLE)                                                                         \
    if (by_rows) {                                                                                 \
      resolve_chunk_rows<OT, WHOLE, kLists>(reinterpret_cast<const unsigned *>(win), s_dir, len,   \
                                            zbits, static_cast<unsigned>(num_rows), base, c0, key, \
                                            valid, answers_from, answers_to, s_groups, s_members,  \
                                            my_groups, s_counts, counting, t, num_targets,        \
                                            kernel_map, sink);                                     \
    } else if (narrow) {                                                                           \
      resolve_chunk<unsigned, OT, WHOLE, kLists>(reinterpret_cast<const unsigned *>(win), top,     \
                                                 base, c0, key, valid, answers_from, answers_to,   \
                                                 s_groups, s_members, my_groups, s_counts,        \
                                                 counting, t, num_targets, kernel_map, sink);      \
    } else {                                                                                       \
      resolve_chunk<unsigned long long, OT, WHOLE, kLists>(win, top, 0ull, c0, key, valid,         \
                                                           answers_from, answers_to, s_groups,     \
                                                           s_members, my_groups, s_counts,        \
                                                           counting, t, num_targets, kernel_map,   \
                                                           sink);                                  \
    }
    if (num_chunks == 1) {
      MNT_RESOLVE(true)
    } else {
      MNT_RESOLVE(false)
    }
#undef MNT_RESOLVE
  }
  if (tile_counts != nullptr) {
    __syncthreads();
    // the offsets of this workgroup's groups: a run of the member table
    const int4 last_group = s_groups[my_groups - 1];
    for (int m = s_groups[0].z + tid; m < last_group.z + last_group.w; m += kQueryThreads) {
      const int o = s_members[m].y;
      const unsigned hits = s_counts[o];
      tile_counts[static_cast<long long>(o) * num_tiles + blockIdx.x] = hits;
      if (kLists && hits != 0) {
        unsigned *totals = sink.row_totals + static_cast<int>(blockIdx.x % sink.total_copies) * sink.total_stride;
        atomicAdd(&totals[o], hits);
        if (halves) atomicAdd(&totals[s_mirror[o]], hits);               // the mirror image has the same hits
      }
    }
    // the zero offset: every target of the tile is its own hit
    if (kLists && halves && tid == 0 && s_zero_offset >= 0) {
      unsigned *totals = sink.row_totals + static_cast<int>(blockIdx.x % sink.total_copies) * sink.total_stride;
      atomicAdd(&totals[s_zero_offset], static_cast<unsigned>(t_end - t0));
    }
  }
  if (kLists && tid == 0) sink.tile_mode[blockIdx.x] = num_chunks == 1 ? 0u : 1u;
}

// The query for frames too wide for a packed key (more than 63 bits of
// coordinate ranges, kernel reach and batch id): the reference's own way,
// a binary search per (offset, target) pair that compares whole coordinate
// tuples (csrc/minuet/common/functions.h:94-105,
// csrc/minuet/cuda/kernels/query_sorted_index_with_offsets.cuh:36-77), inside
// the target's batch.  Slow next to query_kernel (no shared window, log2 S
// dependent reads per pair) and only taken when that one cannot run.
// offsets: [O, ndim] as (low, high) halves of 64-bit values.
template <typename CT, typename BT, typename OT>
__global__ __launch_bounds__(kQueryBlock) void query_tuples_kernel(
    const CT *__restrict__ sources, long long num_sources, const CT *__restrict__ targets,
    long long num_targets, const int *__restrict__ offsets, int ndim,
    const BT *__restrict__ source_batch_dims, const BT *__restrict__ target_batch_dims,
    int num_batches, OT *__restrict__ kernel_map) {
  const long long t = static_cast<long long>(blockIdx.x) * kQueryBlock + threadIdx.x;
  const int o = blockIdx.y;
  if (t >= num_targets) return;
  long long q[MNT_MAX_NDIM];
  load_row<CT>(targets + t * ndim, ndim, q);
  bool representable = true;
#pragma unroll
  for (int k = 0; k < MNT_MAX_NDIM; ++k) {
    if (k < ndim) {
      const unsigned lo = static_cast<unsigned>(offsets[(o * ndim + k) * 2 + 0]);
      const unsigned hi = static_cast<unsigned>(offsets[(o * ndim + k) * 2 + 1]);
      const long long d = static_cast<long long>((static_cast<unsigned long long>(hi) << 32) | lo);
      long long sum;
      // a shifted coordinate beyond the coordinate type equals no source
      representable = representable && !__builtin_add_overflow(q[k], d, &sum) &&
                      sum == static_cast<long long>(static_cast<CT>(sum));
      q[k] = sum;
    }
  }
  long long lo = 0, hi = num_sources;
  if (source_batch_dims != nullptr) {
    const int b = batch_of<BT>(t, target_batch_dims, num_batches);
    lo = static_cast<long long>(source_batch_dims[b]);
    hi = static_cast<long long>(source_batch_dims[b + 1]);
  }
  const long long end = hi;
  // first source row of the batch that is not below q (lexicographic, dimension 0 first)
  while (representable && lo < hi) {
    const long long mid = lo + ((hi - lo) >> 1);
    long long c[MNT_MAX_NDIM];
    load_row<CT>(sources + mid * ndim, ndim, c);
    bool below = false, decided = false;
#pragma unroll
    for (int k = 0; k < MNT_MAX_NDIM; ++k) {
      if (k < ndim && !decided && c[k] != q[k]) {
        below = c[k] < q[k];
        decided = true;
      }
    }
    if (below) {
      lo = mid + 1;
    } else {
      hi = mid;
    }
  }
  bool found = representable && lo < end;
  if (found) {
    long long c[MNT_MAX_NDIM];
    load_row<CT>(sources + lo * ndim, ndim, c);
#pragma unroll
    for (int k = 0; k < MNT_MAX_NDIM; ++k) found = found && (k >= ndim || c[k] == q[k]);
  }
  kernel_map[static_cast<long long>(o) * num_targets + t] = found ? static_cast<OT>(lo) : static_cast<OT>(-1);
}

// Hit counts of every (row, tile of 512 targets) of an existing dense map.
template <typename IT>
__global__ __launch_bounds__(kQueryBlock) void count_tiles_kernel(
    const IT *__restrict__ kernel_map, long long num_targets, unsigned *__restrict__ tile_counts,
    int num_tiles) {
  __shared__ unsigned s_sum;
  const int o = blockIdx.y;
  const long long t0 = static_cast<long long>(blockIdx.x) * kTargetsPerTile;
  if (threadIdx.x == 0) s_sum = 0;
  __syncthreads();
  unsigned hits = 0;
#pragma unroll
  for (int r = 0; r < kTargetsPerTile / kQueryBlock; ++r) {
    const long long t = t0 + r * kQueryBlock + threadIdx.x;
    const bool hit = t < num_targets && kernel_map[static_cast<long long>(o) * num_targets + t] != static_cast<IT>(-1);
    hits += __popcll(__ballot(hit));
  }
  if (lane_id() == 0 && hits) atomicAdd(&s_sum, hits);
  __syncthreads();
  if (threadIdx.x == 0) tile_counts[static_cast<long long>(o) * num_tiles + blockIdx.x] = s_sum;
}

// One workgroup per row: exclusive scan of its tile counts in place and the
// row total.
__global__ __launch_bounds__(256) void tile_scan_kernel(unsigned *__restrict__ tile_counts,
                                                        int num_tiles,
                                                        unsigned *__restrict__ row_sizes) {
  __shared__ unsigned wave_sums[256 / kWave];
  unsigned *row = tile_counts + static_cast<long long>(blockIdx.x) * num_tiles;
  const int t = threadIdx.x;
  const int lane = lane_id();
  const int chunk = (num_tiles + 255) / 256;
  const int lo = t * chunk;
  const int hi = lo + chunk < num_tiles ? lo + chunk : num_tiles;
  unsigned sum = 0;
  for (int i = lo; i < hi; ++i) sum += row[i];
  unsigned inclusive = sum;
  for (int off = 1; off < kWave; off <<= 1) {
    const unsigned u = __shfl_up(inclusive, off);
    if (lane >= off) inclusive += u;
  }
  if (lane == kWave - 1) wave_sums[t >> 6] = inclusive;
  __syncthreads();
  unsigned before = 0, total = 0;
#pragma unroll
  for (int w = 0; w < 256 / kWave; ++w) {
    const unsigned x = wave_sums[w];
    before += w < (t >> 6) ? x : 0u;
    total += x;
  }
  unsigned run = before + inclusive - sum;
  for (int i = lo; i < hi; ++i) {
    unsigned v = row[i];
    row[i] = run;
    run += v;
  }
  if (t == 0) row_sizes[blockIdx.x] = total;
}

// The row order from the row totals, stable ascending by size (reorder) or
// identity, its inverse, the sizes in row order and their exclusive prefix;
// run by one whole workgroup.
// plan layout (unsigned): order[O] | position_of[O] | sorted_sizes[O] | prefix[O+1];
// the first three blocks are mirrored into plan_host (pinned host memory) and
// the sequence flag tells the host that they are there.
__device__ __forceinline__ void plan_from_sizes(const unsigned *row_sizes, int num_offsets, int reorder,
                                                unsigned *__restrict__ plan,
                                                unsigned *__restrict__ plan_host,
                                                unsigned long long *flag,
                                                unsigned long long sequence) {
  const int t = threadIdx.x;
  unsigned *order = plan;
  unsigned *position_of = plan + num_offsets;
  unsigned *sorted_sizes = plan + 2 * num_offsets;
  unsigned *prefix = plan + 3 * num_offsets;
  for (int o = t; o < num_offsets; o += blockDim.x) {
    const unsigned mine = row_sizes[o];
    int pos = o;
    if (reorder) {
      pos = 0;
      for (int p = 0; p < num_offsets; ++p) {
        const unsigned other = row_sizes[p];
        pos += (other < mine || (other == mine && p < o)) ? 1 : 0;
      }
    }
    order[pos] = o;
    position_of[o] = pos;
    sorted_sizes[pos] = mine;
    if (plan_host != nullptr) {
      plan_host[pos] = o;
      plan_host[num_offsets + o] = pos;
      plan_host[2 * num_offsets + pos] = mine;
    }
  }
  // thread 0 raises the flag behind a system-scope fence, which covers the
  // host writes of its own wavefront; the other wavefronts see to theirs
  if (plan_host != nullptr && t >= kWave && t < num_offsets) __threadfence_system();
  __syncthreads();
  if (t == 0) {
    unsigned total = 0;
    for (int j = 0; j < num_offsets; ++j) {
      prefix[j] = total;
      total += sorted_sizes[j];
    }
    prefix[num_offsets] = total;
    if (flag != nullptr) {
      __threadfence_system();
      __hip_atomic_store(flag, sequence, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
    }
  }
}

// One workgroup, launched after tile_scan_kernel.  (A separate launch instead
// of a "last workgroup" ticket inside tile_scan_kernel: the device-wide fence
// every workgroup would need costs more than the launch.  One workgroup doing
// both jobs was measured slower than the two launches as well.)
__global__ __launch_bounds__(256) void map_plan_kernel(const unsigned *__restrict__ row_sizes,
                                                       int num_offsets, int reorder,
                                                       unsigned *__restrict__ plan,
                                                       unsigned *__restrict__ plan_host,
                                                       unsigned long long *flag,
                                                       unsigned long long sequence) {
  plan_from_sizes(row_sizes, num_offsets, reorder, plan, plan_host, flag, sequence);
}

template <typename T>
__global__ __launch_bounds__(256) void fill_kernel(T *__restrict__ data, long long n, T value) {
  const long long stride = static_cast<long long>(gridDim.x) * blockDim.x;
  for (long long i = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += stride) {
    data[i] = value;
  }
}

// One wavefront per (row, tile): walks the 512 targets of the tile in order and
// ranks the hits.  Writes any of: target rank table, source rank table, pair
// lists.  `position_of` maps an offset to its output row (null = identity) and
// `row_base` gives the list position of the first hit of an output row.
template <typename IT>
__global__ __launch_bounds__(kQueryBlock) void emit_kernel(
    const IT *__restrict__ kernel_map, long long num_sources, long long num_targets,
    int num_offsets, const unsigned *__restrict__ tile_bases, int num_tiles,
    const unsigned *__restrict__ position_of, const unsigned *__restrict__ row_base,
    IT *__restrict__ source_masks, IT *__restrict__ target_masks, int *__restrict__ in_idx,
    int *__restrict__ out_idx, const unsigned *__restrict__ plan, int *__restrict__ sizes_out,
    int *__restrict__ order_out) {
  if (plan != nullptr && blockIdx.x == 0 && blockIdx.y == 0) {
    // device copies of the row order and the sizes in row order
    for (int j = threadIdx.x; j < num_offsets; j += kQueryBlock) {
      if (order_out) order_out[j] = static_cast<int>(plan[j]);
      if (sizes_out) sizes_out[j] = static_cast<int>(plan[2 * num_offsets + j]);
    }
  }
  const int o = blockIdx.y * (kQueryBlock / kWave) + (threadIdx.x >> 6);
  if (o >= num_offsets) return;
  const int lane = lane_id();
  const long long row = position_of ? position_of[o] : o;
  const long long t0 = static_cast<long long>(blockIdx.x) * kTargetsPerTile;
  unsigned running = tile_bases[static_cast<long long>(o) * num_tiles + blockIdx.x];
  const long long list_base = row_base ? static_cast<long long>(row_base[row]) : 0;
  const unsigned long long below = (1ull << lane) - 1ull;
#pragma unroll 2
  for (int r = 0; r < kTargetsPerTile / kWave; ++r) {
    const long long t = t0 + r * kWave + lane;
    const bool valid = t < num_targets;
    const IT m = valid ? kernel_map[static_cast<long long>(o) * num_targets + t] : static_cast<IT>(-1);
    const bool hit = m != static_cast<IT>(-1);
    const unsigned long long votes = __ballot(hit);
    const unsigned rank = running + __popcll(votes & below);
    if (valid && target_masks) target_masks[row * num_targets + t] = hit ? static_cast<IT>(rank) : static_cast<IT>(-1);
    if (hit) {
      if (source_masks) source_masks[row * num_sources + static_cast<long long>(m)] = static_cast<IT>(rank);
      if (in_idx) {
        in_idx[list_base + rank] = static_cast<int>(m);
        out_idx[list_base + rank] = static_cast<int>(t);
      }
    }
    running += __popcll(votes);
  }
}


// Final pair lists from the staged hits of a lists-mode query launch.  Row o
// of the lists starts where the rows ordered before it end (ascending hit
// count with ties in offset order when reorder is set, offset order
// otherwise); inside the row the tiles follow each other.  A workgroup takes
// kPlaceTiles consecutive tiles of one offset: it works out the list position
// of its first hit from the row totals and the tile counts before it (every
// workgroup sums those for itself; there is no scan pass), then each
// wavefront copies its tiles 64 targets at a time: the ballot says which
// targets hit, their sources are read from the staging slots and both go to
// consecutive list entries.  Workgroup (0, 0) also ranks the rows for the
// host (plan_from_sizes) and writes the device copies of sizes and order.
constexpr int kPlaceTiles = 4;
constexpr int kPlaceBlock = 256;

template <bool kChain>
__global__ __launch_bounds__(kPlaceBlock) void place_kernel(
    const int *__restrict__ stage, const unsigned long long *__restrict__ masks,
    const unsigned *__restrict__ tile_counts, const unsigned *row_totals,
    const unsigned *__restrict__ tile_mode, long long num_targets, int num_offsets, int num_tiles,
    long long num_wave_tiles, int reorder, int *__restrict__ in_idx, int *__restrict__ out_idx,
    unsigned *__restrict__ plan, unsigned *__restrict__ plan_host, unsigned long long *flag,
    unsigned long long sequence, int *__restrict__ sizes_out, int *__restrict__ order_out,
    const DevicePlan *__restrict__ chain_plan, const long long *__restrict__ folded_bounds,
    long long *chain_host, const unsigned *__restrict__ repeats, int total_copies, int total_stride) {
  __shared__ unsigned s_partial[kPlaceBlock / kWave];
  __shared__ unsigned s_partial_mirror[kPlaceBlock / kWave];
  __shared__ unsigned s_totals[kPlanMaxOffsets];
  static_assert(kPlaceTiles == kPlaceBlock / kWave, "one tile per wavefront");
  const int tid = threadIdx.x;
  const int lane = lane_id();
  const int w = tid >> 6;
  if (kChain && blockIdx.y == 0) {
    // Row 0 of a chain's grid places nothing: its first workgroup tells the
    // host how the chain went (verdict, coordinate bounds, sizes, order) and
    // leaves the device copies of sizes and order.  It reads three things in
    // one trip to memory and is among the first workgroups to start, so the
    // host hears of the sizes while the lists are still being placed.
    if (blockIdx.x != 0) return;
    int verdict = chain_plan->verdict;
    const unsigned repeated = repeats != nullptr ? repeats[0] : 0u;
    unsigned total = 0;
    {
      unsigned part[kMaxTotalCopies];
#pragma unroll
      for (int c = 0; c < kMaxTotalCopies; ++c) {
        part[c] = c < total_copies && tid < num_offsets ? row_totals[c * total_stride + tid] : 0u;
      }
#pragma unroll
      for (int c = 0; c < kMaxTotalCopies; ++c) total += part[c];
    }
    if (repeated != 0 && verdict == 0) verdict = 3;     // equal rows: the halves do not mirror each other
    if (tid == 0) {
#pragma unroll
      for (int slot = 0; slot < 2 * MNT_MAX_NDIM; ++slot) chain_host[slot] = folded_bounds[slot];
      chain_host[2 * MNT_MAX_NDIM] = static_cast<long long>(verdict);
      if (verdict != 0) {
        __threadfence_system();
        __hip_atomic_store(flag, sequence, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
      }
    }
    if (verdict != 0) return;
    if (tid < num_offsets && tid < kPlanMaxOffsets) s_totals[tid] = total;
    __syncthreads();
    plan_from_sizes(s_totals, num_offsets, reorder, plan, plan_host, flag, sequence);
    for (int j = tid; j < num_offsets; j += kPlaceBlock) {
      if (order_out) order_out[j] = static_cast<int>(plan[j]);
      if (sizes_out) sizes_out[j] = static_cast<int>(plan[2 * num_offsets + j]);
    }
    return;
  }
  const int tile0 = blockIdx.x * kPlaceTiles;
  const int tile = tile0 + w;
  constexpr int kSegments = kTargetsPerTile / kWave;

  // ---- Everything the workgroup reads from memory is asked for here, and
  // waited for ONCE: a trip to memory takes about two microseconds, and seven of
  // them one after the other (verdict, totals, tile counts, ballots, staged hits
  // ...) were most of this kernel's time.  What does not depend on the row this
  // workgroup writes comes first; the row's offset itself is read from the
  // chain's plan.  The staged hits are read as whole segments, lane l slot l,
  // instead of the slot a hit's rank names once the ballots are in.  After a
  // chain that declined the scratch arrays hold whatever was there: reading
  // that is harmless (every index is in range), nothing is written then.
  int verdict = 0, packed = blockIdx.y;
  unsigned repeated = 0;
  if (kChain) {
    verdict = chain_plan->verdict;
    packed = chain_plan->rows[blockIdx.y - 1];                       // row 0 of the grid is the teller above
    repeated = repeats != nullptr ? repeats[0] : 0u;
  }
  unsigned total_mine = 0;                       // hits of offset tid (tid < num_offsets <= 64 when there are copies)
  if (total_copies > 1) {
    unsigned part[kMaxTotalCopies];
#pragma unroll
    for (int c = 0; c < kMaxTotalCopies; ++c) {
      part[c] = c < total_copies && tid < num_offsets ? row_totals[c * total_stride + tid] : 0u;
    }
#pragma unroll
    for (int c = 0; c < kMaxTotalCopies; ++c) total_mine += part[c];
  }
  const unsigned mode = tile < num_tiles ? tile_mode[tile] : 0u;
  // Half of the offsets looked up (see DevicePlan): the workgroups of a
  // looked-up offset write the rows of its mirror image as well, those of the
  // zero offset write the identity, and mirror images have no workgroups.
  packed = __builtin_amdgcn_readfirstlane(packed);
  const int o = kChain ? packed & 0xff : packed;
  const int kind = kChain ? (packed >> 8) & 0xff : 0;
  const int twin = kChain ? ((packed >> 16) & 0xff) - 1 : -1;
  const bool live = tile < num_tiles && kind == 0;                    // uniform per wavefront
  const long long t_tile = static_cast<long long>(tile) * kTargetsPerTile;
  const long long row = static_cast<long long>(o) * num_targets;
  int entry[kSegments];
#pragma unroll
  for (int s = 0; s < kSegments; ++s) {
    const long long t = t_tile + s * kWave + lane;
    entry[s] = live && t < num_targets ? stage[row + t] : -1;
  }
  const long long wave_tile = (t_tile >> 6) + lane;
  const unsigned long long my_mask =
      live && lane < kSegments && wave_tile < num_wave_tiles
          ? masks[static_cast<long long>(o) * num_wave_tiles + wave_tile] : 0ull;
  const unsigned *counts = tile_counts + static_cast<long long>(o) * num_tiles;
  const int my_tile = tile0 + lane;
  const unsigned count = kind == 0 && lane < kPlaceTiles && my_tile < num_tiles ? counts[my_tile] : 0u;
  unsigned tiles_before = 0;
  if (kind == 0) {
    for (int i = tid; i < tile0; i += kPlaceBlock) tiles_before += counts[i];
  }
  // the one wait: everything above has been asked for by now
  {
    unsigned lo = static_cast<unsigned>(my_mask), hi = static_cast<unsigned>(my_mask >> 32);
    asm volatile("" : "+v"(entry[0]), "+v"(entry[1]), "+v"(entry[2]), "+v"(entry[3]), "+v"(entry[4]),
                 "+v"(entry[5]), "+v"(entry[6]), "+v"(entry[7]), "+v"(lo), "+v"(hi));
  }
  if (repeated != 0 && verdict == 0) verdict = 3;       // equal rows: the halves do not mirror each other
  if (verdict != 0) return;
  if (total_copies > 1) {
    if (tid < num_offsets) s_totals[tid] = total_mine;
    __syncthreads();
    row_totals = s_totals;
  }
  if (!kChain && blockIdx.x == 0 && blockIdx.y == 0) {
    // sizes, order and the flag for the host; device copies of sizes and order
    plan_from_sizes(row_totals, num_offsets, reorder, plan, plan_host, flag, sequence);
    for (int j = tid; j < num_offsets; j += kPlaceBlock) {
      if (order_out) order_out[j] = static_cast<int>(plan[j]);
      if (sizes_out) sizes_out[j] = static_cast<int>(plan[2 * num_offsets + j]);
    }
  }
  if (kind == 1) return;                       // written by the workgroups of its mirror image
  // rows before row o and before the mirror image's row
  const unsigned mine = row_totals[o];
  unsigned before = 0, before_twin = 0;
  for (int p = tid; p < num_offsets; p += kPlaceBlock) {
    const unsigned other = row_totals[p];
    const bool first = reorder ? (other < mine || (other == mine && p < o)) : p < o;
    before += first ? other : 0u;
    const bool first_twin = reorder ? (other < mine || (other == mine && p < twin)) : p < twin;
    before_twin += twin >= 0 && first_twin ? other : 0u;
  }
  if (kind == 2) {
    // the zero offset: hit number t of the row is target t with source t
    for (int off = 32; off > 0; off >>= 1) before += __shfl_xor(before, off);
    if (lane == 0) s_partial[w] = before;
    __syncthreads();
    unsigned row_start = 0;
#pragma unroll
    for (int ww = 0; ww < kPlaceBlock / kWave; ++ww) row_start += s_partial[ww];
    const long long first = static_cast<long long>(tile0) * kTargetsPerTile;
    for (long long t = first + tid; t < first + kPlaceTiles * kTargetsPerTile && t < num_targets; t += kPlaceBlock) {
      in_idx[row_start + t] = static_cast<int>(t);
      out_idx[row_start + t] = static_cast<int>(t);
    }
    return;
  }
  // list position of the first hit of (o, tile0): rows before, tiles before tile0
  before += tiles_before;
  before_twin += tiles_before;
  for (int off = 32; off > 0; off >>= 1) {
    before += __shfl_xor(before, off);
    before_twin += __shfl_xor(before_twin, off);
  }
  if (lane == 0) {
    s_partial[w] = before;
    s_partial_mirror[w] = before_twin;
  }
  __syncthreads();
  unsigned base = 0, base_twin = 0;
#pragma unroll
  for (int ww = 0; ww < kPlaceBlock / kWave; ++ww) {
    base += s_partial[ww];
    base_twin += s_partial_mirror[ww];
  }
  // entry number e of row o is entry number e of the mirror image's row with source and target exchanged
  const unsigned to_twin = base_twin - base;
  // tiles of this workgroup: exclusive prefix of their counts
  unsigned inclusive = count;
  for (int off = 1; off < kPlaceTiles; off <<= 1) {
    const unsigned u = __shfl_up(inclusive, off);
    if (lane >= off) inclusive += u;
  }
  const unsigned exclusive = inclusive - count;
  const unsigned long long below = lanes_below();
  if (tile >= num_tiles || __shfl(count, w) == 0) return;              // uniform per wavefront
  unsigned at = base + __shfl(exclusive, w);
  if (mode == 0) {
    // lane s holds the ballot of segment s and the hits before it
    const unsigned my_hits = __popcll(my_mask);
    unsigned seg_inclusive = my_hits;
    for (int off = 1; off < kSegments; off <<= 1) {
      const unsigned u = __shfl_up(seg_inclusive, off);
      if (lane >= off) seg_inclusive += u;
    }
    const unsigned seg_exclusive = seg_inclusive - my_hits;
#pragma unroll
    for (int s = 0; s < kSegments; ++s) {
      const unsigned long long mask = __shfl(my_mask, s);
      const bool hit = (mask >> lane) & 1ull;
      const unsigned r = __popcll(mask & below);
      // the hit of this lane's target is the r-th staged entry of the segment, which lane r read
      const int found = __shfl(entry[s], static_cast<int>(r));
      const unsigned rank = at + __shfl(seg_exclusive, s) + r;
      if (hit) {
        const int target = static_cast<int>(t_tile + s * kWave + lane);
        in_idx[rank] = found;
        out_idx[rank] = target;
        if (twin >= 0) {
          in_idx[rank + to_twin] = target;
          out_idx[rank + to_twin] = found;
        }
      }
    }
  } else {
#pragma unroll
    for (int s = 0; s < kSegments; ++s) {
      const bool hit = entry[s] != -1;
      const unsigned long long mask = __ballot(hit);
      if (hit) {
        const unsigned r = at + __popcll(mask & below);
        const int target = static_cast<int>(t_tile + s * kWave + lane);
        in_idx[r] = entry[s];
        out_idx[r] = target;
        if (twin >= 0) {
          in_idx[r + to_twin] = target;
          out_idx[r + to_twin] = entry[s];
        }
      }
      at += __popcll(mask);
    }
  }
}

// Target-major row lists of a kernel map, for the list-driven Scatter.  The
// pair lists number the hits row by row (list position p = row prefix + rank
// of the target among the row's hits); here every target gets the run
// row_ptr[t] .. row_ptr[t + 1] - 1 of a second numbering, by target first and
// by row (in list order) second, and out_pos[p] says where hit p sits in it.
// One workgroup per tile of 512 targets, one target per lane:
//   1. every wavefront ballots its 64 targets against each offset's row of the
//      dense map and leaves the ballots in LDS; a lane counts its own hits;
//   2. the counts are scanned (row_ptr) and the ballots of an offset turned
//      into the rank of each wavefront's first hit;
//   3. every lane walks the rows in list order and numbers its hits.
// tables: order[O] (list row j -> offset), list_start[O] (first list position
// of row j).  tile_bases: exclusive per-offset scan of the per-tile hit counts.
// Dynamic LDS: O * (64 + 32 + 4) bytes + 64.
__global__ __launch_bounds__(kQueryThreads) void row_lists_kernel(
    const int *__restrict__ kernel_map, long long num_targets, int num_offsets,
    const unsigned *__restrict__ tile_bases, int num_tiles, const int *__restrict__ tables,
    int *__restrict__ row_ptr, int *__restrict__ out_pos) {
  extern __shared__ __align__(16) unsigned char s_rows[];
  constexpr int kWaves = kQueryThreads / kWave;
  unsigned long long *s_ballot = reinterpret_cast<unsigned long long *>(s_rows);            // [O][waves]
  unsigned *s_first = reinterpret_cast<unsigned *>(s_ballot + static_cast<size_t>(num_offsets) * kWaves);  // [O][waves]
  unsigned *s_base = s_first + static_cast<size_t>(num_offsets) * kWaves;                   // [O], by list row
  unsigned *s_wave = s_base + num_offsets;                                                  // [waves + 2]
  const int tid = threadIdx.x;
  const int lane = lane_id();
  const int w = tid >> 6;
  const int tile = blockIdx.x;
  const long long t = static_cast<long long>(tile) * kTargetsPerTile + tid;
  const bool valid = t < num_targets;
  const int *order = tables;
  const int *list_start = tables + num_offsets;
  if (tid == 0) s_wave[kWaves] = 0;
  __syncthreads();
  unsigned count = 0;
  for (int o = 0; o < num_offsets; ++o) {
    const bool hit = valid && kernel_map[static_cast<long long>(o) * num_targets + t] != -1;
    const unsigned long long votes = __builtin_amdgcn_ballot_w64(hit);
    if (lane == 0) s_ballot[o * kWaves + w] = votes;
    count += hit ? 1u : 0u;
  }
  // hits of this tile before each target, and of all tiles before this one
  unsigned inclusive = count;
  for (int off = 1; off < kWave; off <<= 1) {
    const unsigned u = __shfl_up(inclusive, off);
    if (lane >= off) inclusive += u;
  }
  if (lane == kWave - 1) s_wave[w] = inclusive;
  unsigned earlier = 0;
  for (int o = tid; o < num_offsets; o += kQueryThreads) {
    earlier += tile_bases[static_cast<long long>(o) * num_tiles + tile];
  }
  for (int off = 32; off > 0; off >>= 1) earlier += __shfl_xor(earlier, off);
  if (lane == 0 && earlier != 0) atomicAdd(&s_wave[kWaves], earlier);
  __syncthreads();
  for (int j = tid; j < num_offsets; j += kQueryThreads) {
    // list row j: the rank of each wavefront's first hit, and the list position of the tile's first
    const int o = order[j];
    unsigned run = 0;
#pragma unroll
    for (int ww = 0; ww < kWaves; ++ww) {
      s_first[o * kWaves + ww] = run;
      run += __popcll(s_ballot[o * kWaves + ww]);
    }
    s_base[j] = static_cast<unsigned>(list_start[j]) + tile_bases[static_cast<long long>(o) * num_tiles + tile];
  }
  unsigned before = s_wave[kWaves];
  unsigned tile_hits = 0;
#pragma unroll
  for (int ww = 0; ww < kWaves; ++ww) {
    before += ww < w ? s_wave[ww] : 0u;
    tile_hits += s_wave[ww];
  }
  unsigned at = before + inclusive - count;
  if (valid) row_ptr[t] = static_cast<int>(at);
  if (t == num_targets - 1) row_ptr[num_targets] = static_cast<int>(s_wave[kWaves] + tile_hits);
  __syncthreads();
  const unsigned long long below = lanes_below();
  for (int j = 0; j < num_offsets; ++j) {
    const int o = order[j];
    const unsigned long long votes = s_ballot[o * kWaves + w];
    if ((votes >> lane) & 1ull) {
      const unsigned p = s_base[j] + s_first[o * kWaves + w] + __popcll(votes & below);
      out_pos[p] = static_cast<int>(at);
      ++at;
    }
  }
}

template <typename IT>
__global__ __launch_bounds__(256) void export_sizes_kernel(const unsigned *__restrict__ sizes,
                                                           int n, IT *__restrict__ out) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) out[i] = static_cast<IT>(sizes[i]);
}

// ------------------------------------------------------------------ host ----

static int width_of(unsigned long long range) {
  return range == 0 ? 0 : 64 - __builtin_clzll(range);
}

struct QueryPlan {
  Frame frame;
  std::vector<int> tables;               // group and member tables of query_kernel
  int num_groups;
  long long delta_min, delta_max;
  bool groups_in_rows;                   // the offsets of every group differ in the last coordinate only
  bool fits;                             // the frame packs into one 64-bit key; otherwise nothing else is filled in
};

// Builds the packing frame from the coordinate bounds of sources and targets
// (h_bounds: 8 slots each, min then max) and the kernel offsets.
static QueryPlan make_plan(const long long *src_bounds, const long long *tgt_bounds,
                           const int64_t *offsets, int64_t num_offsets, int ndim,
                           int64_t num_batches) {
  QueryPlan plan;
  memset(&plan.frame, 0, sizeof(Frame));
  plan.fits = true;
  plan.num_groups = 0;
  plan.delta_min = plan.delta_max = 0;
  plan.groups_in_rows = false;
  Frame &f = plan.frame;
  f.ndim = ndim;
  int bits = 0;
  for (int k = ndim - 1; k >= 0; --k) {
    long long omin = 0, omax = 0;
    for (int64_t o = 0; o < num_offsets; ++o) {
      long long d = offsets[o * ndim + k];
      omin = d < omin ? d : omin;
      omax = d > omax ? d : omax;
    }
    __int128 lo = static_cast<__int128>(tgt_bounds[k]) + omin;
    __int128 hi = static_cast<__int128>(tgt_bounds[MNT_MAX_NDIM + k]) + omax;
    if (src_bounds[k] < lo) lo = src_bounds[k];
    if (src_bounds[MNT_MAX_NDIM + k] > hi) hi = src_bounds[MNT_MAX_NDIM + k];
    __int128 range = hi - lo;
    if (!(range >= 0 && range < (static_cast<__int128>(1) << 63) && lo >= INT64_MIN && lo <= INT64_MAX)) {
      plan.fits = false;
      return plan;
    }
    f.lo[k] = static_cast<long long>(lo);
    f.width[k] = width_of(static_cast<unsigned long long>(range));
    f.shift[k] = bits < 63 ? bits : 63;
    bits += f.width[k];
  }
  f.batch_width = num_batches > 1 ? width_of(static_cast<unsigned long long>(num_batches - 1)) : 0;
  f.batch_shift = bits < 63 ? bits : 63;
  bits += f.batch_width;
  f.total_bits = bits;
  // coordinate ranges plus kernel reach plus batch id beyond 63 bits: the caller
  // takes the tuple-comparing query instead
  if (bits > 63) {
    plan.fits = false;
    return plan;
  }
  std::vector<std::pair<long long, int>> keyed(num_offsets);
  for (int64_t o = 0; o < num_offsets; ++o) {
    long long d = 0;
    for (int k = 0; k < ndim; ++k) {
      d += static_cast<long long>(static_cast<unsigned long long>(offsets[o * ndim + k]) << f.shift[k]);
    }
    keyed[o] = std::make_pair(d, static_cast<int>(o));
  }
  std::stable_sort(keyed.begin(), keyed.end(),
                   [](const std::pair<long long, int> &x, const std::pair<long long, int> &y) {
                     return x.first < y.first;
                   });
  std::vector<int> group_start;
  for (int64_t i = 0; i < num_offsets; ++i) {
    // a group spans at most kGroupSpan in key and holds at most kGroupSpan + 1
    // members (repeated offsets would otherwise overfill it)
    if (i == 0 || keyed[i].first - keyed[group_start.back()].first > kGroupSpan ||
        i - group_start.back() > kGroupSpan) {
      group_start.push_back(static_cast<int>(i));
    }
  }
  plan.num_groups = static_cast<int>(group_start.size());
  group_start.push_back(static_cast<int>(num_offsets));
  plan.tables.assign(4 * plan.num_groups + 2 * num_offsets, 0);
  for (int g = 0; g < plan.num_groups; ++g) {
    const unsigned long long first = static_cast<unsigned long long>(keyed[group_start[g]].first);
    plan.tables[4 * g + 0] = static_cast<int>(static_cast<unsigned>(first & 0xffffffffull));
    plan.tables[4 * g + 1] = static_cast<int>(static_cast<unsigned>(first >> 32));
    plan.tables[4 * g + 2] = group_start[g];
    plan.tables[4 * g + 3] = group_start[g + 1] - group_start[g];
    for (int i = group_start[g]; i < group_start[g + 1]; ++i) {
      plan.tables[4 * plan.num_groups + 2 * i + 0] = static_cast<int>(keyed[i].first - keyed[group_start[g]].first);
      plan.tables[4 * plan.num_groups + 2 * i + 1] = keyed[i].second;
    }
  }
  plan.groups_in_rows = true;
  for (int g = 0; g < plan.num_groups; ++g) {
    const int64_t first = keyed[group_start[g]].second;
    for (int i = group_start[g] + 1; i < group_start[g + 1]; ++i) {
      for (int k = 0; k + 1 < ndim; ++k) {
        if (offsets[keyed[i].second * ndim + k] != offsets[first * ndim + k]) plan.groups_in_rows = false;
      }
    }
  }
  plan.delta_min = num_offsets > 0 ? keyed.front().first : 0;
  plan.delta_max = num_offsets > 0 ? keyed.back().first : 0;
  return plan;
}

struct QueryArgs {
  const void *sources;
  int64_t num_sources;
  const void *targets;
  int64_t num_targets;
  int ndim;
  int coord_dtype;
  const void *source_batch_dims;
  const void *target_batch_dims;
  int64_t num_batches;
  int batch_dtype;
};

static void check_query_args(const QueryArgs &a, int64_t num_offsets) {
  MNT_CHECK(a.ndim >= 1 && a.ndim <= MNT_MAX_NDIM, "ndim must be in [1, %d] but found %d",
            MNT_MAX_NDIM, a.ndim);
  MNT_CHECK(a.num_sources >= 0 && a.num_sources <= INT32_MAX && a.num_targets >= 0 &&
                a.num_targets <= INT32_MAX,
            "number of sources / targets out of range");
  MNT_CHECK(num_offsets >= 0 && num_offsets <= 65535, "number of offsets %lld out of range",
            static_cast<long long>(num_offsets));
  MNT_CHECK((a.source_batch_dims == nullptr) == (a.target_batch_dims == nullptr),
            "source_batch_dims and target_batch_dims must be both provided or neither provided");
  int_size(a.coord_dtype);
  if (a.source_batch_dims) {
    int_size(a.batch_dtype);
    MNT_CHECK(a.num_batches >= 1, "batch dims must have at least 2 entries");
  }
}

template <typename CT, typename BT, typename OT, bool kLists>
static void launch_query(const QueryArgs &a, const QueryPlan &plan, const int *d_tables,
                         int num_offsets, OT *kernel_map, unsigned *tile_counts, int num_tiles,
                         const HitSink &sink, hipStream_t stream) {
  KeyReader<CT, BT> src{static_cast<const CT *>(a.sources), static_cast<const BT *>(a.source_batch_dims),
                        static_cast<int>(a.num_batches), a.num_sources};
  KeyReader<CT, BT> tgt{static_cast<const CT *>(a.targets), static_cast<const BT *>(a.target_batch_dims),
                        static_cast<int>(a.num_batches), a.num_targets};
  // room for the row directory where the last coordinate is wide enough for it
  const bool small_tables = plan.tables.size() * sizeof(int) <= 2048;
  const int dir_rows =
      plan.groups_in_rows && small_tables && plan.frame.width[plan.frame.ndim - 1] >= 3 ? kDirectoryRows : 0;
  const size_t dyn = sizeof(unsigned) * (plan.tables.size() + static_cast<size_t>(num_offsets) + 4) +
                     sizeof(unsigned short) * static_cast<size_t>(dir_rows);
  CarriedTables carried;
  memset(&carried, 0, sizeof(carried));
  if (d_tables == nullptr) memcpy(carried.v, plan.tables.data(), sizeof(int) * plan.tables.size());
  // a cloud of fewer tiles than compute units: the offset groups of a tile go
  // to several workgroups (not under kLists, whose staging is per tile)
  int split = 1;
  if (!kLists && plan.num_groups > 1 && num_tiles > 0) {
    const int wanted = std::min(plan.num_groups, std::max(1, compute_units() / num_tiles));
    const int share = static_cast<int>(div_ceil(plan.num_groups, wanted));
    split = static_cast<int>(div_ceil(plan.num_groups, share));
  }
  const dim3 grid(static_cast<unsigned>(num_tiles), static_cast<unsigned>(split));
  query_kernel<CT, BT, OT, kLists><<<grid, kQueryThreads, dyn, stream>>>(
      src, tgt, plan.frame, d_tables, carried, plan.num_groups, num_offsets, plan.delta_min,
      plan.delta_max, kernel_map, tile_counts, num_tiles, dir_rows, sink, nullptr);
  check_launch("query_kernel");
}

// Coordinate bounds of both operands: taken from the caller when given (8
// values each: min[4], max[4]), otherwise reduced on the device (one launch
// and one synchronisation).  bounds_out (nullable, 16 values) receives them.
static void resolve_bounds(const QueryArgs &a, const int64_t *source_bounds, const int64_t *target_bounds,
                           long long bounds[16], int64_t *bounds_out, Scope &scope, hipStream_t stream) {
  const bool need_src = source_bounds == nullptr;
  const bool need_tgt = target_bounds == nullptr;
  if (need_src || need_tgt) {
    long long fresh[16];
    read_bounds(need_src ? a.sources : nullptr, need_src ? a.num_sources : 0,
                need_tgt ? a.targets : nullptr, need_tgt ? a.num_targets : 0, a.ndim, a.coord_dtype,
                fresh, scope, stream);
    memcpy(bounds, fresh, sizeof(fresh));
  }
  if (!need_src) memcpy(bounds, source_bounds, sizeof(long long) * 8);
  if (!need_tgt) memcpy(bounds + 8, target_bounds, sizeof(long long) * 8);
  if (bounds_out != nullptr) memcpy(bounds_out, bounds, sizeof(long long) * 16);
}

static void enqueue_count_tiles(const void *kernel_map, int index_dtype, int64_t num_offsets,
                                int64_t num_targets, unsigned *tile_counts, int num_tiles,
                                hipStream_t stream);

// The query of a frame that does not fit a packed key: tuple comparisons
// (query_tuples_kernel), then the per-tile hit counts from the map it wrote.
static void run_wide_query(const QueryArgs &a, const int64_t *offsets_host, int64_t num_offsets,
                           bool batched, void *kernel_map, int out_dtype, unsigned *tile_counts,
                           int num_tiles, Scope &scope, hipStream_t stream) {
  std::vector<int> halves(static_cast<size_t>(num_offsets) * a.ndim * 2);
  for (size_t i = 0; i < halves.size() / 2; ++i) {
    const unsigned long long v = static_cast<unsigned long long>(offsets_host[i]);
    halves[2 * i + 0] = static_cast<int>(static_cast<unsigned>(v & 0xffffffffull));
    halves[2 * i + 1] = static_cast<int>(static_cast<unsigned>(v >> 32));
  }
  int *d_offsets = scope.alloc<int>(halves.size());
  upload_ints(halves, d_offsets, stream);
  const dim3 grid(static_cast<unsigned>(div_ceil(a.num_targets, kQueryBlock)), static_cast<unsigned>(num_offsets));
  const int nb = static_cast<int>(a.num_batches);
#define MNT_QT(CT, BT, OT)                                                                         \
  query_tuples_kernel<CT, BT, OT><<<grid, kQueryBlock, 0, stream>>>(                               \
      static_cast<const CT *>(a.sources), a.num_sources, static_cast<const CT *>(a.targets),       \
      a.num_targets, d_offsets, a.ndim, batched ? static_cast<const BT *>(a.source_batch_dims) : nullptr, \
      batched ? static_cast<const BT *>(a.target_batch_dims) : nullptr, nb, static_cast<OT *>(kernel_map))
  const bool c32 = a.coord_dtype == MNT_INT32;
  const bool b32 = !batched || a.batch_dtype == MNT_INT32;
  const bool o32 = out_dtype == MNT_INT32;
  if (c32 && b32 && o32) MNT_QT(int32_t, int32_t, int32_t);
  else if (c32 && b32) MNT_QT(int32_t, int32_t, int64_t);
  else if (c32 && o32) MNT_QT(int32_t, int64_t, int32_t);
  else if (c32) MNT_QT(int32_t, int64_t, int64_t);
  else if (b32 && o32) MNT_QT(int64_t, int32_t, int32_t);
  else if (b32) MNT_QT(int64_t, int32_t, int64_t);
  else if (o32) MNT_QT(int64_t, int64_t, int32_t);
  else MNT_QT(int64_t, int64_t, int64_t);
#undef MNT_QT
  check_launch("query_tuples_kernel");
  if (tile_counts != nullptr) {
    enqueue_count_tiles(kernel_map, out_dtype, num_offsets, a.num_targets, tile_counts, num_tiles, stream);
  }
}

// Runs the query into kernel_map (element type out_dtype) and, when tile_counts
// is given, the per-(offset, tile) hit counts.  offsets_host: int64 [O, ndim].
// With a sink the hits are staged for the pair lists instead and kernel_map
// is not touched (tile_counts is needed then).  Returns false, with nothing
// launched, when a sink was given but the frame is too wide for packed keys:
// the staged form needs them, the caller goes through a dense map instead.
static bool run_query(const QueryArgs &a, const int64_t *offsets_host, int64_t num_offsets,
                      const int64_t *source_bounds, const int64_t *target_bounds,
                      int64_t *bounds_out, void *kernel_map, int out_dtype, unsigned *tile_counts,
                      Scope &scope, hipStream_t stream, const HitSink *sink = nullptr) {
  const int num_tiles = static_cast<int>(div_ceil(a.num_targets, kTargetsPerTile));
  const bool batched = a.source_batch_dims != nullptr && a.num_batches > 1;
  profile_mark("enter:query", stream);
  long long bounds[16];
  resolve_bounds(a, source_bounds, target_bounds, bounds, bounds_out, scope, stream);
  profile_mark("query_bounds+sync", stream);
  QueryPlan plan = make_plan(bounds, bounds + 8, offsets_host, num_offsets, a.ndim,
                             batched ? a.num_batches : 1);
  if (!plan.fits) {
    if (sink != nullptr) return false;
    run_wide_query(a, offsets_host, num_offsets, batched, kernel_map, out_dtype, tile_counts, num_tiles,
                   scope, stream);
    profile_mark("query", stream);
    return true;
  }
  // Large tables are uploaded as kernel arguments of a tiny copy kernel: nothing
  // to keep alive on the host and no staging buffer another call could overwrite.
  const int no = static_cast<int>(num_offsets);
  MNT_CHECK(plan.tables.size() * sizeof(int) + sizeof(unsigned) * (num_offsets + 4) <= 24 * 1024,
            "too many kernel offsets (%lld) for the query kernel's table space",
            static_cast<long long>(num_offsets));
  int *d_tables = nullptr;                 // small tables ride in the kernel arguments
  if (plan.tables.size() > static_cast<size_t>(kCarriedInts)) {
    d_tables = scope.alloc<int>(plan.tables.size());
    upload_ints(plan.tables, d_tables, stream);
  }
  QueryArgs b = a;
  if (!batched) {
    b.source_batch_dims = nullptr;
    b.target_batch_dims = nullptr;
    b.num_batches = 1;
  }
  const bool c32 = a.coord_dtype == MNT_INT32;
  const bool b32 = !batched || a.batch_dtype == MNT_INT32;
  const bool o32 = out_dtype == MNT_INT32;
  if (sink != nullptr) {
#define MNT_QL(CT, BT)                                                                          \
  launch_query<CT, BT, int32_t, true>(b, plan, d_tables, no, nullptr, tile_counts, num_tiles, *sink, stream)
    if (c32 && b32) MNT_QL(int32_t, int32_t);
    else if (c32) MNT_QL(int32_t, int64_t);
    else if (b32) MNT_QL(int64_t, int32_t);
    else MNT_QL(int64_t, int64_t);
#undef MNT_QL
    profile_mark("query", stream);
    return true;
  }
  const HitSink none{nullptr, nullptr, nullptr, nullptr, 0, 0, nullptr, 1, 0};
#define MNT_Q(CT, BT, OT)                                                                        \
  launch_query<CT, BT, OT, false>(b, plan, d_tables, no, static_cast<OT *>(kernel_map), tile_counts, \
                                  num_tiles, none, stream)
  if (c32 && b32 && o32) MNT_Q(int32_t, int32_t, int32_t);
  else if (c32 && b32) MNT_Q(int32_t, int32_t, int64_t);
  else if (c32 && o32) MNT_Q(int32_t, int64_t, int32_t);
  else if (c32) MNT_Q(int32_t, int64_t, int64_t);
  else if (b32 && o32) MNT_Q(int64_t, int32_t, int32_t);
  else if (b32) MNT_Q(int64_t, int32_t, int64_t);
  else if (o32) MNT_Q(int64_t, int64_t, int32_t);
  else MNT_Q(int64_t, int64_t, int64_t);
#undef MNT_Q
  profile_mark("query", stream);
  return true;
}

template <typename T>
static void enqueue_fill(T *data, int64_t n, T value, hipStream_t stream) {
  if (n <= 0) return;
  fill_kernel<T><<<grid_for(n, 256 * 4, 8192), 256, 0, stream>>>(data, n, value);
  check_launch("fill_kernel");
}

static void enqueue_count_tiles(const void *kernel_map, int index_dtype, int64_t num_offsets,
                                int64_t num_targets, unsigned *tile_counts, int num_tiles,
                                hipStream_t stream) {
  dim3 grid(num_tiles, static_cast<unsigned>(num_offsets));
  if (index_dtype == MNT_INT32) {
    count_tiles_kernel<int32_t><<<grid, kQueryBlock, 0, stream>>>(
        static_cast<const int32_t *>(kernel_map), num_targets, tile_counts, num_tiles);
  } else {
    count_tiles_kernel<int64_t><<<grid, kQueryBlock, 0, stream>>>(
        static_cast<const int64_t *>(kernel_map), num_targets, tile_counts, num_tiles);
  }
  check_launch("count_tiles_kernel");
}

template <typename IT>
static void enqueue_emit(const IT *kernel_map, int64_t num_sources, int64_t num_targets,
                         int num_offsets, const unsigned *tile_bases, int num_tiles,
                         const unsigned *position_of, const unsigned *row_base, IT *source_masks,
                         IT *target_masks, int *in_idx, int *out_idx, hipStream_t stream,
                         const unsigned *plan = nullptr, int *sizes_out = nullptr,
                         int *order_out = nullptr) {
  if (source_masks) enqueue_fill<IT>(source_masks, static_cast<int64_t>(num_offsets) * num_sources, static_cast<IT>(-1), stream);
  if (num_offsets == 0) return;
  dim3 grid(num_tiles > 0 ? num_tiles : 1, static_cast<unsigned>(div_ceil(num_offsets, kQueryBlock / kWave)));
  emit_kernel<IT><<<grid, kQueryBlock, 0, stream>>>(kernel_map, num_sources, num_targets, num_offsets,
                                                   tile_bases, num_tiles, position_of, row_base,
                                                   source_masks, target_masks, in_idx, out_idx,
                                                   plan, sizes_out, order_out);
  check_launch("emit_kernel");
}

// persistent-state header of the two-phase kernel-map build
struct MapState {
  int64_t num_sources, num_targets, num_offsets;
  int num_tiles;
  int reorder;
  const void *kernel_map;
};

// Second half of the first phase of a kernel-map build: per-offset sizes and
// the stable size order from the per-tile hit counts, mirrored into pinned
// host memory (past the bounds slots), then the state the emit call reads.
static unsigned long long enqueue_sizes(Arena &arena, const MapState &state, unsigned *tile_counts,
                                        unsigned *row_sizes, unsigned *plan, hipStream_t stream) {
  const int64_t num_offsets = state.num_offsets;
  unsigned *d_plan_host = reinterpret_cast<unsigned *>(static_cast<char *>(arena.pinned_device()) + Arena::kPlanOffset);
  const unsigned long long sequence = arena.next_sequence();
  tile_scan_kernel<<<static_cast<unsigned>(num_offsets), 256, 0, stream>>>(tile_counts, state.num_tiles,
                                                                           row_sizes);
  check_launch("tile_scan_kernel");
  map_plan_kernel<<<1, 256, 0, stream>>>(row_sizes, static_cast<int>(num_offsets), state.reorder, plan,
                                         d_plan_host, arena.flag_device(1), sequence);
  check_launch("map_plan_kernel");
  return sequence;
}

// Waits for the sizes enqueued under `sequence` and hands them to the host arrays.
static void collect_sizes(Arena &arena, unsigned long long sequence, int64_t num_offsets,
                          int64_t *sizes_host_out, int64_t *order_host_out) {
  const unsigned *h_plan =
      reinterpret_cast<const unsigned *>(static_cast<char *>(arena.pinned()) + Arena::kPlanOffset);
  arena.wait_flag(1, sequence);
  for (int64_t j = 0; j < num_offsets; ++j) {
    order_host_out[j] = h_plan[j];
    sizes_host_out[j] = h_plan[2 * num_offsets + j];
  }
}

static void finish_sizes(Arena &arena, const MapState &state, unsigned *tile_counts,
                         unsigned *row_sizes, unsigned *plan, int64_t *sizes_host_out,
                         int64_t *order_host_out, hipStream_t stream) {
  const unsigned long long sequence = enqueue_sizes(arena, state, tile_counts, row_sizes, plan, stream);
  collect_sizes(arena, sequence, state.num_offsets, sizes_host_out, order_host_out);
  profile_mark("map_sizes_order+sync", stream);
  memcpy(arena.map_state, &state, sizeof(state));
  arena.map_state_valid = true;
}

}  // namespace mnt

using namespace mnt;

extern "C" int mnt_query_sorted_index_with_offsets(
    const void *sources, int64_t num_sources, const void *targets, int64_t num_targets,
    const void *offsets, int64_t num_offsets, int ndim, int coord_dtype,
    const void *source_batch_dims, const void *target_batch_dims, int64_t num_batches,
    int batch_dtype, void *kernel_map_out, int out_dtype, void *stream_) {
  return guarded([&] {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    QueryArgs a{sources, num_sources, targets, num_targets, ndim, coord_dtype,
                source_batch_dims, target_batch_dims, num_batches, batch_dtype};
    check_query_args(a, num_offsets);
    const int osz = int_size(out_dtype);
    if (num_targets == 0 || num_offsets == 0) return;
    MNT_CHECK(kernel_map_out != nullptr && offsets != nullptr, "null argument");
    if (num_sources == 0) {
      MNT_HIP(hipMemsetAsync(kernel_map_out, 0xFF, static_cast<size_t>(osz) * num_offsets * num_targets, stream));
      return;
    }
    Scope scope(stream);
    // offsets live on the device in the reference interface: bring them over
    const int csz = int_size(coord_dtype);
    std::vector<unsigned char> raw(static_cast<size_t>(csz) * num_offsets * ndim);
    MNT_HIP(hipMemcpyAsync(raw.data(), offsets, raw.size(), hipMemcpyDeviceToHost, stream));
    MNT_HIP(hipStreamSynchronize(stream));
    std::vector<int64_t> host_offsets(static_cast<size_t>(num_offsets) * ndim);
    for (size_t i = 0; i < host_offsets.size(); ++i) {
      host_offsets[i] = csz == 4 ? static_cast<int64_t>(reinterpret_cast<int32_t *>(raw.data())[i])
                                 : reinterpret_cast<int64_t *>(raw.data())[i];
    }
    run_query(a, host_offsets.data(), num_offsets, nullptr, nullptr, nullptr, kernel_map_out, out_dtype, nullptr, scope, stream);
  });
}

extern "C" int mnt_compute_kernel_map_sizes(const void *kernel_map, int64_t num_offsets,
                                            int64_t num_targets, int index_dtype,
                                            void *sizes_out, void *stream_) {
  return guarded([&] {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const int isz = int_size(index_dtype);
    MNT_CHECK(num_offsets >= 0 && num_targets >= 0 && num_targets <= INT32_MAX, "bad shape");
    if (num_offsets == 0) return;
    if (num_targets == 0) {
      MNT_HIP(hipMemsetAsync(sizes_out, 0, static_cast<size_t>(isz) * num_offsets, stream));
      return;
    }
    Scope scope(stream);
    const int num_tiles = static_cast<int>(div_ceil(num_targets, kTargetsPerTile));
    unsigned *tile_counts = scope.alloc<unsigned>(static_cast<size_t>(num_offsets) * num_tiles);
    unsigned *row_sizes = scope.alloc<unsigned>(num_offsets);
    enqueue_count_tiles(kernel_map, index_dtype, num_offsets, num_targets, tile_counts, num_tiles, stream);
    tile_scan_kernel<<<static_cast<unsigned>(num_offsets), 256, 0, stream>>>(tile_counts, num_tiles, row_sizes);
    check_launch("tile_scan_kernel");
    const unsigned grid = grid_for(num_offsets, 256);
    if (index_dtype == MNT_INT32) {
      export_sizes_kernel<int32_t><<<grid, 256, 0, stream>>>(row_sizes, static_cast<int>(num_offsets), static_cast<int32_t *>(sizes_out));
    } else {
      export_sizes_kernel<int64_t><<<grid, 256, 0, stream>>>(row_sizes, static_cast<int>(num_offsets), static_cast<int64_t *>(sizes_out));
    }
    check_launch("export_sizes_kernel");
  });
}

extern "C" int mnt_compute_kernel_map_masks(const void *kernel_map, int64_t num_offsets,
                                            int64_t num_sources, int64_t num_targets,
                                            int index_dtype, void *source_masks_out,
                                            void *target_masks_out, void *stream_) {
  return guarded([&] {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    int_size(index_dtype);
    MNT_CHECK(num_offsets >= 0 && num_offsets <= 65535 && num_targets >= 0 && num_targets <= INT32_MAX &&
                  num_sources >= 0 && num_sources <= INT32_MAX,
              "bad shape");
    if (num_offsets == 0) return;
    Scope scope(stream);
    const int num_tiles = static_cast<int>(div_ceil(num_targets > 0 ? num_targets : 1, kTargetsPerTile));
    unsigned *tile_counts = scope.alloc<unsigned>(static_cast<size_t>(num_offsets) * num_tiles);
    unsigned *row_sizes = scope.alloc<unsigned>(num_offsets);
    if (num_targets > 0) {
      enqueue_count_tiles(kernel_map, index_dtype, num_offsets, num_targets, tile_counts, num_tiles, stream);
      tile_scan_kernel<<<static_cast<unsigned>(num_offsets), 256, 0, stream>>>(tile_counts, num_tiles, row_sizes);
      check_launch("tile_scan_kernel");
    }
    if (index_dtype == MNT_INT32) {
      enqueue_emit<int32_t>(static_cast<const int32_t *>(kernel_map), num_sources, num_targets,
                            static_cast<int>(num_offsets), tile_counts, num_tiles, nullptr, nullptr,
                            static_cast<int32_t *>(source_masks_out),
                            static_cast<int32_t *>(target_masks_out), nullptr, nullptr, stream);
    } else {
      enqueue_emit<int64_t>(static_cast<const int64_t *>(kernel_map), num_sources, num_targets,
                            static_cast<int>(num_offsets), tile_counts, num_tiles, nullptr, nullptr,
                            static_cast<int64_t *>(source_masks_out),
                            static_cast<int64_t *>(target_masks_out), nullptr, nullptr, stream);
    }
  });
}

extern "C" int mnt_kernel_map_pair_lists(const int32_t *kernel_map, int64_t num_offsets,
                                         int64_t num_targets, const int64_t *cumsum_host,
                                         int32_t *in_idx_out, int32_t *out_idx_out,
                                         void *stream_) {
  return guarded([&] {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    MNT_CHECK(num_offsets >= 0 && num_offsets <= 65535 && num_targets >= 0 && num_targets <= INT32_MAX, "bad shape");
    if (num_offsets == 0 || num_targets == 0) return;
    MNT_CHECK(cumsum_host != nullptr && in_idx_out != nullptr && out_idx_out != nullptr, "null argument");
    Scope scope(stream);
    const int num_tiles = static_cast<int>(div_ceil(num_targets, kTargetsPerTile));
    unsigned *tile_counts = scope.alloc<unsigned>(static_cast<size_t>(num_offsets) * num_tiles);
    unsigned *row_sizes = scope.alloc<unsigned>(num_offsets);
    unsigned *row_base = scope.alloc<unsigned>(num_offsets + 1);
    std::vector<unsigned> base(num_offsets + 1);
    for (int64_t o = 0; o <= num_offsets; ++o) base[o] = static_cast<unsigned>(cumsum_host[o]);
    MNT_HIP(hipMemcpyAsync(row_base, base.data(), sizeof(unsigned) * (num_offsets + 1), hipMemcpyHostToDevice, stream));
    enqueue_count_tiles(kernel_map, MNT_INT32, num_offsets, num_targets, tile_counts, num_tiles, stream);
    tile_scan_kernel<<<static_cast<unsigned>(num_offsets), 256, 0, stream>>>(tile_counts, num_tiles, row_sizes);
    check_launch("tile_scan_kernel");
    enqueue_emit<int32_t>(kernel_map, 0, num_targets, static_cast<int>(num_offsets), tile_counts,
                          num_tiles, nullptr, row_base, nullptr, nullptr, in_idx_out, out_idx_out, stream);
    MNT_HIP(hipStreamSynchronize(stream));   // `base` is pageable host memory
  });
}

extern "C" int mnt_kernel_map_query(const void *sources, int64_t num_sources, const void *targets,
                                    int64_t num_targets, const int64_t *offsets_host,
                                    int64_t num_offsets, int ndim, int coord_dtype,
                                    const void *source_batch_dims, const void *target_batch_dims,
                                    int64_t num_batches, int batch_dtype, int reorder,
                                    const int64_t *source_bounds_host,
                                    const int64_t *target_bounds_host, int64_t *bounds_host_out,
                                    int32_t *kernel_map_out, int64_t *sizes_host_out,
                                    int64_t *order_host_out, void *stream_) {
  return guarded([&] {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    QueryArgs a{sources, num_sources, targets, num_targets, ndim, coord_dtype,
                source_batch_dims, target_batch_dims, num_batches, batch_dtype};
    check_query_args(a, num_offsets);
    MNT_CHECK(offsets_host != nullptr && sizes_host_out != nullptr && order_host_out != nullptr, "null argument");
    Arena &arena = Arena::of(stream);
    const int num_tiles = static_cast<int>(div_ceil(num_targets > 0 ? num_targets : 1, kTargetsPerTile));
    // persistent block: MapState | tile bases [O*tiles] | row sizes [O] | plan [4*O+1]
    const size_t words = static_cast<size_t>(num_offsets) * num_tiles + num_offsets + 4 * num_offsets + 1;
    char *keep = static_cast<char *>(arena.persistent(1, 256 + words * sizeof(unsigned)));
    unsigned *tile_counts = reinterpret_cast<unsigned *>(keep + 256);
    unsigned *row_sizes = tile_counts + static_cast<size_t>(num_offsets) * num_tiles;
    unsigned *plan = row_sizes + num_offsets;
    MapState state{num_sources, num_targets, num_offsets, num_tiles, reorder, kernel_map_out};
    arena.map_state_valid = false;
    if (bounds_host_out != nullptr) {
      for (int i = 0; i < 16; ++i) bounds_host_out[i] = (i & 4) ? INT64_MIN : INT64_MAX;
    }
    if (num_offsets == 0) {
      memcpy(arena.map_state, &state, sizeof(state));
      arena.map_state_valid = true;
      return;
    }
    MNT_CHECK(sizeof(unsigned) * 3 * num_offsets + 1024 <= Arena::kPinnedBytes,
              "too many kernel offsets (%lld)", static_cast<long long>(num_offsets));
    if (num_targets == 0 || num_sources == 0) {
      if (num_targets > 0) {
        MNT_CHECK(kernel_map_out != nullptr, "kernel_map_out is null");
        MNT_HIP(hipMemsetAsync(kernel_map_out, 0xFF, sizeof(int32_t) * num_offsets * num_targets, stream));
      }
      MNT_HIP(hipMemsetAsync(tile_counts, 0, words * sizeof(unsigned), stream));
    } else {
      MNT_CHECK(kernel_map_out != nullptr, "kernel_map_out is null");
      Scope scope(stream);
      run_query(a, offsets_host, num_offsets, source_bounds_host, target_bounds_host, bounds_host_out,
                kernel_map_out, MNT_INT32, tile_counts, scope, stream);
    }
    finish_sizes(arena, state, tile_counts, row_sizes, plan, sizes_host_out, order_host_out, stream);
  });
}

extern "C" int mnt_kernel_map_build(const void *sources, int64_t num_sources, const void *targets,
                                    int64_t num_targets, const int64_t *offsets_host,
                                    int64_t num_offsets, int ndim, int coord_dtype,
                                    const void *source_batch_dims, const void *target_batch_dims,
                                    int64_t num_batches, int batch_dtype, int reorder,
                                    const int64_t *source_bounds_host,
                                    const int64_t *target_bounds_host, int64_t *bounds_host_out,
                                    int32_t *kernel_map_out, int32_t *source_masks_out,
                                    int32_t *target_masks_out, int32_t *in_idx_out,
                                    int32_t *out_idx_out, int64_t list_capacity,
                                    int32_t *sizes_dev_out, int32_t *order_dev_out,
                                    int64_t *sizes_host_out, int64_t *order_host_out, void *stream_) {
  return guarded([&] {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    QueryArgs a{sources, num_sources, targets, num_targets, ndim, coord_dtype,
                source_batch_dims, target_batch_dims, num_batches, batch_dtype};
    check_query_args(a, num_offsets);
    MNT_CHECK(offsets_host != nullptr && sizes_host_out != nullptr && order_host_out != nullptr, "null argument");
    MNT_CHECK(num_sources > 0 && num_targets > 0 && num_offsets > 0,
              "mnt_kernel_map_build needs sources, targets and offsets (use mnt_kernel_map_query / _emit "
              "for empty operands)");
    MNT_CHECK(kernel_map_out != nullptr, "kernel_map_out is null");
    MNT_CHECK((in_idx_out == nullptr) == (out_idx_out == nullptr), "in_idx_out and out_idx_out go together");
    MNT_CHECK(in_idx_out == nullptr || list_capacity >= num_offsets * num_targets,
              "list_capacity = %lld cannot hold every (offset, target) pair (%lld)",
              (long long)list_capacity, (long long)(num_offsets * num_targets));
    MNT_CHECK(sizeof(unsigned) * 3 * num_offsets + 1024 <= Arena::kPinnedBytes,
              "too many kernel offsets (%lld)", static_cast<long long>(num_offsets));
    Arena &arena = Arena::of(stream);
    arena.map_state_valid = false;
    const int num_tiles = static_cast<int>(div_ceil(num_targets, kTargetsPerTile));
    const size_t words = static_cast<size_t>(num_offsets) * num_tiles + num_offsets + 4 * num_offsets + 1;
    char *keep = static_cast<char *>(arena.persistent(1, 256 + words * sizeof(unsigned)));
    unsigned *tile_counts = reinterpret_cast<unsigned *>(keep + 256);
    unsigned *row_sizes = tile_counts + static_cast<size_t>(num_offsets) * num_tiles;
    unsigned *plan = row_sizes + num_offsets;
    const MapState state{num_sources, num_targets, num_offsets, num_tiles, reorder, kernel_map_out};
    if (bounds_host_out != nullptr) {
      for (int i = 0; i < 16; ++i) bounds_host_out[i] = (i & 4) ? INT64_MIN : INT64_MAX;
    }
    {
      Scope scope(stream);
      run_query(a, offsets_host, num_offsets, source_bounds_host, target_bounds_host, bounds_host_out,
                kernel_map_out, MNT_INT32, tile_counts, scope, stream);
    }
    // the tables are written while the host waits for the sizes
    const unsigned long long sequence = enqueue_sizes(arena, state, tile_counts, row_sizes, plan, stream);
    const int no = static_cast<int>(num_offsets);
    enqueue_emit<int32_t>(kernel_map_out, num_sources, num_targets, no, tile_counts, num_tiles, plan + no,
                          plan + 3 * no, source_masks_out, target_masks_out, in_idx_out, out_idx_out,
                          stream, plan, sizes_dev_out, order_dev_out);
    collect_sizes(arena, sequence, num_offsets, sizes_host_out, order_host_out);
    profile_mark("map_sizes_order+emit+sync", stream);
  });
}

extern "C" int mnt_kernel_map_lists(const void *sources, int64_t num_sources, const void *targets,
                                    int64_t num_targets, const int64_t *offsets_host,
                                    int64_t num_offsets, int ndim, int coord_dtype,
                                    const void *source_batch_dims, const void *target_batch_dims,
                                    int64_t num_batches, int batch_dtype, int reorder,
                                    const int64_t *source_bounds_host,
                                    const int64_t *target_bounds_host, int64_t *bounds_host_out,
                                    int32_t *in_idx_out, int32_t *out_idx_out, int64_t list_capacity,
                                    int32_t *sizes_dev_out, int32_t *order_dev_out,
                                    int64_t *sizes_host_out, int64_t *order_host_out, void *stream_) {
  return guarded([&] {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    QueryArgs a{sources, num_sources, targets, num_targets, ndim, coord_dtype,
                source_batch_dims, target_batch_dims, num_batches, batch_dtype};
    check_query_args(a, num_offsets);
    MNT_CHECK(offsets_host != nullptr && sizes_host_out != nullptr && order_host_out != nullptr, "null argument");
    MNT_CHECK(num_sources > 0 && num_targets > 0 && num_offsets > 0,
              "mnt_kernel_map_lists needs sources, targets and offsets (use mnt_kernel_map_query / _emit "
              "for empty operands)");
    MNT_CHECK(in_idx_out != nullptr && out_idx_out != nullptr, "in_idx_out / out_idx_out is null");
    MNT_CHECK(list_capacity >= num_offsets * num_targets,
              "list_capacity = %lld cannot hold every (offset, target) pair (%lld)",
              (long long)list_capacity, (long long)(num_offsets * num_targets));
    MNT_CHECK(sizeof(unsigned) * 3 * num_offsets + 1024 <= Arena::kPinnedBytes,
              "too many kernel offsets (%lld)", static_cast<long long>(num_offsets));
    Arena &arena = Arena::of(stream);
    arena.map_state_valid = false;
    if (bounds_host_out != nullptr) {
      for (int i = 0; i < 16; ++i) bounds_host_out[i] = (i & 4) ? INT64_MIN : INT64_MAX;
    }
    Scope scope(stream);
    const int no = static_cast<int>(num_offsets);
    const int num_tiles = static_cast<int>(div_ceil(num_targets, kTargetsPerTile));
    const int64_t num_wave_tiles = div_ceil(num_targets, kWave);
    int *stage = scope.alloc<int>(static_cast<size_t>(num_offsets) * num_targets);
    unsigned long long *masks = scope.alloc<unsigned long long>(static_cast<size_t>(num_offsets) * num_wave_tiles);
    unsigned *tile_counts = scope.alloc<unsigned>(static_cast<size_t>(num_offsets) * num_tiles);
    unsigned *tile_mode = scope.alloc<unsigned>(num_tiles);
    unsigned *row_totals = scope.alloc<unsigned>(num_offsets);
    unsigned *plan = scope.alloc<unsigned>(4 * num_offsets + 1);
    enqueue_fill<unsigned>(row_totals, num_offsets, 0u, stream);
    const HitSink sink{stage, masks, row_totals, tile_mode, num_wave_tiles, no, nullptr, 1, no};
    if (!run_query(a, offsets_host, num_offsets, source_bounds_host, target_bounds_host, bounds_host_out,
                   nullptr, MNT_INT32, tile_counts, scope, stream, &sink)) {
      // a frame too wide for packed keys: dense map by tuple comparisons (the
      // staging block has the right size for it), then the lists from that map
      int64_t known[16];
      if (bounds_host_out != nullptr) memcpy(known, bounds_host_out, sizeof(known));
      const int64_t *src_known = bounds_host_out != nullptr ? known : source_bounds_host;
      const int64_t *tgt_known = bounds_host_out != nullptr ? known + 8 : target_bounds_host;
      run_query(a, offsets_host, num_offsets, src_known, tgt_known, nullptr, stage, MNT_INT32, tile_counts,
                scope, stream);
      unsigned *row_sizes = scope.alloc<unsigned>(num_offsets);
      const MapState state{num_sources, num_targets, num_offsets, num_tiles, reorder, stage};
      const unsigned long long sequence = enqueue_sizes(arena, state, tile_counts, row_sizes, plan, stream);
      enqueue_emit<int32_t>(stage, num_sources, num_targets, no, tile_counts, num_tiles, plan + no, plan + 3 * no,
                            nullptr, nullptr, in_idx_out, out_idx_out, stream, plan, sizes_dev_out,
                            order_dev_out);
      collect_sizes(arena, sequence, num_offsets, sizes_host_out, order_host_out);
      profile_mark("map_sizes_order+emit+sync", stream);
      return;
    }
    unsigned *d_plan_host = reinterpret_cast<unsigned *>(static_cast<char *>(arena.pinned_device()) + Arena::kPlanOffset);
    const unsigned long long sequence = arena.next_sequence();
    dim3 grid(static_cast<unsigned>(div_ceil(num_tiles, kPlaceTiles)), static_cast<unsigned>(num_offsets));
    place_kernel<false><<<grid, kPlaceBlock, 0, stream>>>(stage, masks, tile_counts, row_totals, tile_mode,
                                                   num_targets, no, num_tiles, num_wave_tiles, reorder,
                                                   in_idx_out, out_idx_out, plan, d_plan_host,
                                                   arena.flag_device(1), sequence, sizes_dev_out,
                                                   order_dev_out, nullptr, nullptr, nullptr, nullptr, 1, no);
    check_launch("place_kernel");
    collect_sizes(arena, sequence, num_offsets, sizes_host_out, order_host_out);
    profile_mark("map_place+sync", stream);
  });
}

// ---- sort -> query -> pair lists as one chain of six launches and one wait ----

namespace mnt {

static int total_copies() {
  static const int value = [] {
    const char *text = getenv("MINUET_TOTAL_COPIES");
    const int v = text != nullptr && *text != 0 ? atoi(text) : 4;
    return v < 1 ? 1 : v > kMaxTotalCopies ? kMaxTotalCopies : v;
  }();
  return value;
}

// MINUET_MAP_HALVES=0 looks every offset up (for comparisons).
static bool map_halves_enabled() {
  static const bool value = [] {
    const char *text = getenv("MINUET_MAP_HALVES");
    return text == nullptr || *text == 0 || atoi(text) != 0;
  }();
  return value;
}

constexpr size_t kChainHostOffset = 128;      // pinned block: bounds (8 words), then the chain's verdict

template <typename CT>
static void launch_query_chain(const CT *sorted, int64_t n, int ndim, int num_offsets,
                               unsigned *tile_counts, int num_tiles, const HitSink &sink,
                               const DevicePlan *plan, hipStream_t stream) {
  KeyReader<CT, int32_t> rows{sorted, nullptr, 1, n};
  Frame frame;
  memset(&frame, 0, sizeof(frame));
  frame.ndim = ndim;
  CarriedTables carried;
  memset(&carried, 0, sizeof(carried));
  // LDS for the largest tables these offsets can make and for the row directory
  const size_t dyn = sizeof(unsigned) * (6 * static_cast<size_t>(num_offsets) + num_offsets + 4) +
                     sizeof(unsigned short) * static_cast<size_t>(kDirectoryRows);
  query_kernel<CT, int32_t, int32_t, true><<<num_tiles, kQueryThreads, dyn, stream>>>(
      rows, rows, frame, nullptr, carried, 0, num_offsets, 0, 0, nullptr, tile_counts, num_tiles,
      kDirectoryRows, sink, plan);
  check_launch("query_kernel");
}

}  // namespace mnt

extern "C" int mnt_sorted_kernel_map_lists(const void *coords, int64_t n, int ndim, int coord_dtype,
                                           const int64_t *offsets_host, int64_t num_offsets,
                                           int reorder, int32_t *indices_out, void *sorted_coords_out,
                                           int32_t *in_idx_out, int32_t *out_idx_out,
                                           int64_t list_capacity, int32_t *sizes_dev_out,
                                           int32_t *order_dev_out, int64_t *bounds_host_out,
                                           int64_t *sizes_host_out, int64_t *order_host_out,
                                           void *stream_) {
  return guarded([&] {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    MNT_CHECK(ndim >= 1 && ndim <= MNT_MAX_NDIM, "ndim must be in [1, %d] but found %d", MNT_MAX_NDIM, ndim);
    MNT_CHECK(n > 0 && n <= INT32_MAX, "number of coordinates %lld out of range", static_cast<long long>(n));
    MNT_CHECK(num_offsets > 0 && num_offsets <= 65535, "number of offsets %lld out of range",
              static_cast<long long>(num_offsets));
    int_size(coord_dtype);
    MNT_CHECK(coords != nullptr && offsets_host != nullptr && indices_out != nullptr &&
                  sorted_coords_out != nullptr && in_idx_out != nullptr && out_idx_out != nullptr &&
                  bounds_host_out != nullptr && sizes_host_out != nullptr && order_host_out != nullptr,
              "null argument");
    MNT_CHECK(list_capacity >= num_offsets * n,
              "list_capacity = %lld cannot hold every (offset, target) pair (%lld)",
              (long long)list_capacity, (long long)(num_offsets * n));
    bool small_offsets = true;
    for (int64_t i = 0; i < num_offsets * ndim; ++i) {
      small_offsets = small_offsets && offsets_host[i] >= INT32_MIN / 2 && offsets_host[i] <= INT32_MAX / 2;
    }
    if (small_offsets && chain_sort_takes(n, 1, static_cast<int>(num_offsets))) {
      profile_mark("enter:map_chain", stream);
      Arena &arena = Arena::of(stream);
      arena.map_state_valid = false;
      Scope scope(stream);
      const int no = static_cast<int>(num_offsets);
      const int buckets = 1 << chain_sort_msd_bits(n);
      const int num_tiles = static_cast<int>(div_ceil(n, kTargetsPerTile));
      const int64_t num_wave_tiles = div_ceil(n, kWave);
      ChainSortBuffers buf;
      buf.partial = scope.alloc<long long>(128 * 8);
      buf.folded = scope.alloc<long long>(2 * MNT_MAX_NDIM);
      // bucket totals, cursors, the copies of the hits per offset, the equal-rows flag
      // (and the sort's status words, which must start at zero like the rest)
      buf.counter_words = 2 * buckets + kMaxTotalCopies * kPlanMaxOffsets + 1 + 4;
      buf.counters = scope.alloc<unsigned>(buf.counter_words);
      buf.info = scope.alloc<unsigned>(4);
      buf.status = buf.counters + (buf.counter_words - 4);
      buf.chunks = scope.alloc<uint4>(chain_sort_max_pairs(n));
      buf.words = scope.alloc<unsigned long long>(chain_sort_words(n));
      buf.starts = scope.alloc<unsigned>(buckets + 1);
      buf.plan = scope.alloc<DevicePlan>(1);
      unsigned *row_totals = buf.counters + 2 * buckets;
      int *stage = scope.alloc<int>(static_cast<size_t>(num_offsets) * n);
      unsigned long long *masks = scope.alloc<unsigned long long>(static_cast<size_t>(num_offsets) * num_wave_tiles);
      unsigned *tile_counts = scope.alloc<unsigned>(static_cast<size_t>(num_offsets) * num_tiles);
      unsigned *tile_mode = scope.alloc<unsigned>(num_tiles);
      unsigned *plan = scope.alloc<unsigned>(4 * num_offsets + 1);
      OffsetTable table;
      memset(&table, 0, sizeof(table));
      for (int o = 0; o < no; ++o) {
        for (int k = 0; k < ndim; ++k) table.v[o][k] = static_cast<int>(offsets_host[o * ndim + k]);
      }
      // the cloud is mapped onto itself: offsets that come in pairs d / -d need one look-up per pair
      classify_offset_pairs(table, no, ndim, map_halves_enabled());
      int num_rows = 0;                            // offsets with rows of their own to write (DevicePlan::rows)
      for (int o = 0; o < no; ++o) num_rows += table.kind[o] != 1 ? 1 : 0;
      enqueue_chain_sort(coords, n, ndim, coord_dtype, indices_out, sorted_coords_out, buf, table, no, stream);
      unsigned *repeats = row_totals + kMaxTotalCopies * kPlanMaxOffsets;
      const HitSink sink{stage, masks, row_totals, tile_mode, num_wave_tiles, no, repeats, total_copies(),
                         kPlanMaxOffsets};
      char *pinned_device = static_cast<char *>(arena.pinned_device());
      unsigned *d_plan_host = reinterpret_cast<unsigned *>(pinned_device + Arena::kPlanOffset);
      long long *d_chain_host = reinterpret_cast<long long *>(pinned_device + kChainHostOffset);
      const unsigned long long sequence = arena.next_sequence();
      if (coord_dtype == MNT_INT32) {
        launch_query_chain<int32_t>(static_cast<const int32_t *>(sorted_coords_out), n, ndim, no, tile_counts,
                                    num_tiles, sink, buf.plan, stream);
      } else {
        launch_query_chain<int64_t>(static_cast<const int64_t *>(sorted_coords_out), n, ndim, no, tile_counts,
                                    num_tiles, sink, buf.plan, stream);
      }
      profile_mark("query", stream);
      // a workgroup per four tiles and per offset that is looked up (or is the zero offset); row 0 tells the host
      dim3 grid(static_cast<unsigned>(div_ceil(num_tiles, kPlaceTiles)), static_cast<unsigned>(num_rows + 1));
      place_kernel<true><<<grid, kPlaceBlock, 0, stream>>>(stage, masks, tile_counts, row_totals, tile_mode, n, no,
                                                     num_tiles, num_wave_tiles, reorder, in_idx_out,
                                                     out_idx_out, plan, d_plan_host, arena.flag_device(1),
                                                     sequence, sizes_dev_out, order_dev_out, buf.plan,
                                                     buf.folded, d_chain_host, repeats, total_copies(), kPlanMaxOffsets);
      check_launch("place_kernel");
      arena.wait_flag(1, sequence);
      const long long *h_chain = reinterpret_cast<const long long *>(static_cast<char *>(arena.pinned()) + kChainHostOffset);
      profile_mark("map_place+sync", stream);
      if (h_chain[2 * MNT_MAX_NDIM] == 0) {
        const unsigned *h_plan = reinterpret_cast<const unsigned *>(static_cast<char *>(arena.pinned()) + Arena::kPlanOffset);
        for (int64_t j = 0; j < num_offsets; ++j) {
          order_host_out[j] = h_plan[j];
          sizes_host_out[j] = h_plan[2 * num_offsets + j];
        }
        memcpy(bounds_host_out, h_chain, sizeof(long long) * 2 * MNT_MAX_NDIM);
        return;
      }
      // the chain declined (strong clustering, keys too wide): the calls below start over
    }
    if (mnt_arg_sort_coordinates(coords, n, ndim, coord_dtype, nullptr, 1, MNT_INT32, indices_out,
                                 sorted_coords_out, bounds_host_out, stream_) != 0) {
      throw Error{mnt_last_error()};
    }
    if (mnt_kernel_map_lists(sorted_coords_out, n, sorted_coords_out, n, offsets_host, num_offsets, ndim,
                             coord_dtype, nullptr, nullptr, 1, MNT_INT32, reorder, bounds_host_out,
                             bounds_host_out, nullptr, in_idx_out, out_idx_out, list_capacity,
                             sizes_dev_out, order_dev_out, sizes_host_out, order_host_out, stream_) != 0) {
      throw Error{mnt_last_error()};
    }
  });
}

extern "C" int mnt_kernel_map_row_lists(const int32_t *kernel_map, int64_t num_offsets,
                                        int64_t num_targets, const int64_t *sizes_host,
                                        const int64_t *order_host, int32_t *row_ptr_out,
                                        int32_t *out_pos_out, void *stream_) {
  return guarded([&] {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    MNT_CHECK(num_offsets >= 0 && num_offsets <= 1024 && num_targets >= 0 && num_targets <= INT32_MAX,
              "bad shape O=%lld T=%lld (at most 1024 offsets)", (long long)num_offsets, (long long)num_targets);
    MNT_CHECK(row_ptr_out != nullptr, "row_ptr_out is null");
    if (num_targets == 0 || num_offsets == 0) {
      enqueue_fill<int32_t>(row_ptr_out, num_targets + 1, 0, stream);
      return;
    }
    MNT_CHECK(kernel_map != nullptr && sizes_host != nullptr, "null argument");
    int64_t nnz = 0;
    std::vector<int> tables(2 * num_offsets);
    std::vector<char> seen(num_offsets, 0);
    for (int64_t j = 0; j < num_offsets; ++j) {
      const int64_t o = order_host != nullptr ? order_host[j] : j;
      MNT_CHECK(o >= 0 && o < num_offsets && !seen[o], "order_host is not a permutation of the offsets");
      seen[o] = 1;
      MNT_CHECK(sizes_host[j] >= 0 && sizes_host[j] <= num_targets, "size of list row %lld is out of range",
                (long long)j);
      tables[j] = static_cast<int>(o);
      tables[num_offsets + j] = static_cast<int>(nnz);
      nnz += sizes_host[j];
    }
    MNT_CHECK(nnz <= INT32_MAX, "more than 2^31 - 1 hits");
    MNT_CHECK(nnz == 0 || out_pos_out != nullptr, "out_pos_out is null");
    Scope scope(stream);
    const int num_tiles = static_cast<int>(div_ceil(num_targets, kTargetsPerTile));
    unsigned *tile_counts = scope.alloc<unsigned>(static_cast<size_t>(num_offsets) * num_tiles);
    unsigned *row_sizes = scope.alloc<unsigned>(num_offsets);
    int *d_tables = scope.alloc<int>(tables.size());
    upload_ints(tables, d_tables, stream);
    enqueue_count_tiles(kernel_map, MNT_INT32, num_offsets, num_targets, tile_counts, num_tiles, stream);
    tile_scan_kernel<<<static_cast<unsigned>(num_offsets), 256, 0, stream>>>(tile_counts, num_tiles, row_sizes);
    check_launch("tile_scan_kernel");
    const size_t lds = static_cast<size_t>(num_offsets) * (kQueryThreads / kWave) * (sizeof(unsigned long long) + sizeof(unsigned)) +
                       static_cast<size_t>(num_offsets) * sizeof(unsigned) + 64;
    row_lists_kernel<<<num_tiles, kQueryThreads, lds, stream>>>(kernel_map, num_targets,
                                                                static_cast<int>(num_offsets), tile_counts,
                                                                num_tiles, d_tables, row_ptr_out, out_pos_out);
    check_launch("row_lists_kernel");
  });
}

extern "C" int mnt_kernel_map_dense(const void *sources, int64_t num_sources, const void *targets,
                                    int64_t num_targets, const int64_t *offsets_host,
                                    int64_t num_offsets, int ndim, int coord_dtype,
                                    const void *source_batch_dims, const void *target_batch_dims,
                                    int64_t num_batches, int batch_dtype,
                                    const int64_t *source_bounds_host,
                                    const int64_t *target_bounds_host, int64_t *bounds_host_out,
                                    int32_t *kernel_map_out, void *stream_) {
  return guarded([&] {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    QueryArgs a{sources, num_sources, targets, num_targets, ndim, coord_dtype,
                source_batch_dims, target_batch_dims, num_batches, batch_dtype};
    check_query_args(a, num_offsets);
    MNT_CHECK(offsets_host != nullptr, "null argument");
    if (bounds_host_out != nullptr) {
      for (int i = 0; i < 16; ++i) bounds_host_out[i] = (i & 4) ? INT64_MIN : INT64_MAX;
    }
    if (num_offsets == 0 || num_targets == 0) return;
    MNT_CHECK(kernel_map_out != nullptr, "kernel_map_out is null");
    if (num_sources == 0) {
      enqueue_fill<int32_t>(kernel_map_out, num_offsets * num_targets, -1, stream);
      return;
    }
    Scope scope(stream);
    run_query(a, offsets_host, num_offsets, source_bounds_host, target_bounds_host, bounds_host_out,
              kernel_map_out, MNT_INT32, nullptr, scope, stream);
  });
}

extern "C" int mnt_kernel_map_tables(const int32_t *kernel_map, int64_t num_sources,
                                     int64_t num_targets, int64_t num_offsets, int reorder,
                                     int64_t *sizes_host_out, int64_t *order_host_out,
                                     void *stream_) {
  return guarded([&] {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    MNT_CHECK(num_sources >= 0 && num_targets >= 0 && num_offsets >= 0 && num_sources <= INT32_MAX &&
                  num_targets <= INT32_MAX && num_offsets <= 65535,
              "bad shape S=%lld T=%lld O=%lld", (long long)num_sources, (long long)num_targets,
              (long long)num_offsets);
    MNT_CHECK(sizes_host_out != nullptr && order_host_out != nullptr, "null argument");
    Arena &arena = Arena::of(stream);
    const int num_tiles = static_cast<int>(div_ceil(num_targets > 0 ? num_targets : 1, kTargetsPerTile));
    const size_t words = static_cast<size_t>(num_offsets) * num_tiles + num_offsets + 4 * num_offsets + 1;
    char *keep = static_cast<char *>(arena.persistent(1, 256 + words * sizeof(unsigned)));
    unsigned *tile_counts = reinterpret_cast<unsigned *>(keep + 256);
    unsigned *row_sizes = tile_counts + static_cast<size_t>(num_offsets) * num_tiles;
    unsigned *plan = row_sizes + num_offsets;
    MapState state{num_sources, num_targets, num_offsets, num_tiles, reorder, kernel_map};
    arena.map_state_valid = false;
    if (num_offsets == 0) {
      memcpy(arena.map_state, &state, sizeof(state));
      arena.map_state_valid = true;
      return;
    }
    MNT_CHECK(sizeof(unsigned) * 3 * num_offsets + 1024 <= Arena::kPinnedBytes,
              "too many kernel offsets (%lld)", static_cast<long long>(num_offsets));
    if (num_targets == 0) {
      enqueue_fill<unsigned>(tile_counts, static_cast<int64_t>(words), 0u, stream);
    } else {
      MNT_CHECK(kernel_map != nullptr, "kernel_map is null");
      enqueue_count_tiles(kernel_map, MNT_INT32, num_offsets, num_targets, tile_counts, num_tiles, stream);
    }
    finish_sizes(arena, state, tile_counts, row_sizes, plan, sizes_host_out, order_host_out, stream);
  });
}

extern "C" int mnt_kernel_map_emit(int32_t *source_masks_out, int32_t *target_masks_out,
                                   int32_t *in_idx_out, int32_t *out_idx_out,
                                   int32_t *sizes_dev_out, int32_t *order_dev_out, void *stream_) {
  return guarded([&] {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    Arena &arena = Arena::of(stream);
    MNT_CHECK(arena.map_state_valid, "mnt_kernel_map_emit called without a preceding mnt_kernel_map_query");
    MapState state;
    memcpy(&state, arena.map_state, sizeof(state));
    arena.map_state_valid = false;
    MNT_CHECK((in_idx_out == nullptr) == (out_idx_out == nullptr), "in_idx_out and out_idx_out go together");
    if (state.num_offsets == 0) return;
    char *keep = static_cast<char *>(arena.persistent(1, 0));
    unsigned *tile_bases = reinterpret_cast<unsigned *>(keep + 256);
    unsigned *row_sizes = tile_bases + static_cast<size_t>(state.num_offsets) * state.num_tiles;
    unsigned *plan = row_sizes + state.num_offsets;
    const int no = static_cast<int>(state.num_offsets);
    profile_mark("enter:emit", stream);
    enqueue_emit<int32_t>(static_cast<const int32_t *>(state.kernel_map), state.num_sources,
                          state.num_targets, no, tile_bases, state.num_tiles, plan + no,
                          plan + 3 * no, source_masks_out, target_masks_out, in_idx_out, out_idx_out,
                          stream, plan, sizes_dev_out, order_dev_out);
    profile_mark("map_emit", stream);
  });
}

// ---- the sizes of a kernel map without any allocation ------------------------
//
// Same kernels as mnt_compute_kernel_map_sizes; the per-(row, tile) hit counts
// and the row totals live in a file-scope device array instead of the arena.
// Each GPU holds its own copy of the array for the life of the process; its
// address is looked up once per device and kept.

namespace mnt {

constexpr size_t kStaticScratchWords = MNT_STATIC_SCRATCH_WORDS;   // 4 MiB per GPU
static __device__ __align__(256) unsigned scratch[kStaticScratchWords];

constexpr int kMaxDevices = 64;
static unsigned *g_scratch_address[kMaxDevices] = {nullptr};
static std::mutex g_scratch_mutex;

// Device address of the current device's copy of `scratch` (the array's name
// is only a host-side stand-in and must never reach a kernel).
static unsigned *static_scratch() {
  int device = 0;
  MNT_HIP(hipGetDevice(&device));
  MNT_CHECK(device >= 0 && device < kMaxDevices, "device index %d out of range", device);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_address[device] == nullptr) {
    void *address = nullptr;
    MNT_HIP(hipGetSymbolAddress(&address, HIP_SYMBOL(scratch)));
    MNT_CHECK(address != nullptr, "the static scratch array has no device address");
    g_scratch_address[device] = static_cast<unsigned *>(address);
  }
  return g_scratch_address[device];
}

}  // namespace mnt

extern "C" int mnt_compute_kernel_map_sizes_static(const void *kernel_map, int64_t num_offsets,
                                                   int64_t num_targets, int index_dtype,
                                                   void *sizes_out, void *stream_) {
  return guarded([&] {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    int_size(index_dtype);
    MNT_CHECK(num_offsets >= 0 && num_targets >= 0 && num_targets <= INT32_MAX && num_offsets <= 65535,
              "bad shape O=%lld T=%lld", (long long)num_offsets, (long long)num_targets);
    if (num_offsets == 0) return;
    MNT_CHECK(sizes_out != nullptr, "sizes_out is null");
    if (num_targets == 0) {
      // a fill kernel, not a memset node: the call may be under stream capture
      if (index_dtype == MNT_INT32) enqueue_fill<int32_t>(static_cast<int32_t *>(sizes_out), num_offsets, 0, stream);
      else enqueue_fill<int64_t>(static_cast<int64_t *>(sizes_out), num_offsets, 0, stream);
      return;
    }
    MNT_CHECK(kernel_map != nullptr, "kernel_map is null");
    const int num_tiles = static_cast<int>(div_ceil(num_targets, kTargetsPerTile));
    const size_t words = static_cast<size_t>(num_offsets) * num_tiles + static_cast<size_t>(num_offsets);
    MNT_CHECK(words <= kStaticScratchWords,
              "mnt_compute_kernel_map_sizes_static: %lld offsets x %d tiles of %d targets need %zu words "
              "of scratch, the static array holds %zu (use mnt_compute_kernel_map_sizes)",
              (long long)num_offsets, num_tiles, kTargetsPerTile, words, kStaticScratchWords);
    unsigned *base = static_scratch();
    unsigned *tile_counts = base;                  // every word in use is written by count_tiles_kernel
    unsigned *row_sizes = base + static_cast<size_t>(num_offsets) * num_tiles;
    enqueue_count_tiles(kernel_map, index_dtype, num_offsets, num_targets, tile_counts, num_tiles, stream);
    tile_scan_kernel<<<static_cast<unsigned>(num_offsets), 256, 0, stream>>>(tile_counts, num_tiles, row_sizes);
    check_launch("tile_scan_kernel");
    const unsigned grid = grid_for(num_offsets, 256);
    if (index_dtype == MNT_INT32) {
      export_sizes_kernel<int32_t><<<grid, 256, 0, stream>>>(row_sizes, static_cast<int>(num_offsets), static_cast<int32_t *>(sizes_out));
    } else {
      export_sizes_kernel<int64_t><<<grid, 256, 0, stream>>>(row_sizes, static_cast<int>(num_offsets), static_cast<int64_t *>(sizes_out));
    }
    check_launch("export_sizes_kernel");
  });
}
