// Building blocks of the coordinate sort that other stages reuse.
#pragma once

#include "common.h"

namespace mnt {

// Per-dimension min / max of coords a[na, ndim] and (optionally) b[nb, ndim]:
// out[0..3] = min of a, out[4..7] = max of a, out[8..15] the same for b
// (INT64_MAX / INT64_MIN for an empty array).  Two launches, then a wait on
// a completion flag; the second kernel writes the results into pinned host memory.
void read_bounds(const void *a, int64_t na, const void *b, int64_t nb, int ndim, int coord_dtype,
                 long long out[16], Scope &scope, hipStream_t stream);

// Copies a small host int array to device memory as arguments of a tiny copy
// kernel: no staging buffer to protect, no synchronisation.
void upload_ints(const std::vector<int> &host, int *dst, hipStream_t stream);

// In-place exclusive prefix sum of `total` 32-bit counters (one workgroup).
void enqueue_exclusive_scan(unsigned *data, int64_t total, hipStream_t stream);

// Number of 32-bit counters radix_sort_pairs needs for n items.
size_t radix_counts_len(int64_t n);

// Number of passes radix_sort_pairs makes over n keys of `bits` significant
// bits: the sorted keys end up in the first buffer when it is even, in the
// alternate one when it is odd.
int radix_sort_passes(int64_t n, int bits);

// Stable LSD radix sort of (key, value) pairs over the low `bits` bits.  The
// sorted data ends up in keys / vals (the pointers are swapped with the
// *_alt scratch buffers as passes complete).
void radix_sort_pairs(unsigned long long *&keys, unsigned *&vals, unsigned long long *&keys_alt,
                      unsigned *&vals_alt, int64_t n, int bits, unsigned *counts,
                      hipStream_t stream);

// ---- the bucket sort as a chain of launches that never waits for the host ----

struct OffsetTable;
struct DevicePlan;

// Device memory of one chain (all of it scratch).  `counters` is cleared by
// the first launch: totals[buckets] | cursors[buckets] | whatever the caller
// keeps behind them (counter_words in all).
struct ChainSortBuffers {
  long long *partial;            // [128 * 8] partial extremes
  long long *folded;             // [8] coordinate minima, then maxima
  unsigned *counters;
  int counter_words;
  unsigned *info;                // [4]
  unsigned *status;              // [4], inside `counters` (zero when the dealing kernel starts): [0] non-zero:
                                 // the sort declined, [2] (bucket, chunk) pairs of the ranking launch
                                 // (histogram form only)
  uint4 *chunks;                 // [chain_sort_max_pairs(n)]
  unsigned long long *words;     // [chain_sort_words(n)]
  unsigned *starts;              // [buckets + 1] first sorted row of every bucket (slab form only)
  DevicePlan *plan;              // query plan written by the ranking launch (nullable)
};

// Whether the chain takes a cloud of n rows (one batch) with this many offsets;
// the final word is the chain's own (status[0]), known once it has run.
bool chain_sort_takes(int64_t n, int64_t num_batches, int num_offsets);
// log2 of the number of buckets the chain uses for n rows, and the most
// (bucket, chunk) pairs its ranking launch can have.
int chain_sort_msd_bits(int64_t n);
int64_t chain_sort_max_pairs(int64_t n);
// Words of ChainSortBuffers::words the chain needs for n rows (a slab per
// bucket when the dealing launch works without a histogram).
size_t chain_sort_words(int64_t n);
// Enqueues bounds -> histogram -> dealing -> ranking (int32 permutation and
// sorted rows); the ranking launch also writes the query plan for `offsets`.
void enqueue_chain_sort(const void *coords, int64_t n, int ndim, int coord_dtype, int32_t *indices_out,
                        void *sorted_out, const ChainSortBuffers &buf, const OffsetTable &offsets,
                        int num_offsets, hipStream_t stream);

}  // namespace mnt
