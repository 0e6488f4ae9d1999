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

}  // namespace mnt
