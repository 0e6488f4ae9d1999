// Building blocks of the coordinate sort that other stages reuse.
#pragma once

#include "common.h"

namespace mnt {

// Per-dimension min (slots 0..3) and max (slots 4..7) of coords[n, ndim] into
// d_bounds (8 x int64, device).  With init the slots are reset first; without
// it the call folds into what is already there.
void enqueue_bounds(const void *coords, int64_t n, int ndim, int coord_dtype, long long *d_bounds,
                    bool init, hipStream_t stream);

// In-place exclusive prefix sum of `total` 32-bit counters (one workgroup).
void enqueue_exclusive_scan(unsigned *data, int64_t total, hipStream_t stream);

// Number of 32-bit counters radix_sort_pairs needs for n items.
size_t radix_counts_len(int64_t n);

// Stable LSD radix sort of (key, value) pairs over the low `bits` bits.  The
// sorted data ends up in keys / vals (the pointers are swapped with the
// *_alt scratch buffers as passes complete).
void radix_sort_pairs(unsigned long long *&keys, unsigned *&vals, unsigned long long *&keys_alt,
                      unsigned *&vals_alt, int64_t n, int bits, unsigned *counts,
                      hipStream_t stream);

}  // namespace mnt
