// Device-side helpers shared by the Map kernels.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

#include "common.h"

namespace mnt {

constexpr int kWave = 64;

__device__ __forceinline__ unsigned lane_id() { return threadIdx.x & (kWave - 1); }

__device__ __forceinline__ unsigned long long lanes_below() {
  return (1ull << lane_id()) - 1ull;
}

// A 64-bit value that is the same in every lane, moved to scalar registers.
__device__ __forceinline__ long long uniform64(long long v) {
  const unsigned lo = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(v));
  const unsigned hi = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(static_cast<unsigned long long>(v) >> 32));
  return static_cast<long long>((static_cast<unsigned long long>(hi) << 32) | lo);
}

// A load that goes through to the memory every compute die sees (device-scope
// atomic load): what device-scope atomics of other workgroups, possibly on
// another die, have left there, not what this die's caches hold.
template <typename T>
__device__ __forceinline__ T load_through(const T *p) {
  return __hip_atomic_load(const_cast<T *>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Batch of row i: the g with dims[g] <= i < dims[g+1] (dims has num_batches+1
// entries).  Rows at or past dims[num_batches] land in the last batch.
template <typename IT>
__device__ __forceinline__ int batch_of(long long i, const IT *__restrict__ dims,
                                        int num_batches) {
  int lo = 0, hi = num_batches - 1;
  while (lo < hi) {
    int mid = (lo + hi) >> 1;
    if (static_cast<long long>(dims[mid + 1]) > i) {
      hi = mid;
    } else {
      lo = mid + 1;
    }
  }
  return lo;
}

// Whether some batch ends exactly at row index `end` (exclusive end).
template <typename IT>
__device__ __forceinline__ bool is_batch_end(long long end, const IT *__restrict__ dims,
                                             int num_batches) {
  int lo = 0, hi = num_batches;
  while (lo < hi) {
    int mid = (lo + hi) >> 1;
    if (static_cast<long long>(dims[mid]) < end) {
      lo = mid + 1;
    } else {
      hi = mid;
    }
  }
  return lo <= num_batches && static_cast<long long>(dims[lo]) == end;
}

// Loads the (up to four) coordinates of one row without branching on the
// number of dimensions: slots past ndim re-read coordinate 0, so all loads
// are issued together instead of one after another.
template <typename CT>
__device__ __forceinline__ void load_row_raw(const CT *__restrict__ row, int ndim,
                                             CT (&raw)[MNT_MAX_NDIM]) {
#pragma unroll
  for (int k = 0; k < MNT_MAX_NDIM; ++k) raw[k] = row[k < ndim ? k : 0];
}

template <typename CT>
__device__ __forceinline__ void load_row(const CT *__restrict__ row, int ndim,
                                         long long (&c)[MNT_MAX_NDIM]) {
  CT raw[MNT_MAX_NDIM];
  load_row_raw<CT>(row, ndim, raw);
#pragma unroll
  for (int k = 0; k < MNT_MAX_NDIM; ++k) c[k] = static_cast<long long>(raw[k]);
}

// Key of one row under a Frame (see common.h).  `batch` is ignored when the
// frame has no batch field.
template <typename CT>
__device__ __forceinline__ unsigned long long pack_row(const CT *__restrict__ row,
                                                       const Frame &f, int batch) {
  long long c[MNT_MAX_NDIM];
  load_row<CT>(row, f.ndim, c);
  unsigned long long key = 0;
#pragma unroll
  for (int k = 0; k < MNT_MAX_NDIM; ++k) {
    const unsigned long long v =
        static_cast<unsigned long long>(c[k]) - static_cast<unsigned long long>(f.lo[k]);
    key |= k < f.ndim ? (v << f.shift[k]) : 0ull;
  }
  if (f.batch_width > 0) key |= static_cast<unsigned long long>(batch) << f.batch_shift;
  return key;
}

}  // namespace mnt
