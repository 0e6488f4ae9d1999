// Gather -> grouped MFMA GEMM -> Scatter for gfx950, plus the host-side padding
// plan, the forward driver and the autotuner's stage timers.
//
// Data flow and addressing follow SparseConvolutionForward::operator()
// (csrc/minuet/cuda/functions/sparse_convolution.cu:504-661): row `rank` of
// offset o lives at buffer row cumsum_padded[o] + rank; the gather is
// source-stationary over source_masks[O,S]
// (kernels/padded_gather_warp_optimized.cuh:43-59) and the scatter is
// target-stationary over target_masks[O,T] with offsets summed in row order and
// no atomics (kernels/padded_scatter_warp_optimized.cuh:33-62).  All offsets
// are multiplied in ONE grouped launch whose tiles never cross an offset, so
// padded rows are never computed.
#include <algorithm>
#include <cstring>

#include "conv_device.h"
#include "device_utils.h"
#include "sort.h"

namespace mnt {

// ------------------------------------------------------------ host plan ----

static void padding_buckets(const int64_t *sizes, int64_t n, bool has_threshold, double threshold,
                            std::vector<int64_t> &buckets) {
  buckets.clear();
  buckets.push_back(0);
  int64_t i = 0;
  while (i < n) {
    const int64_t first = i;
    uint64_t actual = static_cast<uint64_t>(sizes[i]);
    uint64_t summit = actual;
    while (i + 1 < n) {
      actual += static_cast<uint64_t>(sizes[i + 1]);
      summit = std::max<uint64_t>(summit, static_cast<uint64_t>(sizes[i + 1]));
      const uint64_t padded = summit * static_cast<uint64_t>((i + 1) - first + 1);
      if (has_threshold) {
        if (threshold < 0) break;
        // 0/0 is NaN in the reference and never exceeds the threshold
        if (actual > 0 && static_cast<double>(padded - actual) / static_cast<double>(actual) > threshold) break;
      }
      ++i;
    }
    buckets.push_back(i + 1);
    ++i;
  }
}

static void cumsum_padded(const int64_t *sizes, int64_t n, const std::vector<int64_t> &buckets,
                          std::vector<int64_t> &cum) {
  cum.assign(n + 1, 0);
  for (size_t b = 0; b + 1 < buckets.size(); ++b) {
    int64_t summit = 0;
    for (int64_t j = buckets[b]; j < buckets[b + 1]; ++j) summit = std::max(summit, sizes[j]);
    for (int64_t j = buckets[b]; j < buckets[b + 1]; ++j) cum[j + 1] = cum[j] + summit;
  }
}

// ----------------------------------------------------------------- gather ----

// One lane group per source row: the row is read once, then copied to the
// buffer row of every offset that uses it.  Rank-table entries are fetched
// eight offsets at a time so that their latencies overlap.
constexpr int kMaskBatch = 8;

template <int VB, int NV, typename IT>
__global__ __launch_bounds__(256) void gather_kernel(const unsigned char *__restrict__ sources,
                                                     unsigned char *__restrict__ buffer,
                                                     const IT *__restrict__ source_masks,
                                                     const int *__restrict__ row_start,
                                                     long long num_sources, int num_offsets,
                                                     int row_bytes, int lanes_per_row) {
  typedef typename VecOf<VB>::type V;
  const long long gtid = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
  const long long s = gtid / lanes_per_row;
  const int lr = static_cast<int>(gtid % lanes_per_row);
  if (s >= num_sources) return;
  V value[NV];
  const unsigned char *src = sources + s * row_bytes;
#pragma unroll
  for (int i = 0; i < NV; ++i) value[i] = *reinterpret_cast<const V *>(src + (lr + i * lanes_per_row) * VB);
  for (int o0 = 0; o0 < num_offsets; o0 += kMaskBatch) {
    long long d[kMaskBatch];
#pragma unroll
    for (int j = 0; j < kMaskBatch; ++j) {
      const int o = o0 + j < num_offsets ? o0 + j : num_offsets - 1;
      d[j] = static_cast<long long>(source_masks[static_cast<long long>(o) * num_sources + s]);
    }
#pragma unroll
    for (int j = 0; j < kMaskBatch; ++j) {
      if (o0 + j < num_offsets && d[j] >= 0) {
        unsigned char *dst = buffer + (static_cast<long long>(row_start[o0 + j]) + d[j]) * row_bytes;
#pragma unroll
        for (int i = 0; i < NV; ++i) *reinterpret_cast<V *>(dst + (lr + i * lanes_per_row) * VB) = value[i];
      }
    }
  }
}

// ---------------------------------------------------------------- scatter ----

template <typename T, typename V, int E, int NV>
__device__ __forceinline__ void finish_row(float (&acc)[NV][E], const Epilogue &ep, long long t,
                                           int channels, int lr, int lanes_per_row,
                                           unsigned char *__restrict__ dst, float unscale = 1.0f) {
  constexpr int VB = E * static_cast<int>(sizeof(T));
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int piece = lr + i * lanes_per_row;
    if (ep.range != nullptr) {
#pragma unroll
      for (int k = 0; k < E; ++k) acc[i][k] *= unscale;
    }
    if (ep.scale != nullptr) {
#pragma unroll
      for (int k = 0; k < E; ++k) acc[i][k] *= ep.scale[piece * E + k];
    }
    if (ep.shift != nullptr) {
#pragma unroll
      for (int k = 0; k < E; ++k) acc[i][k] += ep.shift[piece * E + k];
    }
    if (ep.residual != nullptr) {
      const V raw = *reinterpret_cast<const V *>(static_cast<const unsigned char *>(ep.residual) +
                                                 t * channels * static_cast<long long>(sizeof(T)) +
                                                 piece * VB);
      const T *e = reinterpret_cast<const T *>(&raw);
#pragma unroll
      for (int k = 0; k < E; ++k) acc[i][k] += to_float(e[k]);
    }
    if (ep.activation == MNT_ACT_RELU) {
#pragma unroll
      for (int k = 0; k < E; ++k) acc[i][k] = fmaxf(acc[i][k], 0.0f);
    } else if (ep.activation == MNT_ACT_LEAKY_RELU) {
#pragma unroll
      for (int k = 0; k < E; ++k) acc[i][k] = acc[i][k] > 0.0f ? acc[i][k] : acc[i][k] * ep.slope;
    } else if (ep.activation == MNT_ACT_RELU6) {
#pragma unroll
      for (int k = 0; k < E; ++k) acc[i][k] = fminf(fmaxf(acc[i][k], 0.0f), 6.0f);
    }
    V raw;
    T *e = reinterpret_cast<T *>(&raw);
#pragma unroll
    for (int k = 0; k < E; ++k) e[k] = static_cast<T>(acc[i][k]);
    *reinterpret_cast<V *>(dst + piece * VB) = raw;
  }
}

// Fallback for kernels with more offsets than the listed form below stages:
// one lane group per target row sums its buffer rows in offset order in fp32
// and writes the row once.  The buffer holds elements of type TB (the output
// type, or fp32 when the output type is too coarse to round partial products
// to), the output elements of type T.  `direct` (nullable) holds one more
// buffer row per target, indexed by the target itself: the centre-offset
// product of the shortcut, which needs no rank table.
template <typename TB, typename T, int VB, int NV, typename IT>
__global__ __launch_bounds__(256) void scatter_wide_kernel(const TB *__restrict__ buffer,
                                                      unsigned char *__restrict__ targets,
                                                      const IT *__restrict__ target_masks,
                                                      const int *__restrict__ row_start,
                                                      long long num_targets, int num_offsets,
                                                      int channels, int lanes_per_row,
                                                      const TB *__restrict__ direct, Epilogue ep) {
  typedef typename VecOf<VB>::type V;
  const float unscale = 1.0f / range_scale(ep.range);            // every lane is still here
  constexpr int E = VB / static_cast<int>(sizeof(T));
  constexpr int BB = E * static_cast<int>(sizeof(TB));          // buffer bytes per vector
  typedef typename VecOf<(BB > 16 ? 16 : BB)>::type BV;
  constexpr int NBV = BB > 16 ? BB / 16 : 1;
  const long long gtid = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
  const long long t = gtid / lanes_per_row;
  const int lr = static_cast<int>(gtid % lanes_per_row);
  if (t >= num_targets) return;
  float acc[NV][E];
  unsigned char *dst = targets + t * channels * static_cast<long long>(sizeof(T));
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    if (direct != nullptr) {
      const TB *piece = direct + t * channels + (lr + i * lanes_per_row) * E;
      BV raw[NBV];
#pragma unroll
      for (int v = 0; v < NBV; ++v) raw[v] = reinterpret_cast<const BV *>(piece)[v];
      const TB *e = reinterpret_cast<const TB *>(raw);
#pragma unroll
      for (int k = 0; k < E; ++k) acc[i][k] = to_float(e[k]);
    } else {
#pragma unroll
      for (int k = 0; k < E; ++k) acc[i][k] = 0.0f;
    }
  }
  // rank-table entries are fetched 32 offsets at a time and buffer rows a
  // sub-batch at a time (all loads of a batch in flight together), then
  // summed in offset order
  constexpr int kMasks = 32;
  // rows in flight per lane group: 2 to 5 measure the same, more cost a wavefront of occupancy
  constexpr int kRows = 4;
  for (int o0 = 0; o0 < num_offsets; o0 += kMasks) {
    int d[kMasks];
#pragma unroll
    for (int j = 0; j < kMasks; ++j) {
      const int o = o0 + j < num_offsets ? o0 + j : num_offsets - 1;
      const int v = static_cast<int>(target_masks[static_cast<long long>(o) * num_targets + t]);
      d[j] = o0 + j < num_offsets ? v : -1;
    }
#pragma unroll
    for (int j0 = 0; j0 < kMasks; j0 += kRows) {
      if (o0 + j0 >= num_offsets) break;
      BV raw[kRows][NV][NBV];
#pragma unroll
      for (int j = 0; j < kRows; ++j) {
        if (d[j0 + j] >= 0) {
          const TB *src = buffer + (static_cast<long long>(row_start[o0 + j0 + j]) + d[j0 + j]) * channels;
#pragma unroll
          for (int i = 0; i < NV; ++i) {
            const TB *piece = src + (lr + i * lanes_per_row) * E;
#pragma unroll
            for (int v = 0; v < NBV; ++v) raw[j][i][v] = reinterpret_cast<const BV *>(piece)[v];
          }
        }
      }
#pragma unroll
      for (int j = 0; j < kRows; ++j) {
        if (d[j0 + j] >= 0) {
#pragma unroll
          for (int i = 0; i < NV; ++i) {
            const TB *e = reinterpret_cast<const TB *>(raw[j][i]);
#pragma unroll
            for (int k = 0; k < E; ++k) acc[i][k] += to_float(e[k]);
          }
        }
      }
    }
  }
  finish_row<T, V, E, NV>(acc, ep, t, channels, lr, lanes_per_row, dst, unscale);
}

// Scatter for kernel maps of at most MAXO rank rows (offset groups, 2 x 2 x 2
// kernels): one lane group per target reads its MAXO rank entries in one trip
// and all of its buffer rows in a second one, sums them in row order in fp32
// and writes the target once; no row list, no barrier.
template <typename TB, typename T, int VB, int NV, typename IT, int MAXO>
__global__ __launch_bounds__(256) void scatter_few_kernel(const TB *__restrict__ buffer,
                                                          unsigned char *__restrict__ targets,
                                                          const IT *__restrict__ target_masks,
                                                          const int *__restrict__ row_start,
                                                          long long num_targets, int num_offsets,
                                                          int channels, int lanes_per_row,
                                                          const TB *__restrict__ direct, Epilogue ep) {
  typedef typename VecOf<VB>::type V;
  const float unscale = 1.0f / range_scale(ep.range);            // every lane is still here
  constexpr int E = VB / static_cast<int>(sizeof(T));
  constexpr int BB = E * static_cast<int>(sizeof(TB));          // buffer bytes per vector
  typedef typename VecOf<(BB > 16 ? 16 : BB)>::type BV;
  constexpr int NBV = BB > 16 ? BB / 16 : 1;
  const long long gtid = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
  const long long t = gtid / lanes_per_row;
  const int lr = static_cast<int>(gtid % lanes_per_row);
  if (t >= num_targets) return;
  int d[MAXO];
#pragma unroll
  for (int j = 0; j < MAXO; ++j) {
    d[j] = j < num_offsets ? static_cast<int>(target_masks[static_cast<long long>(j) * num_targets + t]) : -1;
  }
  BV first[NV][NBV];
  if (direct != nullptr) {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const TB *piece = direct + t * channels + (lr + i * lanes_per_row) * E;
#pragma unroll
      for (int v = 0; v < NBV; ++v) first[i][v] = reinterpret_cast<const BV *>(piece)[v];
    }
  }
  BV raw[MAXO][NV][NBV];
#pragma unroll
  for (int j = 0; j < MAXO; ++j) {
    if (d[j] >= 0) {
      const TB *src = buffer + (static_cast<long long>(row_start[j]) + d[j]) * channels;
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const TB *piece = src + (lr + i * lanes_per_row) * E;
#pragma unroll
        for (int v = 0; v < NBV; ++v) raw[j][i][v] = reinterpret_cast<const BV *>(piece)[v];
      }
    }
  }
  float acc[NV][E];
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const TB *e = reinterpret_cast<const TB *>(first[i]);
#pragma unroll
    for (int k = 0; k < E; ++k) acc[i][k] = direct != nullptr ? to_float(e[k]) : 0.0f;
  }
#pragma unroll
  for (int j = 0; j < MAXO; ++j) {
    if (d[j] >= 0) {
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const TB *e = reinterpret_cast<const TB *>(raw[j][i]);
#pragma unroll
        for (int k = 0; k < E; ++k) acc[i][k] += to_float(e[k]);
      }
    }
  }
  unsigned char *dst = targets + t * channels * static_cast<long long>(sizeof(T));
  finish_row<T, V, E, NV>(acc, ep, t, channels, lr, lanes_per_row, dst, unscale);
}

// Scatter in two phases per workgroup of `tile_targets` (a power of two)
// consecutive targets.
//   1. Listing: thread (part, target) reads its share of the target's rank
//      table column (consecutive lanes read consecutive addresses), and the
//      valid entries are compacted, in offset order, into a per-target list of
//      buffer rows in LDS.
//   2. Summation: one lane group per target walks that list, a batch of rows in
//      flight at a time, sums in fp32 in offset order and writes the row once.
// The buffer holds elements of type TB (the output type, or fp32 when the
// output type is too coarse to round partial products to), the output elements
// of type T.  `direct` (nullable) holds one more buffer row per target, indexed
// by the target itself: the centre-offset product of the shortcut, which needs
// no rank table.  Dynamic LDS: (num_offsets + 256 / tile_targets) * tile_targets
// ints.
constexpr int kScatterBlock = 256;
constexpr int kScatterFewOffsets = 9;   // rank rows that scatter_few_kernel keeps in flight at once

template <typename TB, typename T, int VB, int NV, typename IT>
__global__ __launch_bounds__(kScatterBlock) void scatter_kernel(
    const TB *__restrict__ buffer, unsigned char *__restrict__ targets,
    const IT *__restrict__ target_masks, const int *__restrict__ row_start, long long num_targets,
    int num_offsets, int channels, int lanes_per_row, const TB *__restrict__ direct,
    int tile_shift, Epilogue ep) {
  typedef typename VecOf<VB>::type V;
  const float unscale = 1.0f / range_scale(ep.range);            // every lane is still here
  constexpr int E = VB / static_cast<int>(sizeof(T));
  constexpr int BB = E * static_cast<int>(sizeof(TB));          // buffer bytes per vector
  typedef typename VecOf<(BB > 16 ? 16 : BB)>::type BV;
  constexpr int NBV = BB > 16 ? BB / 16 : 1;
  constexpr int kBatch = 8;
  extern __shared__ int scatter_lds[];
  const int tile = 1 << tile_shift;
  const int parts = kScatterBlock >> tile_shift;
  int *list = scatter_lds;                       // [num_offsets][tile]
  int *counts = scatter_lds + num_offsets * tile;  // [parts][tile]
  const int tid = static_cast<int>(threadIdx.x);
  const long long t0 = static_cast<long long>(blockIdx.x) << tile_shift;

  {
    const int tt = tid & (tile - 1);
    const int part = tid >> tile_shift;
    const int share = (num_offsets + parts - 1) / parts;
    const int o_lo = part * share;
    const int o_hi = min(num_offsets, o_lo + share);
    const long long t = min(t0 + tt, num_targets - 1);
    const IT *column = target_masks + t;
    // the first batch stays in registers across the barrier; later batches
    // (kernels with more than 8 * parts offsets) are read again
    int first[kBatch];
    int count = 0;
#pragma unroll
    for (int j = 0; j < kBatch; ++j) {
      const int o = o_lo + j;
      first[j] = o < o_hi ? static_cast<int>(column[static_cast<long long>(o) * num_targets]) : -1;
    }
#pragma unroll
    for (int j = 0; j < kBatch; ++j) count += first[j] >= 0 ? 1 : 0;
    for (int o0 = o_lo + kBatch; o0 < o_hi; o0 += kBatch) {
      int more[kBatch];
#pragma unroll
      for (int j = 0; j < kBatch; ++j) {
        const int o = o0 + j;
        more[j] = o < o_hi ? static_cast<int>(column[static_cast<long long>(o) * num_targets]) : -1;
      }
#pragma unroll
      for (int j = 0; j < kBatch; ++j) count += more[j] >= 0 ? 1 : 0;
    }
    counts[part * tile + tt] = count;
    __syncthreads();
    int at = 0;
    for (int p = 0; p < part; ++p) at += counts[p * tile + tt];
#pragma unroll
    for (int j = 0; j < kBatch; ++j) {
      if (first[j] >= 0) {
        list[at * tile + tt] = row_start[o_lo + j] + first[j];
        ++at;
      }
    }
    for (int o0 = o_lo + kBatch; o0 < o_hi; o0 += kBatch) {
      int more[kBatch];
#pragma unroll
      for (int j = 0; j < kBatch; ++j) {
        const int o = o0 + j;
        more[j] = o < o_hi ? static_cast<int>(column[static_cast<long long>(o) * num_targets]) : -1;
      }
#pragma unroll
      for (int j = 0; j < kBatch; ++j) {
        if (more[j] >= 0) {
          list[at * tile + tt] = row_start[o0 + j] + more[j];
          ++at;
        }
      }
    }
    __syncthreads();
  }

  // rows in flight per lane group: 2 to 5 measure the same, more cost a wavefront of occupancy
  constexpr int kRows = 4;
  const int groups = kScatterBlock / lanes_per_row;
  const int group = tid / lanes_per_row;
  const int lr = tid - group * lanes_per_row;
  if (group >= groups) return;
  for (int tt = group; tt < tile; tt += groups) {
    const long long t = t0 + tt;
    if (t >= num_targets) break;
    int n = 0;
    for (int p = 0; p < parts; ++p) n += counts[p * tile + tt];
    float acc[NV][E];
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      if (direct != nullptr) {
        const TB *piece = direct + t * channels + (lr + i * lanes_per_row) * E;
        BV raw[NBV];
#pragma unroll
        for (int v = 0; v < NBV; ++v) raw[v] = reinterpret_cast<const BV *>(piece)[v];
        const TB *e = reinterpret_cast<const TB *>(raw);
#pragma unroll
        for (int k = 0; k < E; ++k) acc[i][k] = to_float(e[k]);
      } else {
#pragma unroll
        for (int k = 0; k < E; ++k) acc[i][k] = 0.0f;
      }
    }
    for (int k0 = 0; k0 < n; k0 += kRows) {
      int row[kRows];
#pragma unroll
      for (int j = 0; j < kRows; ++j) row[j] = k0 + j < n ? list[(k0 + j) * tile + tt] : -1;
      BV raw[kRows][NV][NBV];
#pragma unroll
      for (int j = 0; j < kRows; ++j) {
        if (row[j] >= 0) {
          const TB *src = buffer + static_cast<long long>(row[j]) * channels;
#pragma unroll
          for (int i = 0; i < NV; ++i) {
            const TB *piece = src + (lr + i * lanes_per_row) * E;
#pragma unroll
            for (int v = 0; v < NBV; ++v) raw[j][i][v] = reinterpret_cast<const BV *>(piece)[v];
          }
        }
      }
#pragma unroll
      for (int j = 0; j < kRows; ++j) {
        if (row[j] >= 0) {
#pragma unroll
          for (int i = 0; i < NV; ++i) {
            const TB *e = reinterpret_cast<const TB *>(raw[j][i]);
#pragma unroll
            for (int k = 0; k < E; ++k) acc[i][k] += to_float(e[k]);
          }
        }
      }
    }
    unsigned char *dst = targets + t * channels * static_cast<long long>(sizeof(T));
    finish_row<T, V, E, NV>(acc, ep, t, channels, lr, lanes_per_row, dst, unscale);
  }
}

// Scatter of the list-driven dataflow: the GEMM has written its products in
// target-major order, so target t sums the CONSECUTIVE buffer rows
// row_ptr[t] .. row_ptr[t + 1] - 1 (in the order of the kernel map's rows, the
// centre offset last, which is the reference's order of summation,
// sparse_convolution.cu:642-660) and no rank table or row list is read: the
// buffer streams through once.  One lane group per target, `tile` targets per
// workgroup.
template <typename TB, typename T, int VB, int NV>
__global__ __launch_bounds__(kScatterBlock) void scatter_rows_kernel(
    const TB *__restrict__ buffer, unsigned char *__restrict__ targets, const int *__restrict__ row_ptr,
    long long num_targets, int channels, int lanes_per_row, int tile, Epilogue ep) {
  typedef typename VecOf<VB>::type V;
  const float unscale = 1.0f / range_scale(ep.range);            // every lane is still here
  constexpr int E = VB / static_cast<int>(sizeof(T));
  constexpr int BB = E * static_cast<int>(sizeof(TB));          // buffer bytes per vector
  typedef typename VecOf<(BB > 16 ? 16 : BB)>::type BV;
  constexpr int NBV = BB > 16 ? BB / 16 : 1;
  constexpr int kRows = 4;                                       // rows in flight per lane group
  const int tid = static_cast<int>(threadIdx.x);
  const int groups = kScatterBlock / lanes_per_row;
  const int group = tid / lanes_per_row;
  const int lr = tid - group * lanes_per_row;
  if (group >= groups) return;
  const long long t0 = static_cast<long long>(blockIdx.x) * tile;
  for (int tt = group; tt < tile; tt += groups) {
    const long long t = t0 + tt;
    if (t >= num_targets) break;
    const int lo = row_ptr[t], hi = row_ptr[t + 1];
    float acc[NV][E];
#pragma unroll
    for (int i = 0; i < NV; ++i) {
#pragma unroll
      for (int k = 0; k < E; ++k) acc[i][k] = 0.0f;
    }
    for (int k0 = lo; k0 < hi; k0 += kRows) {
      BV raw[kRows][NV][NBV];
#pragma unroll
      for (int j = 0; j < kRows; ++j) {
        if (k0 + j < hi) {
          const TB *src = buffer + static_cast<long long>(k0 + j) * channels;
#pragma unroll
          for (int i = 0; i < NV; ++i) {
            const TB *piece = src + (lr + i * lanes_per_row) * E;
#pragma unroll
            for (int v = 0; v < NBV; ++v) raw[j][i][v] = reinterpret_cast<const BV *>(piece)[v];
          }
        }
      }
#pragma unroll
      for (int j = 0; j < kRows; ++j) {
        if (k0 + j < hi) {
#pragma unroll
          for (int i = 0; i < NV; ++i) {
            const TB *e = reinterpret_cast<const TB *>(raw[j][i]);
#pragma unroll
            for (int k = 0; k < E; ++k) acc[i][k] += to_float(e[k]);
          }
        }
      }
    }
    unsigned char *dst = targets + t * channels * static_cast<long long>(sizeof(T));
    finish_row<T, V, E, NV>(acc, ep, t, channels, lr, lanes_per_row, dst, unscale);
  }
}

// Element type of the GEMM-output / scatter-input buffer for feature type T.
// bfloat16 keeps only 8 significant bits, so rounding every partial product
// to it would cost more accuracy than the output rounding itself: its rows are
// IEEE half words under the per-pass power-of-two scale of range_kernel.
template <typename T>
struct BufferOf { typedef T type; };
template <>
struct BufferOf<bf16_t> { typedef half_t type; };
template <typename T>
struct ScaledBuffer { static constexpr bool value = false; };
template <>
struct ScaledBuffer<bf16_t> { static constexpr bool value = true; };

// ------------------------------------------------------------ grouped GEMM ----

constexpr int kGemmBlock = 256;
constexpr int kGemmRows = 128;          // rows of A per workgroup (32 per wavefront)
constexpr int kMaxChannelBlocks = 4;    // 32-channel blocks per workgroup (128 channels)

// meta: [G | tile_prefix (G+1) | row_start (G+1) | rows (G) | weight (G) | list_start (G)]
//
// One workgroup multiplies 128 buffer rows of one offset by that offset's
// weights: out^T = W^T x A^T.  The first MFMA operand holds 32 output
// channels, the second 32 data rows, so every lane ends up with 4 consecutive
// channels of ONE data row per accumulator group (how the rows are written:
// see the output pass at the end of the kernel).  CH > 0: K is exactly CH
// chunks of 128 bytes (CH <= 2) and the whole tile is loaded before the first
// product; CH == 0: any K, one chunk ahead.
//
// A never passes through LDS: lane (r, h) of a wavefront loads, for step kk of
// a 128-byte chunk of row r, the 16 bytes at offset 32*kk + 16*h — exactly its
// MFMA operand.  The same K permutation is applied to the weights (lane half
// h of step kk reads the same bytes of its channel row), which leaves the
// dot products unchanged.  Only the weights (W^T, K-contiguous, padded) are
// staged in LDS, shared by the four wavefronts; the NB channel blocks of a
// workgroup (up to 128 channels) are accumulated in registers, so A is read
// once per 128-channel slice of the output.
//
// With `gather_index` (nullable) the Gather step is folded into the A load:
// data row i of group g is then row gather_index[list_start[g] + i] of `a`
// (the source features) instead of buffer row row_start[g] + i, and no gather
// buffer exists; a group with list_start < 0 reads row i of `a` itself (the
// centre offset of the shortcut).  The output rows stay in buffer order,
// unless `out_pos` (nullable, needs gather_index and no such centre group)
// says where each goes: the product of list entry p = list_start[g] + i is
// then written to buffer row out_pos[p] (the target-major layout that the
// list-driven Scatter sums without an index).
//
// The tables reach the kernel either in device memory (grouped_gemm_kernel) or
// as a by-value argument (grouped_gemm_riding_kernel: meta starts at entry
// meta_at of `table`); workgroup (0, 0) of the latter also copies the whole
// table to `table_out` for the kernels that follow in the stream, so that no
// separate upload runs.  Reading the tables from the argument segment costs
// every workgroup a little, so large passes use the first form.
struct MetaInMemory {
  const int *meta;
  __device__ __forceinline__ int operator()(int i) const { return meta[i]; }
};
struct MetaInArguments {
  const PlanChunk *table;
  int meta_at;
  __device__ __forceinline__ int operator()(int i) const { return table->v[meta_at + i]; }
};

// Offset groups (GM > 0): the GM offsets of a group are multiplied in ONE
// product whose K dimension is their GM weight matrices one after the other.
// A data row then stands for a target that ANY offset of its group reaches,
// and holds that target's GM source rows end to end (zeros where an offset has
// no source), so a group needs as many buffer rows as it has such targets
// instead of one per (offset, target) pair: offsets that differ along an axis
// in which the cloud is dense share most of their targets.  The tables come
// from group_emit_kernel: head[0] is the axis the groups lie along (chosen on
// the device), head[1 + j] the rows of group j; src[j * stride + i] holds the
// source rows (x, y, z; -1: none) of data row i of group j, which is also its
// buffer row; offset_of[axis][j][m] is the offset (weight matrix) of member m.
// Needs K * sizeof(T) to be whole 128-byte chunks.
constexpr int kGroupCount = 9;
constexpr int kGroupMembers = 3;
struct GroupView {
  const int *head;
  const int4 *src;
  long long stride;
  int tiles_per_group;
  int offset_of[3 * kGroupCount * kGroupMembers];
};

template <typename T, typename TC, int NB, bool VEC, int CH, typename Meta, int GM = 0>
__device__ __forceinline__ void grouped_gemm_body(const T *__restrict__ a, TC *__restrict__ c,
                                                  const T *__restrict__ wt, const Meta &entry, int K,
                                                  int N, int Kp, int Np,
                                                  const int *__restrict__ gather_index,
                                                  const int *__restrict__ out_pos,
                                                  const float *__restrict__ range,
                                                  const GroupView *__restrict__ groups = nullptr) {
  // product rows of a scaled buffer leave as acc * scale (a power of two)
  const float scale = ScaledBuffer<T>::value ? range_scale(range) : 1.0f;
  constexpr int EPC = 16 / static_cast<int>(sizeof(T));        // elements per 16-byte piece
  constexpr int KC = kChunkBytes / static_cast<int>(sizeof(T));
  constexpr int TN = NB * 32;
  constexpr int kLdsChunks = CH > 0 ? CH : 1;
  // the output pass turns one 32 x 32 block per wavefront around in the same memory
  constexpr int kTurnRow = 32 * static_cast<int>(sizeof(TC)) + 16;
  constexpr int kTurnBytes = 32 * kTurnRow;
  constexpr int kWeightBytes = kLdsChunks * TN * kLdsRowBytes;
  constexpr int kLdsBytes = kWeightBytes > 4 * kTurnBytes ? kWeightBytes : 4 * kTurnBytes;
  __shared__ __align__(16) unsigned char b_lds[kLdsBytes];

  const int G = GM > 0 ? kGroupCount : entry(0);
  const int at_prefix = 1, at_start = at_prefix + G + 1, at_rows = at_start + G + 1, at_weight = at_rows + G,
            at_list = at_weight + G;

  const int n0 = blockIdx.y * TN;
  // A workgroup walks the tiles blockIdx.x, blockIdx.x + gridDim.x, ...: the
  // grid is what the compute units hold at once, since workgroups that live for
  // a few microseconds are launched more slowly than they finish.
  const int num_tiles = GM > 0 ? kGroupCount * groups->tiles_per_group : entry(at_prefix + G);

  // What a tile is made of is worked out from tables that do not depend on the
  // tile: they are fetched once per workgroup (lane i keeps the entries of
  // group i), and finding a tile's group is a ballot.  The one thing a tile
  // still has to fetch before its operands, the source row(s) of each data
  // row, is asked for one tile ahead, while the tile before it is multiplied:
  // a tile then waits for ONE trip to memory (its operands) instead of three.
  struct TileAt {
    bool ok;
    int prefix, rows, start, weight, list, group;
  };
  const int lane0 = threadIdx.x & 63;
  int m_prefix = 0, m_rows = 0, m_start = 0, m_weight = 0, m_list = 0, m_total = 0, axis = 0;
  if constexpr (GM > 0) {
    // tiles are numbered over the rows the groups really have (the grid only
    // knows the worst case): a scan over the nine lanes that hold the groups'
    // row counts gives every group's first tile
    m_rows = groups->head[1 + min(lane0, kGroupCount - 1)];
    axis = groups->head[0];
    const int tiles = (m_rows + kGemmRows - 1) / kGemmRows;
    int upto = tiles;
#pragma unroll
    for (int d = 1; d < 16; d <<= 1) {
      const int below = __shfl_up(upto, d);
      if (lane0 >= d) upto += below;
    }
    m_total = __builtin_amdgcn_readlane(upto, kGroupCount - 1);
    m_prefix = upto - tiles;
  } else {
    m_total = num_tiles;
    if (G <= kWave) {
      const int i = min(lane0, G - 1);
      m_prefix = entry(at_prefix + i);
      m_rows = entry(at_rows + i);
      m_start = entry(at_start + i);
      m_weight = entry(at_weight + i);
      m_list = entry(at_list + i);
    }
  }
  auto tile_at = [&](int tile) {
    TileAt t = {tile < m_total, 0, 0, 0, 0, 0, 0};
    if (!t.ok) return t;
    if (GM > 0 || G <= kWave) {
      const int g = __popcll(__ballot(lane0 < G && m_prefix <= tile)) - 1;
      t.group = g;
      t.prefix = __builtin_amdgcn_readlane(m_prefix, g);
      t.rows = __builtin_amdgcn_readlane(m_rows, g);
      t.start = __builtin_amdgcn_readlane(m_start, g);
      t.weight = __builtin_amdgcn_readlane(m_weight, g);
      t.list = __builtin_amdgcn_readlane(m_list, g);
    } else {
      int lo = 0, hi = G - 1;
      while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (entry(at_prefix + mid) <= tile) {
          lo = mid;
        } else {
          hi = mid - 1;
        }
      }
      t.prefix = entry(at_prefix + lo);
      t.rows = entry(at_rows + lo);
      t.start = entry(at_start + lo);
      t.weight = entry(at_weight + lo);
      t.list = entry(at_list + lo);
    }
    return t;
  };
  // the source row (plain) or the member source rows (groups) of this lane's data row of a tile
  auto rows_of = [&](const TileAt &t, int tile) {
    int4 v = make_int4(-1, -1, -1, 0);
    if (!t.ok) return v;
    const int row = (threadIdx.x >> 6) * 32 + (threadIdx.x & 31);
    const int r0 = (tile - t.prefix) * kGemmRows;
    const bool row_ok = row < t.rows - r0;
    if constexpr (GM > 0) {
      if (row_ok) v = groups->src[t.group * groups->stride + r0 + row];
    } else {
      if (gather_index != nullptr && t.list >= 0 && row_ok) {
        v.x = gather_index[static_cast<long long>(t.list) + r0 + row];
      }
    }
    return v;
  };

  int tile = blockIdx.x;
  TileAt here = tile_at(tile);
  if (!here.ok) return;                              // the same for the whole workgroup
  int4 here_rows = rows_of(here, tile);
  for (;;) {
  // (the thread's number is made opaque per tile: what is derived from it is
  // worked out again for every tile instead of being kept in registers)
  int tid = threadIdx.x;
  asm volatile("" : "+v"(tid));
  const int lane = tid & 63;
  const int wv = tid >> 6;
  const int r = lane & 31;
  const int h = lane >> 5;
  const int g_prefix = here.prefix, g_rows = here.rows, g_start = here.start, g_weight = here.weight,
            g_list = here.list, group = here.group;
  const int next_tile = tile + gridDim.x;
  const TileAt next = tile_at(next_tile);
  int4 next_rows = make_int4(-1, -1, -1, 0);
  const int r0 = (tile - g_prefix) * kGemmRows;
  const int valid = min(kGemmRows, g_rows - r0);
  const long long row_base = (GM > 0 ? group * groups->stride : static_cast<long long>(g_start)) + r0;
  const T *w_base = wt + (static_cast<long long>(g_weight) * Np + n0) * Kp;
  const int list_at = g_list;

  const int row = wv * 32 + r;
  const bool row_ok = row < valid;
  long long a_index = row_base + row;
  if (gather_index != nullptr) {
    a_index = list_at < 0 ? r0 + row : (row_ok ? here_rows.x : 0);
  }
  const T *a_row = a + a_index * K;
  const int4 member_rows = here_rows;
  // where this tile's rows go, for the lists of the output pass (null: buffer order)
  const int *pos_list = out_pos != nullptr ? out_pos + (static_cast<long long>(list_at) + r0) : nullptr;

  floatx16 acc[NB];
#pragma unroll
  for (int b = 0; b < NB; ++b) {
#pragma unroll
    for (int j = 0; j < 16; ++j) acc[b][j] = 0.0f;
  }

  // Software pipeline over the K chunks: the A pieces and the W^T pieces of
  // chunk i+1 are loaded into registers while chunk i is multiplied.
  constexpr int kSteps = kChunkBytes / 32;
  constexpr int kWPieces = (TN * 8 + kGemmBlock - 1) / kGemmBlock;

  auto load_a = [&](int k0, uint4 (&dst)[kSteps]) {
#pragma unroll
    for (int kk = 0; kk < kSteps; ++kk) {
      const int k = k0 + kk * 2 * EPC + h * EPC;
      uint4 v = make_uint4(0u, 0u, 0u, 0u);
      if (row_ok) {
        if (VEC && k + EPC <= K) {
          v = *reinterpret_cast<const uint4 *>(a_row + k);
        } else {
          T *e = reinterpret_cast<T *>(&v);
#pragma unroll
          for (int x = 0; x < EPC; ++x) {
            if (k + x < K) e[x] = a_row[k + x];
          }
        }
      }
      dst[kk] = v;
    }
  };
  auto load_w = [&](int k0, uint4 (&wpiece)[kWPieces]) {
#pragma unroll
    for (int i = 0; i < kWPieces; ++i) {
      const int piece = tid + i * kGemmBlock;
      const int n = piece >> 3;
      const int q = piece & 7;
      uint4 v = make_uint4(0u, 0u, 0u, 0u);
      if (piece < TN * 8 && n0 + n < Np) {
        v = *reinterpret_cast<const uint4 *>(w_base + static_cast<long long>(n) * Kp + k0 + q * EPC);
      }
      wpiece[i] = v;
    }
  };

  auto store_w = [&](int chunk, const uint4 (&wpiece)[kWPieces]) {
#pragma unroll
    for (int i = 0; i < kWPieces; ++i) {
      const int piece = tid + i * kGemmBlock;
      if (piece < TN * 8) {
        *reinterpret_cast<uint4 *>(b_lds + chunk * (TN * kLdsRowBytes) + (piece >> 3) * kLdsRowBytes +
                                   (piece & 7) * 16) = wpiece[i];
      }
    }
  };
  auto multiply = [&](int chunk, const uint4 (&frag)[kSteps]) {
#pragma unroll
    for (int kk = 0; kk < kSteps; ++kk) {
      const int off = kk * 32 + h * 16;
#pragma unroll
      for (int b = 0; b < NB; ++b) {
        const uint4 chan_frag = *reinterpret_cast<const uint4 *>(b_lds + chunk * (TN * kLdsRowBytes) +
                                                                 (b * 32 + r) * kLdsRowBytes + off);
        acc[b] = Mfma<T>::run(chan_frag, frag[kk], acc[b]);
      }
    }
  };

  if constexpr (GM > 0) {
    // The concatenated K is walked in stages of SC chunks (SC = CH here: 2 where
    // a member's row is an even number of chunks, else 1).  A stage lies inside
    // one member: its A pieces come from that member's source row, its W^T
    // pieces from that member's weight matrix.  All loads of a stage are issued
    // together; the W^T pieces of the next stage are asked for as soon as this
    // stage's are in LDS (their registers are free then), the A pieces after
    // the products that still read the present ones.
    constexpr int SC = CH;
    const int per_member = Kp / KC;
    const int stages = GM * per_member / SC;
    auto load_a_of = [&](int st, uint4 (&dst)[SC][kSteps]) {
      const int chunk = st * SC;
      const int m = chunk / per_member;
      const int s = m == 0 ? member_rows.x : m == 1 ? member_rows.y : member_rows.z;
      const T *from = a + static_cast<long long>(s < 0 ? 0 : s) * K + (chunk - m * per_member) * KC + h * EPC;
#pragma unroll
      for (int c2 = 0; c2 < SC; ++c2) {
#pragma unroll
        for (int kk = 0; kk < kSteps; ++kk) {
          uint4 v = make_uint4(0u, 0u, 0u, 0u);
          if (s >= 0) v = *reinterpret_cast<const uint4 *>(from + c2 * KC + kk * 2 * EPC);
          dst[c2][kk] = v;
        }
      }
    };
    auto load_w_of = [&](int st, uint4 (&wpiece)[SC][kWPieces]) {
      const int chunk = st * SC;
      const int m = chunk / per_member;
      const int offset = groups->offset_of[(axis * kGroupCount + group) * kGroupMembers + m];
      const T *from = wt + (static_cast<long long>(offset) * Np + n0) * Kp + (chunk - m * per_member) * KC;
#pragma unroll
      for (int c2 = 0; c2 < SC; ++c2) {
#pragma unroll
        for (int p = 0; p < kWPieces; ++p) {
          const int piece = tid + p * kGemmBlock;
          uint4 v = make_uint4(0u, 0u, 0u, 0u);
          if (piece < TN * 8 && n0 + (piece >> 3) < Np) {
            v = *reinterpret_cast<const uint4 *>(from + c2 * KC + static_cast<long long>(piece >> 3) * Kp +
                                                 (piece & 7) * EPC);
          }
          wpiece[c2][p] = v;
        }
      }
    };
    uint4 frag[SC][kSteps];
    uint4 wpiece[SC][kWPieces];
    load_w_of(0, wpiece);
    load_a_of(0, frag);
    next_rows = rows_of(next, next_tile);
    for (int st = 0; st < stages; ++st) {
      if (st > 0) __syncthreads();                   // previous stage of W^T fully consumed
#pragma unroll
      for (int c2 = 0; c2 < SC; ++c2) store_w(c2, wpiece[c2]);
      __syncthreads();
      const bool more = st + 1 < stages;
      if (more) load_w_of(st + 1, wpiece);
#pragma unroll
      for (int c2 = 0; c2 < SC; ++c2) multiply(c2, frag[c2]);
      if (more) load_a_of(st + 1, frag);
    }
  } else if constexpr (CH > 0) {
    // K of CH chunks (Kp == CH * KC): every load of the tile is issued at
    // once, so the tile pays for one trip to memory instead of one per chunk.
    uint4 frags[CH][kSteps];
    uint4 wpieces[CH][kWPieces];
#pragma unroll
    for (int c = 0; c < CH; ++c) load_w(c * KC, wpieces[c]);
#pragma unroll
    for (int c = 0; c < CH; ++c) load_a(c * KC, frags[c]);
    next_rows = rows_of(next, next_tile);
#pragma unroll
    for (int c = 0; c < CH; ++c) store_w(c, wpieces[c]);
    __syncthreads();
#pragma unroll
    for (int c = 0; c < CH; ++c) multiply(c, frags[c]);
  } else {
    uint4 frag[kSteps], frag_next[kSteps];
    uint4 wpiece[kWPieces];
    load_a(0, frag);
    load_w(0, wpiece);
    next_rows = rows_of(next, next_tile);
    for (int k0 = 0; k0 < Kp; k0 += KC) {
      if (k0 > 0) __syncthreads();                   // previous chunk of W^T fully consumed
      store_w(0, wpiece);
      __syncthreads();
      const bool more = k0 + KC < Kp;
      if (more) {
        load_a(k0 + KC, frag_next);
        load_w(k0 + KC, wpiece);
      }
      multiply(0, frag);
      if (more) {
#pragma unroll
        for (int kk = 0; kk < kSteps; ++kk) frag[kk] = frag_next[kk];
      }
    }
  }

  // Output.  A lane holds 4 consecutive channels of one row per accumulator
  // group, and neighbouring lanes hold different rows: stored as they are,
  // every lane's 8 or 16 bytes are a write request of their own.  Where rows
  // are whole 16-byte pieces each wavefront turns its 32 x 32 blocks around in
  // LDS first, so that a store instruction covers rows in contiguous pieces of
  // 64 bytes (16-bit buffers) or 128 (32-bit).
  if (VEC && (static_cast<long long>(N) * sizeof(TC)) % 16 == 0) {
    constexpr int EPV = 16 / static_cast<int>(sizeof(TC));       // channels per 16-byte piece
    constexpr int kRowPieces = 32 / EPV;                          // pieces of a block's row
    constexpr int kPieces = 32 * kRowPieces / kWave;              // per lane and block
    // buffer row of every row piece this lane will write
    long long out_row[kPieces];
#pragma unroll
    for (int i = 0; i < kPieces; ++i) {
      const int rr = wv * 32 + (lane + i * kWave) / kRowPieces;
      out_row[i] = pos_list != nullptr ? (rr < valid ? static_cast<long long>(pos_list[rr]) : 0ll) : row_base + rr;
    }
    __syncthreads();                                              // every product has read its weights
    unsigned char *turn = b_lds + wv * kTurnBytes;
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      if (n0 + b * 32 >= N) break;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        TC four[4];
#pragma unroll
        for (int x = 0; x < 4; ++x) four[x] = static_cast<TC>(ScaledBuffer<T>::value ? acc[b][q * 4 + x] * scale : acc[b][q * 4 + x]);
        unsigned char *at = turn + r * kTurnRow + (q * 8 + h * 4) * static_cast<int>(sizeof(TC));
        if (sizeof(TC) == 2) {
          *reinterpret_cast<uint2 *>(at) = *reinterpret_cast<const uint2 *>(four);
        } else {
          *reinterpret_cast<uint4 *>(at) = *reinterpret_cast<const uint4 *>(four);
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
      for (int i = 0; i < kPieces; ++i) {
        const int piece = lane + i * kWave;
        const int pr = piece / kRowPieces, part = piece % kRowPieces;
        const int ch = n0 + b * 32 + part * EPV;
        const uint4 v = *reinterpret_cast<const uint4 *>(turn + pr * kTurnRow + part * 16);
        if (wv * 32 + pr < valid && ch < N) {                     // N % EPV == 0: a piece is all in or all out
          *reinterpret_cast<uint4 *>(c + out_row[i] * N + ch) = v;
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
  } else if (row_ok) {
    TC *dst = c + (pos_list != nullptr ? static_cast<long long>(pos_list[row]) : row_base + row) * N;
#pragma unroll
    for (int b = 0; b < NB; ++b) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int ch = n0 + b * 32 + q * 8 + h * 4;
        if (VEC && ch + 4 <= N) {
          TC out[4];
#pragma unroll
          for (int x = 0; x < 4; ++x) out[x] = static_cast<TC>(ScaledBuffer<T>::value ? acc[b][q * 4 + x] * scale : acc[b][q * 4 + x]);
          if (sizeof(TC) == 2) {
            *reinterpret_cast<uint2 *>(dst + ch) = *reinterpret_cast<const uint2 *>(out);
          } else {
            *reinterpret_cast<uint4 *>(dst + ch) = *reinterpret_cast<const uint4 *>(out);
          }
        } else {
#pragma unroll
          for (int x = 0; x < 4; ++x) {
            if (ch + x < N) dst[ch + x] = static_cast<TC>(ScaledBuffer<T>::value ? acc[b][q * 4 + x] * scale : acc[b][q * 4 + x]);
          }
        }
      }
    }
  }
  if (!next.ok) break;                  // the same for the whole workgroup
  __syncthreads();                      // the next tile's weights go where this one's were (and its turned blocks)
  tile = next_tile;
  here = next;
  here_rows = next_rows;
  }
}

template <typename T, typename TC, int NB, bool VEC, int CH>
__global__ __launch_bounds__(kGemmBlock, 3) void grouped_gemm_kernel(
    const T *__restrict__ a, TC *__restrict__ c, const T *__restrict__ wt,
    const int *__restrict__ meta, int K, int N, int Kp, int Np,
    const int *__restrict__ gather_index, const int *__restrict__ out_pos, const float *__restrict__ range) {
  grouped_gemm_body<T, TC, NB, VEC, CH>(a, c, wt, MetaInMemory{meta}, K, N, Kp, Np, gather_index, out_pos, range);
}

// The same with the tables as a by-value argument.
template <typename T, typename TC, int NB, bool VEC, int CH>
__global__ __launch_bounds__(kGemmBlock, 3) void grouped_gemm_riding_kernel(
    const T *__restrict__ a, TC *__restrict__ c, const T *__restrict__ wt, int K, int N, int Kp, int Np,
    const int *__restrict__ gather_index, PlanChunk table, int table_count, int meta_at,
    int *__restrict__ table_out, const int *__restrict__ out_pos, const float *__restrict__ range) {
  if (blockIdx.x == 0 && blockIdx.y == 0) {
    for (int i = threadIdx.x; i < table_count; i += kGemmBlock) table_out[i] = table.v[i];
  }
  grouped_gemm_body<T, TC, NB, VEC, CH>(a, c, wt, MetaInArguments{&table, meta_at}, K, N, Kp, Np,
                                        gather_index, out_pos, range);
}

// The grouped GEMM over offset groups (see GroupView).  Workgroup (0, 0) also
// leaves the buffer row at which every group starts, for the Scatter that
// follows in the stream.
template <typename T, typename TC, int NB, int SC>
__global__ __launch_bounds__(kGemmBlock, 3) void group_gemm_kernel(
    const T *__restrict__ a, TC *__restrict__ c, const T *__restrict__ wt, int K, int N, int Kp, int Np,
    GroupView groups, int *__restrict__ row_start_out, const float *__restrict__ range) {
  if (blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x <= kGroupCount) {
    row_start_out[threadIdx.x] = static_cast<int>(threadIdx.x * groups.stride);
  }
  grouped_gemm_body<T, TC, NB, true, SC, MetaInMemory, kGroupMembers>(a, c, wt, MetaInMemory{nullptr}, K, N, Kp, Np,
                                                                      nullptr, nullptr, range, &groups);
}

// ---------------------------------------------------- offset-group tables ----
//
// From the dense kernel map M [27, T] of a 3 x 3 x 3 layer: for each of the
// three axes the 27 offsets fall into 9 groups of 3 that differ along that
// axis only.  A target belongs to a group when any of the group's offsets
// reaches a source.  Three launches, no wait on the host:
//   group_count_kernel   targets per (axis, group, tile of 256 targets);
//   group_scan_kernel    one workgroup: totals per axis, the axis with the
//                        fewest rows wins (the lowest on a tie), its tile counts
//                        become exclusive prefixes, head = [axis, rows of the
//                        9 groups];
//   group_emit_kernel    rank of every target inside its groups (-1: none) and
//                        the member source rows of every data row.
struct GroupOffsets {
  int o[3 * kGroupCount * kGroupMembers];     // offset of member m of group j along axis a: [a][j][m]
};
constexpr int kGroupTile = 256;

__device__ __forceinline__ bool group_reaches(const int *__restrict__ dense, long long num_targets,
                                              const GroupOffsets &tab, int slot, long long t, int (&row)[3]) {
  bool any = false;
#pragma unroll
  for (int m = 0; m < kGroupMembers; ++m) {
    row[m] = dense[static_cast<long long>(tab.o[slot * kGroupMembers + m]) * num_targets + t];
    any |= row[m] >= 0;
  }
  return any;
}

__global__ __launch_bounds__(kGroupTile) void group_count_kernel(const int *__restrict__ dense,
                                                                  long long num_targets, GroupOffsets tab,
                                                                  int tiles, int *__restrict__ tile_counts) {
  __shared__ int s_count[kGroupTile / kWave];
  const int slot = blockIdx.y;                                   // axis * 9 + group
  const long long t = static_cast<long long>(blockIdx.x) * kGroupTile + threadIdx.x;
  int row[3];
  const bool any = t < num_targets && group_reaches(dense, num_targets, tab, slot, t, row);
  const int count = __popcll(__ballot(any));
  if ((threadIdx.x & (kWave - 1)) == 0) s_count[threadIdx.x / kWave] = count;
  __syncthreads();
  if (threadIdx.x == 0) {
    int sum = 0;
#pragma unroll
    for (int w = 0; w < kGroupTile / kWave; ++w) sum += s_count[w];
    tile_counts[slot * tiles + blockIdx.x] = sum;
  }
}

__global__ __launch_bounds__(1024) void group_scan_kernel(int *__restrict__ tile_counts, int tiles,
                                                           int *__restrict__ head) {
  constexpr int kWaves = 1024 / kWave;
  constexpr int kBatch = 8;                          // loads a lane keeps in flight
  __shared__ int s_part[3][kWaves];
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  // totals per axis: every lane adds up a strided share, kBatch loads at a time
  const int per_axis = kGroupCount * tiles;
  for (int axis = 0; axis < 3; ++axis) {
    const int *counts = tile_counts + axis * per_axis;
    int mine = 0;
    for (int base = tid; base < per_axis; base += kBatch * 1024) {
      int v[kBatch];
#pragma unroll
      for (int k = 0; k < kBatch; ++k) v[k] = base + k * 1024 < per_axis ? counts[base + k * 1024] : 0;
#pragma unroll
      for (int k = 0; k < kBatch; ++k) mine += v[k];
    }
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) mine += __shfl_xor(mine, d);
    if (lane == 0) s_part[axis][wave] = mine;
  }
  __syncthreads();
  int total[3] = {0, 0, 0};
#pragma unroll
  for (int axis = 0; axis < 3; ++axis) {
#pragma unroll
    for (int w = 0; w < kWaves; ++w) total[axis] += s_part[axis][w];
  }
  int axis = 0;
  if (total[1] < total[axis]) axis = 1;
  if (total[2] < total[axis]) axis = 2;
  if (tid == 0) head[0] = axis;
  // exclusive prefixes of the winning axis' tile counts: a wavefront per group,
  // kBatch x 64 counts fetched at a time and scanned in registers
  if (wave >= kGroupCount) return;
  int *counts = tile_counts + (axis * kGroupCount + wave) * tiles;
  int carry = 0;
  for (int base = 0; base < tiles; base += kBatch * kWave) {
    int v[kBatch];
#pragma unroll
    for (int k = 0; k < kBatch; ++k) {
      const int i = base + k * kWave + lane;
      v[k] = i < tiles ? counts[i] : 0;
    }
#pragma unroll
    for (int k = 0; k < kBatch; ++k) {
      int scan = v[k];                                           // inclusive scan inside the wavefront
#pragma unroll
      for (int d = 1; d < kWave; d <<= 1) {
        const int up = __shfl_up(scan, d);
        if (lane >= d) scan += up;
      }
      const int i = base + k * kWave + lane;
      if (i < tiles) counts[i] = carry + scan - v[k];
      carry += __builtin_amdgcn_readlane(scan, kWave - 1);
    }
  }
  if (lane == 0) head[1 + wave] = carry;
}

__global__ __launch_bounds__(kGroupTile) void group_emit_kernel(const int *__restrict__ dense,
                                                                 long long num_targets, GroupOffsets tab,
                                                                 int tiles, const int *__restrict__ tile_counts,
                                                                 const int *__restrict__ head,
                                                                 int *__restrict__ rank_out,
                                                                 int4 *__restrict__ src_out) {
  __shared__ int s_count[kGroupTile / kWave];
  const int axis = head[0];
  const int group = blockIdx.y;
  const int slot = axis * kGroupCount + group;
  const int base = tile_counts[slot * tiles + blockIdx.x];
  const long long t = static_cast<long long>(blockIdx.x) * kGroupTile + threadIdx.x;
  int row[3] = {-1, -1, -1};
  const bool any = t < num_targets && group_reaches(dense, num_targets, tab, slot, t, row);
  const unsigned long long ballot = __ballot(any);
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  if (lane == 0) s_count[wave] = __popcll(ballot);
  __syncthreads();
  int before = base;
  for (int w = 0; w < wave; ++w) before += s_count[w];
  const int rank = before + __popcll(ballot & ((1ull << lane) - 1ull));
  if (t < num_targets) {
    rank_out[static_cast<long long>(group) * num_targets + t] = any ? rank : -1;
    if (any) src_out[static_cast<long long>(group) * num_targets + rank] = make_int4(row[0], row[1], row[2], 0);
  }
}

// ---------------------------------------------------------- host launchers ----

static int pow2_vec(int64_t bytes_per_lane, int64_t row_bytes, const void *p0, const void *p1) {
  const uintptr_t align = reinterpret_cast<uintptr_t>(p0) | reinterpret_cast<uintptr_t>(p1);
  for (int vb = 16; vb >= 2; vb >>= 1) {
    if (bytes_per_lane % vb == 0 && row_bytes % vb == 0 && align % vb == 0) return vb;
  }
  return 0;
}

struct LaneShape {
  int vb;
  int nv;
  int lanes_per_row;
};

// Maps the reference's "tile size" (feature elements per thread, must divide
// the channel count) to vector width and vectors per lane.  tile == 0 picks
// 16 bytes per lane.
static LaneShape lane_shape(int64_t tile, int64_t channels, int esize, const void *p0, const void *p1,
                            const char *what) {
  const int64_t row_bytes = channels * esize;
  if (tile <= 0) {
    tile = 16 / esize;
    while (tile > 1 && channels % tile != 0) tile >>= 1;
  }
  MNT_CHECK(channels % tile == 0, "Unsupported %s = %lld with tile size = %lld", what,
            static_cast<long long>(channels), static_cast<long long>(tile));
  const int64_t bytes_per_lane = tile * esize;
  LaneShape shape;
  shape.vb = pow2_vec(bytes_per_lane, row_bytes, p0, p1);
  MNT_CHECK(shape.vb >= esize && shape.vb > 0, "feature rows are not aligned to their element size");
  shape.nv = static_cast<int>(bytes_per_lane / shape.vb);
  MNT_CHECK(shape.nv >= 1 && shape.nv <= 8 && (shape.nv & (shape.nv - 1)) == 0,
            "Unsupported %s = %lld with tile size = %lld", what, static_cast<long long>(channels),
            static_cast<long long>(tile));
  shape.lanes_per_row = static_cast<int>(row_bytes / bytes_per_lane);
  return shape;
}

template <typename IT>
static void launch_gather(const LaneShape &sh, const void *sources, void *buffer, const IT *masks,
                          const int *row_start, int64_t num_sources, int num_offsets, int row_bytes,
                          hipStream_t stream) {
  if (num_sources == 0 || num_offsets == 0) return;
  const unsigned grid = static_cast<unsigned>(div_ceil(num_sources * sh.lanes_per_row, 256));
#define MNT_G(VB, NV)                                                                            \
  gather_kernel<VB, NV, IT><<<grid, 256, 0, stream>>>(static_cast<const unsigned char *>(sources), \
                                                      static_cast<unsigned char *>(buffer), masks,  \
                                                      row_start, num_sources, num_offsets,          \
                                                      row_bytes, sh.lanes_per_row)
#define MNT_GV(VB)                 \
  switch (sh.nv) {                 \
    case 1: MNT_G(VB, 1); break;   \
    case 2: MNT_G(VB, 2); break;   \
    case 4: MNT_G(VB, 4); break;   \
    default: MNT_G(VB, 8); break;  \
  }
  switch (sh.vb) {
    case 16: MNT_GV(16); break;
    case 8: MNT_GV(8); break;
    case 4: MNT_GV(4); break;
    default: MNT_GV(2); break;
  }
#undef MNT_GV
#undef MNT_G
  check_launch("gather_kernel");
}

// Largest kernel (offset count) the listed scatter stages in LDS; larger ones
// take the direct form.
constexpr int kScatterListedOffsets = 343;

template <typename TB, typename T, typename IT>
static void launch_scatter(const LaneShape &sh, const TB *buffer, void *targets, const IT *masks,
                           const int *row_start, int64_t num_targets, int num_offsets, int channels,
                           const TB *direct, const Epilogue &ep, hipStream_t stream) {
  if (num_targets == 0) return;
  if (num_offsets <= kScatterFewOffsets && sh.nv <= 2 && sizeof(TB) <= sizeof(T)) {
    const unsigned few_grid = static_cast<unsigned>(div_ceil(num_targets * sh.lanes_per_row, 256));
#define MNT_F(VB, NV)                                                                                          \
  scatter_few_kernel<TB, T, VB, NV, IT, kScatterFewOffsets><<<few_grid, 256, 0, stream>>>(                      \
      buffer, static_cast<unsigned char *>(targets), masks, row_start, num_targets, num_offsets, channels,     \
      sh.lanes_per_row, direct, ep)
#define MNT_FV(VB)       \
  if (sh.nv == 1) {      \
    MNT_F(VB, 1);        \
  } else {               \
    MNT_F(VB, 2);        \
  }
    if (sh.vb == 16) {
      MNT_FV(16);
      check_launch("scatter_few_kernel");
      return;
    }
    if (sh.vb == 8) {
      MNT_FV(8);
      check_launch("scatter_few_kernel");
      return;
    }
#undef MNT_FV
#undef MNT_F
  }
  const bool listed = num_offsets <= kScatterListedOffsets && sh.lanes_per_row <= kScatterBlock;
  // 64 targets per workgroup (32 for large kernels, so that the row lists fit
  // in LDS); fewer when that would leave most of the chip without a workgroup,
  // but never fewer than the lane groups of a workgroup
  int tile_shift = num_offsets <= 128 ? 6 : 5;
  const int groups = std::max(1, kScatterBlock / sh.lanes_per_row);
  while (tile_shift > 3 && (num_targets >> tile_shift) < 1024 && (1 << (tile_shift - 1)) >= groups) {
    --tile_shift;
  }
  const unsigned grid =
      listed ? static_cast<unsigned>(div_ceil(num_targets, int64_t{1} << tile_shift))
             : static_cast<unsigned>(div_ceil(num_targets * sh.lanes_per_row, 256));
  const size_t lds =
      static_cast<size_t>(num_offsets + (kScatterBlock >> tile_shift)) * sizeof(int) << tile_shift;
#define MNT_S(VB, NV)                                                                               \
  if (listed) {                                                                                     \
    scatter_kernel<TB, T, VB, NV, IT><<<grid, kScatterBlock, lds, stream>>>(                        \
        buffer, static_cast<unsigned char *>(targets), masks, row_start, num_targets, num_offsets,  \
        channels, sh.lanes_per_row, direct, tile_shift, ep);                                        \
  } else {                                                                                          \
    scatter_wide_kernel<TB, T, VB, NV, IT><<<grid, 256, 0, stream>>>(                               \
        buffer, static_cast<unsigned char *>(targets), masks, row_start, num_targets, num_offsets,  \
        channels, sh.lanes_per_row, direct, ep);                                                    \
  }
#define MNT_SV(VB)                 \
  switch (sh.nv) {                 \
    case 1: MNT_S(VB, 1); break;   \
    case 2: MNT_S(VB, 2); break;   \
    case 4: MNT_S(VB, 4); break;   \
    default: MNT_S(VB, 8); break;  \
  }
  if (sh.vb == 16) {
    MNT_SV(16);
  } else if (sh.vb == 8) {
    MNT_SV(8);
  } else if (sh.vb == 4) {
    MNT_SV(4);
  } else {
    if constexpr (sizeof(T) == 2) {
      MNT_SV(2);
    } else {
      MNT_FAIL("feature rows are not aligned to their element size");
    }
  }
#undef MNT_SV
#undef MNT_S
  check_launch("scatter_kernel");
}

// Integer tables that ride a GEMM launch as a kernel argument (count == 0:
// none, the kernel reads `meta` from device memory).
// Passes of at most this many GEMM tiles take their tables as an argument of
// the GEMM (one launch less); larger ones upload them first, which costs a
// launch but keeps the tables in device memory for thousands of workgroups.
constexpr int kRidingMaxTiles = 4096;

struct RidingTable {
  const std::vector<int> *ints = nullptr;
  int meta_at = 0;
  int *out = nullptr;
};

template <typename T, typename TC, int NB>
static void launch_gemm_nb(const T *a, TC *c, const T *wt, const int *meta, int num_tiles, int K, int N,
                           int Kp, int Np, bool vec, const int *gather_index, const RidingTable &riding,
                           hipStream_t stream, const int *out_pos, const float *range) {
  // as many workgroups as the compute units hold at once (by registers); each
  // walks its share of the tiles
  const int slices = static_cast<int>(div_ceil(Np, NB * 32));
  const int resident = compute_units() * (NB >= 3 ? 3 : NB == 2 ? 4 : 6);
  dim3 grid(static_cast<unsigned>(std::min(num_tiles, std::max(1, resident / slices))),
            static_cast<unsigned>(slices));
  // rows of one or two chunks are loaded whole, ahead of the first product
  const int chunks = Kp / (kChunkBytes / static_cast<int>(sizeof(T)));
  const int held = vec && chunks <= 2 ? chunks : 0;
  if (riding.ints != nullptr) {
    PlanChunk chunk;
    const int count = static_cast<int>(riding.ints->size());
    std::memcpy(chunk.v, riding.ints->data(), count * sizeof(int));
#define MNT_RIDING(VEC, CH)                                                                 \
  grouped_gemm_riding_kernel<T, TC, NB, VEC, CH><<<grid, kGemmBlock, 0, stream>>>(          \
      a, c, wt, K, N, Kp, Np, gather_index, chunk, count, riding.meta_at, riding.out, out_pos, range)
    if (held == 1) {
      MNT_RIDING(true, 1);
    } else if (held == 2) {
      MNT_RIDING(true, 2);
    } else if (vec) {
      MNT_RIDING(true, 0);
    } else {
      MNT_RIDING(false, 0);
    }
#undef MNT_RIDING
  } else {
#define MNT_PLAIN(VEC, CH)                                                                  \
  grouped_gemm_kernel<T, TC, NB, VEC, CH><<<grid, kGemmBlock, 0, stream>>>(a, c, wt, meta, K, N, Kp, Np, \
                                                                           gather_index, out_pos, range)
    if (held == 1) {
      MNT_PLAIN(true, 1);
    } else if (held == 2) {
      MNT_PLAIN(true, 2);
    } else if (vec) {
      MNT_PLAIN(true, 0);
    } else {
      MNT_PLAIN(false, 0);
    }
#undef MNT_PLAIN
  }
}

template <typename T, typename TC>
static void launch_gemm(const T *a, TC *c, const T *wt, const int *meta, int num_tiles, int K, int N,
                        int Kp, int Np, const int *gather_index, hipStream_t stream,
                        const RidingTable &riding = RidingTable(), const int *out_pos = nullptr,
                        const float *range = nullptr) {
  if (num_tiles == 0) return;
  const bool vec = (static_cast<int64_t>(K) * sizeof(T)) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(a) % 16 == 0 && N % 4 == 0 &&
                   reinterpret_cast<uintptr_t>(c) % 16 == 0;
  // All channels in one workgroup up to 128; wider outputs are cut into equal
  // slices of at most 128 channels (A is then read once per slice).  Eight
  // blocks per workgroup would read A once at 256 channels, but their 128
  // accumulator registers leave one workgroup per CU and measured slower.
  const int blocks = Np / 32;
  const int slices = static_cast<int>(div_ceil(blocks, kMaxChannelBlocks));
  switch (static_cast<int>(div_ceil(blocks, slices))) {
    case 1: launch_gemm_nb<T, TC, 1>(a, c, wt, meta, num_tiles, K, N, Kp, Np, vec, gather_index, riding, stream, out_pos, range); break;
    case 2: launch_gemm_nb<T, TC, 2>(a, c, wt, meta, num_tiles, K, N, Kp, Np, vec, gather_index, riding, stream, out_pos, range); break;
    case 3: launch_gemm_nb<T, TC, 3>(a, c, wt, meta, num_tiles, K, N, Kp, Np, vec, gather_index, riding, stream, out_pos, range); break;
    default: launch_gemm_nb<T, TC, 4>(a, c, wt, meta, num_tiles, K, N, Kp, Np, vec, gather_index, riding, stream, out_pos, range); break;
  }
  check_launch("grouped_gemm_kernel");
}

// ------------------------------------------------------------ forward plan ----

struct ForwardPlan {
  int64_t active_offsets;            // offsets that go through gather/GEMM/scatter
  bool shortcut;
  std::vector<int64_t> cum;          // padded row prefix, active_offsets + 1
  std::vector<int> meta;             // grouped-GEMM meta (see kernel)
  std::vector<int> row_start;        // int copy of cum for gather / scatter
  int num_tiles;
  int64_t total_rows;
};

static ForwardPlan make_forward_plan(const int64_t *sizes, int64_t num_offsets, int64_t num_sources,
                                     int64_t num_targets, bool allow_shortcut, bool has_threshold,
                                     double threshold) {
  ForwardPlan plan;
  plan.shortcut = allow_shortcut && num_offsets > 0 && sizes[num_offsets - 1] == num_targets &&
                  sizes[num_offsets - 1] == num_sources;
  plan.active_offsets = plan.shortcut ? num_offsets - 1 : num_offsets;
  std::vector<int64_t> buckets;
  padding_buckets(sizes, plan.active_offsets, has_threshold, threshold, buckets);
  cumsum_padded(sizes, plan.active_offsets, buckets, plan.cum);
  plan.total_rows = plan.cum[plan.active_offsets];
  MNT_CHECK(plan.total_rows <= INT32_MAX, "gather buffer of %lld rows exceeds the 32-bit row index",
            static_cast<long long>(plan.total_rows));
  plan.row_start.resize(plan.active_offsets + 1);
  for (int64_t j = 0; j <= plan.active_offsets; ++j) plan.row_start[j] = static_cast<int>(plan.cum[j]);
  std::vector<int> groups;
  for (int64_t j = 0; j < plan.active_offsets; ++j) {
    if (sizes[j] > 0) groups.push_back(static_cast<int>(j));
  }
  const int G = static_cast<int>(groups.size());
  plan.meta.assign(1 + (G + 1) + (G + 1) + G + G + G, 0);
  plan.meta[0] = G;
  int *tile_prefix = plan.meta.data() + 1;
  int *row_start = tile_prefix + G + 1;
  int *rows = row_start + G + 1;
  int *weight = rows + G;
  int *list_start = weight + G;
  int tiles = 0;
  int64_t listed = 0;
  int next = 0;
  for (int i = 0; i < G; ++i) {
    const int j = groups[i];
    for (; next < j; ++next) listed += sizes[next];
    list_start[i] = static_cast<int>(listed);
    tile_prefix[i] = tiles;
    row_start[i] = static_cast<int>(plan.cum[j]);
    rows[i] = static_cast<int>(sizes[j]);
    weight[i] = j;
    tiles += static_cast<int>(div_ceil(sizes[j], kGemmRows));
  }
  tile_prefix[G] = tiles;
  row_start[G] = static_cast<int>(plan.total_rows);
  plan.num_tiles = tiles;
  return plan;
}

static std::vector<int> direct_meta(int64_t rows, int weight_index) {
  // one group: all rows of the source tensor against one weight matrix
  std::vector<int> meta = {1, 0, static_cast<int>(div_ceil(rows, kGemmRows)), 0, static_cast<int>(rows),
                           static_cast<int>(rows), weight_index, 0};
  return meta;
}

static void read_sizes(const void *sizes_dev, int index_dtype, int64_t num_offsets,
                       std::vector<int64_t> &out, hipStream_t stream) {
  out.resize(num_offsets);
  if (num_offsets == 0) return;
  const int isz = int_size(index_dtype);
  std::vector<unsigned char> raw(static_cast<size_t>(isz) * num_offsets);
  MNT_HIP(hipMemcpyAsync(raw.data(), sizes_dev, raw.size(), hipMemcpyDeviceToHost, stream));
  MNT_HIP(hipStreamSynchronize(stream));
  for (int64_t j = 0; j < num_offsets; ++j) {
    out[j] = isz == 4 ? static_cast<int64_t>(reinterpret_cast<int32_t *>(raw.data())[j])
                      : reinterpret_cast<int64_t *>(raw.data())[j];
  }
}


// Range of the pass's product rows (see range_kernel): null unless the
// buffer of feature type T is a scaled one.
template <typename T>
static float *measure_range(Scope &scope, const T *features, int64_t count, const T *wt, int64_t columns,
                            int Kp, hipStream_t stream) {
  if (!ScaledBuffer<T>::value) return nullptr;
  float *range = scope.alloc<float>(kRangeParts);
  range_kernel<T><<<kRangeParts, 256, 0, stream>>>(features, static_cast<long long>(count), wt,
                                                   static_cast<long long>(columns), Kp, range);
  check_launch("range_kernel");
  profile_mark("range", stream);
  return range;
}

template <typename T, typename IT>
static void forward_typed(int64_t gather_tile, int64_t scatter_tile, const ForwardPlan &plan,
                          const T *sources, const T *weights, const IT *source_masks,
                          const IT *target_masks, const IT *order, const int *gather_index,
                          const Epilogue &epilogue, const T *packed, const int64_t *order_host,
                          int64_t S, int64_t Tn, int64_t O, int64_t K, int64_t N, T *out,
                          hipStream_t stream) {
  Scope scope(stream);
  const int kc = kChunkBytes / static_cast<int>(sizeof(T));
  const int Kp = static_cast<int>(div_ceil(K, kc) * kc);
  const int Np = static_cast<int>(div_ceil(N, 32) * 32);
  const int active = static_cast<int>(plan.active_offsets);

  profile_mark("enter:forward", stream);
  const bool folded = gather_index != nullptr;      // Gather folded into the GEMM's A load
  const bool ahead = packed != nullptr;             // weights packed by the caller
  const size_t rows = static_cast<size_t>(plan.total_rows > 0 ? plan.total_rows : 1);
  const int64_t centre = ahead && order_host != nullptr && O > 0 ? order_host[O - 1] : O - 1;

  // One integer table for the whole pass: row starts, then the GEMM groups.
  // With the folded gather both products read the source features, so the
  // centre offset of the shortcut joins the grouped launch as one more group
  // (rows taken as they are, output after the other buffer rows); otherwise
  // its single-group descriptor follows for a launch of its own.
  std::vector<int> meta(plan.meta);
  int num_tiles = plan.num_tiles;
  if (ahead && order_host != nullptr) {
    // weights packed ahead of time are in the layer's own offset order: point
    // every GEMM group at the matrix of the offset its row stands for
    const int G = meta[0];
    int *weight = meta.data() + 1 + (G + 1) + (G + 1) + G;
    for (int i = 0; i < G; ++i) weight[i] = static_cast<int>(order_host[weight[i]]);
  }
  const bool merged = plan.shortcut && folded;
  if (merged) {
    const int G = meta[0];
    const int *tile_prefix = meta.data() + 1, *row_start = tile_prefix + G + 1, *count = row_start + G + 1,
              *weight = count + G, *list_start = weight + G;
    const int extra = static_cast<int>(div_ceil(S, kGemmRows));
    std::vector<int> grown;
    grown.push_back(G + 1);
    grown.insert(grown.end(), tile_prefix, tile_prefix + G + 1);
    grown.push_back(tile_prefix[G] + extra);
    grown.insert(grown.end(), row_start, row_start + G);
    grown.push_back(static_cast<int>(rows));
    grown.push_back(static_cast<int>(rows + S));
    grown.insert(grown.end(), count, count + G);
    grown.push_back(static_cast<int>(S));
    grown.insert(grown.end(), weight, weight + G);
    grown.push_back(static_cast<int>(centre));
    grown.insert(grown.end(), list_start, list_start + G);
    grown.push_back(-1);
    meta.swap(grown);
    num_tiles += extra;
  }
  std::vector<int> ints(plan.row_start);
  const size_t meta_at = ints.size();
  ints.insert(ints.end(), meta.begin(), meta.end());
  const size_t direct_at = ints.size();
  std::vector<int> dmeta;
  if (plan.shortcut && !merged) {
    dmeta = direct_meta(S, static_cast<int>(centre));
    ints.insert(ints.end(), dmeta.begin(), dmeta.end());
  }
  int *d_ints = scope.alloc<int>(ints.size());
  int *d_row_start = d_ints;
  int *d_meta = d_ints + meta_at;
  int *d_direct = d_ints + direct_at;
  const bool fits = ints.size() <= static_cast<size_t>(kPlanInts);
  // the table travels as an argument of the first kernel of the pass: the
  // packing kernel, or with packed weights and the folded gather the GEMM
  RidingTable riding;
  const T *wt = packed;
  if (ahead) {
    if (fits && folded && num_tiles > 0 && num_tiles <= kRidingMaxTiles) {
      riding.ints = &ints;
      riding.meta_at = static_cast<int>(meta_at);
      riding.out = d_ints;
    } else {
      upload_ints(ints, d_ints, stream);
    }
  } else {
    T *fresh = scope.alloc<T>(static_cast<size_t>(O) * Np * Kp);
    wt = fresh;
    PlanChunk chunk;
    int count = 0;
    if (fits) {
      count = static_cast<int>(ints.size());
      std::memcpy(chunk.v, ints.data(), ints.size() * sizeof(int));
    } else {
      upload_ints(ints, d_ints, stream);
    }
    const long long total = static_cast<long long>(O) * Np * Kp;
    pack_weights_kernel<T, IT><<<grid_for(total, 256, 4096), 256, 0, stream>>>(
        weights, order, static_cast<int>(O), static_cast<int>(K), static_cast<int>(N), Kp, Np, fresh, chunk,
        count, d_ints);
    check_launch("pack_weights_kernel");
  }
  profile_mark("pack_weights", stream);

  typedef typename BufferOf<T>::type TB;
  // with the shortcut the centre offset's product takes one extra buffer row per target
  TB *cbuf = scope.alloc<TB>((rows + (plan.shortcut ? static_cast<size_t>(Tn) : 0)) * N);
  TB *direct = plan.shortcut ? cbuf + rows * N : nullptr;
  const float *range = measure_range<T>(scope, sources, S * K, wt, O * Np, Kp, stream);
  Epilogue finish = epilogue;
  finish.range = range;

  if (folded) {
    launch_gemm<T, TB>(sources, cbuf, wt, d_meta, num_tiles, static_cast<int>(K), static_cast<int>(N), Kp, Np,
                       gather_index, stream, riding, nullptr, range);
  } else {
    T *abuf = scope.alloc<T>(rows * K);
    const LaneShape gsh = lane_shape(gather_tile, K, sizeof(T), sources, abuf, "num_source_features");
    launch_gather<IT>(gsh, sources, abuf, source_masks, d_row_start, S, active,
                      static_cast<int>(K * sizeof(T)), stream);
    profile_mark("gather", stream);
    launch_gemm<T, TB>(abuf, cbuf, wt, d_meta, num_tiles, static_cast<int>(K), static_cast<int>(N), Kp, Np,
                       nullptr, stream, RidingTable(), nullptr, range);
  }
  if (plan.shortcut && !merged) {
    launch_gemm<T, TB>(sources, direct, wt, d_direct, dmeta[2], static_cast<int>(K), static_cast<int>(N), Kp, Np,
                       nullptr, stream, RidingTable(), nullptr, range);
  }
  profile_mark("gemm", stream);

  const LaneShape ssh = lane_shape(scatter_tile, N, sizeof(T), cbuf, out, "num_target_features");
  launch_scatter<TB, T, IT>(ssh, cbuf, out, target_masks, d_row_start, Tn, active,
                            static_cast<int>(N), direct, finish, stream);
  profile_mark("scatter", stream);
}

template <typename TB, typename T>
static void launch_scatter_rows(const LaneShape &sh, const TB *buffer, void *targets, const int *row_ptr,
                                int64_t num_targets, int channels, const Epilogue &ep, hipStream_t stream) {
  if (num_targets == 0) return;
  MNT_CHECK(sh.lanes_per_row <= kScatterBlock, "feature rows of %d lanes do not fit a workgroup", sh.lanes_per_row);
  const int groups = std::max(1, kScatterBlock / sh.lanes_per_row);
  int tile = 64;
  while (tile > 8 && num_targets / tile < 2048 && tile / 2 >= groups) tile /= 2;
  tile = std::max(tile, groups);
  const unsigned grid = static_cast<unsigned>(div_ceil(num_targets, tile));
#define MNT_S(VB, NV)                                                                     \
  scatter_rows_kernel<TB, T, VB, NV><<<grid, kScatterBlock, 0, stream>>>(                 \
      buffer, static_cast<unsigned char *>(targets), row_ptr, num_targets, channels, sh.lanes_per_row, tile, ep)
#define MNT_SV(VB)                 \
  switch (sh.nv) {                 \
    case 1: MNT_S(VB, 1); break;   \
    case 2: MNT_S(VB, 2); break;   \
    case 4: MNT_S(VB, 4); break;   \
    default: MNT_S(VB, 8); break;  \
  }
  if (sh.vb == 16) {
    MNT_SV(16);
  } else if (sh.vb == 8) {
    MNT_SV(8);
  } else if (sh.vb == 4) {
    MNT_SV(4);
  } else {
    if constexpr (sizeof(T) == 2) {
      MNT_SV(2);
    } else {
      MNT_FAIL("feature rows are not aligned to their element size");
    }
  }
#undef MNT_SV
#undef MNT_S
  check_launch("scatter_rows_kernel");
}

// Forward pass of the list-driven dataflow: grouped GEMM reading its rows through
// in_idx and writing them to out_pos, then the streaming Scatter.
template <typename T>
static void forward_rows_typed(int64_t scatter_tile, const ForwardPlan &plan, const T *sources,
                               const T *weights, const int *in_idx, const int *out_pos,
                               const int *row_ptr, const Epilogue &epilogue, const T *packed,
                               const int64_t *order_host, int64_t S, int64_t Tn, int64_t O, int64_t K,
                               int64_t N, T *out, hipStream_t stream) {
  Scope scope(stream);
  const int kc = kChunkBytes / static_cast<int>(sizeof(T));
  const int Kp = static_cast<int>(div_ceil(K, kc) * kc);
  const int Np = static_cast<int>(div_ceil(N, 32) * 32);
  profile_mark("enter:forward", stream);
  // every group points at the matrix of the offset its row stands for (the
  // weights are packed in the layer's own offset order)
  std::vector<int> meta(plan.meta);
  {
    const int G = meta[0];
    int *weight = meta.data() + 1 + (G + 1) + (G + 1) + G;
    if (order_host != nullptr) {
      for (int i = 0; i < G; ++i) weight[i] = static_cast<int>(order_host[weight[i]]);
    }
  }
  std::vector<int> ints(plan.row_start);
  const size_t meta_at = ints.size();
  ints.insert(ints.end(), meta.begin(), meta.end());
  int *d_ints = scope.alloc<int>(ints.size());
  int *d_meta = d_ints + meta_at;
  const bool fits = ints.size() <= static_cast<size_t>(kPlanInts);
  RidingTable riding;
  const T *wt = packed;
  if (packed != nullptr) {
    if (fits && plan.num_tiles > 0 && plan.num_tiles <= kRidingMaxTiles) {
      riding.ints = &ints;
      riding.meta_at = static_cast<int>(meta_at);
      riding.out = d_ints;
    } else {
      upload_ints(ints, d_ints, stream);
    }
  } else {
    T *fresh = scope.alloc<T>(static_cast<size_t>(O) * Np * Kp);
    wt = fresh;
    PlanChunk chunk;
    int count = 0;
    if (fits) {
      count = static_cast<int>(ints.size());
      std::memcpy(chunk.v, ints.data(), ints.size() * sizeof(int));
    } else {
      upload_ints(ints, d_ints, stream);
    }
    const long long total = static_cast<long long>(O) * Np * Kp;
    pack_weights_kernel<T, int32_t><<<grid_for(total, 256, 4096), 256, 0, stream>>>(
        weights, nullptr, static_cast<int>(O), static_cast<int>(K), static_cast<int>(N), Kp, Np, fresh, chunk,
        count, d_ints);
    check_launch("pack_weights_kernel");
  }
  profile_mark("pack_weights", stream);
  typedef typename BufferOf<T>::type TB;
  const size_t rows = static_cast<size_t>(plan.total_rows > 0 ? plan.total_rows : 1);
  TB *cbuf = scope.alloc<TB>(rows * N);
  const float *range = measure_range<T>(scope, sources, S * K, wt, O * Np, Kp, stream);
  Epilogue finish = epilogue;
  finish.range = range;
  launch_gemm<T, TB>(sources, cbuf, wt, d_meta, plan.num_tiles, static_cast<int>(K), static_cast<int>(N), Kp, Np,
                     in_idx, stream, riding, out_pos, range);
  profile_mark("gemm", stream);
  const LaneShape ssh = lane_shape(scatter_tile, N, sizeof(T), cbuf, out, "num_target_features");
  launch_scatter_rows<TB, T>(ssh, cbuf, out, row_ptr, Tn, static_cast<int>(N), finish, stream);
  profile_mark("scatter", stream);
}

}  // namespace mnt

using namespace mnt;

extern "C" int mnt_generate_padding_buckets(const int64_t *sizes_host, int64_t num_offsets,
                                            int has_threshold, double threshold,
                                            int64_t *buckets_out, int64_t *num_boundaries_out) {
  return guarded([&] {
    MNT_CHECK(num_offsets >= 0 && buckets_out != nullptr && num_boundaries_out != nullptr, "bad argument");
    std::vector<int64_t> buckets;
    padding_buckets(sizes_host, num_offsets, has_threshold != 0, threshold, buckets);
    MNT_CHECK(buckets.back() == num_offsets, "bucket boundaries do not cover all offsets");
    for (size_t i = 0; i < buckets.size(); ++i) buckets_out[i] = buckets[i];
    *num_boundaries_out = static_cast<int64_t>(buckets.size());
  });
}

extern "C" int mnt_cumsum_kernel_padded_sizes(const int64_t *sizes_host, int64_t num_offsets,
                                              const int64_t *buckets, int64_t num_boundaries,
                                              int64_t *cumsum_out) {
  return guarded([&] {
    MNT_CHECK(num_offsets >= 0 && num_boundaries >= 1 && cumsum_out != nullptr, "bad argument");
    std::vector<int64_t> b(buckets, buckets + num_boundaries), cum;
    MNT_CHECK(b.front() == 0 && b.back() == num_offsets, "bucket boundaries must run from 0 to the number of offsets");
    cumsum_padded(sizes_host, num_offsets, b, cum);
    for (int64_t j = 0; j <= num_offsets; ++j) cumsum_out[j] = cum[j];
  });
}

#define MNT_DISPATCH_FI(float_dtype, index_dtype, CALL)               \
  do {                                                                \
    const bool i32_ = index_dtype == MNT_INT32;                       \
    if (float_dtype == MNT_FLOAT32) {                                 \
      if (i32_) { CALL(float, int32_t); } else { CALL(float, int64_t); }       \
    } else if (float_dtype == MNT_FLOAT16) {                          \
      if (i32_) { CALL(half_t, int32_t); } else { CALL(half_t, int64_t); }     \
    } else {                                                          \
      if (i32_) { CALL(bf16_t, int32_t); } else { CALL(bf16_t, int64_t); }     \
    }                                                                 \
  } while (0)

extern "C" int mnt_sparse_convolution_forward_fused(
    int64_t gather_tile, int64_t scatter_tile, int allow_shortcut_matmul, int64_t parallel,
    int has_threshold, double threshold, const void *sources, const void *weights,
    const void *source_masks, const void *target_masks, const void *kernel_map_order,
    const void *kernel_map_sizes, const int64_t *sizes_host, int64_t S, int64_t T, int64_t O,
    int64_t K, int64_t N, int index_dtype, int float_dtype, const int32_t *gather_index,
    const float *channel_scale, const float *channel_shift, const void *residual, int activation,
    float negative_slope, const void *packed_weights, const int64_t *order_host, void *out,
    void *stream_) {
  (void)parallel;
  return guarded([&] {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    int_size(index_dtype);
    float_size(float_dtype);
    MNT_CHECK(S >= 0 && T >= 0 && O >= 0 && K >= 1 && N >= 1 && S <= INT32_MAX && T <= INT32_MAX &&
                  O <= 65535 && K <= 65536 && N <= 65536,
              "bad shape S=%lld T=%lld O=%lld Cin=%lld Cout=%lld", (long long)S, (long long)T,
              (long long)O, (long long)K, (long long)N);
    MNT_CHECK(activation >= MNT_ACT_NONE && activation <= MNT_ACT_RELU6, "unknown activation code %d",
              activation);
    MNT_CHECK(reinterpret_cast<uintptr_t>(residual) % 16 == 0 &&
                  reinterpret_cast<uintptr_t>(channel_scale) % 4 == 0 &&
                  reinterpret_cast<uintptr_t>(channel_shift) % 4 == 0,
              "epilogue operands are not aligned (residual: 16 bytes, scale / shift: 4 bytes)");
    MNT_CHECK(packed_weights == nullptr || kernel_map_order == nullptr || order_host != nullptr,
              "weights packed ahead of time need the host copy of kernel_map_order");
    MNT_CHECK(reinterpret_cast<uintptr_t>(packed_weights) % 16 == 0, "packed weights are not 16-byte aligned");
    if (order_host != nullptr) {
      for (int64_t j = 0; j < O; ++j) {
        MNT_CHECK(order_host[j] >= 0 && order_host[j] < O, "order_host[%lld] = %lld is out of range",
                  (long long)j, (long long)order_host[j]);
      }
    }
    if (T == 0) return;
    MNT_CHECK(out != nullptr, "out is null");
    std::vector<int64_t> sizes;
    if (sizes_host != nullptr) {
      sizes.assign(sizes_host, sizes_host + O);
    } else {
      read_sizes(kernel_map_sizes, index_dtype, O, sizes, stream);
    }
    for (int64_t j = 0; j < O; ++j) {
      MNT_CHECK(sizes[j] >= 0 && sizes[j] <= T,
                "kernel map size %lld of offset %lld is out of range", (long long)sizes[j], (long long)j);
    }
    ForwardPlan plan = make_forward_plan(sizes.data(), O, S, T, allow_shortcut_matmul != 0,
                                         has_threshold != 0, threshold);
    const Epilogue epilogue = {channel_scale, channel_shift, residual, activation, negative_slope};
#define MNT_CALL(FT, IT)                                                                          \
  forward_typed<FT, IT>(gather_tile, scatter_tile, plan, static_cast<const FT *>(sources),          \
                        static_cast<const FT *>(weights), static_cast<const IT *>(source_masks),    \
                        static_cast<const IT *>(target_masks), static_cast<const IT *>(kernel_map_order), \
                        gather_index, epilogue, static_cast<const FT *>(packed_weights),             \
                        kernel_map_order != nullptr ? order_host : nullptr, S, T, O, K, N,          \
                        static_cast<FT *>(out), stream)
    MNT_DISPATCH_FI(float_dtype, index_dtype, MNT_CALL);
#undef MNT_CALL
  });
}

extern "C" int mnt_sparse_convolution_forward(
    int64_t gather_tile, int64_t scatter_tile, int allow_shortcut_matmul, int64_t parallel,
    int has_threshold, double threshold, const void *sources, const void *weights,
    const void *source_masks, const void *target_masks, const void *kernel_map_order,
    const void *kernel_map_sizes, const int64_t *sizes_host, int64_t S, int64_t T, int64_t O,
    int64_t K, int64_t N, int index_dtype, int float_dtype, const int32_t *gather_index, void *out,
    void *stream_) {
  return mnt_sparse_convolution_forward_fused(
      gather_tile, scatter_tile, allow_shortcut_matmul, parallel, has_threshold, threshold, sources,
      weights, source_masks, target_masks, kernel_map_order, kernel_map_sizes, sizes_host, S, T, O, K,
      N, index_dtype, float_dtype, gather_index, nullptr, nullptr, nullptr, MNT_ACT_NONE, 0.0f, nullptr,
      nullptr, out, stream_);
}

extern "C" int mnt_sparse_convolution_forward_rows(
    int64_t scatter_tile, const void *sources, const void *weights, const int64_t *sizes_host,
    const int64_t *order_host, const int32_t *in_idx, const int32_t *out_pos, const int32_t *row_ptr,
    int64_t S, int64_t T, int64_t O, int64_t K, int64_t N, int float_dtype, const float *channel_scale,
    const float *channel_shift, const void *residual, int activation, float negative_slope,
    const void *packed_weights, void *out, void *stream_) {
  return guarded([&] {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    float_size(float_dtype);
    MNT_CHECK(S >= 0 && T >= 0 && O >= 0 && K >= 1 && N >= 1 && S <= INT32_MAX && T <= INT32_MAX &&
                  O <= 65535 && K <= 65536 && N <= 65536,
              "bad shape S=%lld T=%lld O=%lld Cin=%lld Cout=%lld", (long long)S, (long long)T,
              (long long)O, (long long)K, (long long)N);
    MNT_CHECK(activation >= MNT_ACT_NONE && activation <= MNT_ACT_RELU6, "unknown activation code %d",
              activation);
    MNT_CHECK(reinterpret_cast<uintptr_t>(residual) % 16 == 0 &&
                  reinterpret_cast<uintptr_t>(channel_scale) % 4 == 0 &&
                  reinterpret_cast<uintptr_t>(channel_shift) % 4 == 0,
              "epilogue operands are not aligned (residual: 16 bytes, scale / shift: 4 bytes)");
    MNT_CHECK(reinterpret_cast<uintptr_t>(packed_weights) % 16 == 0, "packed weights are not 16-byte aligned");
    MNT_CHECK(sizes_host != nullptr, "sizes_host is null");
    if (T == 0) return;
    MNT_CHECK(out != nullptr && row_ptr != nullptr, "null argument");
    int64_t nnz = 0;
    for (int64_t j = 0; j < O; ++j) {
      MNT_CHECK(sizes_host[j] >= 0 && sizes_host[j] <= T, "kernel map size %lld of offset %lld is out of range",
                (long long)sizes_host[j], (long long)j);
      MNT_CHECK(order_host == nullptr || (order_host[j] >= 0 && order_host[j] < O),
                "order_host[%lld] is out of range", (long long)j);
      nnz += sizes_host[j];
    }
    MNT_CHECK(nnz == 0 || (in_idx != nullptr && out_pos != nullptr), "the pair lists are missing");
    MNT_CHECK(nnz == 0 || (sources != nullptr && weights != nullptr), "null operand");
    // no padding and no shortcut: buffer rows are list positions
    ForwardPlan plan = make_forward_plan(sizes_host, O, S, T, false, true, -1.0);
    MNT_CHECK(plan.total_rows == nnz, "the forward plan does not match the pair lists");
    const Epilogue epilogue = {channel_scale, channel_shift, residual, activation, negative_slope};
#define MNT_ROWS(FT)                                                                                  \
  forward_rows_typed<FT>(scatter_tile, plan, static_cast<const FT *>(sources),                        \
                         static_cast<const FT *>(weights), in_idx, out_pos, row_ptr, epilogue,         \
                         static_cast<const FT *>(packed_weights), order_host, S, T, O, K, N,           \
                         static_cast<FT *>(out), stream)
    if (float_dtype == MNT_FLOAT32) {
      MNT_ROWS(float);
    } else if (float_dtype == MNT_FLOAT16) {
      MNT_ROWS(half_t);
    } else {
      MNT_ROWS(bf16_t);
    }
#undef MNT_ROWS
  });
}

// Forward pass over offset groups: the grouped GEMM with K-concatenated members,
// then the ordinary Scatter with the groups' rank table in place of the
// offsets' (9 rows instead of 27).
template <typename T>
static void forward_groups_typed(const T *sources, const T *packed, const int *rank, const int4 *src,
                                 const int *head, const int32_t *offsets_host, int64_t S, int64_t Tn, int64_t K,
                                 int64_t N, const Epilogue &epilogue, T *out, hipStream_t stream) {
  Scope scope(stream);
  const int kc = kChunkBytes / static_cast<int>(sizeof(T));
  const int Kp = static_cast<int>(div_ceil(K, kc) * kc);
  const int Np = static_cast<int>(div_ceil(N, 32) * 32);
  profile_mark("enter:forward", stream);
  typedef typename BufferOf<T>::type TB;
  // room for the worst case (every target in every group); a group's rows start at a multiple of T
  TB *cbuf = scope.alloc<TB>(static_cast<size_t>(kGroupCount) * Tn * N);
  int *d_row_start = scope.alloc<int>(kGroupCount + 1);
  const float *range = measure_range<T>(scope, sources, S * K, packed, int64_t{27} * Np, Kp, stream);
  Epilogue finish = epilogue;
  finish.range = range;
  GroupView view;
  view.head = head;
  view.src = src;
  view.stride = Tn;
  view.tiles_per_group = static_cast<int>(div_ceil(Tn, kGemmRows));
  for (int i = 0; i < 3 * kGroupCount * kGroupMembers; ++i) view.offset_of[i] = offsets_host[i];
  const int blocks = Np / 32;
  const int slices = static_cast<int>(div_ceil(blocks, kMaxChannelBlocks));
  const int nb = static_cast<int>(div_ceil(blocks, slices));
  const int num_tiles = kGroupCount * view.tiles_per_group;
  const int resident = compute_units() * (nb >= 3 ? 3 : nb == 2 ? 4 : 6);
  dim3 grid(static_cast<unsigned>(std::min(num_tiles, std::max(1, resident / slices))), static_cast<unsigned>(slices));
  const bool pairs = (Kp / kc) % 2 == 0;            // stages of two chunks where a member's row divides so
#define MNT_GG(NB)                                                                                              \
  if (pairs) {                                                                                                  \
    group_gemm_kernel<T, TB, NB, 2><<<grid, kGemmBlock, 0, stream>>>(sources, cbuf, packed, static_cast<int>(K), \
                                                                     static_cast<int>(N), Kp, Np, view,         \
                                                                     d_row_start, range);                       \
  } else {                                                                                                      \
    group_gemm_kernel<T, TB, NB, 1><<<grid, kGemmBlock, 0, stream>>>(sources, cbuf, packed, static_cast<int>(K), \
                                                                     static_cast<int>(N), Kp, Np, view,         \
                                                                     d_row_start, range);                       \
  }
  switch (nb) {
    case 1: MNT_GG(1); break;
    case 2: MNT_GG(2); break;
    case 3: MNT_GG(3); break;
    default: MNT_GG(4); break;
  }
#undef MNT_GG
  check_launch("group_gemm_kernel");
  profile_mark("gemm", stream);
  const LaneShape ssh = lane_shape(0, N, sizeof(T), cbuf, out, "num_target_features");
  launch_scatter<TB, T, int32_t>(ssh, cbuf, out, rank, d_row_start, Tn, kGroupCount, static_cast<int>(N), nullptr,
                                 finish, stream);
  profile_mark("scatter", stream);
}

static void check_group_offsets(const int32_t *offsets_host) {
  MNT_CHECK(offsets_host != nullptr, "group_offsets_host is null");
  for (int axis = 0; axis < 3; ++axis) {
    bool seen[27] = {};
    for (int i = 0; i < kGroupCount * kGroupMembers; ++i) {
      const int o = offsets_host[axis * kGroupCount * kGroupMembers + i];
      MNT_CHECK(o >= 0 && o < 27 && !seen[o], "group_offsets_host[%d] does not list each of the 27 offsets once",
                axis);
      seen[o] = true;
    }
  }
}

extern "C" int mnt_kernel_map_offset_groups(const int32_t *kernel_map, int64_t T,
                                            const int32_t *group_offsets_host, int32_t *rank_out,
                                            int32_t *src_out, int32_t *head_out, void *stream_) {
  return guarded([&] {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    MNT_CHECK(T >= 0 && T * kGroupCount <= INT32_MAX, "bad number of targets %lld", (long long)T);
    check_group_offsets(group_offsets_host);
    MNT_CHECK(head_out != nullptr, "head_out is null");
    MNT_CHECK(reinterpret_cast<uintptr_t>(src_out) % 16 == 0, "src_out is not 16-byte aligned");
    Scope scope(stream);
    GroupOffsets tab;
    for (int i = 0; i < 3 * kGroupCount * kGroupMembers; ++i) tab.o[i] = group_offsets_host[i];
    const int tiles = static_cast<int>(std::max<int64_t>(1, div_ceil(T, kGroupTile)));
    int *tile_counts = scope.alloc<int>(static_cast<size_t>(3) * kGroupCount * tiles);
    if (T > 0) MNT_CHECK(kernel_map != nullptr && rank_out != nullptr && src_out != nullptr, "null argument");
    group_count_kernel<<<dim3(tiles, 3 * kGroupCount), kGroupTile, 0, stream>>>(kernel_map, T, tab, tiles,
                                                                                 tile_counts);
    check_launch("group_count_kernel");
    group_scan_kernel<<<1, 1024, 0, stream>>>(tile_counts, tiles, head_out);
    check_launch("group_scan_kernel");
    group_emit_kernel<<<dim3(tiles, kGroupCount), kGroupTile, 0, stream>>>(
        kernel_map, T, tab, tiles, tile_counts, head_out, rank_out, reinterpret_cast<int4 *>(src_out));
    check_launch("group_emit_kernel");
    profile_mark("offset_groups", stream);
  });
}

extern "C" int mnt_sparse_convolution_forward_groups(
    const void *sources, const void *packed_weights, const int32_t *rank, const int32_t *src,
    const int32_t *head, const int32_t *group_offsets_host, int64_t S, int64_t T, int64_t K, int64_t N,
    int float_dtype, const float *channel_scale, const float *channel_shift, const void *residual,
    int activation, float negative_slope, void *out, void *stream_) {
  return guarded([&] {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const int esize = float_size(float_dtype);
    MNT_CHECK(float_dtype != MNT_FLOAT32, "the offset-group forward takes 16-bit features");
    MNT_CHECK(S >= 0 && T >= 0 && K >= 1 && N >= 1 && S <= INT32_MAX && T * kGroupCount <= INT32_MAX &&
                  K <= 65536 && N <= 65536,
              "bad shape S=%lld T=%lld Cin=%lld Cout=%lld", (long long)S, (long long)T, (long long)K, (long long)N);
    MNT_CHECK((K * esize) % kChunkBytes == 0, "source rows of %lld bytes are not whole 128-byte chunks",
              (long long)(K * esize));
    MNT_CHECK(N % 8 == 0, "num_target_features = %lld is not a multiple of 8", (long long)N);
    MNT_CHECK(activation >= MNT_ACT_NONE && activation <= MNT_ACT_RELU6, "unknown activation code %d",
              activation);
    MNT_CHECK(reinterpret_cast<uintptr_t>(residual) % 16 == 0 &&
                  reinterpret_cast<uintptr_t>(channel_scale) % 4 == 0 &&
                  reinterpret_cast<uintptr_t>(channel_shift) % 4 == 0,
              "epilogue operands are not aligned (residual: 16 bytes, scale / shift: 4 bytes)");
    MNT_CHECK(reinterpret_cast<uintptr_t>(packed_weights) % 16 == 0 && reinterpret_cast<uintptr_t>(sources) % 16 == 0 &&
                  reinterpret_cast<uintptr_t>(src) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0,
              "operands are not 16-byte aligned");
    check_group_offsets(group_offsets_host);
    if (T == 0) return;
    MNT_CHECK(sources != nullptr && packed_weights != nullptr && rank != nullptr && src != nullptr &&
                  head != nullptr && out != nullptr,
              "null argument");
    const Epilogue epilogue = {channel_scale, channel_shift, residual, activation, negative_slope};
#define MNT_GROUPS(FT)                                                                                  \
  forward_groups_typed<FT>(static_cast<const FT *>(sources), static_cast<const FT *>(packed_weights), rank, \
                           reinterpret_cast<const int4 *>(src), head, group_offsets_host, S, T, K, N, epilogue, \
                           static_cast<FT *>(out), stream)
    if (float_dtype == MNT_FLOAT16) {
      MNT_GROUPS(half_t);
    } else {
      MNT_GROUPS(bf16_t);
    }
#undef MNT_GROUPS
  });
}

extern "C" int mnt_pack_weights(const void *weights, int64_t O, int64_t K, int64_t N, int float_dtype,
                                void *packed_out, void *stream_) {
  return guarded([&] {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const int esize = float_size(float_dtype);
    MNT_CHECK(O >= 0 && O <= 65535 && K >= 1 && N >= 1 && K <= 65536 && N <= 65536,
              "bad shape O=%lld Cin=%lld Cout=%lld", (long long)O, (long long)K, (long long)N);
    if (O == 0) return;
    MNT_CHECK(weights != nullptr && packed_out != nullptr, "null operand");
    const int kc = kChunkBytes / esize;
    const int Kp = static_cast<int>(div_ceil(K, kc) * kc);
    const int Np = static_cast<int>(div_ceil(N, 32) * 32);
    const long long total = static_cast<long long>(O) * Np * Kp;
#define MNT_PACK(FT)                                                                               \
  pack_weights_kernel<FT, int32_t><<<grid_for(total, 256, 4096), 256, 0, stream>>>(                \
      static_cast<const FT *>(weights), nullptr, static_cast<int>(O), static_cast<int>(K),         \
      static_cast<int>(N), Kp, Np, static_cast<FT *>(packed_out), PlanChunk{}, 0, nullptr)
    if (float_dtype == MNT_FLOAT32) {
      MNT_PACK(float);
    } else if (float_dtype == MNT_FLOAT16) {
      MNT_PACK(half_t);
    } else {
      MNT_PACK(bf16_t);
    }
#undef MNT_PACK
    check_launch("pack_weights_kernel");
  });
}

// ---------------------------------------------------------- stage timers ----

namespace mnt {

static int g_timer_repeats = 1;            // launches between the two events of a stage timer

struct TimerScope {
  hipEvent_t start, stop;
  hipStream_t stream;
  explicit TimerScope(hipStream_t s) : stream(s) {
    MNT_HIP(hipEventCreate(&start));
    MNT_HIP(hipEventCreate(&stop));
  }
  ~TimerScope() {
    (void)hipEventDestroy(start);
    (void)hipEventDestroy(stop);
  }
  void begin() { MNT_HIP(hipEventRecord(start, stream)); }
  float end() {
    MNT_HIP(hipEventRecord(stop, stream));
    MNT_HIP(hipEventSynchronize(stop));
    float ms = 0.0f;
    MNT_HIP(hipEventElapsedTime(&ms, start, stop));
    return ms / static_cast<float>(g_timer_repeats);
  }
};

template <typename T, typename IT>
static float time_gather_typed(int64_t tile, const ForwardPlan &plan, const IT *source_masks,
                               int64_t S, int64_t K, hipStream_t stream) {
  Scope scope(stream);
  const size_t rows = static_cast<size_t>(plan.total_rows > 0 ? plan.total_rows : 1);
  T *sources = scope.alloc<T>(static_cast<size_t>(S > 0 ? S : 1) * K);
  T *abuf = scope.alloc<T>(rows * K);
  int *d_row_start = scope.alloc<int>(plan.row_start.size());
  upload_ints(plan.row_start, d_row_start, stream);
  const LaneShape sh = lane_shape(tile, K, sizeof(T), sources, abuf, "num_source_features");
  TimerScope timer(stream);
  timer.begin();
  for (int r = 0; r < g_timer_repeats; ++r) {
    launch_gather<IT>(sh, sources, abuf, source_masks, d_row_start, S, static_cast<int>(plan.active_offsets),
                      static_cast<int>(K * sizeof(T)), stream);
  }
  return timer.end();
}

template <typename T, typename IT>
static float time_scatter_typed(int64_t tile, const ForwardPlan &plan, const IT *target_masks,
                                int64_t Tn, int64_t N, hipStream_t stream) {
  Scope scope(stream);
  const size_t rows = static_cast<size_t>(plan.total_rows > 0 ? plan.total_rows : 1);
  typedef typename BufferOf<T>::type TB;
  TB *cbuf = scope.alloc<TB>((rows + (plan.shortcut ? static_cast<size_t>(Tn) : 0)) * N);
  T *out = scope.alloc<T>(static_cast<size_t>(Tn > 0 ? Tn : 1) * N);
  int *d_row_start = scope.alloc<int>(plan.row_start.size());
  upload_ints(plan.row_start, d_row_start, stream);
  const LaneShape sh = lane_shape(tile, N, sizeof(T), cbuf, out, "num_target_features");
  TimerScope timer(stream);
  timer.begin();
  for (int r = 0; r < g_timer_repeats; ++r) {
    launch_scatter<TB, T, IT>(sh, cbuf, out, target_masks, d_row_start, Tn,
                              static_cast<int>(plan.active_offsets), static_cast<int>(N),
                              plan.shortcut ? cbuf + rows * N : nullptr, Epilogue{}, stream);
  }
  return timer.end();
}

template <typename T>
static float time_gemm_typed(const ForwardPlan &plan, const T *weights, int64_t S, int64_t O, int64_t K,
                             int64_t N, hipStream_t stream) {
  Scope scope(stream);
  const int kc = kChunkBytes / static_cast<int>(sizeof(T));
  const int Kp = static_cast<int>(div_ceil(K, kc) * kc);
  const int Np = static_cast<int>(div_ceil(N, 32) * 32);
  const size_t rows = static_cast<size_t>(plan.total_rows > 0 ? plan.total_rows : 1);
  typedef typename BufferOf<T>::type TB;
  T *wt = scope.alloc<T>(static_cast<size_t>(O) * Np * Kp);
  T *abuf = scope.alloc<T>(rows * K);
  TB *cbuf = scope.alloc<TB>(rows * N);
  T *direct_a = nullptr;
  TB *direct_c = nullptr;
  int *d_direct = nullptr;
  std::vector<int> dmeta;
  if (plan.shortcut) {
    direct_a = scope.alloc<T>(static_cast<size_t>(S) * K);
    direct_c = scope.alloc<TB>(static_cast<size_t>(S) * N);
    dmeta = direct_meta(S, static_cast<int>(O - 1));
    d_direct = scope.alloc<int>(dmeta.size());
    upload_ints(dmeta, d_direct, stream);
  }
  const long long total = static_cast<long long>(O) * Np * Kp;
  pack_weights_kernel<T, int32_t><<<grid_for(total, 256, 4096), 256, 0, stream>>>(
      weights, nullptr, static_cast<int>(O), static_cast<int>(K), static_cast<int>(N), Kp, Np, wt,
      PlanChunk{}, 0, nullptr);
  check_launch("pack_weights_kernel");
  // operands of a timing run are scratch: clear them so no NaN patterns slow or trap anything
  MNT_HIP(hipMemsetAsync(abuf, 0, rows * K * sizeof(T), stream));
  if (plan.shortcut) MNT_HIP(hipMemsetAsync(direct_a, 0, static_cast<size_t>(S) * K * sizeof(T), stream));
  int *d_meta = scope.alloc<int>(plan.meta.size());
  upload_ints(plan.meta, d_meta, stream);
  TimerScope timer(stream);
  timer.begin();
  for (int r = 0; r < g_timer_repeats; ++r) {
    launch_gemm<T, TB>(abuf, cbuf, wt, d_meta, plan.num_tiles, static_cast<int>(K), static_cast<int>(N), Kp, Np,
                       nullptr, stream);
    if (plan.shortcut) {
      launch_gemm<T, TB>(direct_a, direct_c, wt, d_direct, dmeta[2], static_cast<int>(K), static_cast<int>(N), Kp,
                         Np, nullptr, stream);
    }
  }
  return timer.end();
}

static ForwardPlan timer_plan(const void *sizes_dev, int index_dtype, int64_t S, int64_t T, int64_t O,
                              int allow_shortcut, int has_threshold, double threshold,
                              hipStream_t stream) {
  std::vector<int64_t> sizes;
  read_sizes(sizes_dev, index_dtype, O, sizes, stream);
  return make_forward_plan(sizes.data(), O, S, T, allow_shortcut != 0, has_threshold != 0, threshold);
}

}  // namespace mnt

extern "C" int mnt_timer_repeats(int repeats) {
  return guarded([&] {
    MNT_CHECK(repeats >= 1 && repeats <= 1000, "repeats must be in [1, 1000], found %d", repeats);
    g_timer_repeats = repeats;
  });
}

extern "C" int mnt_time_gather(int64_t tile, int allow_shortcut_matmul, int has_threshold,
                               double threshold, const void *source_masks,
                               const void *kernel_map_sizes, int64_t S, int64_t T, int64_t O,
                               int64_t K, int64_t N, int index_dtype, int float_dtype,
                               float *ms_out, void *stream_) {
  (void)N;
  return guarded([&] {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    float_size(float_dtype);
    ForwardPlan plan = timer_plan(kernel_map_sizes, index_dtype, S, T, O, allow_shortcut_matmul,
                                  has_threshold, threshold, stream);
#define MNT_CALL(FT, IT) \
  *ms_out = time_gather_typed<FT, IT>(tile, plan, static_cast<const IT *>(source_masks), S, K, stream)
    MNT_DISPATCH_FI(float_dtype, index_dtype, MNT_CALL);
#undef MNT_CALL
  });
}

extern "C" int mnt_time_scatter(int64_t tile, int allow_shortcut_matmul, int has_threshold,
                                double threshold, const void *target_masks,
                                const void *kernel_map_sizes, int64_t S, int64_t T, int64_t O,
                                int64_t K, int64_t N, int index_dtype, int float_dtype,
                                float *ms_out, void *stream_) {
  (void)K;
  return guarded([&] {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    float_size(float_dtype);
    ForwardPlan plan = timer_plan(kernel_map_sizes, index_dtype, S, T, O, allow_shortcut_matmul,
                                  has_threshold, threshold, stream);
#define MNT_CALL(FT, IT) \
  *ms_out = time_scatter_typed<FT, IT>(tile, plan, static_cast<const IT *>(target_masks), T, N, stream)
    MNT_DISPATCH_FI(float_dtype, index_dtype, MNT_CALL);
#undef MNT_CALL
  });
}

extern "C" int mnt_time_gemm(int allow_shortcut_matmul, int64_t parallel, int has_threshold,
                             double threshold, const void *weights, const void *kernel_map_sizes,
                             int64_t S, int64_t T, int64_t O, int64_t K, int64_t N,
                             int index_dtype, int float_dtype, float *ms_out, void *stream_) {
  (void)parallel;
  return guarded([&] {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    float_size(float_dtype);
    ForwardPlan plan = timer_plan(kernel_map_sizes, index_dtype, S, T, O, allow_shortcut_matmul,
                                  has_threshold, threshold, stream);
    if (float_dtype == MNT_FLOAT32) {
      *ms_out = time_gemm_typed<float>(plan, static_cast<const float *>(weights), S, O, K, N, stream);
    } else if (float_dtype == MNT_FLOAT16) {
      *ms_out = time_gemm_typed<half_t>(plan, static_cast<const half_t *>(weights), S, O, K, N, stream);
    } else {
      *ms_out = time_gemm_typed<bf16_t>(plan, static_cast<const bf16_t *>(weights), S, O, K, N, stream);
    }
  });
}
