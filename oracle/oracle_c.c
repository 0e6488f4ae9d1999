/*
 * oracle_c.c — plain-C CPU restatement of the sparse-convolution hot path.
 *
 * THIS IS TEST INFRASTRUCTURE: it is the checker of the parity tests and the
 * timed "cpu_baseline" of the benchmark.  The product never links or loads it.
 *
 * Each function restates one stage of the reference (paths relative to the
 * reference checkout) on the host, in the order the reference runs them:
 *   orc_arg_sort      csrc/minuet/cuda/functions/arg_sort_coodrinates.cu:273-360
 *                     (min/max -> mixed-radix flatten, kernels/flatten_coordinates.cuh:18-38
 *                      -> one stable LSD radix sort of (key, index) pairs)
 *   orc_query         csrc/minuet/cuda/kernels/query_sorted_index_with_offsets.cuh:36-77
 *                     (binary search of targets[t]+offsets[o] in the sorted sources)
 *   orc_sizes         csrc/minuet/cuda/functions/scan.cu:220-290
 *   orc_masks         csrc/minuet/cuda/functions/scan.cu:292-365,
 *                     kernels/generate_masks_from_kernel_map.cuh:20-29
 *   orc_pair_lists    inverse of the masks (per-offset (in, out) index lists)
 *   orc_conv_forward  csrc/minuet/cuda/functions/sparse_convolution.cu:504-661
 *                     (gather, per-offset GEMM, target-stationary scatter; fp32)
 *
 * Pinned by tests/test_oracle.py against the NumPy oracle (itself pinned by
 * brute force and library routines) on seeded inputs.  Single point cloud,
 * int32 coordinates, ndim <= 4.
 */
#include <limits.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_MAX_NDIM 4

int orc_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

typedef struct {
  int64_t lo[ORC_MAX_NDIM];
  int64_t pow[ORC_MAX_NDIM];
} orc_frame;

/* cpow[D-1] = 1, cpow[r] = cpow[r+1] * extent[r+1]: dimension 0 most significant.
 * `reach` widens every extent so that a key shifted by a kernel offset stays
 * inside its own field (the reference compares tuples and needs no such room). */
static int make_frame(const int32_t *a, int64_t na, const int32_t *b, int64_t nb, int ndim,
                      int64_t reach, orc_frame *f) {
  int64_t lo[ORC_MAX_NDIM], hi[ORC_MAX_NDIM];
  for (int k = 0; k < ndim; ++k) { lo[k] = INT64_MAX; hi[k] = INT64_MIN; }
  for (int64_t i = 0; i < na; ++i)
    for (int k = 0; k < ndim; ++k) {
      int64_t v = a[i * ndim + k];
      if (v < lo[k]) lo[k] = v;
      if (v > hi[k]) hi[k] = v;
    }
  for (int64_t i = 0; i < nb; ++i)
    for (int k = 0; k < ndim; ++k) {
      int64_t v = b[i * ndim + k];
      if (v < lo[k]) lo[k] = v;
      if (v > hi[k]) hi[k] = v;
    }
  __int128 p = 1;
  for (int k = ndim - 1; k >= 0; --k) {
    f->lo[k] = lo[k] - reach;
    f->pow[k] = (int64_t)p;
    p *= (__int128)(hi[k] - lo[k] + 1 + 2 * reach);
    if (p > ((__int128)1 << 62)) return 1;    /* not flattenable into 64 bits */
  }
  return 0;
}

static inline int64_t flatten(const int32_t *row, int ndim, const orc_frame *f) {
  int64_t key = 0;
  for (int k = 0; k < ndim; ++k) key += ((int64_t)row[k] - f->lo[k]) * f->pow[k];
  return key;
}

/* Stable arg-sort, lexicographic with dimension 0 most significant.
 * indices_out[n]; sorted_out[n*ndim] (nullable).  Returns non-zero when the
 * coordinate range does not fit a 64-bit key. */
int orc_arg_sort(const int32_t *coords, int64_t n, int ndim, int64_t *indices_out,
                 int32_t *sorted_out) {
  if (n == 0) return 0;
  orc_frame f;
  if (make_frame(coords, n, NULL, 0, ndim, 0, &f)) return 1;
  uint64_t *keys = (uint64_t *)malloc(sizeof(uint64_t) * n * 2);
  int64_t *vals = (int64_t *)malloc(sizeof(int64_t) * n * 2);
  uint64_t *k0 = keys, *k1 = keys + n;
  int64_t *v0 = vals, *v1 = vals + n;
  uint64_t all = 0;
  for (int64_t i = 0; i < n; ++i) {
    k0[i] = (uint64_t)flatten(coords + i * ndim, ndim, &f);
    v0[i] = i;
    all |= k0[i];
  }
  for (int shift = 0; shift < 64 && (all >> shift) != 0; shift += 8) {
    int64_t count[257];
    memset(count, 0, sizeof(count));
    for (int64_t i = 0; i < n; ++i) count[((k0[i] >> shift) & 255) + 1]++;
    for (int d = 0; d < 256; ++d) count[d + 1] += count[d];
    for (int64_t i = 0; i < n; ++i) {
      int64_t pos = count[(k0[i] >> shift) & 255]++;
      k1[pos] = k0[i];
      v1[pos] = v0[i];
    }
    uint64_t *tk = k0; k0 = k1; k1 = tk;
    int64_t *tv = v0; v0 = v1; v1 = tv;
  }
  for (int64_t i = 0; i < n; ++i) {
    indices_out[i] = v0[i];
    if (sorted_out) memcpy(sorted_out + i * ndim, coords + v0[i] * ndim, sizeof(int32_t) * ndim);
  }
  free(keys);
  free(vals);
  return 0;
}

/* kernel_map[o*T + t] = index of the source equal to targets[t] + offsets[o], or -1. */
int orc_query(const int32_t *sources, int64_t S, const int32_t *targets, int64_t T,
              const int32_t *offsets, int64_t O, int ndim, int32_t *kernel_map) {
  if (T == 0 || O == 0) return 0;
  if (S == 0) {
    for (int64_t i = 0; i < O * T; ++i) kernel_map[i] = -1;
    return 0;
  }
  int64_t reach = 0;
  for (int64_t i = 0; i < O * ndim; ++i) {
    int64_t v = offsets[i] < 0 ? -(int64_t)offsets[i] : offsets[i];
    if (v > reach) reach = v;
  }
  orc_frame f;
  if (make_frame(sources, S, targets, T, ndim, reach, &f)) return 1;
  int64_t *skeys = (int64_t *)malloc(sizeof(int64_t) * S);
  int64_t *tkeys = (int64_t *)malloc(sizeof(int64_t) * T);
  for (int64_t i = 0; i < S; ++i) skeys[i] = flatten(sources + i * ndim, ndim, &f);
  for (int64_t i = 0; i < T; ++i) tkeys[i] = flatten(targets + i * ndim, ndim, &f);
#pragma omp parallel for schedule(static)
  for (int64_t o = 0; o < O; ++o) {
    int64_t delta = 0;
    for (int k = 0; k < ndim; ++k) delta += (int64_t)offsets[o * ndim + k] * f.pow[k];
    for (int64_t t = 0; t < T; ++t) {
      const int64_t q = tkeys[t] + delta;
      int64_t lo = 0, hi = S;
      while (lo < hi) {
        int64_t mid = (lo + hi) >> 1;
        if (skeys[mid] < q) lo = mid + 1; else hi = mid;
      }
      kernel_map[o * T + t] = (lo < S && skeys[lo] == q) ? (int32_t)lo : -1;
    }
  }
  free(skeys);
  free(tkeys);
  return 0;
}

void orc_sizes(const int32_t *kernel_map, int64_t O, int64_t T, int64_t *sizes) {
  for (int64_t o = 0; o < O; ++o) {
    int64_t c = 0;
    for (int64_t t = 0; t < T; ++t) c += kernel_map[o * T + t] != -1;
    sizes[o] = c;
  }
}

/* Rank tables; rows are taken in the given order (order[j] = offset of row j,
 * NULL = identity). */
void orc_masks(const int32_t *kernel_map, int64_t O, int64_t S, int64_t T, const int64_t *order,
               int32_t *source_masks, int32_t *target_masks) {
  for (int64_t i = 0; i < O * S; ++i) source_masks[i] = -1;
#pragma omp parallel for schedule(static)
  for (int64_t j = 0; j < O; ++j) {
    const int64_t o = order ? order[j] : j;
    int32_t rank = 0;
    for (int64_t t = 0; t < T; ++t) {
      const int32_t s = kernel_map[o * T + t];
      if (s == -1) {
        target_masks[j * T + t] = -1;
      } else {
        target_masks[j * T + t] = rank;
        source_masks[j * S + s] = rank;
        ++rank;
      }
    }
  }
}

/* Hits of every row in target order, rows concatenated; returns nnz. */
int64_t orc_pair_lists(const int32_t *kernel_map, int64_t O, int64_t T, int32_t *in_idx,
                       int32_t *out_idx) {
  int64_t n = 0;
  for (int64_t o = 0; o < O; ++o)
    for (int64_t t = 0; t < T; ++t) {
      const int32_t s = kernel_map[o * T + t];
      if (s != -1) {
        in_idx[n] = s;
        out_idx[n] = (int32_t)t;
        ++n;
      }
    }
  return n;
}

/* out[T, N] = sum_j scatter(gather(F) x W[order[j]]) in fp32, rows j in order. */
void orc_conv_forward(const float *features, const float *weights, const int32_t *source_masks,
                      const int32_t *target_masks, const int64_t *order, const int64_t *sizes,
                      int64_t S, int64_t T, int64_t O, int64_t K, int64_t N, float *out) {
  memset(out, 0, sizeof(float) * T * N);
  int64_t max_size = 0;
  for (int64_t j = 0; j < O; ++j) if (sizes[j] > max_size) max_size = sizes[j];
  float *abuf = (float *)malloc(sizeof(float) * (max_size > 0 ? max_size : 1) * K);
  float *cbuf = (float *)malloc(sizeof(float) * (max_size > 0 ? max_size : 1) * N);
  for (int64_t j = 0; j < O; ++j) {
    if (sizes[j] == 0) continue;
    const float *w = weights + (order ? order[j] : j) * K * N;
    for (int64_t s = 0; s < S; ++s) {
      const int32_t d = source_masks[j * S + s];
      if (d != -1) memcpy(abuf + (int64_t)d * K, features + s * K, sizeof(float) * K);
    }
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < sizes[j]; ++r) {
      float *c = cbuf + r * N;
      for (int64_t n = 0; n < N; ++n) c[n] = 0.0f;
      for (int64_t k = 0; k < K; ++k) {
        const float a = abuf[r * K + k];
        const float *wr = w + k * N;
        for (int64_t n = 0; n < N; ++n) c[n] += a * wr[n];
      }
    }
#pragma omp parallel for schedule(static)
    for (int64_t t = 0; t < T; ++t) {
      const int32_t d = target_masks[j * T + t];
      if (d != -1) {
        const float *c = cbuf + (int64_t)d * N;
        for (int64_t n = 0; n < N; ++n) out[t * N + n] += c[n];
      }
    }
  }
  free(abuf);
  free(cbuf);
}
