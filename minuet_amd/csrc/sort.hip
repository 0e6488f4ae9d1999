// Map step, part 1: coordinate bounds, key packing and a stable LSD radix sort
// of (packed voxel key, row index) pairs for gfx950 (64-wide wavefronts).
//
// Follows the semantics of ArgSortCoordinates / MultiArgSortCoordinates
// (csrc/minuet/cuda/functions/arg_sort_coodrinates.cu:273-469): stable,
// lexicographic with dimension 0 most significant, batch-major.
#include "sort.h"

#include "device_utils.h"

namespace mnt {

// ----------------------------------------------------------------- bounds ----

__global__ void bounds_init_kernel(long long *bounds) {
  int t = threadIdx.x;
  if (t < MNT_MAX_NDIM) bounds[t] = INT64_MAX;
  if (t >= MNT_MAX_NDIM && t < 2 * MNT_MAX_NDIM) bounds[t] = INT64_MIN;
}

template <typename CT>
__global__ __launch_bounds__(256) void bounds_kernel(const CT *__restrict__ coords, long long n,
                                                     int ndim, long long *bounds) {
  long long lo[MNT_MAX_NDIM], hi[MNT_MAX_NDIM];
#pragma unroll
  for (int k = 0; k < MNT_MAX_NDIM; ++k) {
    lo[k] = INT64_MAX;
    hi[k] = INT64_MIN;
  }
  const long long stride = static_cast<long long>(gridDim.x) * blockDim.x;
  for (long long i = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x; i < n;
       i += stride) {
#pragma unroll
    for (int k = 0; k < MNT_MAX_NDIM; ++k) {
      if (k < ndim) {
        long long v = static_cast<long long>(coords[i * ndim + k]);
        lo[k] = v < lo[k] ? v : lo[k];
        hi[k] = v > hi[k] ? v : hi[k];
      }
    }
  }
  __shared__ long long s_lo[4][MNT_MAX_NDIM], s_hi[4][MNT_MAX_NDIM];
#pragma unroll
  for (int k = 0; k < MNT_MAX_NDIM; ++k) {
    for (int off = 32; off > 0; off >>= 1) {
      long long a = __shfl_down(lo[k], off);
      long long b = __shfl_down(hi[k], off);
      lo[k] = a < lo[k] ? a : lo[k];
      hi[k] = b > hi[k] ? b : hi[k];
    }
  }
  const int w = threadIdx.x >> 6;
  if (lane_id() == 0) {
#pragma unroll
    for (int k = 0; k < MNT_MAX_NDIM; ++k) {
      s_lo[w][k] = lo[k];
      s_hi[w][k] = hi[k];
    }
  }
  __syncthreads();
  if (threadIdx.x < ndim) {
    int k = threadIdx.x;
    long long a = s_lo[0][k], b = s_hi[0][k];
    for (int ww = 1; ww < 4; ++ww) {
      a = s_lo[ww][k] < a ? s_lo[ww][k] : a;
      b = s_hi[ww][k] > b ? s_hi[ww][k] : b;
    }
    atomicMin(&bounds[k], a);
    atomicMax(&bounds[MNT_MAX_NDIM + k], b);
  }
}

void enqueue_bounds(const void *coords, int64_t n, int ndim, int coord_dtype, long long *d_bounds,
                    bool init, hipStream_t stream) {
  if (init) {
    bounds_init_kernel<<<1, 64, 0, stream>>>(d_bounds);
    check_launch("bounds_init_kernel");
  }
  if (n == 0) return;
  unsigned grid = grid_for(n, 256 * 4, 1024);
  if (coord_dtype == MNT_INT32) {
    bounds_kernel<int32_t><<<grid, 256, 0, stream>>>(static_cast<const int32_t *>(coords), n,
                                                      ndim, d_bounds);
  } else {
    bounds_kernel<int64_t><<<grid, 256, 0, stream>>>(static_cast<const int64_t *>(coords), n,
                                                      ndim, d_bounds);
  }
  check_launch("bounds_kernel");
}

// ------------------------------------------------------------------ pack ----

// One sort round packs a subset of the fields (dimensions, batch id) into a
// 64-bit key.  Field ndim.. is unused; index MNT_MAX_NDIM is the batch id.
struct SortSpec {
  unsigned long long lo[MNT_MAX_NDIM + 1];
  unsigned long long mask[MNT_MAX_NDIM + 1];
  int shift[MNT_MAX_NDIM + 1];
  int ndim;
  int num_batches;
};

template <typename CT, typename IT>
__global__ __launch_bounds__(256) void pack_keys_kernel(const CT *__restrict__ coords,
                                                        long long n, SortSpec spec,
                                                        const IT *__restrict__ batch_dims,
                                                        const unsigned *__restrict__ perm_in,
                                                        unsigned long long *__restrict__ keys,
                                                        unsigned *__restrict__ vals) {
  const long long stride = static_cast<long long>(gridDim.x) * blockDim.x;
  for (long long i = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x; i < n;
       i += stride) {
    const long long row = perm_in ? static_cast<long long>(perm_in[i]) : i;
    unsigned long long key = 0;
#pragma unroll
    for (int k = 0; k < MNT_MAX_NDIM; ++k) {
      if (k < spec.ndim && spec.mask[k]) {
        unsigned long long v =
            static_cast<unsigned long long>(static_cast<long long>(coords[row * spec.ndim + k])) -
            spec.lo[k];
        key |= (v & spec.mask[k]) << spec.shift[k];
      }
    }
    if (spec.mask[MNT_MAX_NDIM]) {
      unsigned long long b = batch_of<IT>(row, batch_dims, spec.num_batches);
      key |= (b & spec.mask[MNT_MAX_NDIM]) << spec.shift[MNT_MAX_NDIM];
    }
    keys[i] = key;
    vals[i] = static_cast<unsigned>(row);
  }
}

// ------------------------------------------------------------ radix sort ----

constexpr int kRadixBits = 8;
constexpr int kRadix = 1 << kRadixBits;
constexpr int kSortBlock = 256;

template <int ITEMS>
__global__ __launch_bounds__(kSortBlock) void radix_hist_kernel(
    const unsigned long long *__restrict__ keys, long long n, int shift,
    unsigned *__restrict__ counts, int num_tiles) {
  __shared__ unsigned hist[kRadix];
  hist[threadIdx.x] = 0;
  __syncthreads();
  const long long base = static_cast<long long>(blockIdx.x) * (kSortBlock * ITEMS);
#pragma unroll
  for (int r = 0; r < ITEMS; ++r) {
    long long i = base + r * kSortBlock + threadIdx.x;
    if (i < n) atomicAdd(&hist[(keys[i] >> shift) & (kRadix - 1)], 1u);
  }
  __syncthreads();
  counts[static_cast<long long>(threadIdx.x) * num_tiles + blockIdx.x] = hist[threadIdx.x];
}

// Exclusive scan of a flat array by one workgroup (digit-major tile counts).
__global__ __launch_bounds__(1024) void scan_counts_kernel(unsigned *__restrict__ data,
                                                           long long total) {
  __shared__ unsigned partial[1024];
  const int t = threadIdx.x;
  const long long chunk = (total + 1023) / 1024;
  const long long lo = t * chunk;
  const long long hi = lo + chunk < total ? lo + chunk : total;
  unsigned sum = 0;
  for (long long i = lo; i < hi; ++i) sum += data[i];
  partial[t] = sum;
  __syncthreads();
  for (int off = 1; off < 1024; off <<= 1) {
    unsigned v = t >= off ? partial[t - off] : 0;
    __syncthreads();
    partial[t] += v;
    __syncthreads();
  }
  unsigned run = partial[t] - sum;
  for (long long i = lo; i < hi; ++i) {
    unsigned v = data[i];
    data[i] = run;
    run += v;
  }
}

void enqueue_exclusive_scan(unsigned *data, int64_t total, hipStream_t stream) {
  if (total <= 0) return;
  scan_counts_kernel<<<1, 1024, 0, stream>>>(data, total);
  check_launch("scan_counts_kernel");
}

// Stable scatter of one tile.  Wave w owns the contiguous slice
// [w*64*ITEMS, (w+1)*64*ITEMS) of the tile and walks it 64 items at a time, so
// (wave, round, lane) order equals input order; ranks within a digit follow it.
template <int ITEMS>
__global__ __launch_bounds__(kSortBlock) void radix_scatter_kernel(
    const unsigned long long *__restrict__ keys_in, const unsigned *__restrict__ vals_in,
    unsigned long long *__restrict__ keys_out, unsigned *__restrict__ vals_out, long long n,
    int shift, const unsigned *__restrict__ offsets, int num_tiles) {
  constexpr int kWaves = kSortBlock / kWave;
  __shared__ volatile unsigned cnt[kWaves][kRadix];
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int w = tid >> 6;
  for (int i = tid; i < kWaves * kRadix; i += kSortBlock) (&cnt[0][0])[i] = 0;
  __syncthreads();

  const long long base =
      static_cast<long long>(blockIdx.x) * (kSortBlock * ITEMS) + w * (kWave * ITEMS);
  unsigned long long key[ITEMS];
  unsigned val[ITEMS];
  unsigned rank[ITEMS];
  const unsigned long long below_mask = (1ull << lane) - 1ull;
#pragma unroll
  for (int r = 0; r < ITEMS; ++r) {
    const long long i = base + r * kWave + lane;
    const bool valid = i < n;
    key[r] = valid ? keys_in[i] : ~0ull;
    val[r] = valid ? vals_in[i] : 0u;
    const unsigned d = static_cast<unsigned>(key[r] >> shift) & (kRadix - 1);
    unsigned long long peers = __ballot(valid);
#pragma unroll
    for (int b = 0; b < kRadixBits; ++b) {
      const bool bit = (d >> b) & 1u;
      const unsigned long long vote = __ballot(valid && bit);
      peers &= bit ? vote : ~vote;
    }
    const unsigned below = __popcll(peers & below_mask);
    const unsigned prev = cnt[w][d];
    rank[r] = prev + below;
    __builtin_amdgcn_wave_barrier();
    if (valid && below == 0) cnt[w][d] = prev + __popcll(peers);
    __builtin_amdgcn_wave_barrier();
  }
  __syncthreads();
  {
    unsigned run = offsets[static_cast<long long>(tid) * num_tiles + blockIdx.x];
#pragma unroll
    for (int ww = 0; ww < kWaves; ++ww) {
      unsigned c = cnt[ww][tid];
      cnt[ww][tid] = run;
      run += c;
    }
  }
  __syncthreads();
#pragma unroll
  for (int r = 0; r < ITEMS; ++r) {
    const long long i = base + r * kWave + lane;
    if (i < n) {
      const unsigned d = static_cast<unsigned>(key[r] >> shift) & (kRadix - 1);
      const unsigned pos = cnt[w][d] + rank[r];
      keys_out[pos] = key[r];
      vals_out[pos] = val[r];
    }
  }
}

template <int ITEMS>
static void radix_sort_impl(unsigned long long *&keys, unsigned *&vals, unsigned long long *&keys_alt,
                            unsigned *&vals_alt, int64_t n, int bits, unsigned *counts,
                            hipStream_t stream) {
  const int num_tiles = static_cast<int>(div_ceil(n, kSortBlock * ITEMS));
  const int passes = static_cast<int>(div_ceil(bits, kRadixBits));
  for (int p = 0; p < passes; ++p) {
    const int shift = p * kRadixBits;
    radix_hist_kernel<ITEMS><<<num_tiles, kSortBlock, 0, stream>>>(keys, n, shift, counts, num_tiles);
    check_launch("radix_hist_kernel");
    scan_counts_kernel<<<1, 1024, 0, stream>>>(counts, static_cast<long long>(kRadix) * num_tiles);
    check_launch("scan_counts_kernel");
    radix_scatter_kernel<ITEMS><<<num_tiles, kSortBlock, 0, stream>>>(keys, vals, keys_alt, vals_alt,
                                                                       n, shift, counts, num_tiles);
    check_launch("radix_scatter_kernel");
    std::swap(keys, keys_alt);
    std::swap(vals, vals_alt);
  }
}

size_t radix_counts_len(int64_t n) {
  int items = n <= (int64_t(1) << 20) ? 4 : 16;
  return static_cast<size_t>(kRadix) * static_cast<size_t>(div_ceil(n, kSortBlock * items));
}

void radix_sort_pairs(unsigned long long *&keys, unsigned *&vals, unsigned long long *&keys_alt,
                      unsigned *&vals_alt, int64_t n, int bits, unsigned *counts,
                      hipStream_t stream) {
  if (n <= 1 || bits <= 0) return;
  if (n <= (int64_t(1) << 20)) {
    radix_sort_impl<4>(keys, vals, keys_alt, vals_alt, n, bits, counts, stream);
  } else {
    radix_sort_impl<16>(keys, vals, keys_alt, vals_alt, n, bits, counts, stream);
  }
}

// --------------------------------------------------------------- outputs ----

template <typename CT, typename IT>
__global__ __launch_bounds__(256) void emit_sorted_kernel(const CT *__restrict__ coords, long long n,
                                                          int ndim,
                                                          const unsigned *__restrict__ perm,
                                                          IT *__restrict__ indices_out,
                                                          CT *__restrict__ sorted_out) {
  const long long stride = static_cast<long long>(gridDim.x) * blockDim.x;
  for (long long i = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x; i < n;
       i += stride) {
    const unsigned row = perm[i];
    if (indices_out) indices_out[i] = static_cast<IT>(row);
    if (sorted_out) {
      for (int k = 0; k < ndim; ++k) sorted_out[i * ndim + k] = coords[static_cast<long long>(row) * ndim + k];
    }
  }
}

static int bit_width(unsigned long long range) {
  return range == 0 ? 0 : 64 - __builtin_clzll(range);
}

template <typename CT, typename IT>
static void arg_sort_typed(const CT *coords, int64_t n, int ndim, const IT *batch_dims,
                           int64_t num_batches, IT *indices_out, CT *sorted_out,
                           hipStream_t stream) {
  Scope scope(stream);
  const bool batched = batch_dims != nullptr && num_batches > 1;

  profile_mark("enter:arg_sort", stream);
  long long *d_bounds = scope.alloc<long long>(2 * MNT_MAX_NDIM);
  enqueue_bounds(coords, n, ndim, sizeof(CT) == 4 ? MNT_INT32 : MNT_INT64, d_bounds, true, stream);
  long long *h_bounds = static_cast<long long *>(scope.arena().pinned());
  MNT_HIP(hipMemcpyAsync(h_bounds, d_bounds, sizeof(long long) * 2 * MNT_MAX_NDIM,
                         hipMemcpyDeviceToHost, stream));
  MNT_HIP(hipStreamSynchronize(stream));
  profile_mark("sort_bounds+sync", stream);

  // fields from least to most significant: dims ndim-1 .. 0, then the batch id
  int widths[MNT_MAX_NDIM + 1];
  unsigned long long lows[MNT_MAX_NDIM + 1];
  for (int k = 0; k < ndim; ++k) {
    unsigned long long range = static_cast<unsigned long long>(h_bounds[MNT_MAX_NDIM + k]) -
                               static_cast<unsigned long long>(h_bounds[k]);
    widths[k] = bit_width(range);
    lows[k] = static_cast<unsigned long long>(h_bounds[k]);
  }
  widths[MNT_MAX_NDIM] = batched ? bit_width(static_cast<unsigned long long>(num_batches - 1)) : 0;
  lows[MNT_MAX_NDIM] = 0;

  unsigned long long *keys = scope.alloc<unsigned long long>(n);
  unsigned long long *keys_alt = scope.alloc<unsigned long long>(n);
  unsigned *vals = scope.alloc<unsigned>(n);
  unsigned *vals_alt = scope.alloc<unsigned>(n);
  unsigned *counts = scope.alloc<unsigned>(radix_counts_len(n));

  int order[MNT_MAX_NDIM + 1];
  int num_fields = 0;
  for (int k = ndim - 1; k >= 0; --k) order[num_fields++] = k;
  if (batched) order[num_fields++] = MNT_MAX_NDIM;

  const unsigned grid = grid_for(n, 256, 4096);
  bool first = true;
  int f = 0;
  while (f < num_fields) {
    SortSpec spec;
    memset(&spec, 0, sizeof(spec));
    spec.ndim = ndim;
    spec.num_batches = static_cast<int>(num_batches);
    int bits = 0;
    while (f < num_fields && bits + widths[order[f]] <= 64) {
      int k = order[f];
      if (widths[k] > 0) {
        spec.lo[k] = lows[k];
        spec.mask[k] = widths[k] >= 64 ? ~0ull : ((1ull << widths[k]) - 1ull);
        spec.shift[k] = bits;
        bits += widths[k];
      }
      ++f;
    }
    if (bits == 0 && !first) continue;   // nothing to order by in this group
    pack_keys_kernel<CT, IT><<<grid, 256, 0, stream>>>(coords, n, spec, batch_dims,
                                                       first ? nullptr : vals, keys, vals);
    check_launch("pack_keys_kernel");
    first = false;
    profile_mark("sort_pack", stream);
    radix_sort_pairs(keys, vals, keys_alt, vals_alt, n, bits, counts, stream);
    profile_mark("sort_radix", stream);
  }
  emit_sorted_kernel<CT, IT><<<grid, 256, 0, stream>>>(coords, n, ndim, vals, indices_out, sorted_out);
  check_launch("emit_sorted_kernel");
  profile_mark("sort_emit", stream);
}

}  // namespace mnt

using namespace mnt;

extern "C" int mnt_arg_sort_coordinates(const void *coords, int64_t n, int ndim, int coord_dtype,
                                        const void *batch_dims, int64_t num_batches,
                                        int index_dtype, void *indices_out,
                                        void *sorted_coords_out, void *stream_) {
  return guarded([&] {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    MNT_CHECK(ndim >= 1 && ndim <= MNT_MAX_NDIM, "ndim must be in [1, %d] but found %d",
              MNT_MAX_NDIM, ndim);
    MNT_CHECK(n >= 0 && n <= INT32_MAX, "number of coordinates %lld out of range",
              static_cast<long long>(n));
    int_size(coord_dtype);
    int_size(index_dtype);
    if (n == 0) return;
    MNT_CHECK(coords != nullptr, "coords is null");
    if (batch_dims == nullptr) num_batches = 1;
#define MNT_CASE(CT, IT)                                                                     \
  arg_sort_typed<CT, IT>(static_cast<const CT *>(coords), n, ndim,                            \
                         static_cast<const IT *>(batch_dims), num_batches,                    \
                         static_cast<IT *>(indices_out), static_cast<CT *>(sorted_coords_out), \
                         stream)
    if (coord_dtype == MNT_INT32 && index_dtype == MNT_INT32) {
      MNT_CASE(int32_t, int32_t);
    } else if (coord_dtype == MNT_INT32) {
      MNT_CASE(int32_t, int64_t);
    } else if (index_dtype == MNT_INT32) {
      MNT_CASE(int64_t, int32_t);
    } else {
      MNT_CASE(int64_t, int64_t);
    }
#undef MNT_CASE
  });
}
