// Map step, part 2: run-length unique of sorted coordinates and the fused
// target-coordinate generation of strided layers (floor, sort, unique).
//
// Semantics follow UniqueCoordinates / MultiUniqueCoordinates /
// FillUniqueCoordinates (csrc/minuet/cuda/functions/unique_coordinates.cu:10-102,
// csrc/minuet/cuda/kernels/fill_unique_coordinate.cuh:8-22) and
// KernelMapCache.get_target_coordinates (minuet/nn/convolutions.py:84-99).
#include <algorithm>

#include "device_utils.h"
#include "sort.h"

namespace mnt {

constexpr int kScanBlock = 256;
constexpr int kScanItems = 8;
constexpr int kScanTile = kScanBlock * kScanItems;

// Row i closes a run: it is the last row, differs from row i+1, or a batch
// ends right after it.
template <typename CT, typename IT>
__device__ __forceinline__ bool row_ends_run(const CT *__restrict__ coords, long long i,
                                             long long n, int ndim,
                                             const IT *__restrict__ batch_dims, int num_batches) {
  if (i + 1 >= n) return true;
  bool same = true;
  for (int k = 0; k < ndim; ++k) same &= coords[i * ndim + k] == coords[(i + 1) * ndim + k];
  if (!same) return true;
  if (batch_dims != nullptr) return is_batch_end<IT>(i + 1, batch_dims, num_batches);
  return false;
}

// Exclusive scan of `flag` over the workgroup; returns this thread's exclusive
// prefix and the workgroup total through *total.
__device__ __forceinline__ unsigned block_exclusive_scan(unsigned value, unsigned *total) {
  __shared__ unsigned wave_sums[kScanBlock / kWave];
  unsigned inclusive = value;
  for (int off = 1; off < kWave; off <<= 1) {
    unsigned v = __shfl_up(inclusive, off);
    if (static_cast<int>(lane_id()) >= off) inclusive += v;
  }
  const int w = threadIdx.x >> 6;
  if (lane_id() == kWave - 1) wave_sums[w] = inclusive;
  __syncthreads();
  unsigned base = 0, sum = 0;
  for (int ww = 0; ww < kScanBlock / kWave; ++ww) {
    if (ww < w) base += wave_sums[ww];
    sum += wave_sums[ww];
  }
  __syncthreads();
  *total = sum;
  return base + inclusive - value;
}

template <typename CT, typename IT>
__global__ __launch_bounds__(kScanBlock) void unique_tile_sums_kernel(
    const CT *__restrict__ coords, long long n, int ndim, const IT *__restrict__ batch_dims,
    int num_batches, unsigned *__restrict__ tile_sums) {
  const long long base = static_cast<long long>(blockIdx.x) * kScanTile + threadIdx.x * kScanItems;
  unsigned count = 0;
#pragma unroll
  for (int r = 0; r < kScanItems; ++r) {
    long long i = base + r;
    if (i < n) count += row_ends_run<CT, IT>(coords, i, n, ndim, batch_dims, num_batches) ? 1u : 0u;
  }
  unsigned total;
  block_exclusive_scan(count, &total);
  if (threadIdx.x == 0) tile_sums[blockIdx.x] = total;
}

template <typename CT, typename IT>
__global__ __launch_bounds__(kScanBlock) void unique_write_kernel(
    const CT *__restrict__ coords, long long n, int ndim, const IT *__restrict__ batch_dims,
    int num_batches, const unsigned *__restrict__ tile_bases, IT *__restrict__ idx_out) {
  const long long base = static_cast<long long>(blockIdx.x) * kScanTile + threadIdx.x * kScanItems;
  bool flags[kScanItems];
  unsigned count = 0;
#pragma unroll
  for (int r = 0; r < kScanItems; ++r) {
    long long i = base + r;
    flags[r] = i < n && row_ends_run<CT, IT>(coords, i, n, ndim, batch_dims, num_batches);
    count += flags[r] ? 1u : 0u;
  }
  unsigned total;
  unsigned run = block_exclusive_scan(count, &total) + tile_bases[blockIdx.x];
  if (blockIdx.x == 0 && threadIdx.x == 0) idx_out[0] = 0;
#pragma unroll
  for (int r = 0; r < kScanItems; ++r) {
    long long i = base + r;
    run += flags[r] ? 1u : 0u;
    if (i < n) idx_out[i + 1] = static_cast<IT>(run);
  }
}

template <typename CT, typename IT>
__global__ __launch_bounds__(256) void fill_unique_kernel(const CT *__restrict__ coords,
                                                          long long n, int ndim,
                                                          const IT *__restrict__ idx,
                                                          CT *__restrict__ out) {
  const long long stride = static_cast<long long>(gridDim.x) * blockDim.x;
  for (long long i = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x; i < n;
       i += stride) {
    const IT a = idx[i];
    if (a != idx[i + 1]) {
      for (int k = 0; k < ndim; ++k) out[static_cast<long long>(a) * ndim + k] = coords[i * ndim + k];
    }
  }
}

template <typename CT, typename IT>
static void unique_typed(const CT *coords, int64_t n, int ndim, const IT *batch_dims,
                         int64_t num_batches, IT *idx_out, int64_t *num_unique_out,
                         hipStream_t stream) {
  Scope scope(stream);
  const int tiles = static_cast<int>(div_ceil(n, kScanTile));
  unsigned *tile_sums = scope.alloc<unsigned>(tiles);
  unique_tile_sums_kernel<CT, IT><<<tiles, kScanBlock, 0, stream>>>(
      coords, n, ndim, batch_dims, static_cast<int>(num_batches), tile_sums);
  check_launch("unique_tile_sums_kernel");
  enqueue_exclusive_scan(tile_sums, tiles, stream);
  unique_write_kernel<CT, IT><<<tiles, kScanBlock, 0, stream>>>(
      coords, n, ndim, batch_dims, static_cast<int>(num_batches), tile_sums, idx_out);
  check_launch("unique_write_kernel");
  IT *h = static_cast<IT *>(scope.arena().pinned());
  MNT_HIP(hipMemcpyAsync(h, idx_out + n, sizeof(IT), hipMemcpyDeviceToHost, stream));
  MNT_HIP(hipStreamSynchronize(stream));
  *num_unique_out = static_cast<int64_t>(*h);
}

// ------------------------------------------------- fused target coordinates ----

struct TargetSpec {
  long long base[MNT_MAX_NDIM];     // floor(min / stride) per dimension
  long long stride[MNT_MAX_NDIM];
  int shift[MNT_MAX_NDIM];
  unsigned long long mask[MNT_MAX_NDIM];
  int batch_shift;
  int ndim;
  int num_batches;                  // 0 when there is no batch field
};

__device__ __forceinline__ long long floor_div(long long a, long long b) {
  long long q = a / b;
  return (a % b != 0 && ((a < 0) != (b < 0))) ? q - 1 : q;
}

template <typename CT, typename IT>
__global__ __launch_bounds__(256) void pack_target_keys_kernel(
    const CT *__restrict__ coords, long long n, TargetSpec spec,
    const IT *__restrict__ batch_dims, unsigned long long *__restrict__ keys,
    unsigned *__restrict__ vals) {
  const long long stride = static_cast<long long>(gridDim.x) * blockDim.x;
  for (long long i = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x; i < n;
       i += stride) {
    unsigned long long key = 0;
#pragma unroll
    for (int k = 0; k < MNT_MAX_NDIM; ++k) {
      if (k < spec.ndim) {
        long long cell = floor_div(static_cast<long long>(coords[i * spec.ndim + k]), spec.stride[k]);
        key |= (static_cast<unsigned long long>(cell - spec.base[k]) & spec.mask[k]) << spec.shift[k];
      }
    }
    if (spec.num_batches > 0) {
      key |= static_cast<unsigned long long>(batch_of<IT>(i, batch_dims, spec.num_batches))
             << spec.batch_shift;
    }
    keys[i] = key;
    if (vals) vals[i] = static_cast<unsigned>(i);
  }
}

__global__ __launch_bounds__(kScanBlock) void key_tile_sums_kernel(
    const unsigned long long *__restrict__ keys, long long n, unsigned *__restrict__ tile_sums) {
  const long long base = static_cast<long long>(blockIdx.x) * kScanTile + threadIdx.x * kScanItems;
  unsigned count = 0;
#pragma unroll
  for (int r = 0; r < kScanItems; ++r) {
    long long i = base + r;
    if (i < n) count += (i + 1 >= n || keys[i] != keys[i + 1]) ? 1u : 0u;
  }
  unsigned total;
  block_exclusive_scan(count, &total);
  if (threadIdx.x == 0) tile_sums[blockIdx.x] = total;
}

// Writes the exclusive run index of every sorted key: rank[i] = number of runs
// that end before position i (rank[n] = number of runs).  The thread that owns
// the last key also hands the number of runs to the host: value into pinned
// memory, then the sequence flag the host is spinning on.
__global__ __launch_bounds__(kScanBlock) void key_rank_kernel(
    const unsigned long long *__restrict__ keys, long long n,
    const unsigned *__restrict__ tile_bases, unsigned *__restrict__ rank,
    unsigned *host_count, unsigned long long *flag, unsigned long long sequence) {
  const long long base = static_cast<long long>(blockIdx.x) * kScanTile + threadIdx.x * kScanItems;
  bool flags[kScanItems];
  unsigned count = 0;
#pragma unroll
  for (int r = 0; r < kScanItems; ++r) {
    long long i = base + r;
    flags[r] = i < n && (i + 1 >= n || keys[i] != keys[i + 1]);
    count += flags[r] ? 1u : 0u;
  }
  unsigned total;
  unsigned run = block_exclusive_scan(count, &total) + tile_bases[blockIdx.x];
  if (blockIdx.x == 0 && threadIdx.x == 0) rank[0] = 0;
#pragma unroll
  for (int r = 0; r < kScanItems; ++r) {
    long long i = base + r;
    run += flags[r] ? 1u : 0u;
    if (i < n) rank[i + 1] = run;
    if (i == n - 1 && host_count != nullptr) {
      *host_count = run;
      __threadfence_system();
      __hip_atomic_store(flag, sequence, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
    }
  }
}

template <typename CT, typename IT>
__global__ __launch_bounds__(256) void emit_targets_kernel(
    const unsigned long long *__restrict__ keys, const unsigned *__restrict__ rank, long long n,
    TargetSpec spec, const IT *__restrict__ batch_dims_in, CT *__restrict__ out,
    IT *__restrict__ batch_dims_out) {
  const long long stride = static_cast<long long>(gridDim.x) * blockDim.x;
  const long long first = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
  for (long long i = first; i < n; i += stride) {
    const unsigned a = rank[i];
    if (a != rank[i + 1]) {
      const unsigned long long key = keys[i];
#pragma unroll
      for (int k = 0; k < MNT_MAX_NDIM; ++k) {
        if (k < spec.ndim) {
          long long cell = static_cast<long long>((key >> spec.shift[k]) & spec.mask[k]) + spec.base[k];
          out[static_cast<long long>(a) * spec.ndim + k] = static_cast<CT>(cell * spec.stride[k]);
        }
      }
    }
  }
  // Sorted keys are batch-major, so the rows of batch g occupy the same index
  // range as in the input and rank[dims[g]] is the new boundary.
  if (batch_dims_out != nullptr) {
    for (long long g = first; g <= spec.num_batches; g += stride) {
      batch_dims_out[g] = static_cast<IT>(rank[static_cast<long long>(batch_dims_in[g])]);
    }
  }
}

static int bit_width64(unsigned long long range) {
  return range == 0 ? 0 : 64 - __builtin_clzll(range);
}

// ---- bitmap form: when the packed keys span at most 2^28 values, the set of
// distinct keys is a bitmap.  Marking it and walking it in key order yields
// the sorted, duplicate-free targets without any sort.

constexpr int kBitmapMaxBits = 28;                   // 32 MiB of bits
constexpr int kBitmapWords = 8;                      // 32-bit words per thread
constexpr int kBitmapTile = kScanBlock * kBitmapWords;
// persistent block 0 in the bitmap form: the tile bases of the largest bitmap
// first, so that the bitmap itself always starts at the same place
constexpr size_t kBitmapBasesBytes =
    ((((size_t{1} << (kBitmapMaxBits - 5)) / kBitmapTile + 1) * 4 + 255) / 256) * 256;

template <typename CT, typename IT>
__device__ __forceinline__ unsigned long long target_key(const CT *__restrict__ coords, long long i,
                                                         const TargetSpec &spec,
                                                         const IT *__restrict__ batch_dims) {
  unsigned long long key = 0;
#pragma unroll
  for (int k = 0; k < MNT_MAX_NDIM; ++k) {
    if (k < spec.ndim) {
      long long cell = floor_div(static_cast<long long>(coords[i * spec.ndim + k]), spec.stride[k]);
      key |= (static_cast<unsigned long long>(cell - spec.base[k]) & spec.mask[k]) << spec.shift[k];
    }
  }
  if (spec.num_batches > 0) {
    key |= static_cast<unsigned long long>(batch_of<IT>(i, batch_dims, spec.num_batches))
           << spec.batch_shift;
  }
  return key;
}

template <typename CT, typename IT>
__global__ __launch_bounds__(256) void mark_targets_kernel(const CT *__restrict__ coords, long long n,
                                                           TargetSpec spec,
                                                           const IT *__restrict__ batch_dims,
                                                           unsigned *__restrict__ bitmap) {
  // Rows that follow each other in a sorted cloud fall into the same word of
  // the bitmap more often than not (their cells differ in the last coordinate
  // only): a run of neighbouring lanes with one word ORs its bits into the
  // run's first lane, which issues the run's only atomic.
  const long long stride = static_cast<long long>(gridDim.x) * blockDim.x;
  const int lane = static_cast<int>(lane_id());
  for (long long first = static_cast<long long>(blockIdx.x) * blockDim.x; first < n; first += stride) {
    const long long i = first + threadIdx.x;
    const bool valid = i < n;
    const unsigned long long key = valid ? target_key<CT, IT>(coords, i, spec, batch_dims) : 0ull;
    const unsigned word = valid ? static_cast<unsigned>(key >> 5) : 0xffffffffu;   // no word has this index
    unsigned bits = valid ? 1u << (key & 31u) : 0u;
    for (int off = 1; off < kWave; off <<= 1) {
      const unsigned next_word = __shfl_down(word, off);
      const unsigned next_bits = __shfl_down(bits, off);
      if (lane + off < kWave && next_word == word) bits |= next_bits;
    }
    const unsigned word_before = __shfl_up(word, 1);
    if (valid && (lane == 0 || word_before != word)) atomicOr(&bitmap[word], bits);
  }
}

__global__ __launch_bounds__(kScanBlock) void bitmap_tile_sums_kernel(const unsigned *__restrict__ bitmap,
                                                                      long long words,
                                                                      unsigned *__restrict__ tile_sums) {
  const long long base = static_cast<long long>(blockIdx.x) * kBitmapTile + threadIdx.x * kBitmapWords;
  unsigned count = 0;
#pragma unroll
  for (int r = 0; r < kBitmapWords; ++r) {
    if (base + r < words) count += __popc(bitmap[base + r]);
  }
  unsigned total;
  block_exclusive_scan(count, &total);
  if (threadIdx.x == 0) tile_sums[blockIdx.x] = total;
}

// Exclusive scan of the tile sums in place (tiles + 1 entries, the last one
// receives the total) by one workgroup; the total also goes to the host.
__global__ __launch_bounds__(1024) void bitmap_scan_kernel(unsigned *__restrict__ tile_sums, int tiles,
                                                           unsigned *host_count,
                                                           unsigned long long *flag,
                                                           unsigned long long sequence) {
  __shared__ unsigned wave_sums[1024 / kWave];
  const int t = threadIdx.x;
  const int chunk = (tiles + 1023) / 1024;
  const int lo = t * chunk;
  const int hi = min(tiles, lo + chunk);
  unsigned sum = 0;
  for (int i = lo; i < hi; ++i) sum += tile_sums[i];
  // scan of the 1 024 per-thread sums: inside each wavefront by shuffles, then
  // every thread adds the wavefronts before its own
  unsigned inclusive = sum;
  for (int off = 1; off < kWave; off <<= 1) {
    const unsigned v = __shfl_up(inclusive, off);
    if (static_cast<int>(lane_id()) >= off) inclusive += v;
  }
  const int w = t >> 6;
  if (lane_id() == kWave - 1) wave_sums[w] = inclusive;
  __syncthreads();
  unsigned before = 0, all = 0;
  for (int ww = 0; ww < 1024 / kWave; ++ww) {
    const unsigned v = wave_sums[ww];
    before += ww < w ? v : 0u;
    all += v;
  }
  unsigned run = before + inclusive - sum;
  for (int i = lo; i < hi; ++i) {
    const unsigned v = tile_sums[i];
    tile_sums[i] = run;
    run += v;
  }
  if (t == 1023) {
    const unsigned total = all;
    tile_sums[tiles] = total;
    *host_count = total;
    __threadfence_system();
    __hip_atomic_store(flag, sequence, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
  }
}

template <typename CT, typename IT>
__global__ __launch_bounds__(kScanBlock) void bitmap_emit_kernel(
    unsigned *__restrict__ bitmap, long long words, const unsigned *__restrict__ tile_bases,
    int tiles, TargetSpec spec, CT *__restrict__ out, IT *__restrict__ batch_dims_out) {
  const long long base = static_cast<long long>(blockIdx.x) * kBitmapTile + threadIdx.x * kBitmapWords;
  // a tile without a set bit has nothing to write, unless a batch boundary
  // falls into it (then it is read like any other)
  if (batch_dims_out == nullptr && tile_bases[blockIdx.x] == tile_bases[blockIdx.x + 1]) return;
  unsigned word[kBitmapWords];
  unsigned count = 0;
#pragma unroll
  for (int r = 0; r < kBitmapWords; ++r) {
    word[r] = base + r < words ? bitmap[base + r] : 0u;
    count += __popc(word[r]);
  }
  // Set bits cluster (cells that differ in the last coordinate share a word):
  // a thread that walked its own 8 words would hold up its wavefront for up to
  // 256 rows while others have none.  The tile's non-empty words, with the rank
  // of their first row, are therefore listed in LDS and dealt round-robin.
  __shared__ unsigned s_word[kBitmapTile], s_rank[kBitmapTile];
  __shared__ unsigned short s_at[kBitmapTile];
  unsigned total;
  unsigned run = block_exclusive_scan(count, &total) + tile_bases[blockIdx.x];
  unsigned filled = 0;
#pragma unroll
  for (int r = 0; r < kBitmapWords; ++r) filled += word[r] != 0u ? 1u : 0u;
  unsigned listed;
  unsigned slot = block_exclusive_scan(filled, &listed);
#pragma unroll
  for (int r = 0; r < kBitmapWords; ++r) {
    const unsigned long long first_key = static_cast<unsigned long long>(base + r) << 5;
    if (batch_dims_out != nullptr && base + r < words) {
      // batch boundaries g << batch_shift that fall into this word
      const unsigned long long step = 1ull << spec.batch_shift;
      for (unsigned long long g = (first_key + step - 1) >> spec.batch_shift;
           g < static_cast<unsigned long long>(spec.num_batches) && (g << spec.batch_shift) < first_key + 32;
           ++g) {
        const unsigned bit = static_cast<unsigned>((g << spec.batch_shift) - first_key);
        batch_dims_out[g] = static_cast<IT>(run + __popc(word[r] & ((1u << bit) - 1u)));
      }
    }
    if (word[r] != 0u) {
      bitmap[base + r] = 0u;                     // the bitmap goes back all zero: the next build clears nothing
      s_word[slot] = word[r];
      s_rank[slot] = run;
      s_at[slot] = static_cast<unsigned short>(threadIdx.x * kBitmapWords + r);
      ++slot;
      run += __popc(word[r]);
    }
  }
  __syncthreads();
  // Keys of the bitmap form have at most 28 bits, and (field + base) * stride
  // worked out in CT wraps exactly as the wide product cut to CT does: the
  // loop stays in 32-bit arithmetic for 32-bit coordinates.
  const unsigned tile_key = static_cast<unsigned>(static_cast<unsigned long long>(blockIdx.x) * kBitmapTile << 5);
  for (unsigned i = threadIdx.x; i < listed; i += kScanBlock) {
    unsigned bits = s_word[i];
    unsigned at = s_rank[i];
    const unsigned first_key = tile_key + (static_cast<unsigned>(s_at[i]) << 5);
    while (bits != 0u) {
      const unsigned bit = __ffs(bits) - 1;
      bits &= bits - 1u;
      const unsigned key = first_key | bit;
      CT *row = out + static_cast<long long>(at) * spec.ndim;
#pragma unroll
      for (int k = 0; k < MNT_MAX_NDIM; ++k) {
        if (k < spec.ndim) {
          const CT cell = static_cast<CT>((key >> spec.shift[k]) & static_cast<unsigned>(spec.mask[k])) +
                          static_cast<CT>(spec.base[k]);
          row[k] = cell * static_cast<CT>(spec.stride[k]);
        }
      }
      ++at;
    }
  }
  if (batch_dims_out != nullptr && blockIdx.x == 0 && threadIdx.x == 0) {
    batch_dims_out[spec.num_batches] = static_cast<IT>(tile_bases[tiles]);
  }
}

// What phase 2 needs to know about phase 1 (kept in the arena's pending blob).
struct TargetState {
  TargetSpec spec;
  int bitmap;            // 1: bitmap form, 0: sorted keys + ranks
  long long words;
  int tiles;
};

// early_out (nullable): room for n target rows; the targets (and early_dims_out,
// the new batch boundaries) are then written while the host waits for the
// count, and no second call follows.
template <typename CT, typename IT>
static void target_count_typed(const CT *coords, int64_t n, int ndim, const int64_t *target_stride,
                               const IT *batch_dims, int64_t num_batches,
                               const int64_t *source_bounds, int64_t *count_out, hipStream_t stream,
                               CT *early_out = nullptr, IT *early_dims_out = nullptr) {
  Arena &arena = Arena::of(stream);
  arena.pending.valid = false;
  const bool batched = batch_dims != nullptr && num_batches > 1;
  TargetSpec spec;
  memset(&spec, 0, sizeof(spec));
  {
    Scope scope(stream);
    long long h_bounds[16];
    if (source_bounds != nullptr) {
      for (int i = 0; i < 8; ++i) h_bounds[i] = source_bounds[i];
    } else {
      read_bounds(coords, n, nullptr, 0, ndim, sizeof(CT) == 4 ? MNT_INT32 : MNT_INT64, h_bounds, scope, stream);
    }
    int bits = 0;
    spec.ndim = ndim;
    for (int k = ndim - 1; k >= 0; --k) {
      MNT_CHECK(target_stride[k] > 0, "target stride must be positive but found %lld",
                static_cast<long long>(target_stride[k]));
      auto fdiv = [](long long a, long long b) {
        long long q = a / b;
        return (a % b != 0 && ((a < 0) != (b < 0))) ? q - 1 : q;
      };
      long long lo = fdiv(h_bounds[k], target_stride[k]);
      long long hi = fdiv(h_bounds[MNT_MAX_NDIM + k], target_stride[k]);
      int width = bit_width64(static_cast<unsigned long long>(hi) - static_cast<unsigned long long>(lo));
      spec.base[k] = lo;
      spec.stride[k] = target_stride[k];
      spec.shift[k] = bits < 64 ? bits : 63;
      spec.mask[k] = width >= 64 ? ~0ull : ((1ull << width) - 1ull);
      bits += width;
    }
    int batch_width = batched ? bit_width64(static_cast<unsigned long long>(num_batches - 1)) : 0;
    spec.batch_shift = bits < 64 ? bits : 63;
    spec.num_batches = batched ? static_cast<int>(num_batches) : 0;
    bits += batch_width;
    MNT_CHECK(bits <= 64,
              "coordinate range needs %d key bits; strided target generation supports at most 64",
              bits);
    if (bits <= kBitmapMaxBits) {
      const long long words = bits <= 5 ? 1 : (1ll << (bits - 5));
      const int tiles = static_cast<int>(div_ceil(words, kBitmapTile));
      // persistent block: tile bases [tiles + 1] in a fixed-size head, then bitmap [words]
      char *keep = static_cast<char *>(arena.persistent(0, kBitmapBasesBytes + static_cast<size_t>(words) * 4));
      unsigned *tile_bases = reinterpret_cast<unsigned *>(keep);
      unsigned *bitmap = reinterpret_cast<unsigned *>(keep + kBitmapBasesBytes);
      // (the walk of the last build left its words zero; anything else that
      // wrote here, or a build whose walk never ran, has reset the count)
      const long long zero_words = arena.zero_bitmap_words;
      if (zero_words < words) MNT_HIP(hipMemsetAsync(bitmap, 0, static_cast<size_t>(words) * 4, stream));
      arena.zero_bitmap_words = 0;
      arena.zero_bitmap_words_after = std::max(zero_words, words);
      mark_targets_kernel<CT, IT><<<grid_for(n, 256, 4096), 256, 0, stream>>>(coords, n, spec, batch_dims, bitmap);
      check_launch("mark_targets_kernel");
      bitmap_tile_sums_kernel<<<tiles, kScanBlock, 0, stream>>>(bitmap, words, tile_bases);
      check_launch("bitmap_tile_sums_kernel");
      volatile unsigned *h = reinterpret_cast<volatile unsigned *>(static_cast<char *>(arena.pinned()) + 256);
      unsigned *d = reinterpret_cast<unsigned *>(static_cast<char *>(arena.pinned_device()) + 256);
      const unsigned long long sequence = arena.next_sequence();
      bitmap_scan_kernel<<<1, 1024, 0, stream>>>(tile_bases, tiles, d, arena.flag_device(2), sequence);
      check_launch("bitmap_scan_kernel");
      if (early_out != nullptr) {
        bitmap_emit_kernel<CT, IT><<<tiles, kScanBlock, 0, stream>>>(
            bitmap, words, tile_bases, tiles, spec, early_out, batched ? early_dims_out : nullptr);
        check_launch("bitmap_emit_kernel");
        arena.zero_bitmap_words = arena.zero_bitmap_words_after;
      }
      arena.wait_flag(2, sequence);
      *count_out = static_cast<int64_t>(*h);
      if (early_out != nullptr) return;
      TargetState state;
      memset(&state, 0, sizeof(state));
      state.spec = spec;
      state.bitmap = 1;
      state.words = words;
      state.tiles = tiles;
      auto &p = arena.pending;
      p.valid = true;
      p.count = *count_out;
      p.n = n;
      p.num_batches = batched ? num_batches : 0;
      p.ndim = ndim;
      p.coord_dtype = sizeof(CT) == 4 ? MNT_INT32 : MNT_INT64;
      p.index_dtype = sizeof(IT) == 4 ? MNT_INT32 : MNT_INT64;
      static_assert(sizeof(TargetState) <= sizeof(p.blob), "pending blob too small");
      memcpy(p.blob, &state, sizeof(state));
      p.batch_dims = batch_dims;
      return;
    }

    // persistent block: sorted keys [n] then ranks [n+1]
    size_t key_bytes = (static_cast<size_t>(n) * 8 + 255) / 256 * 256;
    char *keep = static_cast<char *>(arena.persistent(0, key_bytes + (static_cast<size_t>(n) + 1) * 4));
    arena.zero_bitmap_words = 0;                 // the sorted keys go where the bitmap form keeps its bitmap
    // the sort ping-pongs between two buffers: start in the one that makes it
    // end in the persistent block
    unsigned long long *kept_keys = reinterpret_cast<unsigned long long *>(keep);
    unsigned long long *spare = scope.alloc<unsigned long long>(n);
    const bool even = radix_sort_passes(n, bits) % 2 == 0;
    unsigned long long *keys = even ? kept_keys : spare;
    unsigned long long *keys_alt = even ? spare : kept_keys;
    unsigned *vals = nullptr, *vals_alt = nullptr;      // keys-only sort
    unsigned *counts = scope.alloc<unsigned>(radix_counts_len(n));
    const unsigned grid = grid_for(n, 256, 4096);
    pack_target_keys_kernel<CT, IT><<<grid, 256, 0, stream>>>(coords, n, spec, batch_dims, keys, vals);
    check_launch("pack_target_keys_kernel");
    radix_sort_pairs(keys, vals, keys_alt, vals_alt, n, bits, counts, stream);
    MNT_CHECK(keys == kept_keys, "sorted keys did not end in the persistent block");
    unsigned *rank = reinterpret_cast<unsigned *>(keep + key_bytes);
    const int tiles = static_cast<int>(div_ceil(n, kScanTile));
    unsigned *tile_sums = scope.alloc<unsigned>(tiles);
    key_tile_sums_kernel<<<tiles, kScanBlock, 0, stream>>>(kept_keys, n, tile_sums);
    check_launch("key_tile_sums_kernel");
    enqueue_exclusive_scan(tile_sums, tiles, stream);
    // the count goes to pinned memory (past the 16 bounds slots) with flag 2
    volatile unsigned *h = reinterpret_cast<volatile unsigned *>(static_cast<char *>(arena.pinned()) + 256);
    unsigned *d = reinterpret_cast<unsigned *>(static_cast<char *>(arena.pinned_device()) + 256);
    const unsigned long long sequence = arena.next_sequence();
    key_rank_kernel<<<tiles, kScanBlock, 0, stream>>>(kept_keys, n, tile_sums, rank, d, arena.flag_device(2),
                                                     sequence);
    check_launch("key_rank_kernel");
    if (early_out != nullptr) {
      emit_targets_kernel<CT, IT><<<grid, 256, 0, stream>>>(kept_keys, rank, n, spec, batch_dims, early_out,
                                                            batched ? early_dims_out : nullptr);
      check_launch("emit_targets_kernel");
    }
    arena.wait_flag(2, sequence);
    *count_out = static_cast<int64_t>(*h);
  }
  if (early_out != nullptr) return;
  auto &p = arena.pending;
  p.valid = true;
  p.count = *count_out;
  p.n = n;
  p.num_batches = batched ? num_batches : 0;
  p.ndim = ndim;
  p.coord_dtype = sizeof(CT) == 4 ? MNT_INT32 : MNT_INT64;
  p.index_dtype = sizeof(IT) == 4 ? MNT_INT32 : MNT_INT64;
  TargetState state;
  memset(&state, 0, sizeof(state));
  state.spec = spec;
  memcpy(p.blob, &state, sizeof(state));
  p.batch_dims = batch_dims;
}

template <typename CT, typename IT>
static void target_fill_typed(CT *out, IT *batch_dims_out, hipStream_t stream) {
  Arena &arena = Arena::of(stream);
  auto &p = arena.pending;
  TargetState state;
  memcpy(&state, p.blob, sizeof(state));
  const TargetSpec spec = state.spec;
  const int64_t n = p.n;
  if (state.bitmap) {
    char *keep = static_cast<char *>(arena.persistent(0, 0));
    const unsigned *tile_bases = reinterpret_cast<const unsigned *>(keep);
    unsigned *bitmap = reinterpret_cast<unsigned *>(keep + kBitmapBasesBytes);
    bitmap_emit_kernel<CT, IT><<<state.tiles, kScanBlock, 0, stream>>>(
        bitmap, state.words, tile_bases, state.tiles, spec, out,
        p.num_batches > 0 ? batch_dims_out : nullptr);
    check_launch("bitmap_emit_kernel");
    arena.zero_bitmap_words = arena.zero_bitmap_words_after;
    p.valid = false;
    return;
  }
  size_t key_bytes = (static_cast<size_t>(n) * 8 + 255) / 256 * 256;
  char *keep = static_cast<char *>(arena.persistent(0, 0));
  const unsigned long long *keys = reinterpret_cast<const unsigned long long *>(keep);
  const unsigned *rank = reinterpret_cast<const unsigned *>(keep + key_bytes);
  const unsigned grid = grid_for(n, 256, 4096);
  emit_targets_kernel<CT, IT><<<grid, 256, 0, stream>>>(
      keys, rank, n, spec, static_cast<const IT *>(p.batch_dims), out,
      p.num_batches > 0 ? batch_dims_out : nullptr);
  check_launch("emit_targets_kernel");
  p.valid = false;
}

}  // namespace mnt

using namespace mnt;

#define MNT_DISPATCH_CI(coord_dtype, index_dtype, CALL) \
  do {                                                  \
    if (coord_dtype == MNT_INT32 && index_dtype == MNT_INT32) { \
      CALL(int32_t, int32_t);                           \
    } else if (coord_dtype == MNT_INT32) {              \
      CALL(int32_t, int64_t);                           \
    } else if (index_dtype == MNT_INT32) {              \
      CALL(int64_t, int32_t);                           \
    } else {                                            \
      CALL(int64_t, int64_t);                           \
    }                                                   \
  } while (0)

extern "C" int mnt_unique_coordinates(const void *sorted_coords, int64_t n, int ndim,
                                      int coord_dtype, const void *batch_dims,
                                      int64_t num_batches, int index_dtype, void *idx_out,
                                      int64_t *num_unique_out, void *stream_) {
  return guarded([&] {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    MNT_CHECK(ndim >= 1 && ndim <= MNT_MAX_NDIM, "ndim must be in [1, %d] but found %d",
              MNT_MAX_NDIM, ndim);
    MNT_CHECK(n >= 0 && n <= INT32_MAX, "number of coordinates %lld out of range",
              static_cast<long long>(n));
    MNT_CHECK(idx_out != nullptr && num_unique_out != nullptr, "null output");
    int_size(coord_dtype);
    const int isz = int_size(index_dtype);
    if (n == 0) {
      MNT_HIP(hipMemsetAsync(idx_out, 0, isz, stream));
      *num_unique_out = 0;
      return;
    }
    if (batch_dims == nullptr) num_batches = 1;
#define MNT_CALL(CT, IT)                                                                      \
  unique_typed<CT, IT>(static_cast<const CT *>(sorted_coords), n, ndim,                         \
                       static_cast<const IT *>(batch_dims), num_batches,                        \
                       static_cast<IT *>(idx_out), num_unique_out, stream)
    MNT_DISPATCH_CI(coord_dtype, index_dtype, MNT_CALL);
#undef MNT_CALL
  });
}

extern "C" int mnt_fill_unique_coordinates(const void *sorted_coords, int64_t n, int ndim,
                                           int coord_dtype, const void *idx, int index_dtype,
                                           void *unique_out, void *stream_) {
  return guarded([&] {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    MNT_CHECK(ndim >= 1 && ndim <= MNT_MAX_NDIM, "ndim must be in [1, %d] but found %d",
              MNT_MAX_NDIM, ndim);
    int_size(coord_dtype);
    int_size(index_dtype);
    if (n == 0) return;
    const unsigned grid = grid_for(n, 256, 4096);
#define MNT_CALL(CT, IT)                                                                  \
  fill_unique_kernel<CT, IT><<<grid, 256, 0, stream>>>(static_cast<const CT *>(sorted_coords), \
                                                       n, ndim, static_cast<const IT *>(idx),   \
                                                       static_cast<CT *>(unique_out))
    MNT_DISPATCH_CI(coord_dtype, index_dtype, MNT_CALL);
#undef MNT_CALL
    check_launch("fill_unique_kernel");
  });
}

extern "C" int mnt_target_coordinates_count(const void *source_coords, int64_t n, int ndim,
                                            int coord_dtype, const int64_t *target_stride,
                                            const void *batch_dims, int64_t num_batches,
                                            int index_dtype, const int64_t *source_bounds_host,
                                            int64_t *num_targets_out, void *stream_) {
  return guarded([&] {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    MNT_CHECK(ndim >= 1 && ndim <= MNT_MAX_NDIM, "ndim must be in [1, %d] but found %d",
              MNT_MAX_NDIM, ndim);
    MNT_CHECK(n >= 0 && n <= INT32_MAX, "number of coordinates %lld out of range",
              static_cast<long long>(n));
    MNT_CHECK(target_stride != nullptr && num_targets_out != nullptr, "null argument");
    int_size(coord_dtype);
    int_size(index_dtype);
    if (n == 0) {
      Arena &arena = Arena::of(stream);
      arena.pending = Arena::Pending();
      arena.pending.valid = true;
      arena.pending.coord_dtype = coord_dtype;
      arena.pending.index_dtype = index_dtype;
      arena.pending.ndim = ndim;
      arena.pending.num_batches = (batch_dims && num_batches > 1) ? num_batches : 0;
      arena.pending.batch_dims = batch_dims;
      *num_targets_out = 0;
      return;
    }
    if (batch_dims == nullptr) num_batches = 1;
#define MNT_CALL(CT, IT)                                                                        \
  target_count_typed<CT, IT>(static_cast<const CT *>(source_coords), n, ndim, target_stride,      \
                             static_cast<const IT *>(batch_dims), num_batches, source_bounds_host, \
                             num_targets_out, stream)
    MNT_DISPATCH_CI(coord_dtype, index_dtype, MNT_CALL);
#undef MNT_CALL
  });
}

extern "C" int mnt_target_coordinates(const void *source_coords, int64_t n, int ndim, int coord_dtype,
                                      const int64_t *target_stride, const void *batch_dims,
                                      int64_t num_batches, int index_dtype,
                                      const int64_t *source_bounds_host, void *target_coords_out,
                                      int64_t capacity, void *target_batch_dims_out,
                                      int64_t *num_targets_out, void *stream_) {
  return guarded([&] {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    MNT_CHECK(ndim >= 1 && ndim <= MNT_MAX_NDIM, "ndim must be in [1, %d] but found %d",
              MNT_MAX_NDIM, ndim);
    MNT_CHECK(n > 0 && n <= INT32_MAX, "number of coordinates %lld out of range (the one-call form needs "
              "at least one)", static_cast<long long>(n));
    MNT_CHECK(target_stride != nullptr && num_targets_out != nullptr && target_coords_out != nullptr,
              "null argument");
    MNT_CHECK(capacity >= n, "capacity = %lld rows cannot hold the targets of %lld sources",
              static_cast<long long>(capacity), static_cast<long long>(n));
    int_size(coord_dtype);
    int_size(index_dtype);
    if (batch_dims == nullptr) num_batches = 1;
    MNT_CHECK(num_batches <= 1 || target_batch_dims_out != nullptr, "target_batch_dims_out is null");
#define MNT_CALL(CT, IT)                                                                        \
  target_count_typed<CT, IT>(static_cast<const CT *>(source_coords), n, ndim, target_stride,      \
                             static_cast<const IT *>(batch_dims), num_batches, source_bounds_host, \
                             num_targets_out, stream, static_cast<CT *>(target_coords_out),       \
                             static_cast<IT *>(target_batch_dims_out))
    MNT_DISPATCH_CI(coord_dtype, index_dtype, MNT_CALL);
#undef MNT_CALL
  });
}

extern "C" int mnt_target_coordinates_fill(void *target_coords_out, void *target_batch_dims_out,
                                           void *stream_) {
  return guarded([&] {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    Arena &arena = Arena::of(stream);
    MNT_CHECK(arena.pending.valid,
              "mnt_target_coordinates_fill called without a preceding mnt_target_coordinates_count");
    const int coord_dtype = arena.pending.coord_dtype;
    const int index_dtype = arena.pending.index_dtype;
    if (arena.pending.n == 0) {
      if (arena.pending.num_batches > 0 && target_batch_dims_out != nullptr) {
        MNT_HIP(hipMemsetAsync(target_batch_dims_out, 0,
                               int_size(index_dtype) * (arena.pending.num_batches + 1), stream));
      }
      arena.pending.valid = false;
      return;
    }
#define MNT_CALL(CT, IT)                                                          \
  target_fill_typed<CT, IT>(static_cast<CT *>(target_coords_out),                  \
                            static_cast<IT *>(target_batch_dims_out), stream)
    MNT_DISPATCH_CI(coord_dtype, index_dtype, MNT_CALL);
#undef MNT_CALL
  });
}
