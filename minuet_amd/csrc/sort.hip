// Map step, part 1: coordinate bounds, key packing and a stable LSD radix sort
// of (packed voxel key, row index) pairs for gfx950 (64-wide wavefronts).
//
// Follows the semantics of ArgSortCoordinates / MultiArgSortCoordinates
// (csrc/minuet/cuda/functions/arg_sort_coodrinates.cu:273-469): stable,
// lexicographic with dimension 0 most significant, batch-major.
#include "sort.h"

#include <algorithm>
#include <cstdlib>
#include <vector>

#include "device_utils.h"
#include "query_plan.h"

namespace mnt {

// ----------------------------------------------------------------- bounds ----

constexpr int kBoundsBlock = 256;
constexpr int kBoundsMaxBlocks = 256;

// Per-dimension min / max of up to two coordinate arrays with no pre-initialised
// memory, in two launches: every workgroup of bounds_kernel writes its partial
// result, bounds_fold_kernel (one workgroup) folds the partials and writes the
// 16 results straight into pinned host memory:
//   out[0..3] = min of a, out[4..7] = max of a, out[8..11] / out[12..15] = b.
// (One launch with a "last workgroup folds" ticket was measured slower: the
// device-wide fence each workgroup needs before it takes its ticket costs more
// than the second launch.)
template <typename CT>
__global__ __launch_bounds__(kBoundsBlock) void bounds_kernel(
    const CT *__restrict__ a, long long na, int blocks_a, const CT *__restrict__ b, long long nb,
    int ndim, long long *__restrict__ partial, unsigned *__restrict__ zero, int zero_count) {
  // counters of the work that follows, cleared on the way (zero may be null)
  for (int i = blockIdx.x * kBoundsBlock + threadIdx.x; i < zero_count; i += gridDim.x * kBoundsBlock) {
    zero[i] = 0u;
  }
  const bool second = static_cast<int>(blockIdx.x) >= blocks_a;
  const CT *coords = second ? b : a;
  const long long n = second ? nb : na;
  const int my_block = second ? blockIdx.x - blocks_a : blockIdx.x;
  const int my_blocks = second ? gridDim.x - blocks_a : blocks_a;
  long long lo[MNT_MAX_NDIM], hi[MNT_MAX_NDIM];
#pragma unroll
  for (int k = 0; k < MNT_MAX_NDIM; ++k) {
    lo[k] = INT64_MAX;
    hi[k] = INT64_MIN;
  }
  // four rows per thread and trip, all loaded before any is compared (rows past
  // the end re-read the last row, which changes no extreme)
  const long long stride = static_cast<long long>(my_blocks) * kBoundsBlock;
  for (long long i0 = static_cast<long long>(my_block) * kBoundsBlock + threadIdx.x; i0 < n;
       i0 += 4 * stride) {
    long long c[4][MNT_MAX_NDIM];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const long long i = i0 + r * stride;
      load_row<CT>(coords + (i < n ? i : n - 1) * ndim, ndim, c[r]);   // slots past ndim repeat coordinate 0
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
#pragma unroll
      for (int k = 0; k < MNT_MAX_NDIM; ++k) {
        lo[k] = c[r][k] < lo[k] ? c[r][k] : lo[k];
        hi[k] = c[r][k] > hi[k] ? c[r][k] : hi[k];
      }
    }
  }
  __shared__ long long s_lo[kBoundsBlock / kWave][MNT_MAX_NDIM], s_hi[kBoundsBlock / kWave][MNT_MAX_NDIM];
#pragma unroll
  for (int k = 0; k < MNT_MAX_NDIM; ++k) {
    for (int off = 32; off > 0; off >>= 1) {
      long long x = __shfl_down(lo[k], off);
      long long y = __shfl_down(hi[k], off);
      lo[k] = x < lo[k] ? x : lo[k];
      hi[k] = y > hi[k] ? y : hi[k];
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
  if (threadIdx.x < 2 * MNT_MAX_NDIM) {
    const int k = threadIdx.x & (MNT_MAX_NDIM - 1);
    const bool is_max = threadIdx.x >= MNT_MAX_NDIM;
    long long v = is_max ? s_hi[0][k] : s_lo[0][k];
    for (int ww = 1; ww < kBoundsBlock / kWave; ++ww) {
      long long u = is_max ? s_hi[ww][k] : s_lo[ww][k];
      v = is_max ? (u > v ? u : v) : (u < v ? u : v);
    }
    partial[static_cast<long long>(blockIdx.x) * 8 + threadIdx.x] = v;
  }
}

__global__ __launch_bounds__(kBoundsBlock) void bounds_fold_kernel(
    const long long *__restrict__ partial, int num_partials, int blocks_a, long long *out,
    unsigned long long *flag, unsigned long long sequence) {
  const int w = threadIdx.x >> 6;
  // thread t takes the partials of workgroups t, t+256, ... of each array
  long long fa[8], fb[8];
#pragma unroll
  for (int slot = 0; slot < 8; ++slot) {
    fa[slot] = slot >= MNT_MAX_NDIM ? INT64_MIN : INT64_MAX;
    fb[slot] = fa[slot];
  }
  for (int blk = threadIdx.x; blk < num_partials; blk += kBoundsBlock) {
    const bool of_b = blk >= blocks_a;
#pragma unroll
    for (int slot = 0; slot < 8; ++slot) {
      const long long u = partial[static_cast<long long>(blk) * 8 + slot];
      long long &dst = of_b ? fb[slot] : fa[slot];
      dst = slot >= MNT_MAX_NDIM ? (u > dst ? u : dst) : (u < dst ? u : dst);
    }
  }
  __shared__ long long s_fold[kBoundsBlock / kWave][16];
#pragma unroll
  for (int slot = 0; slot < 8; ++slot) {
    for (int off = 32; off > 0; off >>= 1) {
      const long long x = __shfl_down(fa[slot], off);
      const long long y = __shfl_down(fb[slot], off);
      if (slot >= MNT_MAX_NDIM) {
        fa[slot] = x > fa[slot] ? x : fa[slot];
        fb[slot] = y > fb[slot] ? y : fb[slot];
      } else {
        fa[slot] = x < fa[slot] ? x : fa[slot];
        fb[slot] = y < fb[slot] ? y : fb[slot];
      }
    }
  }
  if (lane_id() == 0) {
#pragma unroll
    for (int slot = 0; slot < 8; ++slot) {
      s_fold[w][slot] = fa[slot];
      s_fold[w][8 + slot] = fb[slot];
    }
  }
  __syncthreads();
  if (threadIdx.x < 16) {
    const bool is_max = (threadIdx.x & 7) >= MNT_MAX_NDIM;
    long long v = s_fold[0][threadIdx.x];
    for (int ww = 1; ww < kBoundsBlock / kWave; ++ww) {
      const long long u = s_fold[ww][threadIdx.x];
      v = is_max ? (u > v ? u : v) : (u < v ? u : v);
    }
    out[threadIdx.x] = v;                     // wavefront 0, as is the thread that raises the flag
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    __threadfence_system();
    __hip_atomic_store(flag, sequence, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
  }
}

void read_bounds(const void *a, int64_t na, const void *b, int64_t nb, int ndim, int coord_dtype,
                 long long out[16], Scope &scope, hipStream_t stream) {
  for (int i = 0; i < 16; ++i) out[i] = (i & 4) ? INT64_MIN : INT64_MAX;
  if (na <= 0 && nb <= 0) return;
  const int blocks_a = na > 0 ? static_cast<int>(std::min<int64_t>(div_ceil(na, kBoundsBlock * 4), kBoundsMaxBlocks)) : 0;
  const int blocks_b = nb > 0 ? static_cast<int>(std::min<int64_t>(div_ceil(nb, kBoundsBlock * 4), kBoundsMaxBlocks)) : 0;
  const int grid = blocks_a + blocks_b;
  long long *partial = scope.alloc<long long>(static_cast<size_t>(grid) * 8);
  long long *h_out = static_cast<long long *>(scope.arena().pinned());
  long long *d_out = static_cast<long long *>(scope.arena().pinned_device());
  const unsigned long long sequence = scope.arena().next_sequence();
  unsigned long long *flag = scope.arena().flag_device(0);
  if (coord_dtype == MNT_INT32) {
    bounds_kernel<int32_t><<<grid, kBoundsBlock, 0, stream>>>(
        static_cast<const int32_t *>(a), na, blocks_a, static_cast<const int32_t *>(b), nb, ndim,
        partial, nullptr, 0);
  } else {
    bounds_kernel<int64_t><<<grid, kBoundsBlock, 0, stream>>>(
        static_cast<const int64_t *>(a), na, blocks_a, static_cast<const int64_t *>(b), nb, ndim,
        partial, nullptr, 0);
  }
  check_launch("bounds_kernel");
  bounds_fold_kernel<<<1, kBoundsBlock, 0, stream>>>(partial, grid, blocks_a, d_out, flag, sequence);
  check_launch("bounds_fold_kernel");
  scope.arena().wait_flag(0, sequence);
  if (na > 0) memcpy(out, h_out, sizeof(long long) * 8);
  if (nb > 0) memcpy(out + 8, h_out + 8, sizeof(long long) * 8);
}

// ------------------------------------------- small uploads through kernargs ----

constexpr int kUploadInts = 512;
struct IntChunk {
  int v[kUploadInts];
};

__global__ __launch_bounds__(256) void upload_ints_kernel(IntChunk chunk, int count, int *__restrict__ dst) {
  for (int i = threadIdx.x; i < count; i += blockDim.x) dst[i] = chunk.v[i];
}

// Copies a small host int array to device memory as kernel arguments: no
// staging buffer to protect, no synchronisation, safe under stream capture.
void upload_ints(const std::vector<int> &host, int *dst, hipStream_t stream) {
  for (size_t base = 0; base < host.size(); base += kUploadInts) {
    IntChunk chunk;
    const int count = static_cast<int>(std::min<size_t>(kUploadInts, host.size() - base));
    memcpy(chunk.v, host.data() + base, sizeof(int) * count);
    upload_ints_kernel<<<1, 256, 0, stream>>>(chunk, count, dst + base);
    check_launch("upload_ints_kernel");
  }
}

// ------------------------------------------------------------------ keys ----

// One sort round packs a subset of the fields (dimensions, batch id) into a
// 64-bit key.  Field ndim.. is unused; index MNT_MAX_NDIM is the batch id.
struct SortSpec {
  unsigned long long lo[MNT_MAX_NDIM + 1];
  unsigned long long mask[MNT_MAX_NDIM + 1];
  int shift[MNT_MAX_NDIM + 1];
  int ndim;
  int num_batches;
};

// Pass input taken from key / value arrays of an earlier pass (vals may be
// null for a keys-only sort).
struct PlainSource {
  const unsigned long long *keys;
  const unsigned *vals;
  __device__ __forceinline__ void load(long long i, unsigned long long &key, unsigned &val) const {
    key = keys[i];
    val = vals ? vals[i] : 0u;
  }
};

// Pass input computed on the fly from the coordinate rows: the first pass of a
// round never materialises its keys.  perm (nullable) is the order left by
// the previous round.
template <typename CT, typename IT>
struct CoordSource {
  const CT *coords;
  const IT *batch_dims;
  const unsigned *perm;
  SortSpec spec;
  __device__ __forceinline__ void load(long long i, unsigned long long &key, unsigned &val) const {
    const long long row = perm ? static_cast<long long>(perm[i]) : i;
    long long c[MNT_MAX_NDIM];
    load_row<CT>(coords + row * spec.ndim, spec.ndim, c);
    pack(row, c, key, val);
  }
  // Key of row `row` from its coordinates c (fetched earlier, e.g. before the
  // spec was known).
  template <typename VT>
  __device__ __forceinline__ void pack(long long row, const VT (&c)[MNT_MAX_NDIM],
                                       unsigned long long &key, unsigned &val) const {
    unsigned long long k64 = 0;
#pragma unroll
    for (int k = 0; k < MNT_MAX_NDIM; ++k) {
      // fields that are not part of this round (or past ndim) have mask 0
      const unsigned long long v = static_cast<unsigned long long>(static_cast<long long>(c[k])) - spec.lo[k];
      k64 |= (v & spec.mask[k]) << spec.shift[k];
    }
    if (spec.mask[MNT_MAX_NDIM]) {
      unsigned long long b = batch_of<IT>(row, batch_dims, spec.num_batches);
      k64 |= (b & spec.mask[MNT_MAX_NDIM]) << spec.shift[MNT_MAX_NDIM];
    }
    key = k64;
    val = static_cast<unsigned>(row);
  }
};

// Pass output into key / value arrays for the next pass.
struct PlainSink {
  unsigned long long *keys;
  unsigned *vals;
  __device__ __forceinline__ void store(unsigned pos, unsigned long long key, unsigned val) const {
    keys[pos] = key;
    if (vals) vals[pos] = val;
  }
};

// Output of the very last pass: the permutation and (optionally) the sorted
// coordinate rows, so no separate gather pass is needed.
template <typename CT, typename IT>
struct FinalSink {
  const CT *coords;
  int ndim;
  IT *indices;
  CT *sorted;
  __device__ __forceinline__ void store(unsigned pos, unsigned long long, unsigned val) const {
    if (indices) indices[pos] = static_cast<IT>(val);
    if (sorted) {
      for (int k = 0; k < ndim; ++k) {
        sorted[static_cast<long long>(pos) * ndim + k] = coords[static_cast<long long>(val) * ndim + k];
      }
    }
  }
};

// Output of the bucket sort's ranking step.  A one-round key spells its row
// out (every field is c[k] - lo[k], nothing is dropped), so the sorted
// coordinates are unpacked from the key instead of being fetched through the
// permutation: that fetch is a 64-byte sector per 12-byte row at a random
// place of the input.
template <typename CT, typename IT>
struct KeySink {
  SortSpec spec;
  IT *indices;
  CT *sorted;
  __device__ __forceinline__ void store(unsigned pos, unsigned long long key, unsigned val) const {
    if (indices) indices[pos] = static_cast<IT>(val);
    if (sorted) {
#pragma unroll
      for (int k = 0; k < MNT_MAX_NDIM; ++k) {
        if (k < spec.ndim) {
          sorted[static_cast<long long>(pos) * spec.ndim + k] =
              static_cast<CT>(((key >> spec.shift[k]) & spec.mask[k]) + spec.lo[k]);
        }
      }
    }
  }
};

// ------------------------------------------------------------ radix sort ----

constexpr int kMaxRadixBits = 11;
constexpr int kMaxRadix = 1 << kMaxRadixBits;
constexpr int kSortBlock = 256;
constexpr int kSortWaves = kSortBlock / kWave;

// Digit histogram of one tile; counts are digit-major: counts[d * num_tiles + tile].
template <int ITEMS, typename Source>
__global__ __launch_bounds__(kSortBlock) void radix_hist_kernel(Source src, long long n, int shift,
                                                                int radix_bits,
                                                                unsigned *__restrict__ counts,
                                                                int num_tiles) {
  __shared__ unsigned hist[kMaxRadix];
  const int radix = 1 << radix_bits;
  for (int d = threadIdx.x; d < radix; d += kSortBlock) hist[d] = 0;
  __syncthreads();
  const long long base = static_cast<long long>(blockIdx.x) * (kSortBlock * ITEMS);
#pragma unroll
  for (int r = 0; r < ITEMS; ++r) {
    const long long i = base + r * kSortBlock + threadIdx.x;
    if (i < n) {
      unsigned long long key;
      unsigned val;
      src.load(i, key, val);
      atomicAdd(&hist[static_cast<unsigned>(key >> shift) & (radix - 1)], 1u);
    }
  }
  __syncthreads();
  for (int d = threadIdx.x; d < radix; d += kSortBlock) {
    counts[static_cast<long long>(d) * num_tiles + blockIdx.x] = hist[d];
  }
}

// Exclusive scan of a flat array by one workgroup (small arrays only).
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

// Per-digit exclusive prefix over the tiles (one workgroup per digit, counts
// are digit-major) plus the digit totals; the scatter kernel turns the totals
// into digit bases itself.
__global__ __launch_bounds__(kSortBlock) void digit_scan_kernel(unsigned *__restrict__ counts,
                                                                int num_tiles,
                                                                unsigned *__restrict__ totals) {
  __shared__ unsigned wave_sums[kSortWaves];
  __shared__ unsigned carry_s;
  unsigned *row = counts + static_cast<long long>(blockIdx.x) * num_tiles;
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int w = tid >> 6;
  if (tid == 0) carry_s = 0;
  __syncthreads();
  for (int base = 0; base < num_tiles; base += kSortBlock) {
    const int i = base + tid;
    const unsigned v = i < num_tiles ? row[i] : 0u;
    unsigned inc = v;
    for (int off = 1; off < kWave; off <<= 1) {
      unsigned u = __shfl_up(inc, off);
      if (lane >= off) inc += u;
    }
    if (lane == kWave - 1) wave_sums[w] = inc;
    __syncthreads();
    unsigned before = carry_s;
    unsigned all = 0;
    for (int ww = 0; ww < kSortWaves; ++ww) {
      if (ww < w) before += wave_sums[ww];
      all += wave_sums[ww];
    }
    if (i < num_tiles) row[i] = before + inc - v;
    __syncthreads();
    if (tid == 0) carry_s += all;
    __syncthreads();
  }
  if (tid == 0) totals[blockIdx.x] = carry_s;
}

// Stable scatter of one tile.  Wave w owns the contiguous slice
// [w*64*ITEMS, (w+1)*64*ITEMS) of the tile and walks it 64 items at a time, so
// (wave, round, lane) order equals input order.  Lanes with the same digit
// find each other with one ballot per digit bit; the rank of an item is its
// wave's running counter for the digit plus the number of equal lanes below.
template <int ITEMS, typename Source, typename Sink>
__global__ __launch_bounds__(kSortBlock) void radix_scatter_kernel(
    Source src, Sink dst, long long n, int shift, int radix_bits,
    const unsigned *__restrict__ offsets, const unsigned *__restrict__ totals, int num_tiles) {
  __shared__ volatile unsigned cnt[kSortWaves][kMaxRadix];
  __shared__ unsigned scan_sums[kSortWaves];
  const int radix = 1 << radix_bits;
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int w = tid >> 6;
  for (int ww = 0; ww < kSortWaves; ++ww) {
    for (int d = tid; d < radix; d += kSortBlock) cnt[ww][d] = 0;
  }
  __syncthreads();

  const long long base =
      static_cast<long long>(blockIdx.x) * (kSortBlock * ITEMS) + w * (kWave * ITEMS);
  // thread t owns the contiguous digits [t*per, (t+1)*per) when the digit
  // bases are formed below; their totals and this tile's offsets are fetched
  // now, so that the loads overlap the ranking of the keys
  constexpr int kMaxPer = kMaxRadix / kSortBlock;
  const int per = (radix + kSortBlock - 1) / kSortBlock;
  unsigned digit_total[kMaxPer], digit_offset[kMaxPer];
#pragma unroll
  for (int j = 0; j < kMaxPer; ++j) {
    const int d = tid * per + j;
    const bool mine = j < per && d < radix;
    digit_total[j] = mine ? totals[d] : 0u;
    digit_offset[j] = mine ? offsets[static_cast<long long>(d) * num_tiles + blockIdx.x] : 0u;
  }
  unsigned long long key[ITEMS];
  unsigned val[ITEMS];
  unsigned rank[ITEMS];
  const unsigned long long below_mask = (1ull << lane) - 1ull;
#pragma unroll
  for (int r = 0; r < ITEMS; ++r) {
    const long long i = base + r * kWave + lane;
    const bool valid = i < n;
    key[r] = ~0ull;
    val[r] = 0u;
    if (valid) src.load(i, key[r], val[r]);
  }
#pragma unroll
  for (int r = 0; r < ITEMS; ++r) {
    const long long i = base + r * kWave + lane;
    const bool valid = i < n;
    const unsigned d = static_cast<unsigned>(key[r] >> shift) & (radix - 1);
    unsigned long long peers = __ballot(valid);
#pragma unroll
    for (int b = 0; b < kMaxRadixBits; ++b) {
      if (b < radix_bits) {
        const bool bit = (d >> b) & 1u;
        const unsigned long long vote = __ballot(valid && bit);
        peers &= bit ? vote : ~vote;
      }
    }
    const unsigned below = __popcll(peers & below_mask);
    const unsigned prev = cnt[w][d];
    rank[r] = prev + below;
    __builtin_amdgcn_wave_barrier();
    if (valid && below == 0) cnt[w][d] = prev + __popcll(peers);
    __builtin_amdgcn_wave_barrier();
  }
  // digit bases: exclusive scan of the digit totals
  unsigned local_total = 0;
#pragma unroll
  for (int j = 0; j < kMaxPer; ++j) local_total += digit_total[j];
  unsigned inc = local_total;
  for (int off = 1; off < kWave; off <<= 1) {
    unsigned u = __shfl_up(inc, off);
    if (lane >= off) inc += u;
  }
  if (lane == kWave - 1) scan_sums[w] = inc;
  __syncthreads();
  {
    unsigned run = inc - local_total;
    for (int ww = 0; ww < w; ++ww) run += scan_sums[ww];
#pragma unroll
    for (int j = 0; j < kMaxPer; ++j) {
      const int d = tid * per + j;
      if (j < per && d < radix) {
        unsigned at = run + digit_offset[j];
#pragma unroll
        for (int ww = 0; ww < kSortWaves; ++ww) {
          const unsigned c = cnt[ww][d];
          cnt[ww][d] = at;
          at += c;
        }
        run += digit_total[j];
      }
    }
  }
  __syncthreads();
#pragma unroll
  for (int r = 0; r < ITEMS; ++r) {
    const long long i = base + r * kWave + lane;
    if (i < n) {
      const unsigned d = static_cast<unsigned>(key[r] >> shift) & (radix - 1);
      dst.store(cnt[w][d] + rank[r], key[r], val[r]);
    }
  }
}

static int items_for(int64_t n) { return n <= (int64_t(1) << 20) ? 4 : 16; }

static void pass_plan(int bits, int &passes, int &radix_bits);

int radix_sort_passes(int64_t n, int bits) {
  if (n <= 1 || bits <= 0) return 0;
  int passes, radix_bits;
  pass_plan(bits, passes, radix_bits);
  return passes;
}

size_t radix_counts_len(int64_t n) {
  return static_cast<size_t>(kMaxRadix) * static_cast<size_t>(div_ceil(n, kSortBlock * items_for(n))) +
         kMaxRadix;
}

// Number of passes and digit width for `bits` key bits: as few passes as 11-bit
// digits allow, digits then split evenly.
static void pass_plan(int bits, int &passes, int &radix_bits) {
  passes = static_cast<int>(div_ceil(bits, kMaxRadixBits));
  radix_bits = static_cast<int>(div_ceil(bits, passes));
}

template <int ITEMS, typename Source, typename Sink>
static void radix_pass(const Source &src, const Sink &dst, int64_t n, int shift, int radix_bits,
                       unsigned *counts, hipStream_t stream) {
  const int num_tiles = static_cast<int>(div_ceil(n, kSortBlock * ITEMS));
  const int radix = 1 << radix_bits;
  unsigned *totals = counts + static_cast<size_t>(radix) * num_tiles;
  radix_hist_kernel<ITEMS, Source><<<num_tiles, kSortBlock, 0, stream>>>(src, n, shift, radix_bits, counts, num_tiles);
  check_launch("radix_hist_kernel");
  digit_scan_kernel<<<radix, kSortBlock, 0, stream>>>(counts, num_tiles, totals);
  check_launch("digit_scan_kernel");
  radix_scatter_kernel<ITEMS, Source, Sink><<<num_tiles, kSortBlock, 0, stream>>>(
      src, dst, n, shift, radix_bits, counts, totals, num_tiles);
  check_launch("radix_scatter_kernel");
}

template <typename Source, typename Sink>
static void radix_pass_any(const Source &src, const Sink &dst, int64_t n, int shift, int radix_bits,
                           unsigned *counts, hipStream_t stream) {
  if (items_for(n) == 4) {
    radix_pass<4>(src, dst, n, shift, radix_bits, counts, stream);
  } else {
    radix_pass<16>(src, dst, n, shift, radix_bits, counts, stream);
  }
}

void radix_sort_pairs(unsigned long long *&keys, unsigned *&vals, unsigned long long *&keys_alt,
                      unsigned *&vals_alt, int64_t n, int bits, unsigned *counts,
                      hipStream_t stream) {
  if (n <= 1 || bits <= 0) return;
  int passes, radix_bits;
  pass_plan(bits, passes, radix_bits);
  for (int p = 0; p < passes; ++p) {
    radix_pass_any(PlainSource{keys, vals}, PlainSink{keys_alt, vals ? vals_alt : nullptr}, n,
                   p * radix_bits, radix_bits, counts, stream);
    std::swap(keys, keys_alt);
    if (vals) std::swap(vals, vals_alt);
  }
}

// ----------------------------------------------------------- bucket sort ----
//
// Sort of a cloud whose rows fit one 64-bit key: the rows are dealt into
// buckets by the top bits of their key (about 128 rows per bucket), then every
// bucket is ranked in LDS: a workgroup stages the whole bucket and its
// threads count the words below their own; a large bucket is shared by
// several workgroups.  A bucketed row is kept as
// ((rest of the key) << idx_bits) | row, which is unique, so ranks are unique
// and the order inside a bucket needs no stability from the dealing step:
// cursors handed out by atomics will do.
//
// The bucket histogram, its scan and the dealing step are enqueued right
// behind bounds_kernel, with no wait in between: the histogram kernel folds
// the partial bounds itself and the kernels work out the key layout on the
// device.  The host waits once, for the scan kernel, which hands it the
// bounds, the largest bucket and the number of ranking workgroups, and
// launches the ranking while the dealing step still runs.  A cloud with a
// bucket beyond the LDS capacity (strong clustering) takes the radix passes
// instead; the dealing step sees that for itself and does nothing.

constexpr int kBucketMaxBits = 13;
constexpr int kBucketMax = 1 << kBucketMaxBits;
constexpr int kBucketCap = 7680;              // rows of the largest bucket: its words, their padding and
                                              // the ranking kernel's tables fit 64 KiB of LDS
constexpr int kBucketRows = 128;              // rows per bucket aimed at
constexpr int64_t kBucketMinN = 2048;
constexpr size_t kBucketHostOffset = 384;     // pinned block: largest bucket

// Key layout of a sort that takes one round: fields from least to most
// significant are dimensions ndim-1 .. 0, then the batch id.  bounds = lo[4],
// hi[4].  Returns the key width; above 64 the spec is unusable.
__host__ __device__ inline int single_round_spec(const long long *bounds, int ndim,
                                                 int num_batches, SortSpec &spec) {
  int bits = 0;
#pragma unroll
  for (int k = MNT_MAX_NDIM - 1; k >= 0; --k) {
    spec.lo[k] = 0;
    spec.mask[k] = 0;
    spec.shift[k] = 0;
    if (k < ndim) {
      const unsigned long long range = static_cast<unsigned long long>(bounds[MNT_MAX_NDIM + k]) -
                                       static_cast<unsigned long long>(bounds[k]);
      const int w = range == 0 ? 0 : 64 - __builtin_clzll(range);
      // also for a dimension of one value, which takes no key bits: a key is
      // turned back into its row by adding lo to every field
      spec.lo[k] = static_cast<unsigned long long>(bounds[k]);
      if (w > 0) {
        spec.mask[k] = w >= 64 ? ~0ull : ((1ull << w) - 1ull);
        spec.shift[k] = bits & 63;
        bits += w;
      }
    }
  }
  spec.lo[MNT_MAX_NDIM] = 0;
  spec.mask[MNT_MAX_NDIM] = 0;
  spec.shift[MNT_MAX_NDIM] = 0;
  if (num_batches > 1) {
    const int w = 64 - __builtin_clzll(static_cast<unsigned long long>(num_batches - 1));
    spec.mask[MNT_MAX_NDIM] = (1ull << w) - 1ull;
    spec.shift[MNT_MAX_NDIM] = bits & 63;
    bits += w;
  }
  spec.ndim = ndim;
  spec.num_batches = num_batches;
  return bits;
}

struct BucketLayout {
  int msd_bits;     // key bits that select the bucket
  int shift;        // key >> shift = bucket
  int idx_bits;     // width of a row index
  bool ok;          // one key holds a row and one word holds (rest, row)
};

__host__ __device__ inline BucketLayout bucket_layout(int bits, int msd_cap, int idx_bits) {
  BucketLayout l;
  l.msd_bits = bits < msd_cap ? bits : msd_cap;
  l.shift = bits - l.msd_bits;
  l.idx_bits = idx_bits;
  l.ok = bits >= 1 && bits <= 64 && l.shift + idx_bits <= 64;
  return l;
}

// Folds the partial extremes that bounds_kernel left for one array (a row of
// lo[4], hi[4] per workgroup, at most 128 rows) into b.  Every wavefront does
// the whole fold for itself, two rows per lane: no LDS, no barrier.
constexpr int kBucketBoundsBlocks = 128;
__device__ __forceinline__ void fold_bounds(const long long *__restrict__ partial, int num_partials,
                                            long long (&b)[2 * MNT_MAX_NDIM]) {
  const int lane = lane_id();
  const int row = lane < num_partials ? lane : 0;          // a repeated row changes no extreme
  const int row2 = lane + kWave < num_partials ? lane + kWave : 0;
  long long b2[2 * MNT_MAX_NDIM];
#pragma unroll
  for (int slot = 0; slot < 2 * MNT_MAX_NDIM; ++slot) {
    b[slot] = partial[row * 8 + slot];
    b2[slot] = partial[row2 * 8 + slot];
  }
#pragma unroll
  for (int slot = 0; slot < 2 * MNT_MAX_NDIM; ++slot) {
    b[slot] = slot >= MNT_MAX_NDIM ? (b2[slot] > b[slot] ? b2[slot] : b[slot])
                                   : (b2[slot] < b[slot] ? b2[slot] : b[slot]);
  }
#pragma unroll
  for (int slot = 0; slot < 2 * MNT_MAX_NDIM; ++slot) {
    for (int off = 32; off > 0; off >>= 1) {
      const long long u = __shfl_xor(b[slot], off);
      b[slot] = slot >= MNT_MAX_NDIM ? (u > b[slot] ? u : b[slot]) : (u < b[slot] ? u : b[slot]);
    }
    // the same in every lane: say so, which keeps what is derived from it in
    // scalar registers
    const unsigned lo32 = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(b[slot]));
    const unsigned hi32 =
        __builtin_amdgcn_readfirstlane(static_cast<unsigned>(static_cast<unsigned long long>(b[slot]) >> 32));
    b[slot] = static_cast<long long>((static_cast<unsigned long long>(hi32) << 32) | lo32);
  }
}

// Key layout from the folded bounds.
template <typename CT, typename IT>
__device__ __forceinline__ BucketLayout layout_on_device(
    const CT *__restrict__ coords, const IT *__restrict__ batch_dims, int num_batches, int ndim,
    const long long (&b)[2 * MNT_MAX_NDIM], int msd_cap, int idx_bits, CoordSource<CT, IT> &src) {
  src.coords = coords;
  src.batch_dims = batch_dims;
  src.perm = nullptr;
  const int bits = single_round_spec(b, ndim, num_batches, src.spec);
  return bucket_layout(bits, msd_cap, idx_bits);
}

// Rows per bucket; info[0] tells the scan kernel whether the layout holds.
template <typename CT, typename IT, int kBucketItems>
__global__ __launch_bounds__(kSortBlock) void bucket_hist_kernel(
    const CT *__restrict__ coords, const IT *__restrict__ batch_dims, int num_batches, int ndim,
    long long n, const long long *__restrict__ partial, int num_partials, int msd_cap, int idx_bits,
    unsigned *__restrict__ totals, unsigned *__restrict__ info, long long *__restrict__ bounds_out) {
  __shared__ unsigned hist[kBucketMax];
  // the rows first: their loads need nothing from the bounds
  const long long base = static_cast<long long>(blockIdx.x) * (kSortBlock * kBucketItems);
  CT c[kBucketItems][MNT_MAX_NDIM];
#pragma unroll
  for (int r = 0; r < kBucketItems; ++r) {
    const long long i = base + r * kSortBlock + threadIdx.x;
    load_row_raw<CT>(coords + (i < n ? i : n - 1) * ndim, ndim, c[r]);
  }
  long long bounds[2 * MNT_MAX_NDIM];
  fold_bounds(partial, num_partials, bounds);
  if (blockIdx.x == 0 && threadIdx.x == 0) {
#pragma unroll
    for (int slot = 0; slot < 2 * MNT_MAX_NDIM; ++slot) bounds_out[slot] = bounds[slot];
  }
  CoordSource<CT, IT> src;
  const BucketLayout lay =
      layout_on_device<CT, IT>(coords, batch_dims, num_batches, ndim, bounds, msd_cap, idx_bits, src);
  if (blockIdx.x == 0 && threadIdx.x == 0) info[0] = lay.ok ? 1u : 0u;
  if (!lay.ok) return;
  const int buckets = 1 << lay.msd_bits;
  for (int d = threadIdx.x; d < buckets; d += kSortBlock) hist[d] = 0;
  __syncthreads();
#pragma unroll
  for (int r = 0; r < kBucketItems; ++r) {
    const long long i = base + r * kSortBlock + threadIdx.x;
    unsigned long long key;
    unsigned val;
    src.pack(i, c[r], key, val);
    if (i < n) atomicAdd(&hist[static_cast<unsigned>(key >> lay.shift)], 1u);
  }
  __syncthreads();
  for (int d = threadIdx.x; d < buckets; d += kSortBlock) {
    const unsigned count = hist[d];
    if (count != 0) atomicAdd(&totals[d], count);
  }
}

// A bucket of up to 256 rows is ranked by one workgroup, with 1 << mode
// threads sharing a row so that no lane idles (mode 2, 1, 0 for up to 64, 128,
// 256 rows).  A larger bucket (mode kBucketSplit) is ranked 256 rows per
// workgroup after a second split inside LDS.
constexpr unsigned kBucketSplit = 7;

__device__ __forceinline__ unsigned bucket_mode(unsigned m) {
  return m <= 64 ? 2u : m <= 128 ? 1u : m <= 256 ? 0u : kBucketSplit;
}

__device__ __forceinline__ unsigned bucket_pieces(unsigned m) {
  return m == 0 ? 0u : m <= kSortBlock ? 1u : (m + kSortBlock - 1) / kSortBlock;
}

// One workgroup: bucket starts (exclusive scan of the totals, starts[buckets]
// = n), the cursors of the dealing step (a copy of the starts), the list of
// (bucket, chunk of rows) pairs the ranking kernel runs over, info[1] =
// whether the bucket sort goes ahead, and for the host the bounds, the
// largest bucket (all ones when the layout does not hold)
// and the number of pairs.
// chunks[i] = {first row of the bucket, rows of the bucket | mode << 13 |
// chunk << 16, the bucket (the top bits of its rows' keys), 0}.
__global__ __launch_bounds__(1024) void bucket_scan_kernel(
    const unsigned *__restrict__ totals, int buckets, unsigned *__restrict__ info,
    unsigned *__restrict__ starts, unsigned *__restrict__ cursors, uint4 *__restrict__ chunks,
    const long long *__restrict__ folded, long long *host_bounds,
    unsigned *host_out, unsigned long long *flag, unsigned long long sequence) {
  constexpr int kPer = kBucketMax / 1024;
  __shared__ unsigned long long wave_both[1024 / kWave];
  __shared__ unsigned wave_shared[1024 / kWave];
  __shared__ unsigned s_max;
  const int t = threadIdx.x;
  const int per = (buckets + 1023) / 1024;    // consecutive buckets of one thread
  if (t == 0) s_max = 0;
  unsigned v[kPer];
  unsigned sum = 0, biggest = 0, singles = 0, shared = 0;
#pragma unroll
  for (int j = 0; j < kPer; ++j) {
    const int d = t * per + j;
    v[j] = j < per && d < buckets ? totals[d] : 0u;
    sum += v[j];
    biggest = v[j] > biggest ? v[j] : biggest;
    const unsigned mine = v[j] <= kBucketCap ? bucket_pieces(v[j]) : 0u;
    singles += mine == 1 ? 1u : 0u;
    shared += mine > 1 ? mine : 0u;
  }
  // three scans in two sweeps: rows in the low half and one-workgroup buckets
  // in the high half of one word (fewer than 2^31 rows, so the low half never
  // carries into the high one), workgroups of shared buckets in another
  const unsigned long long mine_both =
      static_cast<unsigned long long>(sum) | (static_cast<unsigned long long>(singles) << 32);
  unsigned long long inclusive = mine_both;
  unsigned shared_inclusive = shared;
  for (int off = 1; off < kWave; off <<= 1) {
    const unsigned long long u = __shfl_up(inclusive, off);
    const unsigned u2 = __shfl_up(shared_inclusive, off);
    if (static_cast<int>(lane_id()) >= off) {
      inclusive += u;
      shared_inclusive += u2;
    }
  }
  for (int off = 32; off > 0; off >>= 1) {
    const unsigned u = __shfl_down(biggest, off);
    biggest = u > biggest ? u : biggest;
  }
  if (lane_id() == kWave - 1) {
    wave_both[t >> 6] = inclusive;
    wave_shared[t >> 6] = shared_inclusive;
  }
  __syncthreads();                            // also orders the clearing of s_max
  if (lane_id() == 0 && biggest != 0) atomicMax(&s_max, biggest);
  unsigned long long before = 0, all_both = 0;
  unsigned shared_before = 0, all_shared = 0;
#pragma unroll
  for (int w = 0; w < 1024 / kWave; ++w) {
    const unsigned long long x = wave_both[w];
    const unsigned x2 = wave_shared[w];
    before += w < (t >> 6) ? x : 0ull;
    shared_before += w < (t >> 6) ? x2 : 0u;
    all_both += x;
    all_shared += x2;
  }
  const unsigned long long exclusive = before + inclusive - mine_both;
  unsigned run = static_cast<unsigned>(exclusive);
  // the workgroups of shared buckets run longest and come first in the list
  unsigned shared_at = shared_before + shared_inclusive - shared;
  unsigned single_at = all_shared + static_cast<unsigned>(exclusive >> 32);
#pragma unroll
  for (int j = 0; j < kPer; ++j) {
    const int d = t * per + j;
    if (j < per && d < buckets) {
      starts[d] = run;
      cursors[d] = run;                       // the dealing step hands out places from here
      if (v[j] <= kBucketCap) {
        const unsigned mine = bucket_pieces(v[j]);
        const unsigned head = v[j] | (bucket_mode(v[j]) << 13);
        if (mine == 1) chunks[single_at++] = make_uint4(run, head, d, 0u);
        for (unsigned c = 0; mine > 1 && c < mine; ++c) {
          chunks[shared_at++] = make_uint4(run, head | (c << 16), d, 0u);
        }
      }
    }
    run += v[j];
  }
  if (t == 1023) starts[buckets] = static_cast<unsigned>(all_both);
  __syncthreads();
  if (t == 0) {
    const bool go = info[0] != 0 && s_max <= kBucketCap;
    info[1] = go ? 1u : 0u;
#pragma unroll
    for (int slot = 0; slot < 2 * MNT_MAX_NDIM; ++slot) host_bounds[slot] = folded[slot];
    host_out[0] = info[0] != 0 ? s_max : 0xffffffffu;
    host_out[1] = all_shared + static_cast<unsigned>(all_both >> 32);
    __threadfence_system();
    __hip_atomic_store(flag, sequence, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
  }
}

// Deals the rows of one tile into their buckets as (rest of key, row) words;
// nothing to do when the scan kernel called the bucket sort off (info[1]).
template <typename CT, typename IT, int kBucketItems>
__global__ __launch_bounds__(kSortBlock) void bucket_deal_kernel(
    const CT *__restrict__ coords, const IT *__restrict__ batch_dims, int num_batches, int ndim,
    long long n, const long long *__restrict__ folded, int msd_cap, int idx_bits_,
    const unsigned *__restrict__ info, unsigned *__restrict__ cursors,
    unsigned long long *__restrict__ words) {
  __shared__ unsigned hist[kBucketMax];
  const int tid = threadIdx.x;
  // the rows first: their loads wait for nothing
  const long long base = static_cast<long long>(blockIdx.x) * (kSortBlock * kBucketItems);
  CT c[kBucketItems][MNT_MAX_NDIM];
#pragma unroll
  for (int r = 0; r < kBucketItems; ++r) {
    const long long i = base + r * kSortBlock + tid;
    load_row_raw<CT>(coords + (i < n ? i : n - 1) * ndim, ndim, c[r]);
  }
  const unsigned go = info[1];
  long long bounds[2 * MNT_MAX_NDIM];
#pragma unroll
  for (int slot = 0; slot < 2 * MNT_MAX_NDIM; ++slot) bounds[slot] = folded[slot];
  if (go == 0) return;
  CoordSource<CT, IT> src;
  const BucketLayout lay =
      layout_on_device<CT, IT>(coords, batch_dims, num_batches, ndim, bounds, msd_cap, idx_bits_, src);
  const int shift = lay.shift, idx_bits = lay.idx_bits;
  const int buckets = 1 << lay.msd_bits;
  for (int d = tid; d < buckets; d += kSortBlock) hist[d] = 0;
  __syncthreads();
  const unsigned long long rest_mask = (1ull << shift) - 1ull;
  unsigned long long key[kBucketItems];
  unsigned row[kBucketItems], place[kBucketItems];
#pragma unroll
  for (int r = 0; r < kBucketItems; ++r) {
    const long long i = base + r * kSortBlock + tid;
    src.pack(i, c[r], key[r], row[r]);
    place[r] = 0;
    if (i < n) place[r] = atomicAdd(&hist[static_cast<unsigned>(key[r] >> shift)], 1u);
  }
  __syncthreads();
  // a range of every bucket this tile has rows for: counts fetched first, then
  // all cursor updates in flight together
  constexpr int kPer = kBucketMax / kSortBlock;
  unsigned count[kPer], got[kPer];
#pragma unroll
  for (int j = 0; j < kPer; ++j) {
    const int d = j * kSortBlock + tid;
    count[j] = d < buckets ? hist[d] : 0u;
  }
#pragma unroll
  for (int j = 0; j < kPer; ++j) {
    const int d = j * kSortBlock + tid;
    got[j] = 0;
    if (count[j] != 0) got[j] = atomicAdd(&cursors[d], count[j]);
  }
#pragma unroll
  for (int j = 0; j < kPer; ++j) {
    const int d = j * kSortBlock + tid;
    if (count[j] != 0) hist[d] = got[j];
  }
  __syncthreads();
#pragma unroll
  for (int r = 0; r < kBucketItems; ++r) {
    const long long i = base + r * kSortBlock + tid;
    if (i < n) {
      const unsigned pos = hist[static_cast<unsigned>(key[r] >> shift)] + place[r];
      words[pos] = ((key[r] & rest_mask) << idx_bits) | static_cast<unsigned long long>(row[r]);
    }
  }
}

// One workgroup per (bucket, chunk of rows): stages the whole bucket in LDS
// and writes its chunk of rows to their final places.
//
// Up to 256 rows: 1 << mode threads per row count the words below that row's
// word, each over an interleaved share of the bucket; the sum is the row's
// place in the bucket.
//
// More rows: the bucket is first split again by the top 8 bits of its words
// (a counting sort into LDS: histogram, scan, scatter by cursor, which every
// workgroup of the bucket repeats for itself); a row then only counts inside
// its own part, whose rows the other parts precede or follow as a whole.
// word_bits = width of a word (rest of the key and row index).
struct RankShared {
  unsigned part_cursor[kSortBlock], part_start[kSortBlock + 1], wave_sums[kSortWaves];
};

template <typename CT, typename IT>
__device__ __forceinline__ void rank_bucket_chunk(
    const unsigned long long *__restrict__ words, const uint4 entry, int idx_bits, int word_bits,
    const KeySink<CT, IT> &sink, unsigned long long *s_words, RankShared &sh) {
  unsigned (&part_cursor)[kSortBlock] = sh.part_cursor;
  unsigned (&part_start)[kSortBlock + 1] = sh.part_start;
  unsigned (&wave_sums)[kSortWaves] = sh.wave_sums;
  const unsigned tid = threadIdx.x;
  const unsigned start = entry.x;
  const unsigned m = entry.y & 0x1fffu;
  const unsigned mode = (entry.y >> 13) & 7u;
  const unsigned chunk = entry.y >> 16;
  const unsigned long long idx_mask = (1ull << idx_bits) - 1ull;
  // key of a row = its bucket above the rest of the key that its word carries
  const int rest_bits = word_bits - idx_bits;
  const unsigned long long key_top = rest_bits >= 64 ? 0ull : static_cast<unsigned long long>(entry.z) << rest_bits;

  if (mode != kBucketSplit) {
    // words are read four at a time by each of the 1 << mode sharers
    const unsigned group = 4u << mode;
    const unsigned padded = (m + group - 1u) / group * group;
    for (unsigned i = tid; i < padded; i += kSortBlock) s_words[i] = i < m ? words[start + i] : ~0ull;
    __syncthreads();
    const unsigned part = tid & ((1u << mode) - 1u);
    const unsigned e = tid >> mode;
    const unsigned long long mine = e < m ? s_words[e] : 0ull;
    unsigned rank = 0;
    for (unsigned j = 4u * part; j < padded; j += group) {
      const unsigned long long a = s_words[j], b = s_words[j + 1], c = s_words[j + 2], d = s_words[j + 3];
      rank += (a < mine ? 1u : 0u) + (b < mine ? 1u : 0u) + (c < mine ? 1u : 0u) + (d < mine ? 1u : 0u);
    }
    // the sharers of a row sit in neighbouring lanes
    for (unsigned off = 1; off < (1u << mode); off <<= 1) rank += __shfl_xor(rank, off);
    if (e < m && part == 0) {
      sink.store(start + rank, key_top | (mine >> idx_bits), static_cast<unsigned>(mine & idx_mask));
    }
    return;
  }

  const int part_bits = word_bits < 8 ? word_bits : 8;
  const int part_shift = word_bits - part_bits;
  part_cursor[tid] = 0;
  __syncthreads();
  // the thread's words (every 256th of the bucket) stay in registers for both
  // sweeps; their loads are all in flight together
  constexpr unsigned kMaxPerThread = (kBucketCap + kSortBlock - 1) / kSortBlock;
  unsigned long long w[kMaxPerThread];
#pragma unroll
  for (unsigned k = 0; k < kMaxPerThread; ++k) {
    const unsigned i = k * kSortBlock + tid;
    w[k] = 0ull;
    if (k * kSortBlock < m && i < m) w[k] = words[start + i];
  }
#pragma unroll
  for (unsigned k = 0; k < kMaxPerThread; ++k) {
    const unsigned i = k * kSortBlock + tid;
    if (k * kSortBlock < m && i < m) atomicAdd(&part_cursor[static_cast<unsigned>(w[k] >> part_shift)], 1u);
  }
  __syncthreads();
  {
    const unsigned count = part_cursor[tid];
    unsigned inclusive = count;
    for (int off = 1; off < kWave; off <<= 1) {
      const unsigned u = __shfl_up(inclusive, off);
      if (static_cast<int>(lane_id()) >= off) inclusive += u;
    }
    if (lane_id() == kWave - 1) wave_sums[tid >> 6] = inclusive;
    __syncthreads();
    unsigned before = 0;
    for (unsigned ww = 0; ww < (tid >> 6); ++ww) before += wave_sums[ww];
    part_start[tid] = before + inclusive - count;
    part_cursor[tid] = before + inclusive - count;
    if (tid == kSortBlock - 1) part_start[kSortBlock] = before + inclusive;
  }
  __syncthreads();
#pragma unroll
  for (unsigned k = 0; k < kMaxPerThread; ++k) {
    const unsigned i = k * kSortBlock + tid;
    if (k * kSortBlock < m && i < m) {
      s_words[atomicAdd(&part_cursor[static_cast<unsigned>(w[k] >> part_shift)], 1u)] = w[k];
    }
  }
  __syncthreads();
  // rows are handed out by their place in the dealt bucket: the order inside a
  // part of the LDS copy differs from workgroup to workgroup
  const unsigned e = chunk * kSortBlock + tid;
  if (e < m) {
    const unsigned long long mine = words[start + e];
    const unsigned part = static_cast<unsigned>(mine >> part_shift);
    const unsigned lo = part_start[part], hi = part_start[part + 1];
    unsigned rank = lo;
    unsigned j = lo;
    for (; j + 8 <= hi; j += 8) {              // eight reads in flight, not one
      unsigned long long x[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) x[u] = s_words[j + u];
#pragma unroll
      for (int u = 0; u < 8; ++u) rank += x[u] < mine ? 1u : 0u;
    }
    for (; j < hi; ++j) rank += s_words[j] < mine ? 1u : 0u;
    sink.store(start + rank, key_top | (mine >> idx_bits), static_cast<unsigned>(mine & idx_mask));
  }
}

template <typename CT, typename IT>
__global__ __launch_bounds__(kSortBlock) void bucket_rank_kernel(
    const unsigned long long *__restrict__ words, const uint4 *__restrict__ chunks, int idx_bits,
    int word_bits, KeySink<CT, IT> sink) {
  extern __shared__ __align__(16) unsigned long long s_words[];
  __shared__ RankShared sh;
  rank_bucket_chunk<CT, IT>(words, chunks[blockIdx.x], idx_bits, word_bits, sink, s_words, sh);
}

// Largest cloud the bucket sort takes (MINUET_BUCKET_SORT_MAX_ROWS overrides;
// 0 switches it off).
static int64_t bucket_sort_max_rows() {
  static const int64_t value = [] {
    const char *text = getenv("MINUET_BUCKET_SORT_MAX_ROWS");
    if (text != nullptr && *text != 0) return static_cast<int64_t>(atoll(text));
    return static_cast<int64_t>(1) << 21;
  }();
  return value;
}

// --------------------------------------------------------------- outputs ----

// Identity / gather emit for the cases without any radix pass.
template <typename CT, typename IT>
__global__ __launch_bounds__(256) void emit_sorted_kernel(const CT *__restrict__ coords, long long n,
                                                          int ndim,
                                                          const unsigned *__restrict__ perm,
                                                          IT *__restrict__ indices_out,
                                                          CT *__restrict__ sorted_out) {
  const long long stride = static_cast<long long>(gridDim.x) * blockDim.x;
  for (long long i = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x; i < n;
       i += stride) {
    const long long row = perm ? static_cast<long long>(perm[i]) : i;
    if (indices_out) indices_out[i] = static_cast<IT>(row);
    if (sorted_out) {
      for (int k = 0; k < ndim; ++k) sorted_out[i * ndim + k] = coords[row * ndim + k];
    }
  }
}

static int bit_width(unsigned long long range) {
  return range == 0 ? 0 : 64 - __builtin_clzll(range);
}

// ------------------------------------ bucket sort without a host round trip ----
//
// The same sort enqueued as four launches that need nothing from the host
// (bounds -> histogram -> dealing -> ranking), for a chain that goes on to
// query the sorted rows: the dealing kernel scans the bucket totals for itself
// (every workgroup repeats the scan of at most 8192 counters; there is no scan
// launch), the ranking kernel takes one bucket per workgroup whatever its
// size, so its grid is known beforehand.  What the host would have decided
// after its wait is decided on the device and left in `status`: a word that
// every later kernel of the chain reads first and that the host looks at once,
// at the end.  status[0] != 0: the cloud does not fit this sort (key wider than
// a word, or a bucket beyond kChainBucketCap rows); nothing was written.

constexpr int kChainBucketCap = 4096;         // rows of the largest bucket (32 KiB of LDS)

// Dealing with the scan folded in.  LDS: s_hist[buckets], s_starts[buckets + 1].
template <typename CT, typename IT, int kBucketItems>
__global__ __launch_bounds__(kSortBlock) void bucket_deal_scan_kernel(
    const CT *__restrict__ coords, int ndim, long long n, const long long *__restrict__ folded,
    int msd_cap, int idx_bits_, const unsigned *__restrict__ info,
    const unsigned *__restrict__ totals, unsigned *__restrict__ cursors,
    uint4 *__restrict__ chunks_out, unsigned *__restrict__ status,
    unsigned long long *__restrict__ words) {
  extern __shared__ __align__(16) unsigned s_deal[];
  __shared__ unsigned long long s_wave[kSortWaves];
  __shared__ unsigned s_wave_shared[kSortWaves], s_wave_max[kSortWaves];
  const int tid = threadIdx.x;
  const int lane = lane_id();
  const int buckets = 1 << msd_cap;
  unsigned *s_hist = s_deal;
  unsigned *s_starts = s_deal + buckets;
  // the rows first: their loads wait for nothing
  const long long base = static_cast<long long>(blockIdx.x) * (kSortBlock * kBucketItems);
  CT c[kBucketItems][MNT_MAX_NDIM];
#pragma unroll
  for (int r = 0; r < kBucketItems; ++r) {
    const long long i = base + r * kSortBlock + tid;
    load_row_raw<CT>(coords + (i < n ? i : n - 1) * ndim, ndim, c[r]);
  }
  // bucket starts: thread t scans the consecutive buckets [t * per, (t + 1) * per)
  constexpr int kPer = kBucketMax / kSortBlock;
  const int per = (buckets + kSortBlock - 1) / kSortBlock;
  unsigned v[kPer];
  unsigned sum = 0, biggest = 0, singles = 0, shared = 0;
#pragma unroll
  for (int j = 0; j < kPer; ++j) {
    const int d = tid * per + j;
    v[j] = j < per && d < buckets ? totals[d] : 0u;
    sum += v[j];
    biggest = v[j] > biggest ? v[j] : biggest;
    const unsigned pieces = bucket_pieces(v[j]);
    singles += pieces == 1 ? 1u : 0u;
    shared += pieces > 1 ? pieces : 0u;
  }
  const unsigned layout_ok = info[0];
  long long bounds[2 * MNT_MAX_NDIM];
#pragma unroll
  for (int slot = 0; slot < 2 * MNT_MAX_NDIM; ++slot) bounds[slot] = folded[slot];
  // rows in the low half and one-workgroup buckets in the high half of one word
  // (fewer than 2^31 rows), workgroups of shared buckets in another
  const unsigned long long mine_both =
      static_cast<unsigned long long>(sum) | (static_cast<unsigned long long>(singles) << 32);
  unsigned long long inclusive = mine_both;
  unsigned shared_inclusive = shared;
  for (int off = 1; off < kWave; off <<= 1) {
    const unsigned long long u = __shfl_up(inclusive, off);
    const unsigned u2 = __shfl_up(shared_inclusive, off);
    if (lane >= off) {
      inclusive += u;
      shared_inclusive += u2;
    }
  }
  for (int off = 32; off > 0; off >>= 1) {
    const unsigned u = __shfl_xor(biggest, off);
    biggest = u > biggest ? u : biggest;
  }
  if (lane == kWave - 1) {
    s_wave[tid >> 6] = inclusive;
    s_wave_shared[tid >> 6] = shared_inclusive;
  }
  if (lane == 0) s_wave_max[tid >> 6] = biggest;
  for (int d = tid; d < buckets; d += kSortBlock) s_hist[d] = 0;
  __syncthreads();
  unsigned long long before = 0, all_both = 0;
  unsigned shared_before = 0, all_shared = 0, all_max = 0;
#pragma unroll
  for (int w = 0; w < kSortWaves; ++w) {
    before += w < (tid >> 6) ? s_wave[w] : 0ull;
    shared_before += w < (tid >> 6) ? s_wave_shared[w] : 0u;
    all_both += s_wave[w];
    all_shared += s_wave_shared[w];
    all_max = s_wave_max[w] > all_max ? s_wave_max[w] : all_max;
  }
  const bool go = layout_ok != 0 && all_max <= static_cast<unsigned>(kChainBucketCap);
  if (blockIdx.x == 0 && tid == 0) {
    status[0] = go ? 0u : 1u;
    status[2] = go ? all_shared + static_cast<unsigned>(all_both >> 32) : 0u;      // pairs of the ranking launch
  }
  if (!go) return;                               // the same verdict in every workgroup
  {
    const unsigned long long exclusive = before + inclusive - mine_both;
    unsigned run = static_cast<unsigned>(exclusive);
    // the workgroups of shared buckets run longest and come first in the list
    unsigned shared_at = shared_before + shared_inclusive - shared;
    unsigned single_at = all_shared + static_cast<unsigned>(exclusive >> 32);
#pragma unroll
    for (int j = 0; j < kPer; ++j) {
      const int d = tid * per + j;
      if (j < per && d < buckets) {
        s_starts[d] = run;
        if (blockIdx.x == 0) {
          const unsigned pieces = bucket_pieces(v[j]);
          const unsigned head = v[j] | (bucket_mode(v[j]) << 13);
          if (pieces == 1) chunks_out[single_at++] = make_uint4(run, head, d, 0u);
          for (unsigned c = 0; pieces > 1 && c < pieces; ++c) {
            chunks_out[shared_at++] = make_uint4(run, head | (c << 16), d, 0u);
          }
        }
      }
      run += v[j];
    }
  }
  CoordSource<CT, IT> src;
  const BucketLayout lay = layout_on_device<CT, IT>(coords, nullptr, 1, ndim, bounds, msd_cap, idx_bits_, src);
  const int shift = lay.shift, idx_bits = lay.idx_bits;
  const unsigned long long rest_mask = (1ull << shift) - 1ull;
  unsigned long long key[kBucketItems];
  unsigned row[kBucketItems], place[kBucketItems];
#pragma unroll
  for (int r = 0; r < kBucketItems; ++r) {
    const long long i = base + r * kSortBlock + tid;
    src.pack(i, c[r], key[r], row[r]);
    place[r] = 0;
    if (i < n) place[r] = atomicAdd(&s_hist[static_cast<unsigned>(key[r] >> shift)], 1u);
  }
  __syncthreads();
  // a range of every bucket this tile has rows for (cursors count from zero)
  unsigned count[kPer], got[kPer];
#pragma unroll
  for (int j = 0; j < kPer; ++j) {
    const int d = j * kSortBlock + tid;
    count[j] = d < buckets ? s_hist[d] : 0u;
  }
#pragma unroll
  for (int j = 0; j < kPer; ++j) {
    const int d = j * kSortBlock + tid;
    got[j] = 0;
    if (count[j] != 0) got[j] = atomicAdd(&cursors[d], count[j]);
  }
#pragma unroll
  for (int j = 0; j < kPer; ++j) {
    const int d = j * kSortBlock + tid;
    if (count[j] != 0) s_hist[d] = got[j] + s_starts[d];
  }
  __syncthreads();
#pragma unroll
  for (int r = 0; r < kBucketItems; ++r) {
    const long long i = base + r * kSortBlock + tid;
    if (i < n) {
      const unsigned pos = s_hist[static_cast<unsigned>(key[r] >> shift)] + place[r];
      words[pos] = ((key[r] & rest_mask) << idx_bits) | static_cast<unsigned long long>(row[r]);
    }
  }
}

// bucket_rank_kernel inside the chain: the (bucket, chunk) list and its length
// come from the dealing launch, so the grid is the largest the list can get
// and workgroups past its end leave at once; the word width follows from the
// folded bounds.  Workgroup 0 has no bucket: its first wavefront writes the
// query plan of the launches that follow.
template <typename CT, typename IT>
__global__ __launch_bounds__(kSortBlock) void bucket_rank_chain_kernel(
    const unsigned long long *__restrict__ words, const uint4 *__restrict__ chunks,
    const unsigned *__restrict__ pair_count, int max_pairs, const long long *__restrict__ folded,
    int ndim, int msd_cap, int idx_bits, const unsigned *__restrict__ status, FinalSink<CT, IT> sink,
    OffsetTable offsets, int num_offsets, DevicePlan *__restrict__ plan_out, int slabs,
    const unsigned *__restrict__ bucket_starts) {
  __shared__ __align__(16) unsigned long long s_words[kChainBucketCap + 128];
  __shared__ RankShared sh;
  const unsigned declined = status[0];
  if (blockIdx.x == 0) {
    // runs whatever the sort's verdict: the plan carries the verdict of the whole chain
    if (plan_out != nullptr && threadIdx.x < kWave) {
      PlanScratch &scratch = *reinterpret_cast<PlanScratch *>(s_words);
      static_assert(sizeof(PlanScratch) <= sizeof(s_words), "plan scratch must fit the word staging area");
      make_plan_on_device(folded, offsets, num_offsets, ndim, declined, scratch, plan_out, bucket_starts, msd_cap);
    }
    return;
  }
  const unsigned pair = blockIdx.x - 1;
  const unsigned pairs = pair_count[0];
  const uint4 entry = chunks[pair];                    // the list has room for max_pairs entries
  long long bounds[2 * MNT_MAX_NDIM];
#pragma unroll
  for (int slot = 0; slot < 2 * MNT_MAX_NDIM; ++slot) bounds[slot] = folded[slot];
  if (declined != 0 || pair >= pairs) return;
  SortSpec spec;
  const int key_bits = single_round_spec(bounds, ndim, 1, spec);
  const BucketLayout lay = bucket_layout(key_bits, msd_cap, idx_bits);
  const KeySink<CT, IT> key_sink{spec, sink.indices, sink.sorted};
  // rank_bucket_chunk reads a bucket's words at words[first output row + i]: with a
  // slab per bucket (slabs != 0) they sit at the start of the bucket's slab instead
  const unsigned long long *from =
      slabs != 0 ? words + static_cast<size_t>(entry.z) * kChainBucketCap - entry.x : words;
  rank_bucket_chunk<CT, IT>(from, entry, idx_bits, lay.shift + idx_bits, key_sink, s_words, sh);
}

// The chain without its histogram launch.  The dealing launch needs to know
// where a bucket starts only because buckets are packed end to end; when every
// bucket gets a slab of kChainBucketCap words of its own (the most the ranking
// launch takes anyway), a row's place is its bucket's slab plus what the
// bucket's cursor says, and the cursors, which start at zero, end up as the
// bucket totals.  The dealing launch then folds the bounds itself (what the
// histogram launch did), and a one-workgroup launch turns the totals into the
// ranking launch's list of (bucket, chunk) pairs (every ranking workgroup doing
// that scan for itself was measured: 16 us more on 2 800 workgroups).  A slab
// that would overflow raises status[0] (which starts at zero) like a bad key
// layout does, and the caller takes the separate sort.
template <typename CT, typename IT, int kBucketItems>
__global__ __launch_bounds__(kSortBlock) void bucket_deal_slab_kernel(
    const CT *__restrict__ coords, int ndim, long long n, const long long *__restrict__ partial,
    int num_partials, int msd_cap, int idx_bits_, unsigned *__restrict__ cursors,
    unsigned *__restrict__ status, long long *__restrict__ bounds_out,
    unsigned long long *__restrict__ slabs) {
  extern __shared__ __align__(16) unsigned s_deal[];
  const int tid = threadIdx.x;
  unsigned *s_hist = s_deal;
  // the rows first: their loads wait for nothing
  const long long base = static_cast<long long>(blockIdx.x) * (kSortBlock * kBucketItems);
  CT c[kBucketItems][MNT_MAX_NDIM];
#pragma unroll
  for (int r = 0; r < kBucketItems; ++r) {
    const long long i = base + r * kSortBlock + tid;
    load_row_raw<CT>(coords + (i < n ? i : n - 1) * ndim, ndim, c[r]);
  }
  long long bounds[2 * MNT_MAX_NDIM];
  fold_bounds(partial, num_partials, bounds);
  if (blockIdx.x == 0 && tid == 0) {
#pragma unroll
    for (int slot = 0; slot < 2 * MNT_MAX_NDIM; ++slot) bounds_out[slot] = bounds[slot];
  }
  CoordSource<CT, IT> src;
  const BucketLayout lay = layout_on_device<CT, IT>(coords, nullptr, 1, ndim, bounds, msd_cap, idx_bits_, src);
  if (!lay.ok) {                                 // the same verdict in every workgroup
    if (blockIdx.x == 0 && tid == 0) status[0] = 1u;
    return;
  }
  const int buckets = 1 << lay.msd_bits;
  for (int d = tid; d < buckets; d += kSortBlock) s_hist[d] = 0;
  __syncthreads();
  const int shift = lay.shift, idx_bits = lay.idx_bits;
  const unsigned long long rest_mask = (1ull << shift) - 1ull;
  unsigned long long key[kBucketItems];
  unsigned row[kBucketItems], place[kBucketItems];
#pragma unroll
  for (int r = 0; r < kBucketItems; ++r) {
    const long long i = base + r * kSortBlock + tid;
    src.pack(i, c[r], key[r], row[r]);
    place[r] = 0;
    if (i < n) place[r] = atomicAdd(&s_hist[static_cast<unsigned>(key[r] >> shift)], 1u);
  }
  __syncthreads();
  // a range of every bucket this tile has rows for
  constexpr int kPer = kBucketMax / kSortBlock;
  unsigned count[kPer], got[kPer];
#pragma unroll
  for (int j = 0; j < kPer; ++j) {
    const int d = j * kSortBlock + tid;
    count[j] = d < buckets ? s_hist[d] : 0u;
  }
#pragma unroll
  for (int j = 0; j < kPer; ++j) {
    const int d = j * kSortBlock + tid;
    got[j] = 0;
    if (count[j] != 0) got[j] = atomicAdd(&cursors[d], count[j]);
  }
#pragma unroll
  for (int j = 0; j < kPer; ++j) {
    const int d = j * kSortBlock + tid;
    if (count[j] != 0) s_hist[d] = got[j];
  }
  __syncthreads();
  bool over = false;
#pragma unroll
  for (int r = 0; r < kBucketItems; ++r) {
    const long long i = base + r * kSortBlock + tid;
    if (i < n) {
      const unsigned bucket = static_cast<unsigned>(key[r] >> shift);
      const unsigned pos = s_hist[bucket] + place[r];
      if (pos < static_cast<unsigned>(kChainBucketCap)) {
        slabs[static_cast<size_t>(bucket) * kChainBucketCap + pos] =
            ((key[r] & rest_mask) << idx_bits) | static_cast<unsigned long long>(row[r]);
      } else {
        over = true;
      }
    }
  }
  if (over) status[0] = 1u;
}

// One workgroup between the dealing and the ranking launch of the slab form:
// from counts[d] = rows of bucket d (the dealing launch's cursors) the list of
// (bucket, chunk) pairs of the ranking launch, numbered as bucket_scan_kernel
// numbers them (the chunks of buckets that several workgroups share first:
// they run longest), and their number in status[2].
__global__ __launch_bounds__(1024) void bucket_pairs_kernel(const unsigned *__restrict__ counts, int buckets,
                                                            uint4 *__restrict__ chunks,
                                                            unsigned *__restrict__ status,
                                                            unsigned *__restrict__ starts) {
  constexpr int kPer = kBucketMax / 1024;
  __shared__ unsigned long long wave_both[1024 / kWave];
  __shared__ unsigned wave_shared[1024 / kWave];
  const int t = threadIdx.x;
  const int per = (buckets + 1023) / 1024;    // consecutive buckets of one thread
  unsigned v[kPer];
  unsigned sum = 0, singles = 0, shared = 0;
#pragma unroll
  for (int j = 0; j < kPer; ++j) {
    const int d = t * per + j;
    v[j] = j < per && d < buckets ? counts[d] : 0u;
    sum += v[j];
    const unsigned mine = bucket_pieces(v[j]);
    singles += mine == 1 ? 1u : 0u;
    shared += mine > 1 ? mine : 0u;
  }
  if (status[0] != 0) return;                 // declined (a slab overflowed): the counts mean nothing
  const unsigned long long mine_both =
      static_cast<unsigned long long>(sum) | (static_cast<unsigned long long>(singles) << 32);
  unsigned long long inclusive = mine_both;
  unsigned shared_inclusive = shared;
  for (int off = 1; off < kWave; off <<= 1) {
    const unsigned long long u = __shfl_up(inclusive, off);
    const unsigned u2 = __shfl_up(shared_inclusive, off);
    if (static_cast<int>(lane_id()) >= off) {
      inclusive += u;
      shared_inclusive += u2;
    }
  }
  if (lane_id() == kWave - 1) {
    wave_both[t >> 6] = inclusive;
    wave_shared[t >> 6] = shared_inclusive;
  }
  __syncthreads();
  unsigned long long before = 0, all_both = 0;
  unsigned shared_before = 0, all_shared = 0;
#pragma unroll
  for (int w = 0; w < 1024 / kWave; ++w) {
    const unsigned long long x = wave_both[w];
    const unsigned x2 = wave_shared[w];
    before += w < (t >> 6) ? x : 0ull;
    shared_before += w < (t >> 6) ? x2 : 0u;
    all_both += x;
    all_shared += x2;
  }
  const unsigned long long exclusive = before + inclusive - mine_both;
  unsigned run = static_cast<unsigned>(exclusive);
  unsigned shared_at = shared_before + shared_inclusive - shared;
  unsigned single_at = all_shared + static_cast<unsigned>(exclusive >> 32);
#pragma unroll
  for (int j = 0; j < kPer; ++j) {
    const int d = t * per + j;
    if (j < per && d < buckets) {
      starts[d] = run;                        // first sorted row of the bucket
      const unsigned mine = bucket_pieces(v[j]);
      const unsigned head = v[j] | (bucket_mode(v[j]) << 13);
      if (mine == 1) chunks[single_at++] = make_uint4(run, head, d, 0u);
      for (unsigned c = 0; mine > 1 && c < mine; ++c) {
        chunks[shared_at++] = make_uint4(run, head | (c << 16), d, 0u);
      }
    }
    run += v[j];
  }
  if (t == 0) {
    status[2] = all_shared + static_cast<unsigned>(all_both >> 32);
    starts[buckets] = static_cast<unsigned>(all_both);
  }
}

static bool chain_slabs_enabled() {
  static const bool on = [] {
    const char *text = std::getenv("MINUET_CHAIN_SLABS");
    return text == nullptr || std::atoi(text) != 0;
  }();
  return on;
}

static bool chain_windows_enabled() {
  static const bool on = [] {
    const char *text = std::getenv("MINUET_CHAIN_WINDOWS");
    return text == nullptr || std::atoi(text) != 0;
  }();
  return on;
}

size_t chain_sort_words(int64_t n) {
  const size_t packed = static_cast<size_t>(n);
  if (!chain_slabs_enabled()) return packed;
  return std::max(packed, (static_cast<size_t>(1) << chain_sort_msd_bits(n)) * kChainBucketCap);
}

bool chain_sort_takes(int64_t n, int64_t num_batches, int num_offsets) {
  return n >= kBucketMinN && n <= bucket_sort_max_rows() && n <= (int64_t(1) << 21) && num_batches <= 1 &&
         num_offsets >= 1 && num_offsets <= kPlanMaxOffsets;
}

template <typename CT>
static void enqueue_chain_sort_typed(const CT *coords, int64_t n, int ndim, int32_t *indices_out,
                                     CT *sorted_out, const ChainSortBuffers &buf,
                                     const OffsetTable &offsets, int num_offsets, hipStream_t stream) {
  const int idx_bits = bit_width(static_cast<unsigned long long>(n - 1));
  const int msd_cap = chain_sort_msd_bits(n);
  const int buckets = 1 << msd_cap;
  const int num_partials = static_cast<int>(std::min<int64_t>(div_ceil(n, kBoundsBlock * 4), kBucketBoundsBlocks));
  bounds_kernel<CT><<<num_partials, kBoundsBlock, 0, stream>>>(coords, n, num_partials, nullptr, 0, ndim,
                                                               buf.partial, buf.counters, buf.counter_words);
  check_launch("bounds_kernel");
  profile_mark("sort_bounds", stream);
  const bool large = n > (int64_t(1) << 18);
  const unsigned tiles = static_cast<unsigned>(div_ceil(n, kSortBlock * (large ? 16 : 4)));
  unsigned *totals = buf.counters;
  unsigned *cursors = buf.counters + buckets;
  if (chain_slabs_enabled()) {
    // status starts at zero: it sits in the counters that bounds_kernel clears
    const size_t lds = sizeof(unsigned) * static_cast<size_t>(buckets);
    // (rows per thread: more of them mean fewer atomics on the cursors, one per
    // bucket a tile touches, which is what the launch waits for: 8 measure 1.4 us
    // faster than 4 at 200 000 rows, 2 are 2.6 us slower)
    if (large) {
      bucket_deal_slab_kernel<CT, int32_t, 16><<<tiles, kSortBlock, lds, stream>>>(
          coords, ndim, n, buf.partial, num_partials, msd_cap, idx_bits, cursors, buf.status, buf.folded, buf.words);
    } else if (n >= (int64_t(1) << 16)) {
      const unsigned tiles8 = static_cast<unsigned>(div_ceil(n, kSortBlock * 8));
      bucket_deal_slab_kernel<CT, int32_t, 8><<<tiles8, kSortBlock, lds, stream>>>(
          coords, ndim, n, buf.partial, num_partials, msd_cap, idx_bits, cursors, buf.status, buf.folded, buf.words);
    } else {
      bucket_deal_slab_kernel<CT, int32_t, 4><<<tiles, kSortBlock, lds, stream>>>(
          coords, ndim, n, buf.partial, num_partials, msd_cap, idx_bits, cursors, buf.status, buf.folded, buf.words);
    }
    check_launch("bucket_deal_slab_kernel");
    profile_mark("sort_deal", stream);
    bucket_pairs_kernel<<<1, 1024, 0, stream>>>(cursors, buckets, buf.chunks, buf.status, buf.starts);
    check_launch("bucket_pairs_kernel");
    profile_mark("sort_pairs", stream);
    const int max_pairs = static_cast<int>(chain_sort_max_pairs(n));
    bucket_rank_chain_kernel<CT, int32_t><<<max_pairs + 1, kSortBlock, 0, stream>>>(
        buf.words, buf.chunks, buf.status + 2, max_pairs, buf.folded, ndim, msd_cap, idx_bits, buf.status,
        FinalSink<CT, int32_t>{coords, ndim, indices_out, sorted_out}, offsets, num_offsets, buf.plan, 1,
        chain_windows_enabled() ? buf.starts : nullptr);
    check_launch("bucket_rank_chain_kernel");
    profile_mark("sort_rank", stream);
    return;
  }
  if (large) {
    bucket_hist_kernel<CT, int32_t, 16><<<tiles, kSortBlock, 0, stream>>>(
        coords, nullptr, 1, ndim, n, buf.partial, num_partials, msd_cap, idx_bits, totals, buf.info, buf.folded);
  } else {
    bucket_hist_kernel<CT, int32_t, 4><<<tiles, kSortBlock, 0, stream>>>(
        coords, nullptr, 1, ndim, n, buf.partial, num_partials, msd_cap, idx_bits, totals, buf.info, buf.folded);
  }
  check_launch("bucket_hist_kernel");
  profile_mark("sort_hist", stream);
  const size_t lds = sizeof(unsigned) * (2 * static_cast<size_t>(buckets));
  if (large) {
    bucket_deal_scan_kernel<CT, int32_t, 16><<<tiles, kSortBlock, lds, stream>>>(
        coords, ndim, n, buf.folded, msd_cap, idx_bits, buf.info, totals, cursors, buf.chunks, buf.status, buf.words);
  } else {
    bucket_deal_scan_kernel<CT, int32_t, 4><<<tiles, kSortBlock, lds, stream>>>(
        coords, ndim, n, buf.folded, msd_cap, idx_bits, buf.info, totals, cursors, buf.chunks, buf.status, buf.words);
  }
  check_launch("bucket_deal_scan_kernel");
  profile_mark("sort_deal", stream);
  const int max_pairs = static_cast<int>(chain_sort_max_pairs(n));
  bucket_rank_chain_kernel<CT, int32_t><<<max_pairs + 1, kSortBlock, 0, stream>>>(
      buf.words, buf.chunks, buf.status + 2, max_pairs, buf.folded, ndim, msd_cap, idx_bits, buf.status,
      FinalSink<CT, int32_t>{coords, ndim, indices_out, sorted_out}, offsets, num_offsets, buf.plan, 0, nullptr);
  check_launch("bucket_rank_chain_kernel");
  profile_mark("sort_rank", stream);
}

// A bucket of m rows makes at most m / 256 + 1 pairs.
int64_t chain_sort_max_pairs(int64_t n) { return (int64_t(1) << chain_sort_msd_bits(n)) + n / kSortBlock + 1; }

int chain_sort_msd_bits(int64_t n) {
  static const int rows = [] {
    const char *text = std::getenv("MINUET_CHAIN_BUCKET_ROWS");
    const int v = text != nullptr ? std::atoi(text) : 0;
    return v >= 16 && v <= 2048 ? v : kBucketRows;
  }();
  return std::max(1, std::min(kBucketMaxBits, bit_width(static_cast<unsigned long long>(n / rows))));
}

void enqueue_chain_sort(const void *coords, int64_t n, int ndim, int coord_dtype, int32_t *indices_out,
                        void *sorted_out, const ChainSortBuffers &buf, const OffsetTable &offsets,
                        int num_offsets, hipStream_t stream) {
  if (coord_dtype == MNT_INT32) {
    enqueue_chain_sort_typed<int32_t>(static_cast<const int32_t *>(coords), n, ndim, indices_out,
                                      static_cast<int32_t *>(sorted_out), buf, offsets, num_offsets, stream);
  } else {
    enqueue_chain_sort_typed<int64_t>(static_cast<const int64_t *>(coords), n, ndim, indices_out,
                                      static_cast<int64_t *>(sorted_out), buf, offsets, num_offsets, stream);
  }
}

template <typename CT, typename IT>
static void arg_sort_typed(const CT *coords, int64_t n, int ndim, const IT *batch_dims,
                           int64_t num_batches, IT *indices_out, CT *sorted_out,
                           int64_t *bounds_host_out, hipStream_t stream) {
  Scope scope(stream);
  const bool batched = batch_dims != nullptr && num_batches > 1;

  profile_mark("enter:arg_sort", stream);
  long long h_bounds[16];
  // bucket sort, first half: bounds partials, bucket histogram, scan and the
  // dealing step in a row; the scan kernel hands the bounds to the host
  const int batches_in_key = batched ? static_cast<int>(num_batches) : 1;
  const bool try_buckets = n >= kBucketMinN && n <= bucket_sort_max_rows();
  const int idx_bits = bit_width(static_cast<unsigned long long>(n - 1));
  const int msd_cap = std::max(1, std::min(kBucketMaxBits, bit_width(static_cast<unsigned long long>(n / kBucketRows))));
  unsigned *bucket_starts = nullptr;
  uint4 *bucket_chunks = nullptr;
  unsigned long long *bucket_words = nullptr;
  if (try_buckets) {
    Arena &arena = scope.arena();
    unsigned *totals = scope.alloc<unsigned>(kBucketMax + 4);
    unsigned *info = totals + kBucketMax;
    bucket_starts = scope.alloc<unsigned>(kBucketMax + 1);
    unsigned *cursors = scope.alloc<unsigned>(kBucketMax);
    // a bucket of m rows makes at most m / 256 + 1 pairs
    bucket_chunks = scope.alloc<uint4>(kBucketMax + static_cast<size_t>(n / kSortBlock) + 1);
    bucket_words = scope.alloc<unsigned long long>(n);
    const int num_partials = static_cast<int>(std::min<int64_t>(div_ceil(n, kBoundsBlock * 4), kBucketBoundsBlocks));
    long long *partial = scope.alloc<long long>(static_cast<size_t>(num_partials) * 8);
    long long *folded = scope.alloc<long long>(2 * MNT_MAX_NDIM);
    const unsigned long long sequence = arena.next_sequence();
    long long *host_bounds = static_cast<long long *>(arena.pinned_device());
    unsigned *host_out = reinterpret_cast<unsigned *>(static_cast<char *>(arena.pinned_device()) + kBucketHostOffset);
    const IT *dims = batched ? batch_dims : nullptr;
    bounds_kernel<CT><<<num_partials, kBoundsBlock, 0, stream>>>(coords, n, num_partials, nullptr, 0, ndim,
                                                                 partial, totals, kBucketMax + 4);
    check_launch("bounds_kernel");
    // rows per thread of the histogram and dealing kernels: 4, or 16 for a large cloud
    const bool large = n > (int64_t(1) << 18);
    const unsigned tiles = static_cast<unsigned>(div_ceil(n, kSortBlock * (large ? 16 : 4)));
    if (large) {
      bucket_hist_kernel<CT, IT, 16><<<tiles, kSortBlock, 0, stream>>>(
          coords, dims, batches_in_key, ndim, n, partial, num_partials, msd_cap, idx_bits, totals, info,
          folded);
    } else {
      bucket_hist_kernel<CT, IT, 4><<<tiles, kSortBlock, 0, stream>>>(
          coords, dims, batches_in_key, ndim, n, partial, num_partials, msd_cap, idx_bits, totals, info,
          folded);
    }
    check_launch("bucket_hist_kernel");
    bucket_scan_kernel<<<1, 1024, 0, stream>>>(totals, 1 << msd_cap, info, bucket_starts, cursors,
                                               bucket_chunks, folded, host_bounds,
                                               host_out, arena.flag_device(3), sequence);
    check_launch("bucket_scan_kernel");
    if (large) {
      bucket_deal_kernel<CT, IT, 16><<<tiles, kSortBlock, 0, stream>>>(
          coords, dims, batches_in_key, ndim, n, folded, msd_cap, idx_bits, info, cursors, bucket_words);
    } else {
      bucket_deal_kernel<CT, IT, 4><<<tiles, kSortBlock, 0, stream>>>(
          coords, dims, batches_in_key, ndim, n, folded, msd_cap, idx_bits, info, cursors, bucket_words);
    }
    check_launch("bucket_deal_kernel");
    arena.wait_flag(3, sequence);
    memcpy(h_bounds, arena.pinned(), sizeof(long long) * 8);
  } else {
    read_bounds(coords, n, nullptr, 0, ndim, sizeof(CT) == 4 ? MNT_INT32 : MNT_INT64, h_bounds, scope, stream);
  }
  if (bounds_host_out != nullptr) memcpy(bounds_host_out, h_bounds, sizeof(long long) * 8);
  profile_mark(try_buckets ? "sort_bounds+deal+sync" : "sort_bounds+sync", stream);

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

  int order[MNT_MAX_NDIM + 1];
  int num_fields = 0;
  for (int k = ndim - 1; k >= 0; --k) order[num_fields++] = k;
  if (batched) order[num_fields++] = MNT_MAX_NDIM;

  // rounds: greedy groups of fields that fit one 64-bit key
  struct Round {
    SortSpec spec;
    int bits;
  };
  std::vector<Round> rounds;
  int f = 0;
  while (f < num_fields) {
    Round round;
    memset(&round.spec, 0, sizeof(SortSpec));
    round.spec.ndim = ndim;
    round.spec.num_batches = static_cast<int>(num_batches);
    int bits = 0;
    while (f < num_fields && bits + widths[order[f]] <= 64) {
      const int k = order[f];
      if (widths[k] > 0) {
        round.spec.lo[k] = lows[k];
        round.spec.mask[k] = widths[k] >= 64 ? ~0ull : ((1ull << widths[k]) - 1ull);
        round.spec.shift[k] = bits;
        bits += widths[k];
      }
      ++f;
    }
    round.bits = bits;
    if (bits > 0) rounds.push_back(round);
  }

  const unsigned grid = grid_for(n, 256, 4096);
  if (rounds.empty()) {   // all rows equal: the stable order is the identity
    emit_sorted_kernel<CT, IT><<<grid, 256, 0, stream>>>(coords, n, ndim, nullptr, indices_out, sorted_out);
    check_launch("emit_sorted_kernel");
    profile_mark("sort_emit", stream);
    return;
  }

  if (try_buckets) {
    // second half: deal and sort, if the layout holds and no bucket is too big
    CoordSource<CT, IT> src{coords, batched ? batch_dims : nullptr, nullptr, {}};
    const int bits = single_round_spec(h_bounds, ndim, batches_in_key, src.spec);
    const BucketLayout lay = bucket_layout(bits, msd_cap, idx_bits);
    if (lay.ok) {
      Arena &arena = scope.arena();
      volatile unsigned *from_scan =
          reinterpret_cast<volatile unsigned *>(static_cast<char *>(arena.pinned()) + kBucketHostOffset);
      const unsigned biggest = from_scan[0];
      const unsigned pairs = from_scan[1];
      if (biggest <= static_cast<unsigned>(kBucketCap) && pairs > 0) {
        const unsigned long long *words = bucket_words;
        const size_t lds = (static_cast<size_t>(biggest) + 128) * sizeof(unsigned long long);
        bucket_rank_kernel<CT, IT><<<pairs, kSortBlock, lds, stream>>>(
            words, bucket_chunks, lay.idx_bits, lay.shift + lay.idx_bits,
            KeySink<CT, IT>{src.spec, indices_out, sorted_out});
        check_launch("bucket_rank_kernel");
        profile_mark("sort_rank", stream);
        return;
      }
    }
  }

  int total_passes = 0;
  for (const Round &round : rounds) {
    int passes, rb;
    pass_plan(round.bits, passes, rb);
    total_passes += passes;
  }
  unsigned long long *keys = nullptr, *keys_alt = nullptr;
  unsigned *vals = nullptr, *vals_alt = nullptr;
  if (total_passes > 1) {
    keys = scope.alloc<unsigned long long>(n);
    vals = scope.alloc<unsigned>(n);
    if (total_passes > 2) {
      keys_alt = scope.alloc<unsigned long long>(n);
      vals_alt = scope.alloc<unsigned>(n);
    }
  }
  unsigned *counts = scope.alloc<unsigned>(radix_counts_len(n));
  const FinalSink<CT, IT> final_sink{coords, ndim, indices_out, sorted_out};

  int done = 0;
  const unsigned *perm = nullptr;     // order left by the previous round
  for (size_t r = 0; r < rounds.size(); ++r) {
    int passes, rb;
    pass_plan(rounds[r].bits, passes, rb);
    const CoordSource<CT, IT> coord_src{coords, batch_dims, perm, rounds[r].spec};
    for (int p = 0; p < passes; ++p) {
      const bool first = p == 0;
      const bool last = done + 1 == total_passes;
      const int shift = p * rb;
      if (first && last) {
        radix_pass_any(coord_src, final_sink, n, shift, rb, counts, stream);
      } else if (first) {
        // the previous round's order lives in `vals`; write into the other pair
        unsigned long long *k_out = perm == vals ? keys_alt : keys;
        unsigned *v_out = perm == vals ? vals_alt : vals;
        radix_pass_any(coord_src, PlainSink{k_out, v_out}, n, shift, rb, counts, stream);
        if (perm == vals) {
          std::swap(keys, keys_alt);
          std::swap(vals, vals_alt);
        }
      } else if (last) {
        radix_pass_any(PlainSource{keys, vals}, final_sink, n, shift, rb, counts, stream);
      } else {
        radix_pass_any(PlainSource{keys, vals}, PlainSink{keys_alt, vals_alt}, n, shift, rb, counts, stream);
        std::swap(keys, keys_alt);
        std::swap(vals, vals_alt);
      }
      ++done;
    }
    perm = vals;
  }
  profile_mark("sort_radix", stream);
}

}  // namespace mnt

using namespace mnt;

extern "C" int mnt_arg_sort_coordinates(const void *coords, int64_t n, int ndim, int coord_dtype,
                                        const void *batch_dims, int64_t num_batches,
                                        int index_dtype, void *indices_out,
                                        void *sorted_coords_out, int64_t *bounds_host_out,
                                        void *stream_) {
  return guarded([&] {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    MNT_CHECK(ndim >= 1 && ndim <= MNT_MAX_NDIM, "ndim must be in [1, %d] but found %d",
              MNT_MAX_NDIM, ndim);
    MNT_CHECK(n >= 0 && n <= INT32_MAX, "number of coordinates %lld out of range",
              static_cast<long long>(n));
    int_size(coord_dtype);
    int_size(index_dtype);
    if (bounds_host_out != nullptr) {
      for (int i = 0; i < 8; ++i) bounds_host_out[i] = (i & 4) ? INT64_MIN : INT64_MAX;
    }
    if (n == 0) return;
    MNT_CHECK(coords != nullptr, "coords is null");
    if (batch_dims == nullptr) num_batches = 1;
#define MNT_CASE(CT, IT)                                                                     \
  arg_sort_typed<CT, IT>(static_cast<const CT *>(coords), n, ndim,                            \
                         static_cast<const IT *>(batch_dims), num_batches,                    \
                         static_cast<IT *>(indices_out), static_cast<CT *>(sorted_coords_out), \
                         bounds_host_out, stream)
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
