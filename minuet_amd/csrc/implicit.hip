// Output-stationary forward of a sparse convolution ("implicit GEMM"): the
// whole of Gather -> GEMM -> Scatter
// (csrc/minuet/cuda/functions/sparse_convolution.cu:504-661) in one kernel
// that never materialises the gather or GEMM-output buffers.
//
// It works from the dense kernel map M[O, T] (source row per (offset, target),
// -1 for none; csrc/minuet/cuda/kernels/query_sorted_index_with_offsets.cuh)
// instead of the rank tables.  One wavefront owns 32 consecutive targets and
// keeps their output rows in MFMA accumulators; for every offset it loads the
// source rows M[o, t] straight into its MFMA operand registers (zeros where
// there is no source) and multiplies them by W_o, which the four wavefronts of
// a workgroup share through LDS.  A wavefront skips an offset none of its 32
// targets uses, so the wasted matrix work is bounded by how scattered the hits
// are along the sorted target order.  Sums are kept in fp32 across all offsets
// in ascending offset order and rounded once, after the epilogue.
//
// Rows wider than one step of K (128 bytes) are walked in chunks: the
// pipeline's unit is then an (offset, chunk) pair instead of an offset.  More
// than 128 output channels are split into groups of 128 over blockIdx.y, each
// group reading the source rows again (through L2).
//
// Compared with the three-kernel form this trades HBM traffic (no buffer rows
// written and read back) for matrix work on empty rows; the host entry point
// leaves the choice to the caller.
#include <algorithm>

#include "conv_device.h"
#include "device_utils.h"

namespace mnt {

constexpr int kImplicitBlock = 256;
constexpr int kImplicitTargets = 128;     // per workgroup, 32 per wavefront
constexpr int kImplicitMaxBlocks = 4;     // 32-channel output blocks per channel group (128 channels)
constexpr int kImplicitMaxGroups = 4;     // channel groups (512 channels)
constexpr int kImplicitMaxRowBytes = 2048;
constexpr int64_t kImplicitWideTargets = 1 << 19;   // from here on: two target blocks per wavefront

// wt: packed weights [O][rows][Kp] (W^T, K-contiguous, rows = output channels
// padded to a multiple of 32, Kp = K padded to a multiple of 128 bytes; see
// pack_weights_kernel).  Requires K % (16 / sizeof(T)) == 0 and N % 4 == 0.
// Register sets of the pipeline: 16-byte pieces of one thread's share of a
// weight tile, and of one lane's source row.
template <int N>
struct Pieces {
  uint4 v[N];
};

template <int N>
struct Pieces2 {
  int v[N];
};

typedef unsigned uint4v __attribute__((ext_vector_type(4)));

// Source tensors stay below this many bytes: rows are addressed through 32-bit
// buffer offsets.
constexpr unsigned kMaxSourceBytes = 0xFFFFF000u;

// One output row's worth of epilogue and store: four consecutive channels of
// target t held by this lane.
template <typename T>
__device__ __forceinline__ void finish_four(float (&v)[4], const Epilogue &ep, long long t, int ch, int N,
                                            unsigned char *__restrict__ out) {
  typedef typename VecOf<4 * sizeof(T)>::type V;
  if (ep.scale != nullptr) {
#pragma unroll
    for (int x = 0; x < 4; ++x) v[x] *= ep.scale[ch + x];
  }
  if (ep.shift != nullptr) {
#pragma unroll
    for (int x = 0; x < 4; ++x) v[x] += ep.shift[ch + x];
  }
  if (ep.residual != nullptr) {
    const V raw = *reinterpret_cast<const V *>(static_cast<const unsigned char *>(ep.residual) +
                                               (t * N + ch) * static_cast<long long>(sizeof(T)));
    const T *e = reinterpret_cast<const T *>(&raw);
#pragma unroll
    for (int x = 0; x < 4; ++x) v[x] += to_float(e[x]);
  }
  if (ep.activation == MNT_ACT_RELU) {
#pragma unroll
    for (int x = 0; x < 4; ++x) v[x] = fmaxf(v[x], 0.0f);
  } else if (ep.activation == MNT_ACT_LEAKY_RELU) {
#pragma unroll
    for (int x = 0; x < 4; ++x) v[x] = v[x] > 0.0f ? v[x] : v[x] * ep.slope;
  } else if (ep.activation == MNT_ACT_RELU6) {
#pragma unroll
    for (int x = 0; x < 4; ++x) v[x] = fminf(fmaxf(v[x], 0.0f), 6.0f);
  }
  V raw;
  T *e = reinterpret_cast<T *>(&raw);
#pragma unroll
  for (int x = 0; x < 4; ++x) e[x] = static_cast<T>(v[x]);
  *reinterpret_cast<V *>(out + (t * N + ch) * static_cast<long long>(sizeof(T))) = raw;
}

// The same for one 16-byte piece of an output row (E = 16 / sizeof(T)
// consecutive channels from `ch` on), its sums given in fp32.
template <typename T, int E>
__device__ __forceinline__ void finish_piece(float (&v)[E], const Epilogue &ep, long long t, int ch, int N,
                                             unsigned char *__restrict__ out) {
  if (ep.scale != nullptr) {
#pragma unroll
    for (int x = 0; x < E; ++x) v[x] *= ep.scale[ch + x];
  }
  if (ep.shift != nullptr) {
#pragma unroll
    for (int x = 0; x < E; ++x) v[x] += ep.shift[ch + x];
  }
  if (ep.residual != nullptr) {
    const uint4 raw = *reinterpret_cast<const uint4 *>(static_cast<const unsigned char *>(ep.residual) +
                                                       (t * N + ch) * static_cast<long long>(sizeof(T)));
    const T *e = reinterpret_cast<const T *>(&raw);
#pragma unroll
    for (int x = 0; x < E; ++x) v[x] += to_float(e[x]);
  }
  if (ep.activation == MNT_ACT_RELU) {
#pragma unroll
    for (int x = 0; x < E; ++x) v[x] = fmaxf(v[x], 0.0f);
  } else if (ep.activation == MNT_ACT_LEAKY_RELU) {
#pragma unroll
    for (int x = 0; x < E; ++x) v[x] = v[x] > 0.0f ? v[x] : v[x] * ep.slope;
  } else if (ep.activation == MNT_ACT_RELU6) {
#pragma unroll
    for (int x = 0; x < E; ++x) v[x] = fminf(fmaxf(v[x], 0.0f), 6.0f);
  }
  uint4 raw;
  T *e = reinterpret_cast<T *>(&raw);
#pragma unroll
  for (int x = 0; x < E; ++x) e[x] = static_cast<T>(v[x]);
  *reinterpret_cast<uint4 *>(out + (t * N + ch) * static_cast<long long>(sizeof(T))) = raw;
}

// Epilogue and store of one 32 x 32 block of fp32 sums as the matrix
// instructions leave it (lane (r, h) holds channels q * 8 + h * 4 .. + 3 of
// target block_t0 + r in acc[q * 4 .. + 3]), for output rows that are whole
// 16-byte pieces: the wavefront turns the block around in its own `turn` area
// of LDS (kTurnBytes), so that one store instruction covers rows in contiguous
// pieces of 64 bytes (128 in fp32), and the residual is read the same way.
constexpr int kTurnRow = 32 * 4 + 16;
constexpr int kTurnBytes = 32 * kTurnRow;

template <typename T>
__device__ __forceinline__ void store_turned_block(const floatx16 &acc, unsigned char *turn, int lane, int r,
                                                   int h, long long block_t0, long long num_targets, int ch0,
                                                   int N, const Epilogue &ep, unsigned char *__restrict__ out) {
  constexpr int EPV = 16 / static_cast<int>(sizeof(T));
  constexpr int kOutPieces = 32 / EPV;                          // 16-byte pieces of a block's output row
  constexpr int kPieces = 32 * kOutPieces / 64;                 // per lane
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    *reinterpret_cast<float4 *>(turn + r * kTurnRow + (q * 8 + h * 4) * 4) =
        make_float4(acc[q * 4], acc[q * 4 + 1], acc[q * 4 + 2], acc[q * 4 + 3]);
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
  for (int i = 0; i < kPieces; ++i) {
    const int piece = lane + i * 64;
    const int pr = piece / kOutPieces, part = piece % kOutPieces;
    const int ch = ch0 + part * EPV;
    float v[EPV];
#pragma unroll
    for (int x = 0; x < EPV; x += 4) {
      const float4 f = *reinterpret_cast<const float4 *>(turn + pr * kTurnRow + (part * EPV + x) * 4);
      v[x] = f.x;
      v[x + 1] = f.y;
      v[x + 2] = f.z;
      v[x + 3] = f.w;
    }
    if (block_t0 + pr < num_targets && ch < N) {                // N % EPV == 0: a piece is all in or all out
      finish_piece<T, EPV>(v, ep, block_t0 + pr, ch, N, out);
    }
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// KS: 32-byte steps of K per pipeline stage.  A source row takes `chunks`
// stages of KS * 32 bytes (Kp * sizeof(T) must be a multiple of that when
// chunks > 1).  packed_row = Kp, packed_rows = rows of one offset in wt.
// MW: 32-target blocks per wavefront.  With MW = 2 a wavefront owns 64 targets
// and a workgroup 256: every weight fragment read from LDS feeds two matrix
// operations and the weight tiles are staged half as often per target, at the
// price of twice the accumulators and source-row registers.
// PLAIN: a source row is exactly one stage (no chunks, no ragged end), which
// spares the hot loop the chunk bookkeeping and the end-of-row tests.
template <typename T, int NB, int KS, int MW, bool PLAIN>
__device__ __forceinline__ void implicit_forward_body(
    const T *__restrict__ sources, unsigned source_bytes, const T *__restrict__ wt,
    const int *__restrict__ kernel_map, long long num_targets, int num_offsets, int K, int N,
    int chunks, int packed_row, int packed_rows, unsigned char *__restrict__ out, const Epilogue &ep) {
  constexpr int EPC = 16 / static_cast<int>(sizeof(T));
  constexpr int kSteps = KS;
  constexpr int Np = NB * 32;
  constexpr int kStageBytes = KS * 32;                   // bytes of K per stage
  constexpr int kStageElems = kStageBytes / static_cast<int>(sizeof(T));
  constexpr int kRowPieces = 2 * KS;                     // 16-byte pieces of a weight row per stage
  constexpr int kWPieces = (Np * kRowPieces + kImplicitBlock - 1) / kImplicitBlock;
  // LDS rows of staged weights are padded by 16 bytes against bank conflicts
  constexpr int kLdsRow = kStageBytes + 16;
  constexpr int kBufferBytes = Np * kLdsRow;
  // the output pass turns one 32 x 32 block of fp32 sums per wavefront around in the same memory
  constexpr int kLdsBytes = 2 * kBufferBytes > 4 * kTurnBytes ? 2 * kBufferBytes : 4 * kTurnBytes;
  __shared__ __align__(16) unsigned char w_lds[kLdsBytes];
  const int num_stages = num_offsets * chunks;
  const int first_channel = blockIdx.y * Np;             // channel group of this workgroup

  // (Workgroup -> tile mappings that keep neighbouring tiles on one XCD were
  // measured: contiguous runs per XCD 14 % slower, runs of 8 no change; the
  // rows that tiles share are served by the memory-side cache either way.)
  const long long tile = blockIdx.x;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wv = tid >> 6;
  const int r = lane & 31;
  const int h = lane >> 5;
  long long t[MW], t_safe[MW];
  bool t_ok[MW];
#pragma unroll
  for (int m = 0; m < MW; ++m) {
    t[m] = tile * (kImplicitTargets * MW) + (wv * MW + m) * 32 + r;
    t_ok[m] = t[m] < num_targets;
    t_safe[m] = t_ok[m] ? t[m] : num_targets - 1;
  }

  floatx16 acc[MW][NB];
#pragma unroll
  for (int m = 0; m < MW; ++m) {
#pragma unroll
    for (int b = 0; b < NB; ++b) {
#pragma unroll
      for (int j = 0; j < 16; ++j) acc[m][b][j] = 0.0f;
    }
  }

  // No load below waits for an earlier one's result in its own stage: stage
  // addresses are clamped to the last stage, and a source row's load is masked
  // by a kernel-map entry that was read stages before, so that the loads of
  // later stages never have to be waited for early.
  //
  // Stage s belongs to offset s / chunks and covers chunk s % chunks of the
  // rows.  A stage is a few matrix instructions, so the integer work around
  // them decides the speed: the three load streams walk the stages with
  // running pointers (one step per stage, no multiplication or division), and
  // everything that depends on the lane only is worked out once.  Past the last
  // stage a cursor stays on it and only its count runs on.
  const long long offset_stride = static_cast<long long>(packed_rows) * packed_row * sizeof(T);
  struct Cursor {
    int s, chunk;
    const int *map_row;
    const unsigned char *weights;
  };
  auto next = [&](Cursor c) -> Cursor {
    ++c.s;
    if (c.s < num_stages) {
      if (PLAIN) {
        c.map_row += num_targets;
        c.weights += offset_stride;
      } else if (++c.chunk == chunks) {
        c.chunk = 0;
        c.map_row += num_targets;
        c.weights += offset_stride - static_cast<long long>(chunks - 1) * kStageBytes;
      } else {
        c.weights += kStageBytes;
      }
    }
    return c;
  };
  unsigned map_at[MW];
#pragma unroll
  for (int m = 0; m < MW; ++m) map_at[m] = static_cast<unsigned>(t_safe[m]);
  auto load_index = [&](const Cursor &c) -> Pieces2<MW> {
    Pieces2<MW> set;
#pragma unroll
    for (int m = 0; m < MW; ++m) set.v[m] = c.map_row[map_at[m]];
    return set;
  };
  // piece i of this thread: 16 bytes of weight row (piece / kRowPieces) at
  // position (piece % kRowPieces); threads past the tile repeat its last piece
  unsigned w_at[kWPieces];
#pragma unroll
  for (int i = 0; i < kWPieces; ++i) {
    const int piece = min(tid + i * kImplicitBlock, Np * kRowPieces - 1);
    // a narrower last channel group repeats the last packed row (its outputs are never stored)
    const int row = min(piece / kRowPieces, packed_rows - 1 - first_channel);
    w_at[i] = static_cast<unsigned>((row * packed_row + (piece % kRowPieces) * EPC) * static_cast<int>(sizeof(T)));
  }
  auto load_w = [&](const Cursor &c) -> Pieces<kWPieces> {
    Pieces<kWPieces> set;
#pragma unroll
    for (int i = 0; i < kWPieces; ++i) set.v[i] = *reinterpret_cast<const uint4 *>(c.weights + w_at[i]);
    return set;
  };
  unsigned w_put[kWPieces];
#pragma unroll
  for (int i = 0; i < kWPieces; ++i) {
    const int piece = min(tid + i * kImplicitBlock, Np * kRowPieces - 1);
    w_put[i] = static_cast<unsigned>((piece / kRowPieces) * kLdsRow + (piece % kRowPieces) * 16);
  }
  auto store_w = [&](int buffer, const Pieces<kWPieces> &set) {
#pragma unroll
    for (int i = 0; i < kWPieces; ++i) {
      *reinterpret_cast<uint4 *>(w_lds + buffer * kBufferBytes + w_put[i]) = set.v[i];
    }
  };
  // Source rows come through a buffer resource (32-bit offsets, a scalar part
  // for what all lanes share).
  const __amdgpu_buffer_rsrc_t source_buffer = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<T *>(sources), 0, source_bytes, 0x00020000);
  const unsigned row_bytes = static_cast<unsigned>(K) * sizeof(T);
  auto load_a = [&](const Pieces2<MW> &indices, const Cursor &c) -> Pieces<KS * MW> {
    Pieces<KS * MW> set;
    const bool live = c.s < num_stages;
    const unsigned chunk_at = PLAIN ? 0u : static_cast<unsigned>(c.chunk) * kStageBytes;
#pragma unroll
    for (int m = 0; m < MW; ++m) {
      const int index = (t_ok[m] && live) ? indices.v[m] : -1;
      const unsigned row_at = static_cast<unsigned>(index) * row_bytes + h * 16u;
#pragma unroll
      for (int kk = 0; kk < kSteps; ++kk) {
        // Lanes without a source, and pieces past the end of a ragged row, sit
        // the load out and keep zeros (a lane that loads out of range still
        // takes its turn in the address unit: 7 to 10 % of a layer at 200k
        // voxels).  The step's place in the row is the same for all lanes: it
        // rides in the scalar offset.
        const bool take = index >= 0 && (PLAIN || chunk_at + (kk * 2 + h) * 16u < row_bytes);
        uint4v v = {0u, 0u, 0u, 0u};
        if (take) v = __builtin_amdgcn_raw_buffer_load_b128(source_buffer, row_at, chunk_at + kk * 32u, 0);
        set.v[m * KS + kk] = make_uint4(v.x, v.y, v.z, v.w);
      }
    }
    return set;
  };

  // Software pipeline over the stages (offsets, or chunks of offsets): while
  // stage o is multiplied, the source rows of stage o+2 and the weights of
  // stage o+3 are already on their way, and kernel-map entries are read five
  // stages ahead.  The loop
  // is unrolled by six so that the roles of the register sets (three sets of
  // source rows, three of weights, six kernel-map entries) rotate without
  // copies: a register is never touched while its load is in flight.
  const Cursor c0 = {0, 0, kernel_map,
                     reinterpret_cast<const unsigned char *>(wt + static_cast<long long>(first_channel) * packed_row)};
  const Cursor c1 = next(c0), c2 = next(c1), c3 = next(c2), c4 = next(c3);
  Pieces2<MW> m0 = load_index(c0), m1 = load_index(c1), m2 = load_index(c2), m3 = load_index(c3),
              m4 = load_index(c4), m5 = m4;
  Pieces<KS * MW> a0, a1, a2;
  Pieces<kWPieces> w0, w1, w2;
  w2 = load_w(c0);
  a0 = load_a(m0, c0);
  w0 = load_w(c1);
  a1 = load_a(m1, c1);
  w1 = load_w(c2);
  store_w(0, w2);
  __syncthreads();
  Cursor at_a = c2, at_w = c3, at_m = next(c4);      // stages o + 2, o + 3 and o + 5
  const unsigned w_get = static_cast<unsigned>(r * kLdsRow + h * 16);

  int o = 0;
  // offset o: multiply A_CUR (rows of M_CUR) by the weights in LDS buffer BUF
  // (= o & 1); fetch rows of offset o+2 (entries M_A) into A_NEW, weights of
  // offset o+3 into W_NEW and the kernel-map entries of offset o+5 into M_NEW;
  // put the weights of offset o+1 (W_STORE) into the other LDS buffer.
#define MNT_STAGE(A_CUR, A_NEW, W_STORE, W_NEW, M_CUR, M_A, M_NEW, BUF)                            \
  {                                                                                                \
    W_NEW = load_w(at_w);                                                                          \
    A_NEW = load_a(M_A, at_a);                                                                     \
    M_NEW = load_index(at_m);                                                                      \
    at_w = next(at_w);                                                                             \
    at_a = next(at_a);                                                                             \
    at_m = next(at_m);                                                                             \
    bool live[MW];                                                                                 \
    bool any = false;                                                                              \
    _Pragma("unroll") for (int m = 0; m < MW; ++m) {                                               \
      live[m] = __ballot(t_ok[m] && M_CUR.v[m] >= 0) != 0ull;                                      \
      any = any || live[m];                                                                        \
    }                                                                                              \
    if (any) {                                                                                     \
      const unsigned char *w_buf = w_lds + (BUF) * kBufferBytes + w_get;                           \
      _Pragma("unroll") for (int kk = 0; kk < kSteps; ++kk) {                                      \
        _Pragma("unroll") for (int b = 0; b < NB; ++b) {                                           \
          const uint4 chan = *reinterpret_cast<const uint4 *>(w_buf + b * 32 * kLdsRow + kk * 32); \
          _Pragma("unroll") for (int m = 0; m < MW; ++m) {                                         \
            if (MW == 1 || live[m]) acc[m][b] = Mfma<T>::run(chan, A_CUR.v[m * KS + kk], acc[m][b]); \
          }                                                                                        \
        }                                                                                          \
      }                                                                                            \
    }                                                                                              \
    store_w(1 - (BUF), W_STORE);                                                                   \
    __syncthreads();                                                                               \
    if (++o == num_stages) break;                                                                  \
  }
  while (true) {
    MNT_STAGE(a0, a2, w0, w2, m0, m2, m5, 0)
    MNT_STAGE(a1, a0, w1, w0, m1, m3, m0, 1)
    MNT_STAGE(a2, a1, w2, w1, m2, m4, m1, 0)
    MNT_STAGE(a0, a2, w0, w2, m3, m5, m2, 1)
    MNT_STAGE(a1, a0, w1, w0, m4, m0, m3, 0)
    MNT_STAGE(a2, a1, w2, w1, m5, m1, m4, 1)
  }
#undef MNT_STAGE

  // Output.  A lane holds 4 consecutive channels of one target per accumulator
  // group and neighbouring lanes hold different targets: written as they are,
  // every lane's few bytes are a request of their own.  Where output rows are
  // whole 16-byte pieces each wavefront turns its 32 x 32 blocks around in LDS
  // (free after the last stage's barrier), so that one store instruction
  // covers rows in contiguous pieces of 64 bytes (128 in fp32), and the
  // residual is read the same way.
  if ((static_cast<long long>(N) * sizeof(T)) % 16 == 0) {
    unsigned char *turn = w_lds + wv * kTurnBytes;
#pragma unroll
    for (int m = 0; m < MW; ++m) {
      const long long block_t0 = tile * (kImplicitTargets * MW) + (wv * MW + m) * 32;
      if (block_t0 >= num_targets) break;
#pragma unroll
      for (int b = 0; b < NB; ++b) {
        if (first_channel + b * 32 >= N) break;
        store_turned_block<T>(acc[m][b], turn, lane, r, h, block_t0, num_targets, first_channel + b * 32, N, ep, out);
      }
    }
    return;
  }
#pragma unroll
  for (int m = 0; m < MW; ++m) {
    if (!t_ok[m]) continue;
#pragma unroll
    for (int b = 0; b < NB; ++b) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int ch = first_channel + b * 32 + q * 8 + h * 4;
        if (ch >= N) continue;               // N % 4 == 0: a group of four is all in or all out
        float v[4];
#pragma unroll
        for (int x = 0; x < 4; ++x) v[x] = acc[m][b][q * 4 + x];
        finish_four<T>(v, ep, t[m], ch, N, out);
      }
    }
  }
}

template <typename T, int NB, int KS, int MW, bool PLAIN>
__global__ __launch_bounds__(kImplicitBlock) void implicit_forward_kernel(
    const T *__restrict__ sources, unsigned source_bytes, const T *__restrict__ wt,
    const int *__restrict__ kernel_map, long long num_targets, int num_offsets, int K, int N,
    int chunks, int packed_row, int packed_rows, unsigned char *__restrict__ out, Epilogue ep) {
  implicit_forward_body<T, NB, KS, MW, PLAIN>(sources, source_bytes, wt, kernel_map, num_targets, num_offsets, K, N,
                                       chunks, packed_row, packed_rows, out, ep);
}

// Forward of a layer whose source rows are 4, 8 or 16 bytes of a 16-bit type
// (a stem: 2, 4 or 8 input channels).  A pipeline stage per offset would be
// all overhead for rows that short, so the offsets lie side by side along K
// instead: K' = O * K, 16 elements per matrix instruction, and a lane's
// 16-byte operand piece is 4, 2 or 1 whole source rows of consecutive offsets.
// The weights [O][K][N], read as [O * K][N], are already the matrix to
// multiply by: a workgroup puts them into LDS once, in operand order (piece
// (step, channel block, lane) = 8 elements of K' for one output channel), and
// each wavefront takes its blocks of 32 targets from there.  Nothing is
// pipelined by hand: the kernel is short on registers, and the wavefronts a
// SIMD holds cover each other's trips to memory.
// Dynamic LDS: steps * NB KiB of weight pieces + 4 turn areas.
constexpr int kNarrowBlock = 256;
constexpr int kNarrowBlocksPerWave = 2;    // 32-target blocks a wavefront takes
constexpr int kNarrowSteps = 8;            // steps of K' whose rows are in flight together
constexpr int kNarrowMaxLds = 64 * 1024;

// Whether narrow_forward_kernel takes the layer: 16-bit rows of 4, 8 or 16
// bytes, at most 128 output channels, weights given as they are, and all of
// them in LDS at once.
static bool narrow_fits(int64_t O, int64_t K, int64_t N, int esize, bool has_weights) {
  const int64_t row_bytes = K * esize;
  if (esize != 2 || (row_bytes != 4 && row_bytes != 8 && row_bytes != 16) || !has_weights ||
      N > 32 * kImplicitMaxBlocks) {
    return false;
  }
  const int64_t lds = div_ceil(O * K, 16) * div_ceil(N, 32) * 1024 + (kNarrowBlock / 64) * kTurnBytes;
  return lds <= kNarrowMaxLds;
}

template <typename T, int NB, int RB>
__global__ __launch_bounds__(kNarrowBlock, NB == 1 ? 4 : 2) void narrow_forward_kernel(
    const unsigned char *__restrict__ sources, const T *__restrict__ weights,
    const int *__restrict__ kernel_map, long long num_targets, int num_offsets, int N, int steps,
    unsigned char *__restrict__ out, Epilogue ep) {
  constexpr int SL = 16 / RB;                                   // source rows per operand piece
  constexpr int KR = RB / static_cast<int>(sizeof(T));          // input channels
  typedef typename VecOf<RB>::type RowVec;
  extern __shared__ __align__(16) unsigned char narrow_lds[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wv = tid >> 6;
  const int r = lane & 31;
  const int h = lane >> 5;
  {
    // a thread gathers whole pieces: eight loads in flight, then one LDS store
    const int total_k = num_offsets * KR;
    const int count = steps * NB * 64;
    for (int p = tid; p < count; p += kNarrowBlock) {
      const int ln = p & 63, sb = p >> 6;
      const int b = sb % NB, s = sb / NB;
      const int k0 = 16 * s + 8 * (ln >> 5);
      const int n = b * 32 + (ln & 31);
      T e[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        e[i] = (k0 + i < total_k && n < N) ? weights[static_cast<long long>(k0 + i) * N + n] : static_cast<T>(0.0f);
      }
      reinterpret_cast<uint4 *>(narrow_lds)[p] = *reinterpret_cast<const uint4 *>(e);
    }
  }
  __syncthreads();
  const uint4 *w_pieces = reinterpret_cast<const uint4 *>(narrow_lds) + lane;
  unsigned char *turn = narrow_lds + static_cast<size_t>(steps) * NB * 1024 + wv * kTurnBytes;
  const bool turned = (static_cast<long long>(N) * sizeof(T)) % 16 == 0;
  for (int j = 0; j < kNarrowBlocksPerWave; ++j) {
    const long long block_t0 =
        ((static_cast<long long>(blockIdx.x) * kNarrowBlocksPerWave + j) * (kNarrowBlock / 64) + wv) * 32;
    if (block_t0 >= num_targets) break;
    const long long t = block_t0 + r;
    const bool t_ok = t < num_targets;
    const int *column = kernel_map + (t_ok ? t : num_targets - 1);
    floatx16 acc[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) {
#pragma unroll
      for (int x = 0; x < 16; ++x) acc[b][x] = 0.0f;
    }
    for (int s0 = 0; s0 < steps; s0 += kNarrowSteps) {
      int index[kNarrowSteps][SL];
#pragma unroll
      for (int g = 0; g < kNarrowSteps; ++g) {
#pragma unroll
        for (int q = 0; q < SL; ++q) {
          const int o = (2 * (s0 + g) + h) * SL + q;
          index[g][q] = (t_ok && o < num_offsets) ? column[static_cast<long long>(o) * num_targets] : -1;
        }
      }
      uint4 piece[kNarrowSteps];
#pragma unroll
      for (int g = 0; g < kNarrowSteps; ++g) {
        RowVec rows[SL];
#pragma unroll
        for (int q = 0; q < SL; ++q) {
          rows[q] = RowVec{};
          if (index[g][q] >= 0) {
            rows[q] = *reinterpret_cast<const RowVec *>(sources + static_cast<long long>(index[g][q]) * RB);
          }
        }
        piece[g] = *reinterpret_cast<const uint4 *>(rows);
      }
#pragma unroll
      for (int g = 0; g < kNarrowSteps; ++g) {
        if (s0 + g < steps) {
#pragma unroll
          for (int b = 0; b < NB; ++b) {
            acc[b] = Mfma<T>::run(w_pieces[((s0 + g) * NB + b) * 64], piece[g], acc[b]);
          }
        }
      }
    }
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      if (b * 32 >= N) break;
      if (turned) {
        store_turned_block<T>(acc[b], turn, lane, r, h, block_t0, num_targets, b * 32, N, ep, out);
      } else if (t_ok) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int ch = b * 32 + q * 8 + h * 4;
          if (ch >= N) continue;               // N % 4 == 0: a group of four is all in or all out
          float v[4];
#pragma unroll
          for (int x = 0; x < 4; ++x) v[x] = acc[b][q * 4 + x];
          finish_four<T>(v, ep, t, ch, N, out);
        }
      }
    }
  }
}

// inverse[o][m] = t for every hit kernel_map[o][t] = m (at most one t per
// (o, m): the targets of one offset are distinct translates of their sources).
__global__ __launch_bounds__(256) void invert_map_kernel(const int *__restrict__ kernel_map,
                                                         long long num_targets,
                                                         long long num_sources, long long total,
                                                         int *__restrict__ inverse) {
  const long long stride = static_cast<long long>(gridDim.x) * blockDim.x;
  for (long long i = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x; i < total; i += stride) {
    const int m = kernel_map[i];
    if (m >= 0) {
      const long long o = i / num_targets;
      inverse[o * num_sources + m] = static_cast<int>(i - o * num_targets);
    }
  }
}

__global__ __launch_bounds__(256) void fill_minus_one_kernel(int *__restrict__ data, long long n) {
  const long long stride = static_cast<long long>(gridDim.x) * blockDim.x;
  for (long long i = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += stride) {
    data[i] = -1;
  }
}

template <typename T>
static void implicit_typed(const T *sources, const T *weights, const T *packed, const int *kernel_map,
                           int64_t S, int64_t Tn, int64_t O, int64_t K, int64_t N, const Epilogue &ep,
                           T *out, hipStream_t stream) {
  Scope scope(stream);
  profile_mark("enter:implicit", stream);
  if constexpr (sizeof(T) == 2) {
    if (narrow_fits(O, K, N, sizeof(T), weights != nullptr)) {
      {
        const int64_t narrow_bytes = K * static_cast<int64_t>(sizeof(T));
        const int steps = static_cast<int>(div_ceil(O * K, 16));
        const int blocks = static_cast<int>(div_ceil(N, 32));
        const size_t lds = static_cast<size_t>(steps) * blocks * 1024 + (kNarrowBlock / 64) * kTurnBytes;
        const unsigned grid = static_cast<unsigned>(
            div_ceil(Tn, int64_t{32} * (kNarrowBlock / 64) * kNarrowBlocksPerWave));
#define MNT_NARROW(NB, RB)                                                                              \
  narrow_forward_kernel<T, NB, RB><<<grid, kNarrowBlock, lds, stream>>>(                                \
      reinterpret_cast<const unsigned char *>(sources), weights, kernel_map, Tn, static_cast<int>(O),   \
      static_cast<int>(N), steps, reinterpret_cast<unsigned char *>(out), ep)
#define MNT_NARROW_RB(NB)            \
  if (narrow_bytes == 4) {           \
    MNT_NARROW(NB, 4);               \
  } else if (narrow_bytes == 8) {    \
    MNT_NARROW(NB, 8);               \
  } else {                           \
    MNT_NARROW(NB, 16);              \
  }
        switch (blocks) {
          case 1: MNT_NARROW_RB(1); break;
          case 2: MNT_NARROW_RB(2); break;
          case 3: MNT_NARROW_RB(3); break;
          default: MNT_NARROW_RB(4); break;
        }
#undef MNT_NARROW_RB
#undef MNT_NARROW
        check_launch("narrow_forward_kernel");
        profile_mark("implicit", stream);
        return;
      }
    }
  }
  const int kc = kChunkBytes / static_cast<int>(sizeof(T));
  const int Kp = static_cast<int>(div_ceil(K, kc) * kc);
  const int Np = static_cast<int>(div_ceil(N, 32) * 32);
  const T *wt = packed;
  if (packed == nullptr) {
    T *fresh = scope.alloc<T>(static_cast<size_t>(O) * Np * Kp);
    wt = fresh;
    const long long total = static_cast<long long>(O) * Np * Kp;
    pack_weights_kernel<T, int32_t><<<grid_for(total, 256, 4096), 256, 0, stream>>>(
        weights, nullptr, static_cast<int>(O), static_cast<int>(K), static_cast<int>(N), Kp, Np, fresh,
        PlanChunk{}, 0, nullptr);
    check_launch("pack_weights_kernel");
    profile_mark("pack_weights", stream);
  }
  const unsigned source_bytes = static_cast<unsigned>(S * K * sizeof(T));
  // stage width: 64 bytes for rows up to that, else 128; wider rows go in
  // chunks of 128 bytes (stages of 256 measured two to three times slower:
  // their registers leave one wavefront per SIMD)
  const int row_bytes = Kp * static_cast<int>(sizeof(T));
  const int stage_bytes = K * sizeof(T) <= 64 ? 64 : 128;
  const int chunks = row_bytes <= 128 ? 1 : row_bytes / stage_bytes;
  // channel groups of up to 128 channels; the last group may be narrower
  const int groups = static_cast<int>(div_ceil(Np, 32 * kImplicitMaxBlocks));
  const int blocks = groups > 1 ? kImplicitMaxBlocks : Np / 32;
  // Two target blocks per wavefront where that measured faster: 16-bit
  // features, 33..64 output channels, rows of one stage, and clouds from half
  // a million targets on (0.93 against 0.98 ms at a million targets and 125
  // offsets; at 200 000 targets one block per wavefront is the faster one,
  // 57 against 61 us).
  const bool wide = sizeof(T) == 2 && Np == 64 && chunks == 1 && stage_bytes <= 128 && Tn >= kImplicitWideTargets;
  const dim3 grid(static_cast<unsigned>(div_ceil(Tn, kImplicitTargets * (wide ? 2 : 1))),
                  static_cast<unsigned>(groups));
  const bool plain = chunks == 1 && K * static_cast<int64_t>(sizeof(T)) == stage_bytes;
#define MNT_IMPLICIT(NB, KS, MW)                                                                   \
  if (plain) {                                                                                     \
    implicit_forward_kernel<T, NB, KS, MW, true><<<grid, kImplicitBlock, 0, stream>>>(             \
        sources, source_bytes, wt, kernel_map, Tn, static_cast<int>(O), static_cast<int>(K),       \
        static_cast<int>(N), chunks, Kp, Np, reinterpret_cast<unsigned char *>(out), ep);          \
  } else {                                                                                         \
    implicit_forward_kernel<T, NB, KS, MW, false><<<grid, kImplicitBlock, 0, stream>>>(            \
        sources, source_bytes, wt, kernel_map, Tn, static_cast<int>(O), static_cast<int>(K),       \
        static_cast<int>(N), chunks, Kp, Np, reinterpret_cast<unsigned char *>(out), ep);          \
  }
#define MNT_IMPLICIT_KS(NB, MW)           \
  if (stage_bytes == 64) {                \
    MNT_IMPLICIT(NB, 2, MW);              \
  } else {                                \
    MNT_IMPLICIT(NB, 4, MW);              \
  }
  switch (blocks) {
    case 1: MNT_IMPLICIT_KS(1, 1); break;
    case 2:
      if (wide) {
        MNT_IMPLICIT_KS(2, 2);
      } else {
        MNT_IMPLICIT_KS(2, 1);
      }
      break;
    case 3: MNT_IMPLICIT_KS(3, 1); break;
    default: MNT_IMPLICIT_KS(4, 1); break;
  }
#undef MNT_IMPLICIT_KS
#undef MNT_IMPLICIT
  check_launch("implicit_forward_kernel");
  profile_mark("implicit", stream);
}

}  // namespace mnt

using namespace mnt;

extern "C" int mnt_sparse_convolution_forward_implicit(
    const void *sources, const void *weights, const int32_t *kernel_map, int64_t S, int64_t T,
    int64_t O, int64_t K, int64_t N, int float_dtype, const float *channel_scale,
    const float *channel_shift, const void *residual, int activation, float negative_slope,
    const void *packed_weights, void *out, void *stream_) {
  return guarded([&] {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const int esize = float_size(float_dtype);
    MNT_CHECK(S >= 0 && T >= 0 && O >= 1 && K >= 1 && N >= 1 && S <= INT32_MAX && T <= INT32_MAX &&
                  O <= 65535,
              "bad shape S=%lld T=%lld O=%lld Cin=%lld Cout=%lld", (long long)S, (long long)T,
              (long long)O, (long long)K, (long long)N);
    MNT_CHECK(S * K * esize < static_cast<int64_t>(kMaxSourceBytes),
              "source features of %lld bytes exceed the 4 GiB a buffer resource addresses",
              (long long)(S * K * esize));
    const bool narrow = narrow_fits(O, K, N, esize, weights != nullptr);
    MNT_CHECK(((K * esize) % 16 == 0 || narrow) && K * esize <= kImplicitMaxRowBytes && N % 4 == 0 &&
                  N <= 32 * kImplicitMaxBlocks * kImplicitMaxGroups,
              "Unsupported channel counts for the implicit forward: Cin = %lld (rows must be a multiple "
              "of 16 bytes, at most %d; 16-bit rows of 4 or 8 bytes are taken too where weights are given "
              "unpacked, Cout is at most 128 and the kernel is small), Cout = %lld (a multiple of 4, at most %d)",
              (long long)K, kImplicitMaxRowBytes, (long long)N, 32 * kImplicitMaxBlocks * kImplicitMaxGroups);
    MNT_CHECK(activation >= MNT_ACT_NONE && activation <= MNT_ACT_RELU6, "unknown activation code %d",
              activation);
    MNT_CHECK(reinterpret_cast<uintptr_t>(sources) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0 &&
                  reinterpret_cast<uintptr_t>(residual) % 16 == 0 &&
                  reinterpret_cast<uintptr_t>(channel_scale) % 4 == 0 &&
                  reinterpret_cast<uintptr_t>(channel_shift) % 4 == 0,
              "operands are not aligned (features, out, residual: 16 bytes, scale / shift: 4 bytes)");
    if (T == 0) return;
    MNT_CHECK(out != nullptr && kernel_map != nullptr && (weights != nullptr || packed_weights != nullptr),
              "null operand");
    MNT_CHECK(reinterpret_cast<uintptr_t>(packed_weights) % 16 == 0, "packed weights are not 16-byte aligned");
    const Epilogue ep = {channel_scale, channel_shift, residual, activation, negative_slope};
    if (float_dtype == MNT_FLOAT32) {
      implicit_typed<float>(static_cast<const float *>(sources), static_cast<const float *>(weights),
                            static_cast<const float *>(packed_weights), kernel_map, S, T, O, K, N, ep, static_cast<float *>(out), stream);
    } else if (float_dtype == MNT_FLOAT16) {
      implicit_typed<half_t>(static_cast<const half_t *>(sources), static_cast<const half_t *>(weights),
                             static_cast<const half_t *>(packed_weights), kernel_map, S, T, O, K, N, ep, static_cast<half_t *>(out), stream);
    } else {
      implicit_typed<bf16_t>(static_cast<const bf16_t *>(sources), static_cast<const bf16_t *>(weights),
                             static_cast<const bf16_t *>(packed_weights), kernel_map, S, T, O, K, N, ep, static_cast<bf16_t *>(out), stream);
    }
  });
}

extern "C" int mnt_kernel_map_invert(const int32_t *kernel_map, int64_t num_offsets,
                                     int64_t num_targets, int64_t num_sources,
                                     int32_t *inverse_out, void *stream_) {
  return guarded([&] {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    MNT_CHECK(num_offsets >= 0 && num_targets >= 0 && num_sources >= 0 && num_targets <= INT32_MAX &&
                  num_sources <= INT32_MAX,
              "bad shape O=%lld T=%lld S=%lld", (long long)num_offsets, (long long)num_targets,
              (long long)num_sources);
    const long long filled = num_offsets * num_sources;
    const long long total = num_offsets * num_targets;
    if (filled > 0) {
      MNT_CHECK(inverse_out != nullptr, "inverse_out is null");
      fill_minus_one_kernel<<<grid_for(filled, 256, 8192), 256, 0, stream>>>(inverse_out, filled);
      check_launch("fill_minus_one_kernel");
    }
    if (total > 0 && filled > 0) {
      MNT_CHECK(kernel_map != nullptr, "kernel_map is null");
      invert_map_kernel<<<grid_for(total, 256, 8192), 256, 0, stream>>>(kernel_map, num_targets, num_sources,
                                                                         total, inverse_out);
      check_launch("invert_map_kernel");
    }
  });
}
