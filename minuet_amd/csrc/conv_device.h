// Device-side pieces shared by the feature kernels (grouped GEMM, Scatter,
// the implicit-GEMM forward): element and vector types, the MFMA wrappers,
// the output epilogue and the weight packing kernel.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

#include "common.h"

namespace mnt {

typedef _Float16 half_t;
typedef __bf16 bf16_t;
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));


template <int VB>
struct VecOf;
template <>
struct VecOf<16> { typedef uint4 type; };
template <>
struct VecOf<8> { typedef uint2 type; };
template <>
struct VecOf<4> { typedef unsigned type; };
template <>
struct VecOf<2> { typedef unsigned short type; };


template <typename T>
__device__ __forceinline__ float to_float(T v) { return static_cast<float>(v); }

// What Scatter applies to a summed row before rounding it to the output type:
//   v = act(sum * scale[c] + shift[c] + residual[t][c])
// scale / shift are per-channel fp32 vectors, residual a [T, C] tensor of the
// output type; each is skipped when null.  An inference-mode BatchNorm folds
// into (scale, shift), a bias into shift, a skip connection into residual.
struct Epilogue {
  const float *scale;
  const float *shift;
  const void *residual;
  int activation;      // MNT_ACT_*
  float slope;         // LeakyReLU negative slope
  const float *range;  // see range_kernel: the buffer rows are scaled (null: they are not)
};


template <typename T>
struct Mfma;
template <>
struct Mfma<half_t> {
  __device__ static __forceinline__ floatx16 run(const uint4 &a, const uint4 &b, floatx16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(*reinterpret_cast<const half8 *>(&a),
                                                  *reinterpret_cast<const half8 *>(&b), c, 0, 0, 0);
  }
};
template <>
struct Mfma<bf16_t> {
  __device__ static __forceinline__ floatx16 run(const uint4 &a, const uint4 &b, floatx16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(*reinterpret_cast<const bf16x8 *>(&a),
                                                   *reinterpret_cast<const bf16x8 *>(&b), c, 0, 0, 0);
  }
};
template <>
struct Mfma<float> {
  __device__ static __forceinline__ floatx16 run(const uint4 &a, const uint4 &b, floatx16 c) {
    const float *fa = reinterpret_cast<const float *>(&a);
    const float *fb = reinterpret_cast<const float *>(&b);
#pragma unroll
    for (int i = 0; i < 4; ++i) c = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i], fb[i], c, 0, 0, 0);
    return c;
  }
};


// K is walked in chunks of 128 bytes per row; LDS rows of staged weights are
// padded by 16 bytes against bank conflicts.
constexpr int kChunkBytes = 128;        // bytes of K per row and step
constexpr int kLdsRowBytes = kChunkBytes + 16;

// --------------------------------------------------------- weight packing ----

// wt[j][n][k] = w[order[j]][k][n], zero-padded to [Np][Kp]: the K-contiguous,
// transposed form the GEMM stages into LDS.  Takes the place of PermuteWeights
// (csrc/minuet/cuda/kernels/permute_weights.cuh:8-36).  The same launch also
// carries the forward plan's small integer tables (row starts, GEMM group
// descriptors) to the device as a by-value argument, so that a forward pass
// needs no separate upload.
constexpr int kPlanInts = 512;
struct PlanChunk {
  int v[kPlanInts];
};

template <typename T, typename IT>
__global__ __launch_bounds__(256) void pack_weights_kernel(const T *__restrict__ w,
                                                           const IT *__restrict__ order,
                                                           int num_offsets, int K, int N, int Kp,
                                                           int Np, T *__restrict__ wt, PlanChunk plan,
                                                           int plan_count, int *__restrict__ plan_out) {
  if (blockIdx.x == 0) {
    for (int i = threadIdx.x; i < plan_count; i += blockDim.x) plan_out[i] = plan.v[i];
  }
  const long long total = static_cast<long long>(num_offsets) * Np * Kp;
  const long long stride = static_cast<long long>(gridDim.x) * blockDim.x;
  for (long long i = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x; i < total; i += stride) {
    const int k = static_cast<int>(i % Kp);
    const int n = static_cast<int>((i / Kp) % Np);
    const int j = static_cast<int>(i / (static_cast<long long>(Kp) * Np));
    T value = static_cast<T>(0.0f);
    if (k < K && n < N) {
      const long long src = order ? static_cast<long long>(order[j]) : j;
      value = w[(src * K + k) * N + n];
    }
    wt[i] = value;
  }
}

// ------------------------------------------------- range of the product rows ----

// Product rows of bfloat16 layers travel from the GEMM to Scatter as IEEE half
// words (11 significant bits against bfloat16's 8, so rounding the partial
// products costs less than rounding the output does) times a power of two
// chosen per pass so that no product can leave half's range: every entry of a
// product row is bounded by max|x| * max over (offset, channel) of
// sum_k |w[k][channel]|.  range_kernel leaves the two maxima as kRangeParts
// partial maxima (blocks [0, kRangeFeatureParts): features; the rest: weight
// column sums over the packed weights wt[O][Np][Kp]); range_scale folds them
// (every workgroup of the GEMM and of Scatter does so for itself: 1 KB from
// the L2) into the scale 2^(15 - e), where bound < 2^e.  Non-finite features
// are left out of the maximum (their products are non-finite under any scale).
constexpr int kRangeFeatureParts = 192;
constexpr int kRangeParts = 256;

template <typename T>
__global__ __launch_bounds__(256) void range_kernel(const T *__restrict__ features, long long count,
                                                    const T *__restrict__ wt, long long columns, int Kp,
                                                    float *__restrict__ range) {
  __shared__ float s_part[4];
  float best = 0.0f;
  if (blockIdx.x < kRangeFeatureParts) {
    constexpr int E = 16 / static_cast<int>(sizeof(T));
    const long long stride = static_cast<long long>(kRangeFeatureParts) * 256;
    const long long first = static_cast<long long>(blockIdx.x) * 256 + threadIdx.x;
    if (reinterpret_cast<uintptr_t>(features) % 16 == 0) {
      const long long pieces = count / E;
      for (long long i = first; i < pieces; i += stride) {
        const uint4 raw = reinterpret_cast<const uint4 *>(features)[i];
        const T *e = reinterpret_cast<const T *>(&raw);
#pragma unroll
        for (int k = 0; k < E; ++k) {
          const float v = fabsf(to_float(e[k]));
          best = v <= 3.0e38f ? fmaxf(best, v) : best;
        }
      }
      for (long long i = pieces * E + first; i < count; i += stride) {
        const float v = fabsf(to_float(features[i]));
        best = v <= 3.0e38f ? fmaxf(best, v) : best;
      }
    } else {
      for (long long i = first; i < count; i += stride) {
        const float v = fabsf(to_float(features[i]));
        best = v <= 3.0e38f ? fmaxf(best, v) : best;
      }
    }
  } else {
    // a thread per (offset, channel) row of the packed weights
    const long long stride = static_cast<long long>(kRangeParts - kRangeFeatureParts) * 256;
    for (long long c = static_cast<long long>(blockIdx.x - kRangeFeatureParts) * 256 + threadIdx.x; c < columns;
         c += stride) {
      float sum = 0.0f;
      for (int k = 0; k < Kp; ++k) sum += fabsf(to_float(wt[c * Kp + k]));
      best = fmaxf(best, sum);
    }
  }
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) best = fmaxf(best, __shfl_xor(best, d));
  if ((threadIdx.x & 63) == 0) s_part[threadIdx.x >> 6] = best;
  __syncthreads();
  if (threadIdx.x == 0) range[blockIdx.x] = fmaxf(fmaxf(s_part[0], s_part[1]), fmaxf(s_part[2], s_part[3]));
}

// The scale of the pass (a power of two; 1 without a range or when the bound
// is zero or not finite).  The same in every lane of every workgroup.
__device__ __forceinline__ float range_scale(const float *__restrict__ range) {
  if (range == nullptr) return 1.0f;
  const int lane = threadIdx.x & 63;
  float fx = fmaxf(fmaxf(range[lane], range[lane + 64]), range[lane + 128]);
  float fw = range[kRangeFeatureParts + lane];
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) {
    fx = fmaxf(fx, __shfl_xor(fx, d));
    fw = fmaxf(fw, __shfl_xor(fw, d));
  }
  const float bound = fx * fw;
  if (!(bound > 0.0f) || !(bound <= 3.0e38f)) return 1.0f;
  int e;
  frexpf(bound, &e);                                  // bound = m * 2^e, m in [0.5, 1)
  int shift = 15 - e;
  shift = shift > 120 ? 120 : shift < -120 ? -120 : shift;
  return ldexpf(1.0f, shift);
}

}  // namespace mnt
