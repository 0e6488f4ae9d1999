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


}  // namespace mnt
