// MFMA fragment helpers shared by the gather-GEMM-scatter kernels.
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include "fgms_internal.h"

namespace fgms {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef int int4v __attribute__((ext_vector_type(4)));

template <typename T> struct Elem;
template <> struct Elem<__half> { static constexpr int per_chunk = 8; };
template <> struct Elem<float> { static constexpr int per_chunk = 4; };

template <typename T>
__device__ __forceinline__ void mma(float16v &acc, const int4v &a, const int4v &b) {
  if constexpr (sizeof(T) == 2) {
    acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8, a),
                                                 __builtin_bit_cast(half8, b), acc, 0, 0, 0);
  } else {
    const float4v fa = __builtin_bit_cast(float4v, a), fb = __builtin_bit_cast(float4v, b);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[0], fb[0], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[1], fb[1], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[2], fb[2], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[3], fb[3], acc, 0, 0, 0);
  }
}

__device__ __forceinline__ float swap_with_neighbour(float v) {
  // lane ^ 1 inside each quad: quad_perm [1, 0, 3, 2]
  return __builtin_bit_cast(
      float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));
}

// fp32 value as two bf16 numbers, x = hi + lo + O(2^-17 x) (see the split-bf16 kernels).
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef int int2v __attribute__((ext_vector_type(2)));

__device__ __forceinline__ void split_bf16(float x, __bf16 &hi, __bf16 &lo) {
  hi = (__bf16)x;
  const float h = (float)hi;
  // (an infinite or NaN value stays in hi alone)
  lo = (__bf16)(__builtin_fabsf(h) < __builtin_inff() ? x - h : 0.f);
}

// Re-lays the weights into per-lane MFMA fragment order in the stream's
// workspace (see pack_weights_kernel) and returns the packed buffer.
int pack_weights_any(const GmsArgs &a, int S, const void **packed);
int num_cus();

}  // namespace fgms
