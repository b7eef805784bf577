// Device-side helpers shared by the stage-1 and stage-2 kernels (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fta_internal.h"

namespace fta {

typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) _Float16 f16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;

#define FTA_LDS __attribute__((address_space(3)))

__device__ __forceinline__ float neg_inf() { return -__builtin_huge_valf(); }
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

template <typename T> __device__ __forceinline__ float to_f32(T x) { return static_cast<float>(x); }

__device__ __forceinline__ int64_t load_len(const void* lens, int is_i64, int b) {
  return is_i64 ? static_cast<const int64_t*>(lens)[b] : static_cast<int64_t>(static_cast<const int32_t*>(lens)[b]);
}

// Splits that hold data for a sequence of `t` cached keys: ceil(t / chunk), at
// least one (the tree block always needs a home), at most the grid extent.
__device__ __forceinline__ int splits_for(int t, int chunk, int num_splits) {
  int s = (t + chunk - 1) / chunk;
  s = s < 1 ? 1 : s;
  return s > num_splits ? num_splits : s;
}

struct WorkItem {
  int split, unit, batch, row_block;
};

// Linear workgroup id -> (split, row_block, unit, batch), split fastest.
__device__ __forceinline__ WorkItem decode_work(const KernelParams& p, int id) {
  WorkItem w;
  w.split = id % p.num_splits; id /= p.num_splits;
  w.row_block = id % p.row_blocks; id /= p.row_blocks;
  w.unit = id % p.units;
  w.batch = id / p.units;
  return w;
}

__device__ __forceinline__ float wave_max(float x) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) x = fmaxf(x, __shfl_xor(x, o, 64));
  return x;
}
__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) x += __shfl_xor(x, o, 64);
  return x;
}

}  // namespace fta
