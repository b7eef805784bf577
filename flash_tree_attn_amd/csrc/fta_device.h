// Device-side helpers shared by the stage-1 and stage-2 kernels (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fta_internal.h"

namespace fta {

typedef __attribute__((ext_vector_type(2))) float f32x2;
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
// The workgroup's dynamically sized LDS, as `char name[]`. A macro so that a test harness which runs these
// kernels on host threads can put an ordinary buffer there.
#ifndef FTA_DYNAMIC_LDS
#define FTA_DYNAMIC_LDS(name) extern __shared__ __attribute__((aligned(16))) char name[]
#endif

// Launches `kern(params)` and reports what THIS launch returned (the thread's sticky last-error
// state may hold an older, unrelated failure and is neither read nor cleared).
template <typename Kernel, typename Params>
inline int launch_checked(Kernel kern, dim3 grid, dim3 block, unsigned smem_bytes, hipStream_t stream, const Params& params) {
  void* args[] = {const_cast<Params*>(&params)};
  return hipLaunchKernel(reinterpret_cast<const void*>(kern), grid, block, args, smem_bytes, stream) == hipSuccess ? FTA_OK : FTA_ERR_LAUNCH;
}

__device__ __forceinline__ float neg_inf() { return -__builtin_huge_valf(); }
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

template <typename T> __device__ __forceinline__ float to_f32(T x) { return static_cast<float>(x); }

__device__ __forceinline__ int64_t load_len(const void* lens, int is_i64, int b) {
  return is_i64 ? static_cast<const int64_t*>(lens)[b] : static_cast<int64_t>(static_cast<const int32_t*>(lens)[b]);
}

// Additive mask value of tree key j for the mask row that starts at element `row_start`
// (in elements of the mask's type): the float itself, or 0 / -inf from bit j of a
// packed row.
__device__ __forceinline__ float tree_mask_value(const KernelParams& p, int64_t row_start, int j) {
  if (p.mask_packed) {
    const uint64_t w = static_cast<const uint64_t*>(p.mask)[row_start + (j >> 6)];
    return (w >> (j & 63)) & 1 ? 0.f : neg_inf();
  }
  return static_cast<const float*>(p.mask)[row_start + j];
}

// Element offset of cache position `pos` of sequence b inside the K (or V) tensor, head
// term excluded: batch stride x b for contiguous caches, page stride x page for paged
// ones (stride[0] is the page stride then).
__device__ __forceinline__ int64_t cache_row_offset(const KernelParams& p, const int64_t (&stride)[3], int b, int pos) {
  if (p.block_table) {
    const int page = p.block_table[b * p.table_stride + (pos >> p.page_shift)];
    return page * stride[0] + (pos & ((1 << p.page_shift) - 1)) * stride[2];
  }
  return b * stride[0] + pos * stride[2];
}

// Splits that hold data for a sequence of `t` cached keys: ceil(t / chunk), at
// least one (the tree block always needs a home), at most the grid extent.
__device__ __forceinline__ int splits_for(int t, int chunk, int num_splits) {
  int s = (t + chunk - 1) / chunk;
  s = s < 1 ? 1 : s;
  return s > num_splits ? num_splits : s;
}

struct WorkItem {
  int item, unit, row_block;  // item = (sequence, split) pair, see item_by_order
};

// Linear workgroup id -> (unit, row_block, item).
// Workgroup ids are dealt round-robin to the 8 XCDs, each with its own L2. The row
// blocks of one (batch, unit, split) read the same K/V stream, so they are given ids
// that differ by a multiple of 8 and land on the same XCD: the second block's K/V
// fetches hit in L2 instead of going to HBM again. Groups beyond the last multiple of
// 8 fall back to consecutive ids.
__device__ __forceinline__ WorkItem decode_work(const KernelParams& p, int id) {
  constexpr int kXcds = 8;
  const int rb_n = p.row_blocks;
  const int groups = p.num_splits * p.units * p.bsz;
  const int even_groups = groups - groups % kXcds;
  int g, rb;
  if (id < even_groups * rb_n) {
    const int xcd = id % kXcds, j = id / kXcds;
    rb = j % rb_n;
    g = (j / rb_n) * kXcds + xcd;
  } else {
    const int r = id - even_groups * rb_n;
    rb = r % rb_n;
    g = even_groups + r / rb_n;
  }
  WorkItem w;
  w.row_block = rb;
  // Units vary fastest: the XCDs are served strictly round-robin, so the 8 workgroups of
  // one dispatch round must carry equal work, and the units of one (sequence, split) do.
  // A split index that varied with the XCD would starve the XCDs of the high splits on
  // ragged batches, where short sequences fill only the first splits.
  w.unit = g % p.units;
  w.item = g / p.units;
  return w;
}

// Length of sequence b, clamped to the cache.
__device__ __forceinline__ int clamped_len(const KernelParams& p, int b) {
  const int64_t v = load_len(p.lens, p.len_is_i64, b);
  return static_cast<int>(v < 0 ? 0 : (v > p.cache_len ? p.cache_len : v));
}

// Keys per split of this launch: the plan's entry for the batch's longest sequence
// (len_bound ascends, so the lowest entry that covers max_len wins; lengths above the last
// bound take the last entry).
__device__ __forceinline__ int chunk_for(const KernelParams& p, int max_len) {
  int c = p.chunk_by_len[FTA_LEN_BUCKETS - 1];
#pragma unroll
  for (int i = FTA_LEN_BUCKETS - 2; i >= 0; --i) c = max_len <= p.len_bound[i] ? p.chunk_by_len[i] : c;
  return c;
}

// Maximum of `mine` over the block; every thread of the block must call it, once per kernel
// (it keeps its per-wave slots until the block ends). Blocks of up to 1024 threads.
__device__ __forceinline__ int block_max(int mine) {
  __shared__ int s_wave_max[16];
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) mine = max(mine, __shfl_xor(mine, o, 64));
  if ((threadIdx.x & 63) == 0) s_wave_max[threadIdx.x >> 6] = mine;
  __syncthreads();
  int m = 0;
  for (int w = 0; w < static_cast<int>((blockDim.x + 63) >> 6); ++w) m = max(m, s_wave_max[w]);
  return __builtin_amdgcn_readfirstlane(m);
}

// Batches of up to 64 sequences: lane i of every wave takes sequence i's clamped length (0 beyond the
// batch) and the wave finds the longest by itself, so that no wave waits for another.
constexpr int kMaxWaveBatch = 64;
__device__ __forceinline__ int wave_longest(const KernelParams& p, int* mine) {
  const int lane = threadIdx.x & 63;
  const int len = lane < p.bsz ? clamped_len(p, lane) : 0;
  int m = len;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) m = max(m, __shfl_xor(m, o, 64));
  *mine = len;
  return __builtin_amdgcn_readfirstlane(m);
}

// Keys per split of this launch, from the lengths of the whole batch; every thread of the
// block must call it, once per kernel. Every workgroup of stage 1 and of stage 2 computes
// the same value from the same lengths, so no workgroup has to tell another.
__device__ __forceinline__ int batch_chunk(const KernelParams& p) {
  if (p.bsz == 1) return chunk_for(p, clamped_len(p, 0));
  if (p.bsz <= kMaxWaveBatch) {
    int mine;
    return chunk_for(p, wave_longest(p, &mine));
  }
  int m = 0;
  for (int i = threadIdx.x; i < p.bsz; i += blockDim.x) m = max(m, clamped_len(p, i));
  return chunk_for(p, block_max(m));
}

// Longest-first dispatch for ragged batches. Workgroup ids are handed out in order, and
// round-robin at every level of the machine (XCD, then shader engine), so any run of
// consecutive ids should carry near-equal work and the heaviest items should come first.
// Item k (from the workgroup id) is therefore resolved against the batch's lengths:
// first every full chunk (all equal work; sequence-major), then the last chunk of every
// sequence (partial chunk + tree block) in descending size; what remains of the grid has
// nothing to do. No host look at the lengths and no atomics: every workgroup recomputes
// the order from the bsz lengths (and gets its sequence's clamped length and the
// launch's chunk length back with it). Batches of up to 64 sequences are resolved by every
// wave on its own, in one pass over the lengths held one per lane, without LDS or barriers,
// and in closed form when all sequences are equally long; larger ones up to kMaxOrderedBatch
// go through LDS; batches of one sequence or beyond kMaxOrderedBatch keep the identity
// order. Returns false if the item is empty. Must be called by all threads of the block.
constexpr int kMaxOrderedBatch = 256;
__device__ __forceinline__ bool item_by_order(const KernelParams& p, int k, int* batch, int* split, int* len, int* chunk_out) {
  if (p.bsz == 1 || p.bsz > kMaxOrderedBatch) {
    const int chunk = batch_chunk(p);
    *chunk_out = chunk;
    *batch = k / p.num_splits;
    *split = k % p.num_splits;
    *len = clamped_len(p, *batch);
    return true;
  }
  if (p.bsz <= kMaxWaveBatch) {
    const int lane = threadIdx.x & 63;
    int my_len;
    const int chunk = chunk_for(p, wave_longest(p, &my_len));
    *chunk_out = chunk;
    const bool in_batch = lane < p.bsz;
    const int my_n = splits_for(my_len, chunk, p.num_splits);
    const int my_full = in_batch ? my_n - 1 : 0;          // chunks of this sequence that are full
    const int my_tail = my_len - (my_n - 1) * chunk;      // keys of its last chunk
    const int len0 = __builtin_amdgcn_readlane(my_len, 0);
    if (__builtin_amdgcn_ballot_w64(in_batch && my_len != len0) == 0) {
      // equally long sequences: bsz * full chunks sequence-major, then the last chunks in batch order
      const int full = __builtin_amdgcn_readlane(my_full, 0);
      const int total = p.bsz * full;
      *len = len0;
      if (k < total) {
        *batch = k / full;
        *split = k % full;
        return true;
      }
      *batch = k - total;
      *split = full;
      return k - total < p.bsz;
    }
    int before = 0, total = 0, rank = 0;
    for (int j = 0; j < p.bsz; ++j) {
      const int f = __builtin_amdgcn_readlane(my_full, j), t = __builtin_amdgcn_readlane(my_tail, j);
      total += f;
      before += j < lane ? f : 0;
      rank += (t > my_tail) || (t == my_tail && j < lane);
    }
    const bool full = k >= before && k < before + my_full;
    const uint64_t owner = __builtin_amdgcn_ballot_w64(in_batch && (full || k - total == rank));
    if (owner == 0) return false;
    const int src = __builtin_ctzll(owner);
    *batch = src;
    *split = __builtin_amdgcn_readlane(full ? k - before : my_n - 1, src);
    *len = __builtin_amdgcn_readlane(my_len, src);
    return true;
  }
  __shared__ int s_nsp[kMaxOrderedBatch];
  __shared__ int s_tail[kMaxOrderedBatch];
  __shared__ int s_pick[3];
  const int t = threadIdx.x;
  int longest = 0;
  for (int i = t; i < p.bsz; i += blockDim.x) {
    const int len = clamped_len(p, i);
    s_tail[i] = len;   // parked here until the chunk is known; the same thread comes back for it
    longest = max(longest, len);
  }
  const int chunk = chunk_for(p, block_max(longest));
  *chunk_out = chunk;
  for (int i = t; i < p.bsz; i += blockDim.x) {
    const int len = s_tail[i];
    const int n = splits_for(len, chunk, p.num_splits);
    s_nsp[i] = n;
    s_tail[i] = len - (n - 1) * chunk;
  }
  if (t == 0) s_pick[0] = -1;
  __syncthreads();
  for (int i = t; i < p.bsz; i += blockDim.x) {
    const int mine = s_tail[i];
    int before = 0, total = 0, rank = 0;
    for (int j = 0; j < p.bsz; ++j) {
      const int f = s_nsp[j] - 1;
      total += f;
      before += j < i ? f : 0;
      rank += (s_tail[j] > mine) || (s_tail[j] == mine && j < i);
    }
    const bool full = k >= before && k < before + s_nsp[i] - 1;
    if (full || k - total == rank) {
      s_pick[0] = i;
      s_pick[1] = full ? k - before : s_nsp[i] - 1;
      s_pick[2] = mine + (s_nsp[i] - 1) * chunk;   // the (clamped) length, so that callers need not load it again
    }
  }
  __syncthreads();
  *batch = __builtin_amdgcn_readfirstlane(s_pick[0]);  // uniform: keep them in scalar registers
  *split = __builtin_amdgcn_readfirstlane(s_pick[1]);
  *len = __builtin_amdgcn_readfirstlane(s_pick[2]);
  return *batch >= 0;
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
