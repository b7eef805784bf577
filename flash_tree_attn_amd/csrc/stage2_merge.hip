// Stage 2: log-sum-exp merge of the per-split partials into the final output.
// Replaces flash_tree_attn.py:147-211 and, because the tree block already lives in
// one of the partials, the sigmoid merge of flash_tree_attn.py:373 as well.
//
// One thread owns four consecutive head_dim columns of one output row; the row's
// split weights exp(lse_s - max) are recomputed per thread (the split count is
// small by construction of the heuristic). On request, with many splits and few rows,
// four threads share the walk over the splits (see the kernel and launch()).
#include "fta_device.h"

namespace fta {
namespace {

template <typename T> struct Pack4;
template <> struct Pack4<float> {
  static __device__ __forceinline__ void store(float* dst, f32x4 v) { *reinterpret_cast<f32x4*>(dst) = v; }
};
template <> struct Pack4<_Float16> {
  static __device__ __forceinline__ void store(_Float16* dst, f32x4 v) {
    f16x4 h = {static_cast<_Float16>(v[0]), static_cast<_Float16>(v[1]), static_cast<_Float16>(v[2]),
               static_cast<_Float16>(v[3])};
    *reinterpret_cast<f16x4*>(dst) = h;
  }
};
template <> struct Pack4<__bf16> {
  static __device__ __forceinline__ void store(__bf16* dst, f32x4 v) {
    bf16x4 h = {static_cast<__bf16>(v[0]), static_cast<__bf16>(v[1]), static_cast<__bf16>(v[2]),
                static_cast<__bf16>(v[3])};
    *reinterpret_cast<bf16x4*>(dst) = h;
  }
};

// SG = 1: one thread owns four consecutive head_dim columns of one output row and walks all of the row's
// splits. SG = 4: four threads share those columns and walk every fourth split each, their partial sums
// meet in LDS. The second form is for calls with many splits and few rows (one long sequence): there the
// first leaves the machine a few hundred waves that each issue their loads one split after the other.
template <typename T, int D, int SG>
__global__ void __launch_bounds__(256) stage2_merge_kernel(const KernelParams p) {
  constexpr int kThreadsPerRow = D / 4;
  constexpr int kRowsPerBlock = 256 / (kThreadsPerRow * SG);
  static_assert(kRowsPerBlock >= 1, "a row's threads fit one block");
  const int chunk = batch_chunk(p);   // the same cut stage 1 made (block-wide: before any thread leaves)
  const int64_t total_rows = static_cast<int64_t>(p.bsz) * p.num_q_heads * p.q_len;
  const int r_in_block = threadIdx.x / (kThreadsPerRow * SG);
  const int g = (threadIdx.x / kThreadsPerRow) % SG;
  const int64_t row = static_cast<int64_t>(blockIdx.x) * kRowsPerBlock + r_in_block;
  const bool valid = row < total_rows;
  if (SG == 1 && !valid) return;
  const int64_t row_c = valid ? row : 0;
  const int d = (threadIdx.x % kThreadsPerRow) * 4;
  const int i = static_cast<int>(row_c % p.q_len);
  const int head = static_cast<int>((row_c / p.q_len) % p.num_q_heads);
  const int b = static_cast<int>(row_c / (static_cast<int64_t>(p.q_len) * p.num_q_heads));

  const int S_b = splits_for(clamped_len(p, b), chunk, p.num_splits);

  const float* lse = p.mid_lse + b * p.mid_lse_stride[0] + head * p.mid_lse_stride[1] + i;
  const float* mo = p.mid_o + b * p.mid_o_stride[0] + head * p.mid_o_stride[1] + i * p.mid_o_stride[3] + d;

  float mx = neg_inf();
  for (int s = 0; s < S_b; ++s) mx = fmaxf(mx, lse[s * p.mid_lse_stride[2]]);
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  float wsum = 0.f;
  if (mx != neg_inf()) {
    for (int s = g; s < S_b; s += SG) {
      const float wgt = fast_exp2((lse[s * p.mid_lse_stride[2]] - mx) * kLog2e);
      const f32x4 o = *reinterpret_cast<const f32x4*>(mo + s * p.mid_o_stride[2]);
      acc += wgt * o;
      wsum += wgt;
    }
  }
  if constexpr (SG > 1) {
    __shared__ f32x4 s_acc[kRowsPerBlock][SG][kThreadsPerRow];
    __shared__ float s_w[kRowsPerBlock][SG];
    s_acc[r_in_block][g][threadIdx.x % kThreadsPerRow] = acc;
    if (threadIdx.x % kThreadsPerRow == 0) s_w[r_in_block][g] = wsum;
    __syncthreads();
    if (g != 0 || !valid) return;
#pragma unroll
    for (int o = 1; o < SG; ++o) {
      acc += s_acc[r_in_block][o][threadIdx.x % kThreadsPerRow];
      wsum += s_w[r_in_block][o];
    }
  }
  if (mx != neg_inf()) acc *= 1.f / wsum;
  T* dst = static_cast<T*>(p.out) + b * p.out_stride[0] + head * p.out_stride[1] + i * p.out_stride[2] + d;
  Pack4<T>::store(dst, acc);
}

template <typename T, int D, int SG>
int launch_sg(const KernelParams& p, hipStream_t stream) {
  constexpr int kRowsPerBlock = 256 / ((D / 4) * SG);
  const int64_t total_rows = static_cast<int64_t>(p.bsz) * p.num_q_heads * p.q_len;
  const int64_t grid = (total_rows + kRowsPerBlock - 1) / kRowsPerBlock;
  if (grid <= 0 || grid > 0x7fffffffLL) return FTA_ERR_SHAPE;
  return launch_checked(stage2_merge_kernel<T, D, SG>, dim3(static_cast<unsigned>(grid)), dim3(256), 0, stream, p);
}

template <typename T, int D>
int launch(const KernelParams& p, hipStream_t stream) {
  // The shared walk is for launches that would otherwise leave the machine few waves with long walks: fewer
  // than 16 waves per CU of a 256-CU part in the one-thread-per-column form, eight splits or more. It has not
  // been timed against the plain walk yet, so it only runs on request (FTA_STAGE2_SHARED_WALK=1).
  const int64_t waves = static_cast<int64_t>(p.bsz) * p.num_q_heads * p.q_len * (D / 4) / 64;
  if (env_knobs().stage2_shared_walk && p.num_splits >= 8 && waves < 16 * kDefaultCUs) return launch_sg<T, D, 4>(p, stream);
  return launch_sg<T, D, 1>(p, stream);
}

template <typename T>
int launch_d(const KernelParams& p, int head_dim, hipStream_t stream) {
  switch (head_dim) {
    case 32: return launch<T, 32>(p, stream);
    case 64: return launch<T, 64>(p, stream);
    case 128: return launch<T, 128>(p, stream);
    case 256: return launch<T, 256>(p, stream);
    default: return FTA_ERR_HEAD_DIM;
  }
}

}  // namespace

int launch_stage2_merge(const KernelParams& p, int dtype, int head_dim, void* stream) {
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case FTA_F32: return launch_d<float>(p, head_dim, s);
    case FTA_F16: return launch_d<_Float16>(p, head_dim, s);
    case FTA_BF16: return launch_d<__bf16>(p, head_dim, s);
    default: return FTA_ERR_DTYPE;
  }
}

}  // namespace fta
