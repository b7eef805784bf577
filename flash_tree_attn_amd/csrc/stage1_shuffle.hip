// Stage 1, wavefront-shuffle variant: any dtype (f32/f16/bf16), any head_dim in
// {32,64,128,256}, any number of query rows, any sign of sm_scale. The general
// fallback: fp32 inputs, head_dim 32, non-positive sm_scale.
//
// One workgroup = (batch, unit, split, block of 16 query rows); 4 waves x 4 rows.
// Each 64-key tile of K and V is staged once in LDS and shared by the 16 rows.
// Scores: lane j owns key j of the tile (dot product over head_dim from LDS),
// row max / row sum by wavefront shuffles; P.V: lane owns head_dim columns
// lane, lane+64, ... and walks the 64 keys with P broadcast from LDS.
// Replaces flash_tree_attn.py:49-144 (one split) and, on the split that owns the
// tree block, flash_tree_attn.py:367-373.
#include "fta_device.h"

namespace fta {
namespace {

constexpr int kRowsPerWave = 4;
constexpr int kWaves = 4;
constexpr int kRowsPerWg = kRowsPerWave * kWaves;  // 16

template <typename T, int D>
struct ShuffleSmem {
  static constexpr int kVec = 16 / sizeof(T);          // elements per 128-bit access
  static constexpr int kKPitch = D + kVec;             // padded: lane j reads row j
  static constexpr int kKBytes = kKeyTile * kKPitch * sizeof(T);
  static constexpr int kVBytes = kKeyTile * D * sizeof(T);
  static constexpr int kQBytes = kRowsPerWg * D * sizeof(float);
  static constexpr int kPBytes = kRowsPerWg * kKeyTile * sizeof(float);
  static constexpr int kTotal = kKBytes + kVBytes + kQBytes + kPBytes;
};

template <typename T, int D>
__global__ void __launch_bounds__(256) stage1_shuffle_kernel(const KernelParams p) {
  using S = ShuffleSmem<T, D>;
  constexpr int kVec = S::kVec;
  constexpr int kNC = D >= 64 ? D / 64 : 1;  // head_dim columns per lane in P.V
  FTA_DYNAMIC_LDS(smem);
  T* Ks = reinterpret_cast<T*>(smem);
  T* Vs = reinterpret_cast<T*>(smem + S::kKBytes);
  float* Qs = reinterpret_cast<float*>(smem + S::kKBytes + S::kVBytes);
  float* Ps = reinterpret_cast<float*>(smem + S::kKBytes + S::kVBytes + S::kQBytes);

  const WorkItem w = decode_work(p, blockIdx.x);
  int b, split, T_b, chunk;   // chunk: keys per split of this launch, from the batch's longest sequence
  if (!item_by_order(p, w.item, &b, &split, &T_b, &chunk)) return;
  const int S_b = splits_for(T_b, chunk, p.num_splits);
  if (split >= S_b) return;
  const int kv_start = split * chunk;
  const int kv_end = (split == p.num_splits - 1) ? T_b : min(T_b, kv_start + chunk);
  const bool owns_tree = (split == S_b - 1);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int L = p.q_len;
  const int head0 = w.unit * p.heads_per_unit;
  const int cache_head = head0 / p.kv_group;
  const int cur_head = head0 / p.cur_group;
  const int row0 = w.row_block * kRowsPerWg;

  // Q rows of this workgroup -> LDS as fp32, pre-multiplied by sm_scale*log2(e).
  for (int idx = tid; idx < kRowsPerWg * D; idx += 256) {
    const int r = idx / D, d = idx % D;
    const int row = row0 + r;
    float qv = 0.f;
    if (row < p.rows) {
      const int head = head0 + row / L, i = row % L;
      qv = to_f32(static_cast<const T*>(p.q)[b * p.q_stride[0] + head * p.q_stride[1] + i * p.q_stride[2] + d]);
    }
    Qs[idx] = qv * p.scale_log2;
  }

  float m_run[kRowsPerWave], l_run[kRowsPerWave], acc[kRowsPerWave][kNC];
  int row_head[kRowsPerWave], row_i[kRowsPerWave];
  bool row_ok[kRowsPerWave];
#pragma unroll
  for (int rr = 0; rr < kRowsPerWave; ++rr) {
    m_run[rr] = neg_inf();
    l_run[rr] = 0.f;
#pragma unroll
    for (int c = 0; c < kNC; ++c) acc[rr][c] = 0.f;
    const int row = row0 + wave * kRowsPerWave + rr;
    row_ok[rr] = row < p.rows;
    row_head[rr] = head0 + (row_ok[rr] ? row / L : 0);
    row_i[rr] = row_ok[rr] ? row % L : 0;
  }

  const int cache_tiles = kv_end > kv_start ? (kv_end - kv_start + kKeyTile - 1) / kKeyTile : 0;
  const int tree_tiles = owns_tree ? (L + kKeyTile - 1) / kKeyTile : 0;

  for (int t = 0; t < cache_tiles + tree_tiles; ++t) {
    const bool tree = t >= cache_tiles;
    const int key0 = tree ? (t - cache_tiles) * kKeyTile : kv_start + t * kKeyTile;
    const int key_lim = tree ? L : kv_end;
    // tree rows: [batch, head, row]; cache rows: per position through cache_row_offset (paged or not)
    const T* kbase = tree ? static_cast<const T*>(p.ck) + b * p.ck_stride[0] + cur_head * p.ck_stride[1]
                          : static_cast<const T*>(p.k) + cache_head * p.k_stride[1];
    const T* vbase = tree ? static_cast<const T*>(p.cv) + b * p.cv_stride[0] + cur_head * p.cv_stride[1]
                          : static_cast<const T*>(p.v) + cache_head * p.v_stride[1];

    __syncthreads();  // previous tile fully consumed (also orders the Q staging)
    for (int idx = tid; idx < kKeyTile * (D / kVec); idx += 256) {
      const int j = idx / (D / kVec), c = idx % (D / kVec);
      u32x4 kq = {0, 0, 0, 0}, vq = {0, 0, 0, 0};
      if (key0 + j < key_lim) {
        const int64_t krow = tree ? (key0 + j) * p.ck_stride[2] : cache_row_offset(p, p.k_stride, b, key0 + j);
        const int64_t vrow = tree ? (key0 + j) * p.cv_stride[2] : cache_row_offset(p, p.v_stride, b, key0 + j);
        kq = *reinterpret_cast<const u32x4*>(kbase + krow + c * kVec);
        vq = *reinterpret_cast<const u32x4*>(vbase + vrow + c * kVec);
      }
      *reinterpret_cast<u32x4*>(Ks + j * S::kKPitch + c * kVec) = kq;
      *reinterpret_cast<u32x4*>(Vs + j * D + c * kVec) = vq;
    }
    __syncthreads();

    // scores: lane = key
    float s[kRowsPerWave];
#pragma unroll
    for (int rr = 0; rr < kRowsPerWave; ++rr) s[rr] = 0.f;
    const T* krow = Ks + lane * S::kKPitch;
    const float* qw = Qs + wave * kRowsPerWave * D;
#pragma unroll 4
    for (int d = 0; d < D; d += 4) {
      float kf[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) kf[e] = to_f32(krow[d + e]);
#pragma unroll
      for (int rr = 0; rr < kRowsPerWave; ++rr) {
        const f32x4 qv = *reinterpret_cast<const f32x4*>(qw + rr * D + d);
        s[rr] += qv[0] * kf[0] + qv[1] * kf[1] + qv[2] * kf[2] + qv[3] * kf[3];
      }
    }
    const bool key_ok = key0 + lane < key_lim;
#pragma unroll
    for (int rr = 0; rr < kRowsPerWave; ++rr) {
      float sv = s[rr];
      if (tree && key_ok && row_ok[rr]) {
        const int64_t mrow = b * p.mask_stride[0] + row_head[rr] * p.mask_stride[1] + row_i[rr] * p.mask_stride[2];
        sv += tree_mask_value(p, mrow, key0 + lane) * kLog2e;
      }
      if (!key_ok) sv = neg_inf();
      const float m_new = fmaxf(m_run[rr], wave_max(sv));
      const float alpha = (m_new == neg_inf()) ? 1.f : fast_exp2(m_run[rr] - m_new);
      const float pv = (sv == neg_inf()) ? 0.f : fast_exp2(sv - m_new);
      l_run[rr] = l_run[rr] * alpha + wave_sum(pv);
      m_run[rr] = m_new;
#pragma unroll
      for (int c = 0; c < kNC; ++c) acc[rr][c] *= alpha;
      Ps[(wave * kRowsPerWave + rr) * kKeyTile + lane] = pv;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

    // P.V: lane = head_dim column
    if (D >= 64 || lane < D) {
      const float* pw = Ps + wave * kRowsPerWave * kKeyTile;
#pragma unroll 2
      for (int j = 0; j < kKeyTile; j += 4) {
        f32x4 pj[kRowsPerWave];
#pragma unroll
        for (int rr = 0; rr < kRowsPerWave; ++rr) pj[rr] = *reinterpret_cast<const f32x4*>(pw + rr * kKeyTile + j);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
#pragma unroll
          for (int c = 0; c < kNC; ++c) {
            const float vv = to_f32(Vs[(j + e) * D + lane + 64 * c]);
#pragma unroll
            for (int rr = 0; rr < kRowsPerWave; ++rr) acc[rr][c] += pj[rr][e] * vv;
          }
        }
      }
    }
  }

  // Epilogue: final output (single split) or normalised partial + lse.
  const bool direct = p.num_splits == 1;
#pragma unroll
  for (int rr = 0; rr < kRowsPerWave; ++rr) {
    if (!row_ok[rr]) continue;
    const float inv = l_run[rr] > 0.f ? 1.f / l_run[rr] : 0.f;
    const int head = row_head[rr], i = row_i[rr];
#pragma unroll
    for (int c = 0; c < kNC; ++c) {
      const int d = lane + 64 * c;
      if (d >= D) continue;
      const float o = acc[rr][c] * inv;
      if (direct) {
        static_cast<T*>(p.out)[b * p.out_stride[0] + head * p.out_stride[1] + i * p.out_stride[2] + d] = static_cast<T>(o);
      } else {
        p.mid_o[b * p.mid_o_stride[0] + head * p.mid_o_stride[1] + split * p.mid_o_stride[2] +
                i * p.mid_o_stride[3] + d] = o;
      }
    }
    if (!direct && lane == 0) {
      const float lse = l_run[rr] > 0.f ? (m_run[rr] + fast_log2(l_run[rr])) * kLn2 : neg_inf();
      p.mid_lse[b * p.mid_lse_stride[0] + head * p.mid_lse_stride[1] + split * p.mid_lse_stride[2] + i] = lse;
    }
  }
}

template <typename T, int D>
int launch(const KernelParams& p, hipStream_t stream) {
  using S = ShuffleSmem<T, D>;
  auto kern = stage1_shuffle_kernel<T, D>;
  if (S::kTotal > 64 * 1024) {
    // Raising the dynamic-LDS limit is a driver call: once per kernel and device, not per launch.
    static thread_local int configured_device = -1;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return FTA_ERR_NO_DEVICE;
    if (configured_device != dev) {
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                              S::kTotal) != hipSuccess)
        return FTA_ERR_LAUNCH;
      configured_device = dev;
    }
  }
  const int64_t grid = static_cast<int64_t>(p.bsz) * p.units * p.row_blocks * p.num_splits;
  if (grid <= 0 || grid > 0x7fffffffLL) return FTA_ERR_SHAPE;
  return launch_checked(kern, dim3(static_cast<unsigned>(grid)), dim3(256), S::kTotal, stream, p);
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

int launch_stage1_shuffle(const KernelParams& p, int dtype, int head_dim, void* stream) {
  if (p.rows_per_wg != kRowsPerWg) return FTA_ERR_UNSUPPORTED;
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case FTA_F32: return launch_d<float>(p, head_dim, s);
    case FTA_F16: return launch_d<_Float16>(p, head_dim, s);
    case FTA_BF16: return launch_d<__bf16>(p, head_dim, s);
    default: return FTA_ERR_DTYPE;
  }
}

}  // namespace fta
