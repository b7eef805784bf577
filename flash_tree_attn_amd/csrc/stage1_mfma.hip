// Stage 1, MFMA variant (f16 / bf16, head_dim 64 or 128, >= 16 query rows per unit).
//
// One workgroup = (batch, unit, split, row block). A unit is the set of query heads
// that share one cache head (the GQA group) and one tree head, so its
// rows = heads * q_len query rows all read the same K/V stream: every 64-key tile
// of K and V is fetched from HBM once, staged in LDS, and consumed by all waves.
//
// Each wave owns QB blocks of 32 query rows and computes, per tile,
//     S^T = K Q^T      (v_mfma_f32_32x32x16: A = K rows from LDS, B = Q in registers)
//     online softmax   (lane = query row: max/sum are per-lane, one cross-half swap)
//     O^T += V^T P^T   (A = V^T via transposing LDS reads, B = P^T straight from the
//                       S^T accumulator registers - no LDS round trip)
// In the 32x32 accumulator layout lane (i, h) holds query row i and keys
// 8*(r/4) + 4*h + r%4, r = 0..15; the same lane therefore already holds the B operand
// of the second product if V^T's k-slots are read in that key order.
//
// The split that owns the end of the sequence appends the tree block as extra tiles
// (current_k / current_v with the additive mask), which replaces the eager block and
// sigmoid merge of flash_tree_attn.py:367-373. Output: the final result (one split)
// or a normalised fp32 partial plus its log-sum-exp (flash_tree_attn.py:121-144).
#include <type_traits>

#include "fta_device.h"

namespace fta {
namespace {

template <typename T> struct Mfma;
template <> struct Mfma<__bf16> {
  using Vec8 = bf16x8;
  using Vec4 = bf16x4;
  using Vec2 = bf16x2;
  static __device__ __forceinline__ f32x16 mma(Vec8 a, Vec8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};
template <> struct Mfma<_Float16> {
  using Vec8 = f16x8;
  using Vec4 = f16x4;
  using Vec2 = f16x2;
  static __device__ __forceinline__ f32x16 mma(Vec8 a, Vec8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
};

typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(8))) short s16x8;

template <int D>
struct MfmaSmem {
  static constexpr int kKPitch = D * 2 + 16;  // bytes; +16 keeps row-per-lane 128-bit reads conflict free
  static constexpr int kVPitch = D * 2 + 64;  // bytes; +64 spreads the 4 key rows of a transposing read over all banks
  static constexpr int kKBuf = kKeyTile * kKPitch;
  static constexpr int kVBuf = kKeyTile * kVPitch;
  static constexpr int kTotal = 2 * (kKBuf + kVBuf);
};

// Lanes i and i+32 hold the same query row. v_permlane32_swap exchanges the upper half
// of its first operand with the lower half of its second; the partner's value is then
// in result 1 for lanes < 32 and in result 0 for lanes >= 32 (also when the compiler
// assigns both operands the same register, where both results hold the partner).
__device__ __forceinline__ float half_partner(float x, int lh) {
  auto r = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(unsigned, x), __builtin_bit_cast(unsigned, x), false, false);
  return __builtin_bit_cast(float, lh ? r[0] : r[1]);
}
__device__ __forceinline__ float half_swap_max(float x, int lh) { return fmaxf(x, half_partner(x, lh)); }
__device__ __forceinline__ float half_swap_sum(float x, int lh) { return x + half_partner(x, lh); }

template <typename T, int D, int QB, int NW>
__global__ void __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(QB == 1 ? 2 : 1, QB == 1 ? 2 : 1)))
stage1_mfma_kernel(const KernelParams p) {
  using M = Mfma<T>;
  using Vec8 = typename M::Vec8;
  using SM = MfmaSmem<D>;
  constexpr int kThreads = NW * 64;
  constexpr int KS = D / 16;                         // k-steps of the QK product
  constexpr int DB = D / 32;                         // head_dim blocks of the PV product
  constexpr int kChunks = D / 8;                     // 16-byte chunks per row
  constexpr int kRowsPerPass = kThreads / kChunks;   // rows one pass of the loader covers
  constexpr int kPasses = kKeyTile / kRowsPerPass;
  static_assert(kKeyTile % kRowsPerPass == 0 && kPasses >= 1, "loader mapping");
  constexpr int kRowsPerWave = 32 * QB;
  constexpr int kRowsPerWg = NW * kRowsPerWave;

  extern __shared__ __attribute__((aligned(16))) char smem[];

  const WorkItem w = decode_work(p, blockIdx.x);
  const int b = w.batch;
  int64_t t64 = load_len(p.lens, p.len_is_i64, b);
  const int T_b = static_cast<int>(t64 < 0 ? 0 : (t64 > p.cache_len ? p.cache_len : t64));
  const int S_b = splits_for(T_b, p.chunk, p.num_splits);
  if (w.split >= S_b) return;
  const int kv_start = w.split * p.chunk;
  const int kv_end = (w.split == p.num_splits - 1) ? T_b : min(T_b, kv_start + p.chunk);
  const bool owns_tree = (w.split == S_b - 1);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int li = lane & 31;   // query row within a 32-row block / K row / V^T row
  const int lh = lane >> 5;   // half-wave: selects the k-slot group
  const int L = p.q_len;
  const int head0 = w.unit * p.heads_per_unit;
  const int cache_head = head0 / p.kv_group;
  const int cur_head = head0 / p.cur_group;
  const int wave_row0 = w.row_block * kRowsPerWg + wave * kRowsPerWave;
  const bool wave_active = wave_row0 < p.rows;
  const float c = p.scale_log2;

  const T* kbase = static_cast<const T*>(p.k) + b * p.k_stride[0] + cache_head * p.k_stride[1];
  const T* vbase = static_cast<const T*>(p.v) + b * p.v_stride[0] + cache_head * p.v_stride[1];
  const T* ckbase = static_cast<const T*>(p.ck) + b * p.ck_stride[0] + cur_head * p.ck_stride[1];
  const T* cvbase = static_cast<const T*>(p.cv) + b * p.cv_stride[0] + cur_head * p.cv_stride[1];

  // ---- Q fragments (B operand of S^T = K Q^T), kept in registers for the whole split
  Vec8 qf[QB][KS];
  bool row_ok[QB];
  int row_head[QB], row_i[QB];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    const int row = wave_row0 + qb * 32 + li;
    row_ok[qb] = row < p.rows;
    row_head[qb] = head0 + (row_ok[qb] ? row / L : 0);
    row_i[qb] = row_ok[qb] ? row % L : 0;
    const T* qrow = static_cast<const T*>(p.q) + b * p.q_stride[0] + row_head[qb] * p.q_stride[1] + row_i[qb] * p.q_stride[2];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      u32x4 raw = {0, 0, 0, 0};
      if (row_ok[qb]) raw = *reinterpret_cast<const u32x4*>(qrow + 16 * ks + 8 * lh);
      qf[qb][ks] = __builtin_bit_cast(Vec8, raw);
    }
  }

  f32x16 o[DB][QB];
  float m_run[QB], l_run[QB];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    m_run[qb] = neg_inf();
    l_run[qb] = 0.f;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int r = 0; r < 16; ++r) o[db][qb][r] = 0.f;
  }

  const int cache_tiles = kv_end > kv_start ? (kv_end - kv_start + kKeyTile - 1) / kKeyTile : 0;
  const int tree_tiles = owns_tree ? (L + kKeyTile - 1) / kKeyTile : 0;
  const int ntiles = cache_tiles + tree_tiles;

  // ---- global -> register staging of one K/V tile
  const int ld_row = tid / kChunks;
  const int ld_chunk = tid % kChunks;
  u32x4 kreg[kPasses], vreg[kPasses];
  auto issue_loads = [&](int t) __attribute__((always_inline)) {
    const bool tree = t >= cache_tiles;
    const int key0 = tree ? (t - cache_tiles) * kKeyTile : kv_start + t * kKeyTile;
    const int key_lim = tree ? L : kv_end;
    const T* kb_ = tree ? ckbase : kbase;
    const T* vb_ = tree ? cvbase : vbase;
    const int64_t kts = tree ? p.ck_stride[2] : p.k_stride[2];
    const int64_t vts = tree ? p.cv_stride[2] : p.v_stride[2];
#pragma unroll
    for (int ps = 0; ps < kPasses; ++ps) {
      const int j = key0 + ps * kRowsPerPass + ld_row;
      u32x4 kq = {0, 0, 0, 0}, vq = {0, 0, 0, 0};
      if (j < key_lim) {
        kq = *reinterpret_cast<const u32x4*>(kb_ + j * kts + ld_chunk * 8);
        vq = *reinterpret_cast<const u32x4*>(vb_ + j * vts + ld_chunk * 8);
      }
      kreg[ps] = kq;
      vreg[ps] = vq;
    }
  };
  auto store_lds = [&](int buf) __attribute__((always_inline)) {
    char* kdst = smem + buf * SM::kKBuf;
    char* vdst = smem + 2 * SM::kKBuf + buf * SM::kVBuf;
#pragma unroll
    for (int ps = 0; ps < kPasses; ++ps) {
      const int j = ps * kRowsPerPass + ld_row;
      *reinterpret_cast<u32x4*>(kdst + j * SM::kKPitch + ld_chunk * 16) = kreg[ps];
      *reinterpret_cast<u32x4*>(vdst + j * SM::kVPitch + ld_chunk * 16) = vreg[ps];
    }
  };

  // per-lane LDS byte offsets of the operand reads
  const int k_rd = li * SM::kKPitch + lh * 16;  // + kb*32*pitch + ks*32
  // V^T transposing read: 16-lane group g covers head_dim columns 16*(g%2) .. +15 of a
  // 32-column block; lane s of the group addresses key s/4, columns 4*(s%4) .. +3.
  const int v_rd = (4 * lh + (lane & 15) / 4) * SM::kVPitch + (16 * ((lane >> 4) & 1) + 4 * (lane & 3)) * 2;

  // ---- one 64-key tile: S^T = K Q^T, online softmax, O^T += V^T P^T.
  // MASKED tiles (the tree block, the ragged last cache tile) scale explicitly, add the
  // mask, blank keys past the limit and run a second, compensating P.V product; full
  // cache tiles take the lean path.
  auto process_tile = [&](auto masked_c, int buf, bool tree, int key0, int key_lim) __attribute__((always_inline)) {
    constexpr bool MASKED = decltype(masked_c)::value;
    const char* Kb = smem + buf * SM::kKBuf;
    const char* Vb = smem + 2 * SM::kKBuf + buf * SM::kVBuf;

    f32x16 s[2][QB];
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int qb = 0; qb < QB; ++qb)
#pragma unroll
        for (int r = 0; r < 16; ++r) s[kb][qb][r] = 0.f;
    {
      // K fragments stream through a short register queue: kPF reads ahead of the MFMA
      // that consumes them, so LDS latency hides under the matrix pipeline without
      // holding the whole tile's fragments live.
      constexpr int kFrags = 2 * KS;
      constexpr int kPF = 4;
      Vec8 kf[kFrags];
#pragma unroll
      for (int f = 0; f < kFrags; ++f) {
#ifdef FTA_DBG_NO_LDSREAD
        const u32x4 raw = *reinterpret_cast<const u32x4*>(Kb + k_rd + (f & 1) * 32);
#else
        const u32x4 raw = *reinterpret_cast<const u32x4*>(Kb + k_rd + (f / KS) * 32 * SM::kKPitch + (f % KS) * 32);
#endif
        kf[f] = __builtin_bit_cast(Vec8, raw);
      }
#pragma unroll
      for (int f = 0; f < kFrags; ++f)
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) s[f / KS][qb] = M::mma(kf[f], qf[qb][f % KS], s[f / KS][qb]);
      __builtin_amdgcn_sched_group_barrier(0x100, kPF, 0);
#pragma unroll
      for (int i = 0; i < kFrags - kPF; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, QB, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, kPF * QB, 0);
    }

    // online softmax; P^T packed to T in the B-operand layout of the P.V product
    Vec8 pf[QB][4];
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      const float m_old = m_run[qb];
      if (MASKED) {
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int j = key0 + kb * 32 + (r >> 2) * 8 + 4 * lh + (r & 3);
            float sv = s[kb][qb][r] * c;
            if (tree && j < key_lim && row_ok[qb])
              sv += p.mask[b * p.mask_stride[0] + row_head[qb] * p.mask_stride[1] + row_i[qb] * p.mask_stride[2] + j] * kLog2e;
            s[kb][qb][r] = j < key_lim ? sv : neg_inf();
          }
      }
      float mx0 = fmaxf(s[0][qb][0], s[1][qb][0]), mx1 = fmaxf(s[0][qb][1], s[1][qb][1]);
#pragma unroll
      for (int r = 2; r < 16; r += 2) {
        mx0 = fmaxf(mx0, fmaxf(s[0][qb][r], s[1][qb][r]));
        mx1 = fmaxf(mx1, fmaxf(s[0][qb][r + 1], s[1][qb][r + 1]));
      }
      const float mx = half_swap_max(fmaxf(mx0, mx1), lh);
      const float m_new = fmaxf(m_old, MASKED ? mx : mx * c);
      const float m_use = (MASKED && m_new == neg_inf()) ? 0.f : m_new;
      const float alpha = fast_exp2(m_old - m_use);
      float ps0 = 0.f, ps1 = 0.f;
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int r = 0; r < 16; r += 2) {
#ifdef FTA_DBG_NO_EXP
          const float p0 = __builtin_fmaf(s[kb][qb][r], c, -m_use), p1 = __builtin_fmaf(s[kb][qb][r + 1], c, -m_use);
#else
          const float p0 = MASKED ? fast_exp2(s[kb][qb][r] - m_use) : fast_exp2(__builtin_fmaf(s[kb][qb][r], c, -m_use));
          const float p1 = MASKED ? fast_exp2(s[kb][qb][r + 1] - m_use) : fast_exp2(__builtin_fmaf(s[kb][qb][r + 1], c, -m_use));
#endif
          s[kb][qb][r] = p0;
          s[kb][qb][r + 1] = p1;
          ps0 += p0;
          ps1 += p1;
        }
      l_run[qb] = l_run[qb] * alpha + (ps0 + ps1);
      m_run[qb] = m_new;
      if (__builtin_amdgcn_ballot_w64(m_new > m_old) != 0) {
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
          for (int r = 0; r < 16; ++r) o[db][qb][r] *= alpha;
      }
#pragma unroll
      for (int kk = 0; kk < 4; ++kk) {
        Vec8 pk;
#pragma unroll
        for (int e = 0; e < 8; e += 2) {
          const f32x2 pv = {s[kk >> 1][qb][(kk & 1) * 8 + e], s[kk >> 1][qb][(kk & 1) * 8 + e + 1]};
          const auto pr = __builtin_convertvector(pv, typename M::Vec2);
          pk[e] = pr[0];
          pk[e + 1] = pr[1];
          if (MASKED) {  // keep the rounding residue for the compensating product
            s[kk >> 1][qb][(kk & 1) * 8 + e] = pv[0] - static_cast<float>(pr[0]);
            s[kk >> 1][qb][(kk & 1) * 8 + e + 1] = pv[1] - static_cast<float>(pr[1]);
          }
        }
        pf[qb][kk] = pk;
      }
    }

    auto pv_product = [&]() __attribute__((always_inline)) {
#pragma unroll
      for (int kk = 0; kk < 4; ++kk) {
#pragma unroll
        for (int db = 0; db < DB; ++db) {
#ifdef FTA_DBG_NO_LDSREAD
          const char* va = Vb + v_rd + (kk & 1) * 16 * SM::kVPitch;
#else
          const char* va = Vb + v_rd + (kk * 16) * SM::kVPitch + db * 64;
#endif
          const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 FTA_LDS*)(va));
          const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 FTA_LDS*)(va + 8 * SM::kVPitch));
          const s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
          const Vec8 a = __builtin_bit_cast(Vec8, both);
#pragma unroll
          for (int qb = 0; qb < QB; ++qb) o[db][qb] = M::mma(a, pf[qb][kk], o[db][qb]);
        }
      }
    };
#ifndef FTA_DBG_NO_PV
    pv_product();
#endif
    if (MASKED) {
      // Tree tiles and the ragged last cache tile are where single keys can carry large
      // weights (short sequences); a second product with the low-order part of P removes
      // the 2^-9 rounding of P there. Full cache tiles use one product.
#pragma unroll
      for (int qb = 0; qb < QB; ++qb)
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) {
          Vec8 pk;
#pragma unroll
          for (int e = 0; e < 8; ++e) pk[e] = static_cast<T>(s[kk >> 1][qb][(kk & 1) * 8 + e]);
          pf[qb][kk] = pk;
        }
      pv_product();
    }
  };

  // Two loops over one software pipeline: full cache tiles take the lean body, the
  // ragged last cache tile and the tree tiles the masked one. Tile t+1 is in flight
  // (global -> registers) while tile t is consumed from LDS.
  const int full_tiles = kv_end > kv_start ? (kv_end - kv_start) / kKeyTile : 0;
  issue_loads(0);
  int t = 0;
  for (; t < full_tiles; ++t) {
#ifdef FTA_DBG_NO_GLOBAL
    if (t == 0) { store_lds(0); store_lds(1); }
    __syncthreads();
#else
    store_lds(t & 1);
#ifndef FTA_DBG_NO_BARRIER
    __syncthreads();
#endif
    if (t + 1 < ntiles) issue_loads(t + 1);
#endif
    if (wave_active) process_tile(std::false_type{}, t & 1, false, kv_start + t * kKeyTile, kv_end);
  }
  for (; t < ntiles; ++t) {
    store_lds(t & 1);
    __syncthreads();
    if (t + 1 < ntiles) issue_loads(t + 1);
    const bool tree = t >= cache_tiles;
    const int key0 = tree ? (t - cache_tiles) * kKeyTile : kv_start + t * kKeyTile;
    if (wave_active) process_tile(std::true_type{}, t & 1, tree, key0, tree ? L : kv_end);
  }

  if (!wave_active) return;

  // ---- epilogue
  const bool direct = p.num_splits == 1;
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    const float l_tot = half_swap_sum(l_run[qb], lh);
    if (!row_ok[qb]) continue;
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
    const int head = row_head[qb], i = row_i[qb];
    if (direct) {
      T* dst = static_cast<T*>(p.out) + b * p.out_stride[0] + head * p.out_stride[1] + i * p.out_stride[2];
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int rg = 0; rg < 4; ++rg) {
          typename M::Vec4 v4;
#pragma unroll
          for (int e = 0; e < 4; ++e) v4[e] = static_cast<T>(o[db][qb][rg * 4 + e] * inv);
          *reinterpret_cast<typename M::Vec4*>(dst + db * 32 + rg * 8 + 4 * lh) = v4;
        }
    } else {
      float* dst = p.mid_o + b * p.mid_o_stride[0] + head * p.mid_o_stride[1] + w.split * p.mid_o_stride[2] + i * p.mid_o_stride[3];
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int rg = 0; rg < 4; ++rg) {
          f32x4 v4;
#pragma unroll
          for (int e = 0; e < 4; ++e) v4[e] = o[db][qb][rg * 4 + e] * inv;
          *reinterpret_cast<f32x4*>(dst + db * 32 + rg * 8 + 4 * lh) = v4;
        }
      if (lh == 0) {
        const float lse = l_tot > 0.f ? (m_run[qb] + fast_log2(l_tot)) * kLn2 : neg_inf();
        p.mid_lse[b * p.mid_lse_stride[0] + head * p.mid_lse_stride[1] + w.split * p.mid_lse_stride[2] + i] = lse;
      }
    }
  }
}

template <typename T, int D, int QB, int NW>
int launch(const KernelParams& p, hipStream_t stream) {
  using SM = MfmaSmem<D>;
  auto kern = stage1_mfma_kernel<T, D, QB, NW>;
  if (SM::kTotal > 64 * 1024) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                            SM::kTotal) != hipSuccess)
      return FTA_ERR_LAUNCH;
  }
  const int64_t grid = static_cast<int64_t>(p.bsz) * p.units * p.row_blocks * p.num_splits;
  if (grid <= 0 || grid > 0x7fffffffLL) return FTA_ERR_SHAPE;
  hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>(grid)), dim3(NW * 64), SM::kTotal, stream, p);
  return hipGetLastError() == hipSuccess ? FTA_OK : FTA_ERR_LAUNCH;
}

template <typename T>
int launch_t(const KernelParams& p, int head_dim, hipStream_t stream) {
  if (p.rows_per_wg == 256) {
    if (head_dim == 128) return launch<T, 128, 1, 8>(p, stream);
    if (head_dim == 64) return launch<T, 64, 1, 8>(p, stream);
  } else if (p.rows_per_wg == 128) {
    if (head_dim == 128) return launch<T, 128, 1, 4>(p, stream);
    if (head_dim == 64) return launch<T, 64, 1, 4>(p, stream);
  }
  return FTA_ERR_UNSUPPORTED;
}

}  // namespace

int launch_stage1_mfma(const KernelParams& p, int dtype, int head_dim, void* stream) {
  if (p.scale_log2 <= 0.f) return FTA_ERR_UNSUPPORTED;  // row max is taken before scaling
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case FTA_F16: return launch_t<_Float16>(p, head_dim, s);
    case FTA_BF16: return launch_t<__bf16>(p, head_dim, s);
    default: return FTA_ERR_UNSUPPORTED;
  }
}

}  // namespace fta
