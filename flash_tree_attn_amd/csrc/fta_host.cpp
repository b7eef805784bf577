// Host side of the C ABI: argument validation, the split heuristic and the launch
// sequence. Validation and planning are pure host arithmetic (no HIP calls), so a
// machine without a GPU can exercise them.
#include <hip/hip_runtime_api.h>

#include <cmath>
#include <algorithm>
#include <cstdint>
#include <cstdlib>

#include "fta_internal.h"

namespace fta {

const EnvKnobs& env_knobs() {
  static const EnvKnobs knobs = [] {
    EnvKnobs k{};
    if (const char* e = std::getenv("FTA_ROWS_PER_WG")) k.rows_128 = std::atoi(e) == 128;
    if (const char* e = std::getenv("FTA_FORCE_SPLITS")) k.force_splits = std::max(0, std::atoi(e));
    k.tree_tile_weight = -1;
    if (const char* e = std::getenv("FTA_TREE_TILE_WEIGHT")) k.tree_tile_weight = std::max(0, std::atoi(e));
    if (const char* e = std::getenv("FTA_WIDE_LOOP")) k.wide_loop = e[0] == '1';
    if (const char* e = std::getenv("FTA_SPLIT_KEYS")) k.split_keys = e[0] == '1';
    if (const char* e = std::getenv("FTA_STAGE2_SHARED_WALK")) k.stage2_shared_walk = e[0] == '1';
    return k;
  }();
  return knobs;
}

// Query rows one MFMA workgroup holds: 256 (8 waves x 32 rows, two waves per SIMD, one
// workgroup per CU: the K/V rings take most of the LDS) when the unit has more than 128
// rows, else 128 (4 waves, short rings, two workgroups per CU). FTA_ROWS_PER_WG=128
// forces the 4-wave variant (tuning only). head_dim 256 only exists as the 4-wave variant:
// its tiles are twice as large, two K and two V stages fill the LDS of a CU.
int mfma_rows_per_wg(int rows, int head_dim) {
  if (env_knobs().rows_128) return 128;
  return rows > 128 && head_dim <= 128 ? 256 : 128;
}

namespace {

inline int64_t cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

int esize(int dtype) { return dtype == FTA_F32 ? 4 : 2; }

bool mfma_eligible(const fta_args& a) {
  // The MFMA kernel takes row maxima before scaling, which needs a positive scale.
  // No lower bound on the rows of a unit: rows past its end are blanked per lane, and a
  // unit of one row (plain decode) still streams K/V three times faster through the
  // DMA-fed MFMA kernel than through the shuffle kernel, whose tiles wait on LDS staging.
  return (a.dtype == FTA_F16 || a.dtype == FTA_BF16) && (a.head_dim == 64 || a.head_dim == 128 || a.head_dim == 256) &&
         a.sm_scale > 0.f;
}

// Query heads that share both their cache head and their tree head.
int heads_per_unit(const fta_args& a) {
  const int g = a.num_q_heads / a.num_kv_heads;
  return a.cur_heads == a.num_kv_heads ? g : 1;
}

int validate(const fta_args& a) {
  if (!a.q || !a.k_cache || !a.v_cache || !a.cur_k || !a.cur_v || !a.mask || !a.kv_seq_len || !a.out)
    return FTA_ERR_NULL_POINTER;
  if (a.dtype != FTA_F32 && a.dtype != FTA_F16 && a.dtype != FTA_BF16) return FTA_ERR_DTYPE;
  if (a.len_dtype != FTA_I32 && a.len_dtype != FTA_I64) return FTA_ERR_DTYPE;
  if (a.mask_kind != FTA_MASK_ADDITIVE_F32 && a.mask_kind != FTA_MASK_PACKED_U64) return FTA_ERR_DTYPE;
  if (a.block_table) {
    if (a.page_size != 16 && a.page_size != 32 && a.page_size != 64 && a.page_size != 128) return FTA_ERR_BLOCK_SIZE;
    if (a.block_table_stride < 0 || a.block_table_stride * a.page_size < a.cache_len) return FTA_ERR_SHAPE;
  }
  if (a.head_dim != 32 && a.head_dim != 64 && a.head_dim != 128 && a.head_dim != 256) return FTA_ERR_HEAD_DIM;
  if (a.cache_len != a.v_cache_len) return FTA_ERR_CACHE_LEN_MISMATCH;
  if (a.block_size != 16 && a.block_size != 32 && a.block_size != 64 && a.block_size != 128)
    return FTA_ERR_BLOCK_SIZE;
  if (a.bsz <= 0 || a.num_q_heads <= 0 || a.num_kv_heads <= 0 || a.q_len <= 0 || a.cache_len < 0 ||
      a.max_seq_len_hint < 0 || a.mid_splits < 0 || a.force_splits < 0)
    return FTA_ERR_SHAPE;
  if (a.num_q_heads % a.num_kv_heads != 0) return FTA_ERR_SHAPE;
  if (a.cur_heads != a.num_kv_heads && a.cur_heads != a.num_q_heads) return FTA_ERR_SHAPE;
  if (a.force_kernel < -1 || a.force_kernel > FTA_KERNEL_MFMA_SPLIT_KEYS) return FTA_ERR_UNSUPPORTED;
  // Paged caches with no capacity have no table entry to look up (the kernels clamp positions to cache_len - 1).
  if (a.block_table && a.cache_len == 0) return FTA_ERR_SHAPE;

  // Rows are moved with 128-bit accesses: every row start must be 16-byte aligned.
  const int vec = 16 / esize(a.dtype);
  const int64_t* row_strides[] = {a.q_stride, a.k_stride, a.v_stride, a.ck_stride, a.cv_stride, a.out_stride};
  for (const int64_t* s : row_strides)
    for (int i = 0; i < 3; ++i) {
      if (s[i] < 0) return FTA_ERR_STRIDE;
      if (s[i] % vec != 0) return FTA_ERR_STRIDE;
    }
  const void* row_ptrs[] = {a.q, a.k_cache, a.v_cache, a.cur_k, a.cur_v, a.out};
  for (const void* ptr : row_ptrs)
    if (reinterpret_cast<uintptr_t>(ptr) % 16 != 0) return FTA_ERR_STRIDE;
  for (int i = 0; i < 3; ++i)
    if (a.mask_stride[i] < 0) return FTA_ERR_STRIDE;
  if (reinterpret_cast<uintptr_t>(a.mask) % (a.mask_kind == FTA_MASK_PACKED_U64 ? 8 : 4) != 0) return FTA_ERR_STRIDE;
  return FTA_OK;
}

int plan(const fta_args& a, int num_cus, fta_plan_out* out) {
  if (num_cus <= 0) num_cus = kDefaultCUs;
  const int hpu = heads_per_unit(a);
  const int rows = hpu * a.q_len;
  const int units = a.num_q_heads / hpu;

  int kernel = mfma_eligible(a) ? FTA_KERNEL_MFMA : FTA_KERNEL_SHUFFLE;
  if (a.force_kernel >= 0) {
    if (a.force_kernel != FTA_KERNEL_SHUFFLE && !mfma_eligible(a)) return FTA_ERR_UNSUPPORTED;
    kernel = a.force_kernel == FTA_KERNEL_SHUFFLE ? FTA_KERNEL_SHUFFLE : FTA_KERNEL_MFMA;
  }
  // Units of at most 64 rows, head_dim 64 / 128: two waves per 32-row block, each taking half of a tile's
  // keys, so that all four waves of the workgroup compute (with 32-row waves, three or two of them would only
  // request tiles). Opt-in (force_kernel or FTA_SPLIT_KEYS=1) until it has been timed.
  const bool split_ok = kernel == FTA_KERNEL_MFMA && rows <= 64 && a.head_dim <= 128;
  if (a.force_kernel == FTA_KERNEL_MFMA_SPLIT_KEYS && !split_ok) return FTA_ERR_UNSUPPORTED;
  const bool split_keys = split_ok && (a.force_kernel == FTA_KERNEL_MFMA_SPLIT_KEYS || (a.force_kernel < 0 && env_knobs().split_keys));
  const int rows_per_wg = kernel != FTA_KERNEL_MFMA ? 16 : split_keys ? 64 : mfma_rows_per_wg(rows, a.head_dim);
  // The 64-row-wave loop serves 256-row workgroups on contiguous caches, head_dim 64 / 128. It is
  // opt-in (force_kernel or FTA_WIDE_LOOP=1): its one recorded timing at the headline shape is 5 % behind
  // the 8-wave loop, and bf16 rows carried by a few keys exceed the tolerance in it.
  const bool wide_ok = kernel == FTA_KERNEL_MFMA && rows_per_wg == 256 && !a.block_table && a.head_dim <= 128;
  if (a.force_kernel == FTA_KERNEL_MFMA_WIDE && !wide_ok) return FTA_ERR_UNSUPPORTED;
  const bool wide = wide_ok && (a.force_kernel == FTA_KERNEL_MFMA_WIDE || (a.force_kernel < 0 && env_knobs().wide_loop));
  const int row_blocks = static_cast<int>(cdiv(rows, rows_per_wg));
  // Workgroups one CU holds at a time (LDS- and register-bound, see the kernels): the
  // 128-row MFMA variant is built to share a CU with a second workgroup.
  // The shuffle kernel's workgroups (4 waves, ~40 KB of LDS) fit four to a CU.
  const int wg_per_cu = kernel != FTA_KERNEL_MFMA ? 4 : (rows_per_wg <= 128 && a.head_dim <= 128) ? 2 : 1;

  const int64_t work_items = static_cast<int64_t>(a.bsz) * units * row_blocks;
  const int64_t t_cap = a.max_seq_len_hint > 0 ? std::min(a.max_seq_len_hint, a.cache_len) : a.cache_len;
  const int gran = std::max(a.block_size, kKeyTile);

  // Split count from a cost model of one launch, in microseconds, with every sequence
  // taken at the length cap (lengths are not known on the host):
  //   rounds(S) * wg(S) + tail * wg(S) + merge(S),   wg(S) = fixed + tile_us * tiles(S)
  // rounds = workgroups / CUs rounded up (one workgroup per CU), `fixed` the measured
  // per-workgroup prologue + tree step + epilogue, `tile_us` the steady-state time of
  // one 64-key tile with every CU busy, `tail` the expected idle share of the last
  // round of a ragged batch (a single sequence has nothing to balance), merge the
  // fp32 partials written and read back. Few long chunks win over many short ones:
  // the fixed part is worth 7-10 tiles.
  const int64_t target = static_cast<int64_t>(num_cus) * wg_per_cu;
  struct Cut { int64_t splits, chunk; };
  // The cut for sequences of up to t_len cached keys, with at most s_limit splits (a forced
  // count is only held to the limit when `limit_forced`).
  auto cut_for = [&](int64_t t_len, int64_t s_limit, bool limit_forced) -> Cut {
    t_len = std::max<int64_t>(t_len, 1);
    const int64_t forced_limit = limit_forced ? s_limit : INT64_MAX;
    const int64_t min_chunk = std::max<int64_t>(gran, 4 * kKeyTile);
    const int64_t s_max = std::max<int64_t>(1, std::min<int64_t>(s_limit, t_len / min_chunk));
    const double fixed_us = kernel != FTA_KERNEL_MFMA ? 5.0 : wg_per_cu > 1 ? 12.0 : 20.0;   // partly hidden behind co-resident workgroups
    // per workgroup and 64-key tile, with the CU fully occupied: the pipelined 256-row
    // variant alone on its CU; the plain 128-row variant next to a second workgroup, by
    // the number of its waves that hold rows; the shuffle kernel with four workgroups per CU.
    const int live_waves = std::min(4, static_cast<int>(cdiv(std::min(rows, rows_per_wg), 32)));
    const double tile_us = kernel != FTA_KERNEL_MFMA ? 5.0 : rows_per_wg > 128 ? 2.85 : (1.0 + 0.7 * live_waves) * (a.head_dim > 128 ? 2.0 : 1.0);
    const double tree_tiles = 3.0 * cdiv(a.q_len, kKeyTile);
    const double tail_share = a.bsz > 1 ? 0.25 : 0.0;
    const double partial_mb = 4e-6 * a.bsz * a.num_q_heads * a.q_len * a.head_dim;  // MB per split slot
    int64_t splits = 1;
    double best = 0.0;
    double cost_of[65];
    for (int64_t cand = 1; cand <= s_max; ++cand) {
      const double tiles = std::ceil((t_len / static_cast<double>(kKeyTile) + tree_tiles) / cand);
      const double wg_us = fixed_us + tile_us * tiles;
      const double rounds = static_cast<double>(cdiv(work_items * cand, target));
      const double merge_us = cand > 1 ? 6.0 + cand * partial_mb / 2.0 : 0.0;   // written once, read once, at ~4-5 TB/s
      const double cost = (rounds + tail_share) * wg_us + merge_us;
      cost_of[cand] = cost;
      if (cand == 1 || cost < best * 0.98) {  // a larger count has to win by 2 %
        best = cost;
        splits = cand;
      }
    }
    // A batch whose workgroups all fit the machine at once is only balanced if its sequences
    // are equally long, and the lengths are not known here: the longest sequence then sets the
    // time while most CUs idle. For batches of 8 and more, up to twice the splits are taken
    // where the model prices that at no more than 10 % on an equal-length batch. Measured over
    // split sweeps of 76 ragged and 112 equal-length shapes: -6 % on the ragged ones on
    // average (worst case 2.1x -> 1.3x of the best split count), +1 % on the equal-length ones.
    if (a.bsz >= 8 && a.head_dim <= 128 && work_items * splits <= target) {   // head_dim 256: the model is not calibrated well enough
      const int64_t chosen = splits;
      for (int64_t cand = chosen + 1; cand <= std::min<int64_t>(2 * chosen, s_max); ++cand)
        if (cost_of[cand] <= cost_of[chosen] * 1.10) splits = cand;
    }
    if (a.force_splits > 0) splits = std::min<int64_t>(a.force_splits, forced_limit);
    if (env_knobs().force_splits > 0) splits = std::min<int64_t>(env_knobs().force_splits, forced_limit);
    // Never more splits than blocks of the reference granularity, so that a scratch
    // buffer sized like the reference's (flash_tree_attn.py:274-281) always fits.
    splits = std::min<int64_t>(splits, std::max<int64_t>(1, cdiv(t_len, gran)));
    // The split that owns the end of a sequence also processes the tree block (a masked,
    // latency-bound step worth about three cache tiles per tree tile): count it as extra
    // keys when cutting chunks, so that the last split of a full-length sequence gets a
    // correspondingly shorter cache range.
    // (The 64-row-wave loop's unpipelined masked halves probably weigh more; until a timing says how much it is cut
    // like the 8-wave loop. FTA_TREE_TILE_WEIGHT sets the weight for such a run.)
    const int64_t tree_weight = env_knobs().tree_tile_weight >= 0 ? env_knobs().tree_tile_weight : 3;
    const int64_t tree_keys = splits > 1 ? tree_weight * kKeyTile * cdiv(a.q_len, kKeyTile) : 0;
    int64_t chunk = cdiv(cdiv(t_len + tree_keys, splits), gran) * gran;
    if ((splits - 1) * chunk >= t_len) chunk = cdiv(cdiv(t_len, splits), gran) * gran;
    splits = std::max<int64_t>(1, cdiv(t_len, chunk));
    return Cut{splits, chunk};
  };
  // The grid and the scratch buffers are sized for the length cap. The lengths themselves are
  // only known on the device, and a cap far above them (a cache allocated for the longest
  // context the server admits, a page table's full width) would leave most splits without
  // keys. The kernels therefore take the chunk from a table by the batch's longest sequence:
  // the cut this model makes for that length within the cap's split count. Bounds fall
  // from the cap in steps of 3/4 and 2/3 (1, 3/4, 1/2, 3/8, ...), so the table entry is for
  // a length at most a third above the real one; a batch at the cap gets the cap's own cut.
  const int64_t cap = std::max<int64_t>(t_cap, 1);
  // Scratch the caller brought bounds what the heuristic may pick: a caller of the reference
  // sizes it from the batch's longest sequence (flash_tree_attn.py:274-281), which can be far
  // below the capacity this plan is cut for. (A forced count that does not fit stays an error.)
  // Only where it binds: scratch sized from this plan's own answer leaves the plan as it is.
  const int64_t slots = a.mid_o && a.mid_lse && a.mid_splits > 0 ? a.mid_splits : 64;
  const bool forced = a.force_splits > 0 || env_knobs().force_splits > 0;
  Cut cap_cut = cut_for(cap, 64, false);
  if (!forced && slots < cap_cut.splits) cap_cut = cut_for(cap, slots, false);
  const int64_t splits = cap_cut.splits, chunk = cap_cut.chunk;
  for (int i = 0; i < FTA_LEN_BUCKETS; ++i) {
    const int k = FTA_LEN_BUCKETS - 1 - i;   // steps below the cap
    const int64_t fraction = cdiv((k % 2 ? 3 : 1) * cap, int64_t{1} << (k % 2 ? (k + 3) / 2 : k / 2));
    const int64_t bound = k == 0 ? cap : std::min(cap, cdiv(fraction, gran) * gran);
    out->len_bound[i] = static_cast<int32_t>(bound);
    out->chunk_by_len[i] = static_cast<int32_t>(k == 0 ? chunk : cut_for(bound, splits, true).chunk);
  }

  out->kernel = kernel;
  out->num_splits = static_cast<int32_t>(splits);
  out->chunk = static_cast<int32_t>(chunk);
  out->rows_per_group = rows;
  out->rows_per_wg = rows_per_wg;
  out->row_blocks = row_blocks;
  out->num_workgroups = static_cast<int32_t>(work_items * splits);
  out->mfma_loop = wide ? 1 : split_keys ? 2 : 0;
  out->counter_elems = (splits > 1 && kernel == FTA_KERNEL_MFMA && work_items <= 0x7fffffff) ? static_cast<int32_t>(work_items) : 0;
  // Merging inside stage 1 saves the second launch, but the last workgroup of a sequence
  // merges alone: that pays with two splits and one round of workgroups (short launches,
  // where the second kernel and the gap before it weigh most), not beyond.
  out->single_launch = out->counter_elems > 0 && splits <= 2 && work_items * splits <= target;
  out->mid_lse_elems = splits > 1 ? static_cast<int64_t>(a.bsz) * a.num_q_heads * splits * a.q_len : 0;
  out->mid_o_elems = out->mid_lse_elems * a.head_dim;
  return FTA_OK;
}

}  // namespace
}  // namespace fta

extern "C" {

int fta_abi_version(void) { return FTA_ABI_VERSION; }

const char* fta_strerror(int status) {
  switch (status) {
    case FTA_OK: return "ok";
    case FTA_ERR_NULL_POINTER: return "a required pointer is NULL";
    case FTA_ERR_HEAD_DIM: return "head_dim must be one of 32, 64, 128, 256";
    case FTA_ERR_BLOCK_SIZE: return "block_size must be one of 16, 32, 64, 128";
    case FTA_ERR_CACHE_LEN_MISMATCH: return "k_cache and v_cache have different sequence lengths";
    case FTA_ERR_SCRATCH_TOO_SMALL: return "mid_output / mid_output_lse hold fewer splits than the plan needs";
    case FTA_ERR_DTYPE: return "unsupported dtype";
    case FTA_ERR_SHAPE: return "inconsistent shapes";
    case FTA_ERR_STRIDE: return "unsupported strides: inner stride must be 1 and rows 16-byte aligned";
    case FTA_ERR_UNSUPPORTED: return "no kernel instantiated for this combination";
    case FTA_ERR_LAUNCH: return "HIP kernel launch failed";
    case FTA_ERR_NO_DEVICE: return "no HIP device available";
    default: return "unknown fta status";
  }
}

int fta_validate(const fta_args* args) {
  if (!args) return FTA_ERR_NULL_POINTER;
  return fta::validate(*args);
}

int fta_plan(const fta_args* args, int num_cus, fta_plan_out* plan) {
  if (!args || !plan) return FTA_ERR_NULL_POINTER;
  // Planning needs consistent sizes but no pointers.
  fta_args a = *args;
  // 16-byte aligned stand-in so that validate() only judges the sizes.
  alignas(16) static const char aligned_dummy[16] = {0};
  const void* d = aligned_dummy;
  a.q = a.k_cache = a.v_cache = a.cur_k = a.cur_v = a.kv_seq_len = d;
  a.mask = d;
  a.out = const_cast<void*>(d);
  if (int st = fta::validate(a)) return st;
  return fta::plan(a, num_cus, plan);
}

int fta_device_cus(void) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return FTA_ERR_NO_DEVICE;
  int cus = 0;
  if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return FTA_ERR_NO_DEVICE;
  return cus;
}

namespace {
// stages: bit 0 = stage 1, bit 1 = stage 2
int decode_impl(const fta_args* args, void* hip_stream, int stages) {
  if (!args) return FTA_ERR_NULL_POINTER;
  const fta_args& a = *args;
  if (int st = fta::validate(a)) return st;
  static thread_local int cached_cus = 0;
  if (cached_cus <= 0) {
    cached_cus = fta_device_cus();
    if (cached_cus <= 0) return FTA_ERR_NO_DEVICE;
  }
  fta_plan_out pl;
  if (int st = fta::plan(a, cached_cus, &pl)) return st;
  if (pl.num_splits > 1) {
    if (!a.mid_o || !a.mid_lse) return FTA_ERR_NULL_POINTER;
    if (a.mid_splits < pl.num_splits) return FTA_ERR_SCRATCH_TOO_SMALL;
    for (int i = 0; i < 4; ++i)
      if (a.mid_o_stride[i] < 0 || a.mid_o_stride[i] % 4 != 0) return FTA_ERR_STRIDE;
    for (int i = 0; i < 3; ++i)
      if (a.mid_lse_stride[i] < 0) return FTA_ERR_STRIDE;
    if (reinterpret_cast<uintptr_t>(a.mid_o) % 16 != 0) return FTA_ERR_STRIDE;
  }
  // Single launch: only for the whole path, and only where the plan has such a path.
  const bool fused = stages == 3 && a.counters != nullptr && pl.counter_elems > 0;
  if (fused && a.counter_elems < pl.counter_elems) return FTA_ERR_SCRATCH_TOO_SMALL;

  fta::KernelParams p{};
  p.q = a.q; p.k = a.k_cache; p.v = a.v_cache; p.ck = a.cur_k; p.cv = a.cur_v;
  p.mask = a.mask; p.lens = a.kv_seq_len; p.out = a.out; p.mid_o = a.mid_o; p.mid_lse = a.mid_lse;
  p.counters = fused ? a.counters : nullptr;
  p.block_table = a.block_table;
  p.table_stride = a.block_table_stride;
  p.page_shift = a.page_size == 16 ? 4 : a.page_size == 32 ? 5 : a.page_size == 64 ? 6 : 7;
  p.wide_loop = pl.mfma_loop == 1;
  p.bsz = a.bsz; p.num_q_heads = a.num_q_heads; p.q_len = a.q_len; p.cache_len = a.cache_len;
  p.chunk = pl.chunk; p.num_splits = pl.num_splits;
  for (int i = 0; i < FTA_LEN_BUCKETS; ++i) {
    p.len_bound[i] = pl.len_bound[i];
    p.chunk_by_len[i] = pl.chunk_by_len[i];
  }
  p.heads_per_unit = pl.rows_per_group / a.q_len;
  p.units = a.num_q_heads / p.heads_per_unit;
  p.kv_group = a.num_q_heads / a.num_kv_heads;
  p.cur_group = a.num_q_heads / a.cur_heads;
  p.rows = pl.rows_per_group; p.rows_per_wg = pl.rows_per_wg; p.row_blocks = pl.row_blocks;
  p.len_is_i64 = a.len_dtype == FTA_I64;
  p.mask_packed = a.mask_kind == FTA_MASK_PACKED_U64;
  p.mask_vec4 = !p.mask_packed && reinterpret_cast<uintptr_t>(a.mask) % 16 == 0 && a.mask_stride[0] % 4 == 0 && a.mask_stride[1] % 4 == 0 &&
                a.mask_stride[2] % 4 == 0;
  p.scale_log2 = a.sm_scale * fta::kLog2e;
  for (int i = 0; i < 3; ++i) {
    p.q_stride[i] = a.q_stride[i]; p.k_stride[i] = a.k_stride[i]; p.v_stride[i] = a.v_stride[i];
    p.ck_stride[i] = a.ck_stride[i]; p.cv_stride[i] = a.cv_stride[i]; p.mask_stride[i] = a.mask_stride[i];
    p.out_stride[i] = a.out_stride[i]; p.mid_lse_stride[i] = a.mid_lse_stride[i];
  }
  for (int i = 0; i < 4; ++i) p.mid_o_stride[i] = a.mid_o_stride[i];

  int st = FTA_OK;
  if (stages & 1)
    st = pl.kernel == FTA_KERNEL_MFMA ? fta::launch_stage1_mfma(p, a.dtype, a.head_dim, hip_stream)
                                      : fta::launch_stage1_shuffle(p, a.dtype, a.head_dim, hip_stream);
  if (st) return st;
  if ((stages & 2) && pl.num_splits > 1 && !fused) st = fta::launch_stage2_merge(p, a.dtype, a.head_dim, hip_stream);
  return st;
}
}  // namespace

int fta_decode(const fta_args* args, void* hip_stream) { return decode_impl(args, hip_stream, 3); }
int fta_decode_stage1(const fta_args* args, void* hip_stream) { return decode_impl(args, hip_stream, 1); }
int fta_decode_stage2(const fta_args* args, void* hip_stream) { return decode_impl(args, hip_stream, 2); }

}  // extern "C"
