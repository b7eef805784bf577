// Internal declarations shared by the host side and the HIP kernels.
#pragma once
#include <stdint.h>
#include "fta.h"

namespace fta {

constexpr int kKeyTile = 64;        // keys per LDS tile in every stage-1 kernel
constexpr int kDefaultCUs = 256;    // MI355X: 8 XCDs x 32 CUs
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

// Kernel-side view of one call. A "unit" is a set of `heads_per_unit` consecutive
// query heads that read the same cache head AND the same tree head, so one K/V
// stream serves rows = heads_per_unit * q_len query rows.
struct KernelParams {
  const void* q;
  const void* k;
  const void* v;
  const void* ck;
  const void* cv;
  const void* mask;       // float32 additive values, or uint64 bit words when mask_packed
  const void* lens;
  void* out;
  float* mid_o;
  float* mid_lse;
  const int32_t* block_table;  // null = contiguous caches; else page index per (sequence, position / page size)
  int32_t* counters;      // one per (sequence, unit, row block) when the merge runs inside stage 1, else null

  int32_t bsz;
  int32_t num_q_heads;
  int32_t q_len;
  int32_t cache_len;
  int32_t chunk;          // keys per split at the length cap (the last entry of chunk_by_len)
  int32_t num_splits;
  int32_t heads_per_unit;
  int32_t units;          // num_q_heads / heads_per_unit
  int32_t kv_group;       // query heads per cache head
  int32_t cur_group;      // query heads per tree head
  int32_t rows;           // heads_per_unit * q_len
  int32_t rows_per_wg;
  int32_t row_blocks;
  int32_t len_is_i64;
  int32_t mask_vec4;      // every (float) mask row starts 16-byte aligned
  int32_t mask_packed;    // mask holds one bit per (row, tree key): set = attend
  int32_t page_shift;     // log2(page size) when block_table is set
  int32_t wide_loop;      // 256-row workgroups: 4 waves x 64 rows with the half-tile loop instead of 8 waves x 32 rows
  float scale_log2;       // sm_scale * log2(e)
  int32_t len_bound[FTA_LEN_BUCKETS];     // ascending; the chunk of a launch is chunk_by_len[first i with max length <= len_bound[i]]
  int32_t chunk_by_len[FTA_LEN_BUCKETS];

  int64_t q_stride[3];
  int64_t k_stride[3];
  int64_t v_stride[3];
  int64_t ck_stride[3];
  int64_t cv_stride[3];
  int64_t mask_stride[3];
  int64_t out_stride[3];
  int64_t mid_o_stride[4];
  int64_t mid_lse_stride[3];
  int64_t table_stride;   // block_table elements per sequence
};

// Launchers implemented in the .hip files. Each returns a fta_status.
int launch_stage1_shuffle(const KernelParams& p, int dtype, int head_dim, void* stream);
int launch_stage1_mfma(const KernelParams& p, int dtype, int head_dim, void* stream);
int launch_stage1_mfma_wide(const KernelParams& p, int dtype, int head_dim, void* stream);   // 256-row workgroups of 64-row waves
int launch_stage1_mfma_splitkeys(const KernelParams& p, int dtype, int head_dim, void* stream);   // 64-row workgroups, two waves per row block
int launch_stage2_merge(const KernelParams& p, int dtype, int head_dim, void* stream);

// Rows one MFMA workgroup holds for a unit of `rows` query rows (host + device agree on it).
int mfma_rows_per_wg(int rows, int head_dim);

// Tuning knobs from the environment, read once per process (comparison runs and tests only):
// FTA_ROWS_PER_WG=128, FTA_FORCE_SPLITS=n, FTA_TREE_TILE_WEIGHT=n, FTA_WIDE_LOOP=1, FTA_SPLIT_KEYS=1,
// FTA_STAGE2_SHARED_WALK=1.
struct EnvKnobs {
  bool rows_128;
  int force_splits;      // 0 = none
  int tree_tile_weight;  // < 0 = default
  bool wide_loop;
  bool split_keys;
  bool stage2_shared_walk;   // stage 2: four threads share a row's walk over many splits (not yet timed against the plain walk)
};
const EnvKnobs& env_knobs();

}  // namespace fta
