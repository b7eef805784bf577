// Stage 1, MFMA variant (f16 / bf16, head_dim 64, 128 or 256, positive sm_scale; any number of
// query rows per unit: rows past a unit's end are blanked per lane, and units of a few
// rows still stream K/V faster through this kernel's load path than the shuffle variant).
//
// One workgroup = (batch, unit, split, row block). A unit is the set of query heads
// that share one cache head (the GQA group) and one tree head, so its
// rows = heads * q_len query rows all read the same K/V stream: every 64-key tile
// of K and V is fetched from HBM once, written straight into LDS by the load
// instruction itself (global_load_lds, no register staging) into a ring of NS stages,
// and consumed by all waves of the workgroup.
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
// LDS layout of one K or V tile (64 keys): blocks of RPB = 512/D rows, 1024 bytes each,
// block pitch 1024 + pad. Inside a block the 16-byte chunks of its rows are interleaved
// (chunk c of row r sits at c*16*RPB + r*16), which is what one wave-wide
// global_load_lds writes when lane i fetches chunk i/RPB of row i%RPB. Both operand
// read patterns (16 consecutive K rows at one chunk; 4 consecutive V rows x 64 bytes
// for the transposing read) then fall on distinct banks, and every fragment address is
// a per-lane base plus a compile-time offset.
//
// The split that owns the end of the sequence also runs the tree block, as extra tiles
// ahead of its cache tiles (current_k / current_v with the additive or bit-packed mask),
// which replaces the eager block and sigmoid merge of flash_tree_attn.py:367-373.
// Output: the final result (one split) or a normalised fp32 partial plus its
// log-sum-exp (flash_tree_attn.py:121-144); with counters, the workgroup that finishes
// a sequence last merges the partials itself (flash_tree_attn.py:339-365).
//
// Two loop variants: 8 waves / 256 rows with a software pipeline (softmax of tile t
// sliced behind the MFMAs of P.V(t-1) and K.Q(t+1), K requested 3 tiles ahead into a
// ring of 4 stages / V ring 5, one workgroup per CU), and 4 waves / 128 rows with a plain
// loop and rings of 2 so that two workgroups share a CU (head_dim 256 only has this
// variant, alone on its CU: its tiles are twice as large). Caches are contiguous per
// sequence or paged through a block table (a template parameter, so that the contiguous
// path carries no lookups).
#pragma once
#include <cstdlib>
#include <type_traits>

#include "fta_device.h"
#include "gfx950_ops.h"

namespace fta {
namespace {

template <int D>
struct TileLayout {
  static constexpr int kRowBytes = D * 2;
  static constexpr int kRowsPerBlock = 1024 / kRowBytes;           // 4 (D=128), 8 (D=64), 2 (D=256)
  static constexpr int kChunkStride = 16 * kRowsPerBlock;          // bytes between chunks of one row
  static constexpr int kBlockPitch = 1024 + kChunkStride;          // pad: consecutive blocks shift banks
  static constexpr int kBlocks = kKeyTile / kRowsPerBlock;         // 16, 8, 32
  static constexpr int kTileBytes = kBlocks * kBlockPitch;
  static constexpr int kStageBytes = 2 * kTileBytes;               // K tile then V tile
  // byte offset of 16-byte chunk `c` of tile row `r`
  static __device__ __forceinline__ int at(int r, int c) {
    return (r / kRowsPerBlock) * kBlockPitch + c * kChunkStride + (r % kRowsPerBlock) * 16;
  }
};

// Compile-time loop: f(std::integral_constant<int, I>) for I in [0, N).
template <int I, int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    static_for<I + 1, N>(f);
  }
}

}  // namespace
}  // namespace fta
#include "wide_loop_asm.inc"
namespace fta {
namespace {

// Loop variants (template parameter MODE).
constexpr int kPlain = 0;       // 4 waves x 32 rows, one tile at a time, short rings, two workgroups per CU
constexpr int kPipelined = 1;   // 8 waves x 32 rows, software pipeline over whole tiles
constexpr int kWide = 2;        // 4 waves x 64 rows, software pipeline over half tiles, one wave per SIMD
constexpr int kSplitKeys = 3;   // 4 waves, 64 rows: like kPlain, but two waves share a 32-row block, each taking 32 of a tile's 64 keys

// NSK: how many tiles ahead K is requested. NSK >= 2: K of tile t+1 is read during iteration t
// and must have been requested an iteration earlier. (The K ring has NSK stages, one more in
// the pipelined loop: kKSlots.)
template <typename T, int D, int QB, int NW, int NSK, int MODE, bool PAGED>
__global__ void __launch_bounds__(NW * 64)
FTA_WAVES_PER_EU(((QB == 1 && D <= 128) ? 2 : 1))   // head_dim 256 and 64-row waves need the whole register file
stage1_mfma_kernel(const KernelParams p) {
  using M = Mfma<T>;
  using Vec8 = typename M::Vec8;
  using TL = TileLayout<D>;
  static_assert(NSK >= 2, "K ring too shallow");
  constexpr bool PIPE = MODE == kPipelined;
  constexpr bool WIDE = MODE == kWide;
  constexpr bool KSPLIT = MODE == kSplitKeys;
  static_assert(!KSPLIT || (QB == 1 && NW % 2 == 0), "key halves are written for one row block per wave and pairs of waves");
  static_assert(!WIDE || QB == 2, "the half-tile pipeline is written for two row blocks per wave");
  // V ring: the pipelined loop reads V of a tile one iteration (a whole tile) after its K,
  // the half-tile pipeline half a tile after
  constexpr int NSV = PIPE ? NSK + 2 : WIDE ? NSK + 1 : NSK;
  constexpr int KS = D / 16;                         // k-steps of the QK product
  constexpr int DB = D / 32;                         // head_dim blocks of the PV product
  constexpr int RPB = TL::kRowsPerBlock;
  constexpr int kLoadsPerTensor = TL::kBlocks / NW;  // global_load_lds per wave per tile, per K or V
  static_assert(TL::kBlocks % NW == 0 && kLoadsPerTensor >= 1, "loader mapping");
  constexpr int kLoadsPerTile = 2 * kLoadsPerTensor;
  constexpr int kRowsPerWave = 32 * QB;
  constexpr int kRowsPerWg = (KSPLIT ? NW / 2 : NW) * kRowsPerWave;
  // K stages of the ring. Tiles are requested NSK ahead in every loop; the pipelined loop keeps one
  // stage more, so that K of tile t is still in place behind iteration t, which may want its scores
  // again (kHeavyShare), instead of being overwritten by the tile requested during that iteration.
  constexpr int kKSlots = PIPE ? NSK + 1 : NSK;
  constexpr int kVRing = kKSlots * TL::kTileBytes;   // byte offset of the V ring

  FTA_DYNAMIC_LDS(smem);

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
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int li = lane & 31;   // query row within a 32-row block / K row / V^T row
  const int lh = lane >> 5;   // half-wave: selects the k-slot group
  const int L = p.q_len;
  const int head0 = w.unit * p.heads_per_unit;
  const int cache_head = head0 / p.kv_group;
  const int cur_head = head0 / p.cur_group;
  // kSplitKeys: waves 2r and 2r+1 hold the same 32 rows; wave 2r+h takes keys 32h .. 32h+31 of every tile
  const int kb_own = KSPLIT ? (wave & 1) : 0;
  const int wave_row0 = w.row_block * kRowsPerWg + (KSPLIT ? wave >> 1 : wave) * kRowsPerWave;
  const bool wave_active = wave_row0 < p.rows;
  const float c = p.scale_log2;

  // Contiguous caches: base of this sequence's and head's stream. Paged caches: base of
  // the head inside page 0; the page term comes from the block table per 1 KiB block.
  constexpr bool paged = PAGED;   // the host picks the instantiation by p.block_table
  const char* kbase = reinterpret_cast<const char*>(static_cast<const T*>(p.k) + (paged ? 0 : b * p.k_stride[0]) + cache_head * p.k_stride[1]);
  const char* vbase = reinterpret_cast<const char*>(static_cast<const T*>(p.v) + (paged ? 0 : b * p.v_stride[0]) + cache_head * p.v_stride[1]);
  const int32_t* table = paged ? p.block_table + b * p.table_stride : nullptr;
  const int page_mask = (1 << p.page_shift) - 1;
  const int64_t k_page_bytes = p.k_stride[0] * 2, v_page_bytes = p.v_stride[0] * 2;
  const char* ckbase = reinterpret_cast<const char*>(static_cast<const T*>(p.ck) + b * p.ck_stride[0] + cur_head * p.ck_stride[1]);
  const char* cvbase = reinterpret_cast<const char*>(static_cast<const T*>(p.cv) + b * p.cv_stride[0] + cur_head * p.cv_stride[1]);

  // Tile order: the tree tiles first (their masked, latency-bound handling overlaps the
  // ramp-up of the cache stream), then the cache tiles of this split; only the last cache
  // tile can be ragged.
  const int cache_tiles = kv_end > kv_start ? (kv_end - kv_start + kKeyTile - 1) / kKeyTile : 0;
  const int full_tiles = kv_end > kv_start ? (kv_end - kv_start) / kKeyTile : 0;
  const int tree_tiles = owns_tree ? (L + kKeyTile - 1) / kKeyTile : 0;
  const int ntiles = tree_tiles + cache_tiles;

  // ---- Q rows of this lane (B operand of S^T = K Q^T), kept in registers for the whole split
  Vec8 qf[QB][KS];
  bool row_ok[QB];
  int row_head[QB], row_i[QB];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    const int row = wave_row0 + qb * 32 + li;
    row_ok[qb] = row < p.rows;
    row_head[qb] = head0 + (row_ok[qb] ? row / L : 0);   // rows past the end read row 0 and are zeroed below
    row_i[qb] = row_ok[qb] ? row % L : 0;
  }

  // ---- HBM -> LDS: lane i of a wave-wide load fetches chunk i/RPB of row i%RPB of one
  // block; the hardware writes lane i's 16 bytes at block_base + 16*i. K tiles cycle
  // through a ring of NSK stages, V tiles through NSV = NSK + 2 (V is consumed one
  // iteration after K, see the pipeline below).
  const int ld_rib = lane % RPB;
  const int ld_chunk = lane / RPB;
  const uint32_t k_lane_off = static_cast<uint32_t>(ld_rib * p.k_stride[2] * 2 + ld_chunk * 16);
  const uint32_t v_lane_off = static_cast<uint32_t>(ld_rib * p.v_stride[2] * 2 + ld_chunk * 16);
  const int64_t k_row_bytes = p.k_stride[2] * 2, v_row_bytes = p.v_stride[2] * 2;

  // Paged caches: the page of each of this wave's 1 KiB blocks (RPB consecutive positions,
  // never straddling a page) comes from the block table with wave-uniform (scalar) loads.
  // The entries of the NEXT cache tile are requested when a tile goes out, so that the
  // lookup sits in the slack before the barrier: sync_point fetches them before it waits
  // for the barrier, the tile request after the barrier picks them up.
  int page_of[kLoadsPerTensor];
  int pages_for_tile = -1;   // cache tile whose pages `page_of` holds
  auto load_pages = [&](int ct) __attribute__((always_inline)) {
    const int32_t* ent[kLoadsPerTensor];
#pragma unroll
    for (int i = 0; i < kLoadsPerTensor; ++i) {
      const int key = min(kv_start + ct * kKeyTile + (i * NW + wave) * RPB, p.cache_len - 1);
      ent[i] = table + (key >> p.page_shift);
    }
    static_assert(kLoadsPerTensor == 1 || kLoadsPerTensor % 2 == 0, "entries are fetched singly, in pairs or in fours");
    if constexpr (kLoadsPerTensor == 1) {
      scalar_load_one(ent[0], page_of[0]);
    } else if constexpr (kLoadsPerTensor % 4 == 0) {
#pragma unroll
      for (int i = 0; i < kLoadsPerTensor; i += 4)
        scalar_load_quad(ent[i], ent[i + 1], ent[i + 2], ent[i + 3], page_of[i], page_of[i + 1], page_of[i + 2], page_of[i + 3]);
    } else {
#pragma unroll
      for (int i = 0; i < kLoadsPerTensor; i += 2) scalar_load_pair(ent[i], ent[i + 1], page_of[i], page_of[i + 1]);
    }
    pages_for_tile = ct;
  };
  // Ring slots of the next tile to go out (tiles go out in order, so the slots just count up and wrap).
  int k_slot = 0, v_slot = 0;
  auto advance_slots = [&]() __attribute__((always_inline)) {
    k_slot = k_slot + 1 == kKSlots ? 0 : k_slot + 1;
    v_slot = v_slot + 1 == NSV ? 0 : v_slot + 1;
  };
  const int64_t k_wave_off = static_cast<int64_t>(wave * RPB) * k_row_bytes, v_wave_off = static_cast<int64_t>(wave * RPB) * v_row_bytes;
  const int64_t k_step = static_cast<int64_t>(NW * RPB) * k_row_bytes, v_step = static_cast<int64_t>(NW * RPB) * v_row_bytes;
  const char* k_run = uniform_ptr(kbase + static_cast<int64_t>(kv_start) * k_row_bytes + k_wave_off);   // next full tile, this wave's first block
  const char* v_run = uniform_ptr(vbase + static_cast<int64_t>(kv_start) * v_row_bytes + v_wave_off);
  auto issue_full_tile = [&](int t) __attribute__((always_inline)) {
    char* kst = smem + k_slot * TL::kTileBytes;
    char* vst = smem + kVRing + v_slot * TL::kTileBytes;
    const int key0 = kv_start + (t - tree_tiles) * kKeyTile;
    if constexpr (paged) {
      if (pages_for_tile != t - tree_tiles) load_pages(t - tree_tiles);   // not fetched ahead (first tiles of a split)
    }
    // contiguous caches: full tiles follow each other in memory, so their scalar base just advances;
    // the blocks of this wave sit a fixed stride apart
    const char* ktile = k_run;
    const char* vtile = v_run;
    if constexpr (!paged) {
      k_run = uniform_ptr(k_run + kKeyTile * k_row_bytes);
      v_run = uniform_ptr(v_run + kKeyTile * v_row_bytes);
    }
#pragma unroll
    for (int i = 0; i < kLoadsPerTensor; ++i) {
      const int blk = i * NW + wave;
      const char* ksrc;
      const char* vsrc;
      if (paged) {
        const int key = key0 + blk * RPB;
        ksrc = kbase + page_of[i] * k_page_bytes + static_cast<int64_t>(key & page_mask) * k_row_bytes;
        vsrc = vbase + page_of[i] * v_page_bytes + static_cast<int64_t>(key & page_mask) * v_row_bytes;
      } else {
        ksrc = uniform_ptr(ktile + i * k_step);
        vsrc = uniform_ptr(vtile + i * v_step);
      }
      FTA_LOAD_BLOCK_TO_LDS(ksrc + k_lane_off, kst + blk * TL::kBlockPitch);
      FTA_LOAD_BLOCK_TO_LDS(vsrc + v_lane_off, vst + blk * TL::kBlockPitch);
    }
  };
  // Ragged / tree tiles: rows past the limit re-read the last valid row (finite data
  // that the -inf logits then ignore) instead of touching padding.
  auto issue_edge_tile = [&](int t) __attribute__((always_inline)) {
    char* kst = smem + k_slot * TL::kTileBytes;
    char* vst = smem + kVRing + v_slot * TL::kTileBytes;
    const bool tree = t < tree_tiles;
    const int key0 = tree ? t * kKeyTile : kv_start + (t - tree_tiles) * kKeyTile;
    const int key_lim = tree ? L : kv_end;
    const char* kb_ = tree ? ckbase : kbase;
    const char* vb_ = tree ? cvbase : vbase;
    const int64_t krb = tree ? p.ck_stride[2] * 2 : k_row_bytes;
    const int64_t vrb = tree ? p.cv_stride[2] * 2 : v_row_bytes;
#pragma unroll
    for (int i = 0; i < kLoadsPerTensor; ++i) {
      const int blk = i * NW + wave;
      const int j = min(key0 + blk * RPB + ld_rib, key_lim - 1);
      int64_t koff = j * krb, voff = j * vrb;
      if (paged && !tree) {   // per-lane page: clamped rows may sit in another page than the block's first row
        const int64_t page = table[j >> p.page_shift];
        koff = page * k_page_bytes + (j & page_mask) * krb;
        voff = page * v_page_bytes + (j & page_mask) * vrb;
      }
      FTA_LOAD_BLOCK_TO_LDS(kb_ + koff + ld_chunk * 16, kst + blk * TL::kBlockPitch);
      FTA_LOAD_BLOCK_TO_LDS(vb_ + voff + ld_chunk * 16, vst + blk * TL::kBlockPitch);
    }
  };
  // Tiles are requested in order. A tile may go out once the stage it lands in is free:
  // tile j reuses the K stage of tile j-kKSlots and the V stage of tile j-NSV and goes out when
  // tile j-NSK is done with (for the pipelined loop a stage later than it would have to). `k_done` /
  // `v_done` count the tiles whose K / V every wave has finished reading (as of the last
  // barrier).
  // `cap` bounds the tiles that may go out: ntiles normally; kPadRing lets the ring run
  // past the last tile (the half-tile pipeline keeps one tile going out per
  // synchronisation point so that its waits are constants): such a tile re-reads the last
  // valid cache row into a stage that nobody reads.
  constexpr int kPadRing = 0x7fffffff;
  int next_issue = 0;
  auto issue_ready = [&](int k_done, int v_done, int cap) __attribute__((always_inline)) {
    while (next_issue < cap && next_issue - k_done < NSK && next_issue - v_done < NSV) {
      const int t = next_issue++;
      if (t >= tree_tiles && t - tree_tiles < full_tiles) issue_full_tile(t); else issue_edge_tile(t);
      advance_slots();
    }
  };
  // "All but the loads of the N youngest tiles have landed". The counter holds 63 at most;
  // a larger allowance (deep rings of many-load tiles) is cut to that, which only waits longer.
  auto wait_tiles = [&](auto n_c) __attribute__((always_inline)) {
    constexpr int kAllow = decltype(n_c)::value * kLoadsPerTile;
    wait_vmcnt<(kAllow < 63 ? kAllow : 63)>();
  };
  // One synchronisation point: this wave's share of tile `need` has landed (tiles land in
  // request order; `need` < 0 waits for nothing), then the barrier (everybody's share has
  // landed, and everybody is past the reads that k_done / v_done describe), then every
  // tile whose stages have become free is requested.
  auto sync_point = [&](int need, int k_done, int v_done, int cap) __attribute__((always_inline)) {
    if constexpr (paged) {   // pages of the tile that goes out after the barrier (harmless if none does)
      const int ct = next_issue - tree_tiles;
      load_pages(ct < 0 ? 0 : ct);
    }
    if (need >= 0) {
      const int younger = next_issue - 1 - need;   // tiles requested after `need`
      if (younger >= 4) wait_tiles(std::integral_constant<int, 4>{});
      else if (younger == 3) wait_tiles(std::integral_constant<int, 3>{});
      else if (younger == 2) wait_tiles(std::integral_constant<int, 2>{});
      else if (younger == 1) wait_tiles(std::integral_constant<int, 1>{});
      else wait_vmcnt<0>();
    }
    workgroup_barrier();
    issue_ready(k_done, v_done, cap);
  };
  // The synchronisation point of the half-tile pipeline in the middle of a cache tile:
  // the ring is full (NSK tiles requested beyond the current one), so the tile needed next
  // has exactly two younger ones, and exactly one tile goes out behind the barrier.
  auto sync_steady = [&]() __attribute__((always_inline)) {
    static_assert(!WIDE || (NSK == 4 && NSV == 5), "the constants below are those of a K ring of 4 and a V ring of 5");
    if constexpr (paged) load_pages(next_issue - tree_tiles);
    wait_tiles(std::integral_constant<int, 2>{});
    workgroup_barrier();
    const int t = next_issue++;
    if (t - tree_tiles < full_tiles) issue_full_tile(t); else issue_edge_tile(t);
    advance_slots();
  };

  // The first two tiles go out, then the Q rows are fetched with ordinary loads: the
  // compiler's own wait for them (they are the youngest loads) also covers those tiles,
  // so the prologue needs no hand-counted wait. The rest of the ring follows at the
  // first synchronisation point.
  issue_ready(0, 0, ntiles < 2 ? ntiles : 2);
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    const T* qrow = static_cast<const T*>(p.q) + b * p.q_stride[0] + row_head[qb] * p.q_stride[1] + row_i[qb] * p.q_stride[2] + 8 * lh;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const u32x4 raw = *reinterpret_cast<const u32x4*>(qrow + 16 * ks);
      const u32x4 zero = {0, 0, 0, 0};
      qf[qb][ks] = __builtin_bit_cast(Vec8, row_ok[qb] ? raw : zero);
    }
  }

  f32x16 o[DB][QB];
  float m_run[QB], l_run[QB], alpha_pending[QB];
  bool rescale_pending = false;
  // P goes into the second product rounded to T (flash_tree_attn.py:117). Where a single key carries a
  // large share of a row's weight, that rounding (2^-9 relative for bf16) shows in the output, so a full
  // tile whose largest probability exceeds kHeavyShare of the row's running sum takes the compensating
  // product with the rounding residue as well, like every masked tile. The running sum only grows in
  // units of the final maximum, so no key that ends up with that share of the row escapes. Each lane holds
  // the sum of its part of the keys (half of them, a quarter with key halves); comparing against twice that
  // errs on the side of compensating. The decision is one per wave and tile.
  constexpr float kHeavyShare = 0.25f;
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    m_run[qb] = neg_inf();
    l_run[qb] = 0.f;
    alpha_pending[qb] = 1.f;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int r = 0; r < 16; ++r) o[db][qb][r] = 0.f;
  }

  // per-lane LDS byte addresses of the operand reads (everything else is a constant)
  const uint32_t smem_base = lds_address(smem);
  const uint32_t k_rd = smem_base + TL::at(li, lh);  // + kb * (32/RPB) * pitch + ks * 2 * chunk stride
  // V^T transposing read: 16-lane group g covers head_dim columns 16*(g%2) .. +15 of a
  // 32-column block; lane s of the group addresses key s/4, columns 4*(s%4) .. +3.
  const uint32_t v_rd = smem_base + kVRing + TL::at(4 * lh + (lane & 15) / 4, 2 * ((lane >> 4) & 1) + ((lane >> 1) & 1)) + (lane & 1) * 8;
  constexpr int kVRowsOff8 = (8 / RPB) * TL::kBlockPitch + (8 % RPB) * 16;    // 8 rows further
  constexpr int kVRowsOff16 = (16 / RPB) * TL::kBlockPitch;                   // 16 rows further
  constexpr int kKbOff = (32 / RPB) * TL::kBlockPitch, kKsOff = 2 * TL::kChunkStride;
  constexpr int kKFrags = 2 * KS;   // K fragments per tile (one 128-bit read each)
  constexpr int kVFrags = 4 * DB;   // V^T fragments per tile (two transposing reads each)
  constexpr int kPF = 4;            // fragments requested ahead of the MFMA that consumes them

  // ---- building blocks -------------------------------------------------------------
  // S^T = K Q^T of tile t (fragment queue: kPF reads ahead of the consuming MFMA).
  auto qk_tile = [&](int t, f32x16 (&s)[2][QB]) __attribute__((always_inline)) {
    const uint32_t ka = k_rd + (t % kKSlots) * TL::kTileBytes;
    u32x4 kf[kKFrags];
    static_for<0, kPF>([&](auto f) { kf[f] = lds_read_b128<(f % 2) * kKbOff + (f / 2) * kKsOff>(ka); });
    static_for<0, kKFrags>([&](auto f) {
      constexpr int kNewer = (kKFrags - 1 - f) < (kPF - 1) ? (kKFrags - 1 - f) : (kPF - 1);
      wait_lgkm<kNewer>(kf[f]);
      const Vec8 a = __builtin_bit_cast(Vec8, kf[f]);
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) {
        if constexpr (f / 2 == 0) {
          const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
          s[f % 2][qb] = M::mma(a, qf[qb][f / 2], zero);
        } else {
          s[f % 2][qb] = M::mma(a, qf[qb][f / 2], s[f % 2][qb]);
        }
      }
      if constexpr (f + kPF < kKFrags) kf[f + kPF] = lds_read_b128<((f + kPF) % 2) * kKbOff + ((f + kPF) / 2) * kKsOff>(ka);
    });
  };
  // O^T += V^T P^T of tile t.
  auto pv_tile = [&](int t, const Vec8 (&pf)[QB][4]) __attribute__((always_inline)) {
    const uint32_t va = v_rd + (t % NSV) * TL::kTileBytes;
    u32x2 vlo[kVFrags], vhi[kVFrags];
    auto issue_v = [&](auto g) __attribute__((always_inline)) {
      constexpr int kOff = (g / DB) * kVRowsOff16 + (g % DB) * 4 * TL::kChunkStride;
      vlo[g] = lds_read_tr16_b64<kOff>(va);
      vhi[g] = lds_read_tr16_b64<kOff + kVRowsOff8>(va);
    };
    static_for<0, kPF>(issue_v);
    static_for<0, kVFrags>([&](auto g) {
      constexpr int kNewer = (kVFrags - 1 - g) < (kPF - 1) ? (kVFrags - 1 - g) : (kPF - 1);
      wait_lgkm<2 * kNewer>(vlo[g], vhi[g]);
      const s16x8 both = __builtin_shufflevector(__builtin_bit_cast(s16x4, vlo[g]), __builtin_bit_cast(s16x4, vhi[g]), 0, 1, 2, 3, 4, 5, 6, 7);
      const Vec8 a = __builtin_bit_cast(Vec8, both);
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) o[g % DB][qb] = M::mma(a, pf[qb][g / DB], o[g % DB][qb]);
      if constexpr (g + kPF < kVFrags) issue_v(std::integral_constant<int, g + kPF>{});
    });
  };
  // Both products of one pipelined iteration as ONE fragment stream: P.V of tile t-1
  // (when HAS_PV) followed by K.Q of tile t+1, prefetching across the seam.
  auto mma_stream = [&](auto has_pv_c, int t, const Vec8 (&pf)[QB][4], f32x16 (&s)[2][QB], auto&& valu_slice) __attribute__((always_inline)) {
    constexpr bool HAS_PV = decltype(has_pv_c)::value;
    constexpr int NV = HAS_PV ? kVFrags : 0;
    constexpr int NSTEP = NV + kKFrags;
    const uint32_t va = v_rd + ((t + NSV - 1) % NSV) * TL::kTileBytes;   // tile t-1
    const uint32_t ka = k_rd + ((t + 1) % kKSlots) * TL::kTileBytes;     // tile t+1
    u32x2 vlo[kVFrags], vhi[kVFrags];
    u32x4 kf[kKFrags];
    auto issue = [&](auto i) __attribute__((always_inline)) {
      if constexpr (i < NV) {
        constexpr int g = i;
        constexpr int kOff = (g / DB) * kVRowsOff16 + (g % DB) * 4 * TL::kChunkStride;
        vlo[g] = lds_read_tr16_b64<kOff>(va);
        vhi[g] = lds_read_tr16_b64<kOff + kVRowsOff8>(va);
      } else {
        constexpr int f = i - NV;
        kf[f] = lds_read_b128<(f % 2) * kKbOff + (f / 2) * kKsOff>(ka);
      }
    };
    static_for<0, kPF>(issue);
    static_for<0, NSTEP>([&](auto i) {
      // reads younger than step i's that are already queued: steps i+1 .. i+kPF-1
      constexpr int kLast = (i + kPF - 1) < (NSTEP - 1) ? (i + kPF - 1) : (NSTEP - 1);
      constexpr int kVNewer = (kLast < NV ? kLast : NV - 1) - (i < NV ? i : NV - 1);      // V steps in (i, kLast]
      constexpr int kNewerReads = 2 * (kVNewer > 0 ? kVNewer : 0) + ((kLast - i) - (kVNewer > 0 ? kVNewer : 0));
      if constexpr (i < NV) {
        constexpr int g = i;
        wait_lgkm<kNewerReads>(vlo[g], vhi[g]);
        const s16x8 both = __builtin_shufflevector(__builtin_bit_cast(s16x4, vlo[g]), __builtin_bit_cast(s16x4, vhi[g]), 0, 1, 2, 3, 4, 5, 6, 7);
        const Vec8 a = __builtin_bit_cast(Vec8, both);
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) o[g % DB][qb] = M::mma(a, pf[qb][g / DB], o[g % DB][qb]);
      } else {
        constexpr int f = i - NV;
        wait_lgkm<kNewerReads>(kf[f]);
        const Vec8 a = __builtin_bit_cast(Vec8, kf[f]);
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) {
          if constexpr (f / 2 == 0) {
            const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
            s[f % 2][qb] = M::mma(a, qf[qb][f / 2], zero);
          } else {
            s[f % 2][qb] = M::mma(a, qf[qb][f / 2], s[f % 2][qb]);
          }
        }
      }
      if constexpr (i + kPF < NSTEP) issue(std::integral_constant<int, i + kPF>{});
      // the vector-ALU work that runs in this MFMA's shadow; the fence keeps the compiler
      // from regrouping the two streams (it would put all MFMAs first)
      valu_slice(i, std::integral_constant<int, NSTEP>{});
      schedule_fence();
    });
  };
  // Additive mask values of one tree tile in the accumulator layout (lane = query row,
  // 16 registers = 4 groups of 4 consecutive keys per 32-key block). Indices are clamped
  // instead of branched on, so all loads of a tile are in flight together; rows that
  // start 16-byte aligned fetch each group of 4 keys with one 128-bit load.
  auto load_mask = [&](int key0, float (&mv)[QB][2][16]) __attribute__((always_inline)) {
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      const int64_t mstart = b * p.mask_stride[0] + row_head[qb] * p.mask_stride[1] + row_i[qb] * p.mask_stride[2];
      if (p.mask_packed) {
        // one 64-bit word covers this row's 64 keys of the tile (key0 is a multiple of 64)
        const uint64_t w = static_cast<const uint64_t*>(p.mask)[mstart + (key0 >> 6)];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int j = kb * 32 + (r >> 2) * 8 + 4 * lh + (r & 3);
            mv[qb][kb][r] = (w >> j) & 1 ? 0.f : neg_inf();
          }
        continue;
      }
      const float* mrow = static_cast<const float*>(p.mask) + mstart;
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int rg = 0; rg < 4; ++rg) {
          const int j0 = key0 + kb * 32 + rg * 8 + 4 * lh;
          if (p.mask_vec4 && j0 + 3 < L) {
            const f32x4 v4 = *reinterpret_cast<const f32x4*>(mrow + j0);
#pragma unroll
            for (int e = 0; e < 4; ++e) mv[qb][kb][rg * 4 + e] = v4[e];
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) mv[qb][kb][rg * 4 + e] = mrow[min(j0 + e, L - 1)];
          }
        }
    }
  };
  // Online softmax of one tile's scores: updates m/l, leaves P^T packed to T in `pf` (the
  // B-operand layout of the P.V product) and alpha in alpha_pending / rescale_pending
  // (O is rescaled once the P.V product of the previous tile has been accumulated).
  // MASKED tiles (tree block, ragged last cache tile) scale explicitly, add the mask,
  // blank keys past the limit and keep the rounding residue of P in `s`.
  auto softmax_tile = [&](auto masked_c, f32x16 (&s)[2][QB], Vec8 (&pf)[QB][4], bool tree, int key0, int key_lim, const float (&mv)[QB][2][16]) __attribute__((always_inline)) {
    constexpr bool MASKED = decltype(masked_c)::value;
    bool any_rescale = false;
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
            if (tree) sv = __builtin_fmaf(mv[qb][kb][r], kLog2e, sv);
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
          const float p0 = MASKED ? fast_exp2(s[kb][qb][r] - m_use) : fast_exp2(__builtin_fmaf(s[kb][qb][r], c, -m_use));
          const float p1 = MASKED ? fast_exp2(s[kb][qb][r + 1] - m_use) : fast_exp2(__builtin_fmaf(s[kb][qb][r + 1], c, -m_use));
          s[kb][qb][r] = p0;
          s[kb][qb][r + 1] = p1;
          ps0 += p0;
          ps1 += p1;
        }
      l_run[qb] = l_run[qb] * alpha + (ps0 + ps1);
      m_run[qb] = m_new;
      alpha_pending[qb] = alpha;
      any_rescale |= m_new > m_old;
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
    rescale_pending = wave_any(any_rescale);
  };
  // Whether a full tile with the raw scores `s` holds a heavy key, decided ahead of its softmax (the
  // unfused loops then send it through the masked softmax, which keeps the residue): the row's largest
  // probability against what the lane will at least have summed, its running sum in the new units plus
  // its own largest probability of the tile.
  auto full_tile_is_heavy = [&](const f32x16 (&s)[2][QB]) __attribute__((always_inline)) {
    bool any_heavy = false;
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      float mx0 = fmaxf(s[0][qb][0], s[1][qb][0]), mx1 = fmaxf(s[0][qb][1], s[1][qb][1]);
#pragma unroll
      for (int r = 2; r < 16; r += 2) {
        mx0 = fmaxf(mx0, fmaxf(s[0][qb][r], s[1][qb][r]));
        mx1 = fmaxf(mx1, fmaxf(s[0][qb][r + 1], s[1][qb][r + 1]));
      }
      const float mx_lane = fmaxf(mx0, mx1), mx = half_swap_max(mx_lane, lh);
      const float m_new = fmaxf(m_run[qb], mx * c);
      const float p_top = fast_exp2(__builtin_fmaf(mx, c, -m_new)), p_lane = fast_exp2(__builtin_fmaf(mx_lane, c, -m_new));
      any_heavy |= p_top > 2.f * kHeavyShare * __builtin_fmaf(l_run[qb], fast_exp2(m_run[qb] - m_new), p_lane);
    }
    return wave_any(any_heavy);
  };
  // The rounding residue of a full tile's probabilities `pf`, as a masked tile leaves it in `s`: the
  // scores are computed again (K of the tile is still in its stage) and exponentiated against the
  // running maximum, which is the one `pf` was made with.
  auto residue_of_full_tile = [&](int t, f32x16 (&s)[2][QB], const Vec8 (&pf)[QB][4]) __attribute__((always_inline)) {
    qk_tile(t, s);
#pragma unroll
    for (int qb = 0; qb < QB; ++qb)
#pragma unroll
      for (int kk = 0; kk < 4; ++kk)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int kb = kk >> 1, r = (kk & 1) * 8 + e;
          s[kb][qb][r] = fast_exp2(__builtin_fmaf(s[kb][qb][r], c, -m_run[qb])) - static_cast<float>(pf[qb][kk][e]);
        }
  };
  auto apply_rescale = [&]() __attribute__((always_inline)) {
    if (rescale_pending) {
#pragma unroll
      for (int qb = 0; qb < QB; ++qb)
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
          for (int r = 0; r < 16; ++r) o[db][qb][r] *= alpha_pending[qb];
      rescale_pending = false;
    }
  };
  // ---- the pipeline ----------------------------------------------------------------
  // Iteration t runs the softmax of tile t on the vector ALU while the matrix pipeline
  // works on P.V of tile t-1 and K.Q of tile t+1: two independent instruction streams in
  // one basic block, interleaved by the scheduling hints below. Full cache tiles take
  // this fused body; the ragged last cache tile and the tree tiles run the same three
  // steps one after the other with the masked softmax.
  // Buffers ping-pong between iterations (two statically unrolled roles) so that no
  // register copies are needed: scores sA/sB, packed probabilities pA/pB.
  f32x16 sA[2][QB], sB[2][QB];
  Vec8 pA[QB][4], pB[QB][4];

  // One fused iteration for full tile t: softmax(s_in) -> p_out on the vector ALU while
  // the matrix pipeline does P.V of tile t-1 (p_in, when HAS_PV) and K.Q of tile t+1 -> s_out.
  auto fused = [&](auto has_pv_c, int t, f32x16 (&s_in)[2][QB], f32x16 (&s_out)[2][QB], Vec8 (&p_in)[QB][4], Vec8 (&p_out)[QB][4]) __attribute__((always_inline)) {
    // The lean softmax (full tile: no mask, no key limit) cut into slices, one per MFMA
    // step: steps [0, NA) take the row maximum, step NA exchanges it between the half
    // waves and fixes the new maximum, the following steps exponentiate and pack pairs
    // of values, the last step updates the running sum.
    // The last slice also says whether the tile holds a heavy key (kHeavyShare): then the tile's
    // scores are computed again (K of tile t stays in its stage for this, kKSlots), their rounding
    // residue goes into the registers of the previous tile's probabilities, which the stream has
    // consumed, and is multiplied with V of tile t, which landed with this iteration's
    // synchronisation point. Nothing of this is live across the stream.
    float mx0[QB], mx1[QB], m_new[QB], alpha[QB], ps0[QB], ps1[QB], p_top[QB];
    bool heavy = false;
    auto slice = [&](auto i_c, auto nstep_c) __attribute__((always_inline)) {
      constexpr int I = decltype(i_c)::value, NSTEP = decltype(nstep_c)::value;
      constexpr int NA = NSTEP / 4, EPA = 32 / NA;
      constexpr int NC = NSTEP - NA - 1, PPS = (16 + NC - 1) / NC;
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) {
        if constexpr (I < NA) {
#pragma unroll
          for (int x = I * EPA; x < (I + 1) * EPA; x += 2) {
            const float a0 = s_in[x / 16][qb][x % 16], a1 = s_in[x / 16][qb][x % 16 + 1];
            mx0[qb] = (x == 0) ? a0 : fmaxf(mx0[qb], a0);
            mx1[qb] = (x == 0) ? a1 : fmaxf(mx1[qb], a1);
          }
        } else if constexpr (I == NA) {
          const float mx = half_swap_max(fmaxf(mx0[qb], mx1[qb]), lh);
          m_new[qb] = fmaxf(m_run[qb], mx * c);
          alpha[qb] = fast_exp2(m_run[qb] - m_new[qb]);
          p_top[qb] = fast_exp2(__builtin_fmaf(mx, c, -m_new[qb]));   // the row's largest probability of this tile
          ps0[qb] = 0.f;
          ps1[qb] = 0.f;
        } else {
          constexpr int J0 = (I - NA - 1) * PPS;
#pragma unroll
          for (int j = J0; j < J0 + PPS && j < 16; ++j) {
            const int x = 2 * j, kb = x / 16, r = x % 16;
            const float p0 = fast_exp2(__builtin_fmaf(s_in[kb][qb][r], c, -m_new[qb]));
            const float p1 = fast_exp2(__builtin_fmaf(s_in[kb][qb][r + 1], c, -m_new[qb]));
            const f32x2 pv = {p0, p1};
            const auto pr = __builtin_convertvector(pv, typename M::Vec2);
            if (j & 1) ps1[qb] = M::add_pair(pr, ps1[qb]); else ps0[qb] = M::add_pair(pr, ps0[qb]);
            p_out[qb][kb * 2 + (r >= 8)][r % 8] = pr[0];
            p_out[qb][kb * 2 + (r >= 8)][r % 8 + 1] = pr[1];
          }
        }
      }
      if constexpr (I == NSTEP - 1) {
        bool any_rescale = false, any_heavy = false;
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) {
          l_run[qb] = l_run[qb] * alpha[qb] + (ps0[qb] + ps1[qb]);
          any_rescale |= m_new[qb] > m_run[qb];
          any_heavy |= p_top[qb] > 2.f * kHeavyShare * l_run[qb];
          m_run[qb] = m_new[qb];
          alpha_pending[qb] = alpha[qb];
        }
        rescale_pending = wave_any(any_rescale);
        heavy = wave_any(any_heavy);
      }
    };
    mma_stream(has_pv_c, t, p_in, s_out, slice);
    if (heavy) {
      apply_rescale();   // O in units of this tile's maximum before its residue is added
      residue_of_full_tile(t, s_in, p_out);
#pragma unroll
      for (int qb = 0; qb < QB; ++qb)
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) {
          Vec8 pk;
#pragma unroll
          for (int e = 0; e < 8; ++e) pk[e] = static_cast<T>(s_in[kk >> 1][qb][(kk & 1) * 8 + e]);
          p_in[qb][kk] = pk;
        }
      pv_tile(t, p_in);
    }
  };

  // P.V of a tile whose probabilities are in pA; a masked or heavy tile (`with_residue`) has left P's
  // rounding residue in `res` and takes a second, compensating product with it (packed into pA once the
  // main product has read it).
  auto pv_with_residue = [&](int tile, bool with_residue, f32x16 (&res)[2][QB]) __attribute__((always_inline)) {
    apply_rescale();
    pv_tile(tile, pA);
    if (with_residue) {
#pragma unroll
      for (int qb = 0; qb < QB; ++qb)
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) {
          Vec8 pk;
#pragma unroll
          for (int e = 0; e < 8; ++e) pk[e] = static_cast<T>(res[kk >> 1][qb][(kk & 1) * 8 + e]);
          pA[qb][kk] = pk;
        }
      pv_tile(tile, pA);
    }
  };

  // ---- key halves (MODE == kSplitKeys) -----------------------------------------------
  // Units of a few rows fill one or two waves of a 4-wave workgroup; the others would only
  // request tiles. Here two waves hold the same 32 rows and each takes 32 of a tile's 64 keys
  // (key block kb_own): the same fragments, layouts and steps as the plain loop, half of
  // them per wave, with an online-softmax state of its own that is merged with its
  // partner's through LDS after the last tile (the merge of flash_tree_attn.py:185-211 in
  // its unnormalised form).
  auto qk_half = [&](int t, f32x16& s) __attribute__((always_inline)) {
    const uint32_t ka = k_rd + (t % NSK) * TL::kTileBytes + kb_own * kKbOff;
    u32x4 kf[KS];
    static_for<0, kPF>([&](auto f) { kf[f] = lds_read_b128<f * kKsOff>(ka); });
    static_for<0, KS>([&](auto f) {
      constexpr int kNewer = (KS - 1 - f) < (kPF - 1) ? (KS - 1 - f) : (kPF - 1);
      wait_lgkm<kNewer>(kf[f]);
      const Vec8 a = __builtin_bit_cast(Vec8, kf[f]);
      if constexpr (f == 0) {
        const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        s = M::mma(a, qf[0][f], zero);
      } else {
        s = M::mma(a, qf[0][f], s);
      }
      if constexpr (f + kPF < KS) kf[f + kPF] = lds_read_b128<(f + kPF) * kKsOff>(ka);
    });
  };
  auto pv_half = [&](int t, const Vec8 (&pf)[2]) __attribute__((always_inline)) {
    constexpr int kFrags = 2 * DB;   // two groups of 16 keys x DB blocks of head_dim
    static_assert(KS >= kPF && kFrags >= kPF, "fragment queues deeper than the streams");
    const uint32_t va = v_rd + (t % NSV) * TL::kTileBytes + kb_own * 2 * kVRowsOff16;
    u32x2 vlo[kFrags], vhi[kFrags];
    auto issue_v = [&](auto g) __attribute__((always_inline)) {
      constexpr int kOff = (g / DB) * kVRowsOff16 + (g % DB) * 4 * TL::kChunkStride;
      vlo[g] = lds_read_tr16_b64<kOff>(va);
      vhi[g] = lds_read_tr16_b64<kOff + kVRowsOff8>(va);
    };
    static_for<0, kPF>(issue_v);
    static_for<0, kFrags>([&](auto g) {
      constexpr int kNewer = (kFrags - 1 - g) < (kPF - 1) ? (kFrags - 1 - g) : (kPF - 1);
      wait_lgkm<2 * kNewer>(vlo[g], vhi[g]);
      const s16x8 both = __builtin_shufflevector(__builtin_bit_cast(s16x4, vlo[g]), __builtin_bit_cast(s16x4, vhi[g]), 0, 1, 2, 3, 4, 5, 6, 7);
      o[g % DB][0] = M::mma(__builtin_bit_cast(Vec8, both), pf[g / DB], o[g % DB][0]);
      if constexpr (g + kPF < kFrags) issue_v(std::integral_constant<int, g + kPF>{});
    });
  };
  // Additive mask values of the wave's 32 tree keys from key0 on (load_mask for one key block).
  auto load_mask_half = [&](int key0, float (&mv)[16]) __attribute__((always_inline)) {
    const int64_t mstart = b * p.mask_stride[0] + row_head[0] * p.mask_stride[1] + row_i[0] * p.mask_stride[2];
    if (p.mask_packed) {
      const uint64_t wbits = static_cast<const uint64_t*>(p.mask)[mstart + (key0 >> 6)];
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int j = (key0 & 63) + (r >> 2) * 8 + 4 * lh + (r & 3);
        mv[r] = (wbits >> j) & 1 ? 0.f : neg_inf();
      }
      return;
    }
    const float* mrow = static_cast<const float*>(p.mask) + mstart;
#pragma unroll
    for (int rg = 0; rg < 4; ++rg) {
      const int j0 = key0 + rg * 8 + 4 * lh;
      if (p.mask_vec4 && j0 + 3 < L) {
        const f32x4 v4 = *reinterpret_cast<const f32x4*>(mrow + j0);
#pragma unroll
        for (int e = 0; e < 4; ++e) mv[rg * 4 + e] = v4[e];
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) mv[rg * 4 + e] = mrow[min(j0 + e, L - 1)];
      }
    }
  };
  // softmax_tile for one key block: scores of 32 keys in `s`, P^T of its two 16-key groups out in `pf`.
  auto softmax_half = [&](auto masked_c, f32x16& s, Vec8 (&pf)[2], bool tree, int key0, int key_lim, const float (&mv)[16]) __attribute__((always_inline)) {
    constexpr bool MASKED = decltype(masked_c)::value;
    const float m_old = m_run[0];
    if (MASKED) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int j = key0 + (r >> 2) * 8 + 4 * lh + (r & 3);
        float sv = s[r] * c;
        if (tree) sv = __builtin_fmaf(mv[r], kLog2e, sv);
        s[r] = j < key_lim ? sv : neg_inf();
      }
    }
    float mx0 = s[0], mx1 = s[1];
#pragma unroll
    for (int r = 2; r < 16; r += 2) {
      mx0 = fmaxf(mx0, s[r]);
      mx1 = fmaxf(mx1, s[r + 1]);
    }
    const float mx = half_swap_max(fmaxf(mx0, mx1), lh);
    const float m_new = fmaxf(m_old, MASKED ? mx : mx * c);
    const float m_use = (MASKED && m_new == neg_inf()) ? 0.f : m_new;
    const float alpha = fast_exp2(m_old - m_use);
    float ps0 = 0.f, ps1 = 0.f;
#pragma unroll
    for (int r = 0; r < 16; r += 2) {
      const float p0 = MASKED ? fast_exp2(s[r] - m_use) : fast_exp2(__builtin_fmaf(s[r], c, -m_use));
      const float p1 = MASKED ? fast_exp2(s[r + 1] - m_use) : fast_exp2(__builtin_fmaf(s[r + 1], c, -m_use));
      s[r] = p0;
      s[r + 1] = p1;
      ps0 += p0;
      ps1 += p1;
    }
    l_run[0] = l_run[0] * alpha + (ps0 + ps1);
    m_run[0] = m_new;
    alpha_pending[0] = alpha;
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      Vec8 pk;
#pragma unroll
      for (int e = 0; e < 8; e += 2) {
        const f32x2 pv = {s[kk * 8 + e], s[kk * 8 + e + 1]};
        const auto pr = __builtin_convertvector(pv, typename M::Vec2);
        pk[e] = pr[0];
        pk[e + 1] = pr[1];
        if (MASKED) {  // keep the rounding residue for the compensating product
          s[kk * 8 + e] = pv[0] - static_cast<float>(pr[0]);
          s[kk * 8 + e + 1] = pv[1] - static_cast<float>(pr[1]);
        }
      }
      pf[kk] = pk;
    }
    rescale_pending = wave_any(m_new > m_old);
  };
  auto half_tile_is_heavy = [&](const f32x16& s) __attribute__((always_inline)) {   // full_tile_is_heavy for one key block
    float mx0 = s[0], mx1 = s[1];
#pragma unroll
    for (int r = 2; r < 16; r += 2) {
      mx0 = fmaxf(mx0, s[r]);
      mx1 = fmaxf(mx1, s[r + 1]);
    }
    const float mx_lane = fmaxf(mx0, mx1), mx = half_swap_max(mx_lane, lh);
    const float m_new = fmaxf(m_run[0], mx * c);
    const float p_top = fast_exp2(__builtin_fmaf(mx, c, -m_new)), p_lane = fast_exp2(__builtin_fmaf(mx_lane, c, -m_new));
    return wave_any(p_top > 2.f * kHeavyShare * __builtin_fmaf(l_run[0], fast_exp2(m_run[0] - m_new), p_lane));
  };
  auto pv_half_with_residue = [&](int tile, bool with_residue, const f32x16& res, Vec8 (&pf)[2]) __attribute__((always_inline)) {
    apply_rescale();
    if (with_residue) {   // the compensating product, first: the residue's 16 registers shrink to 4 before any product runs
      Vec8 pr[2];
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) {
        Vec8 pk;
#pragma unroll
        for (int e = 0; e < 8; ++e) pk[e] = static_cast<T>(res[kk * 8 + e]);
        pr[kk] = pk;
      }
      pv_half(tile, pr);
    }
    pv_half(tile, pf);
  };


  // ---- the half-tile pipeline (MODE == kWide) ----------------------------------------
  // A wave holds 64 query rows (two row blocks), so every K or V fragment it reads from LDS
  // feeds two MFMAs. The unit of the pipeline is half a tile (32 keys): the scores of half
  // h of a tile live in sB[h], its probabilities in pA[.][2h], pA[.][2h+1]. The loop over the
  // full cache tiles is hand-scheduled assembly (gen_wide_loop.py -> wide_loop_asm.inc; the
  // schedule and the lazy softmax are described there); the masked halves (tree block, ragged
  // last tile) and everything around the loop are the lambdas below.
  // One masked half tile (32 keys of a tree tile or of the ragged last cache tile), complete:
  // scores, additive mask and key limit, exact online softmax (l and O rescaled at once), P.V,
  // and the compensating P.V product with the rounding residue of P (flash_tree_attn.py:367-373
  // for the tree block). key0 is the first key of the half. The additive terms are gathered
  // here; the step itself is assembly with the register map of the loop (gen_wide_loop.py:
  // gen_masked), so that O, Q, m and l stay where the loop wants them.
  // The additive terms of one half: [qb][16] in the accumulator layout, mask * log2(e), -inf past the key
  // limit. For the tree block these are global loads; phase A issues them ahead of the synchronisation point
  // of their tile, so that they are in flight while the wave waits for the tile and the barrier (the
  // statement takes them as register inputs: gathered right in front of it, their whole latency would show).
  auto gather_madd = [&](auto tree_c, int key0, int key_lim, float (&w_madd)[32]) __attribute__((always_inline)) {
    constexpr bool TREE = decltype(tree_c)::value;
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      float mv[16];
      if constexpr (TREE) {
        const int64_t mstart = b * p.mask_stride[0] + row_head[qb] * p.mask_stride[1] + row_i[qb] * p.mask_stride[2];
        if (p.mask_packed) {
          const uint64_t wbits = static_cast<const uint64_t*>(p.mask)[mstart + (key0 >> 6)];
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int j = (key0 & 63) + (r >> 2) * 8 + 4 * lh + (r & 3);
            mv[r] = (wbits >> j) & 1 ? 0.f : neg_inf();
          }
        } else {
          const float* mrow = static_cast<const float*>(p.mask) + mstart;
#pragma unroll
          for (int rg = 0; rg < 4; ++rg) {
            const int j0 = key0 + rg * 8 + 4 * lh;
            if (p.mask_vec4 && j0 + 3 < L) {
              const f32x4 v4 = *reinterpret_cast<const f32x4*>(mrow + j0);
#pragma unroll
              for (int e = 0; e < 4; ++e) mv[rg * 4 + e] = v4[e];
            } else {
#pragma unroll
              for (int e = 0; e < 4; ++e) mv[rg * 4 + e] = mrow[min(j0 + e, L - 1)];
            }
          }
        }
      }
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int j = key0 + (r >> 2) * 8 + 4 * lh + (r & 3);
        const float add = TREE ? mv[r] * kLog2e : 0.f;
        w_madd[qb * 16 + r] = j < key_lim ? add : neg_inf();
      }
    }
  };
  auto masked_half = [&](auto h_c, int t, const float (&w_madd)[32]) __attribute__((always_inline)) {
    constexpr int H = decltype(h_c)::value;
    float w_o[32 * DB], w_m[2] = {m_run[0], m_run[1]}, w_l[2] = {l_run[0], l_run[1]};
    uint32_t w_q[8 * KS];
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) w_o[(db * 2 + qb) * 16 + r] = o[db][qb][r];
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const u32x4 raw = __builtin_bit_cast(u32x4, qf[qb][ks]);
#pragma unroll
        for (int e = 0; e < 4; ++e) w_q[(qb * KS + ks) * 4 + e] = raw[e];
      }
    }
    const uint32_t w_koffs = (t % NSK) * TL::kTileBytes + H * kKbOff, w_voffs = (t % NSV) * TL::kTileBytes + H * 2 * kVRowsOff16;
    const uint32_t w_krd = k_rd, w_vrd = v_rd;
    const float w_c = c;
    if constexpr (D == 128 && std::is_same<T, __bf16>::value) { if constexpr (H == 0) FTA_WIDE_MASKED_128_BF16_H0(); else FTA_WIDE_MASKED_128_BF16_H1(); }
    else if constexpr (D == 128) { if constexpr (H == 0) FTA_WIDE_MASKED_128_F16_H0(); else FTA_WIDE_MASKED_128_F16_H1(); }
    else if constexpr (std::is_same<T, __bf16>::value) { if constexpr (H == 0) FTA_WIDE_MASKED_64_BF16_H0(); else FTA_WIDE_MASKED_64_BF16_H1(); }
    else { if constexpr (H == 0) FTA_WIDE_MASKED_64_F16_H0(); else FTA_WIDE_MASKED_64_F16_H1(); }
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[db][qb][r] = w_o[(db * 2 + qb) * 16 + r];
      m_run[qb] = w_m[qb];
      l_run[qb] = w_l[qb];
    }
  };

  float mask_vals[QB][2][16];
  const int c0 = tree_tiles;   // first cache tile
  if constexpr (MODE == kPlain) {
    // Plain variant: every tile runs scores -> softmax -> P.V back to back, with the next
    // tile in flight. Its small LDS footprint lets two workgroups share a CU; their
    // phases (matrix, vector, waiting, prologue, epilogue) overlap each other instead
    // of being interleaved by hand.
    for (int t = 0; t < ntiles; ++t) {
      sync_point(t, t, t, ntiles);
      if (!wave_active) continue;
      const bool tree = t < tree_tiles;
      const bool masked = tree || t - c0 >= full_tiles;
      const int key0 = tree ? t * kKeyTile : kv_start + (t - c0) * kKeyTile;
      if (tree) load_mask(key0, mask_vals);   // in flight while the scores are computed
      qk_tile(t, sB);
      const bool with_residue = masked || full_tile_is_heavy(sB);   // (a full tile passes the key limit of the masked softmax whole)
      if (with_residue) softmax_tile(std::true_type{}, sB, pA, tree, key0, tree ? L : kv_end, mask_vals);
      else softmax_tile(std::false_type{}, sB, pA, false, key0, kv_end, mask_vals);
      pv_with_residue(t, with_residue, sB);
    }
    if (!wave_active) return;
  } else if constexpr (KSPLIT) {
    f32x16 s_half;
    Vec8 p_half[2];
    float mask_half[16];
    for (int t = 0; t < ntiles; ++t) {
      sync_point(t, t, t, ntiles);
      if (!wave_active) continue;
      const bool tree = t < tree_tiles;
      const int key0 = (tree ? t * kKeyTile : kv_start + (t - c0) * kKeyTile) + 32 * kb_own;
      if (tree) load_mask_half(key0, mask_half);   // in flight while the scores are computed
      qk_half(t, s_half);
      // tree and ragged tiles, and full tiles in which this wave's 32 keys hold a heavy one (against the
      // wave's own running sum: its partner's keys only add to the row's), keep the residue
      const bool masked = tree || t - c0 >= full_tiles || half_tile_is_heavy(s_half);
      if (masked) softmax_half(std::true_type{}, s_half, p_half, tree, key0, tree ? L : kv_end, mask_half);
      else softmax_half(std::false_type{}, s_half, p_half, false, key0, kv_end, mask_half);
      pv_half_with_residue(t, masked, s_half, p_half);
    }
    // The two waves of a row block merge their states: the wave of the upper key block parks
    // m, l and O in LDS (the rings are idle: every tile has landed and been read once all
    // waves are past the first barrier), the wave of the lower one folds them into its own
    // and goes on to the epilogue. Lane-major layout: word k of lane i at (k * 64 + i).
    constexpr int kStateWords = 2 + 16 * DB;
    static_assert((NW / 2) * kStateWords * 64 * 4 <= 2 * NSK * TL::kTileBytes, "the parked states fit the rings");
    float* park = reinterpret_cast<float*>(smem) + (wave >> 1) * kStateWords * 64 + lane;
    __syncthreads();
    if (kb_own == 1 && wave_active) {
      park[0] = m_run[0];
      park[64] = l_run[0];
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) park[(2 + db * 16 + r) * 64] = o[db][0][r];
    }
    __syncthreads();
    if (kb_own == 1 || !wave_active) return;
    {
      const float m_other = park[0], l_other = park[64];
      const float m_both = fmaxf(m_run[0], m_other);
      const float m_use = m_both == neg_inf() ? 0.f : m_both;
      const float a_own = fast_exp2(m_run[0] - m_use), a_other = fast_exp2(m_other - m_use);
      l_run[0] = l_run[0] * a_own + l_other * a_other;
      m_run[0] = m_both;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[db][0][r] = o[db][0][r] * a_own + park[(2 + db * 16 + r) * 64] * a_other;
    }
  } else if constexpr (WIDE) {
    constexpr std::integral_constant<int, 0> h0{};
    constexpr std::integral_constant<int, 1> h1{};
    // phase A: the tree tiles, half by half, each half a complete masked step
    for (int u = 0; u < tree_tiles; ++u) {
      // (only the first half's terms go ahead: the second half's would have to live through the first statement,
      // which leaves the compiler too few registers to hold them; their cache lines are warm by then)
      float madd[32];
      if (wave_active) gather_madd(std::true_type{}, u * kKeyTile, L, madd);
      sync_point(u, u, u, ntiles);
      if (!wave_active) continue;
      masked_half(h0, u, madd);
      if (u * kKeyTile + 32 < L) {
        gather_madd(std::true_type{}, u * kKeyTile + 32, L, madd);
        masked_half(h1, u, madd);
      }
    }
    // phase B: the full cache tiles through the half-tile pipeline. One synchronisation
    // point per tile, between its two steps: by then every wave has read all of K of tile
    // t (its second half went into the scores during step (t, 0)) and all of V of tile t-1.
    // The hot loop is branch-free apart from its exits: a step that overflowed leaves the
    // loop, is redone exactly outside of it, and the loop is entered again.
    const int full_end = c0 + full_tiles;
    if (full_tiles >= 1) {
      sync_point(c0, c0, c0, kPadRing);   // fills the ring: c0 + NSK tiles requested from here on
      if (wave_active) {
        // Operands of the assembly loop, each one 32-bit value bound to the register the loop
        // names (gen_wide_loop.py: operands()).
        float w_o[32 * DB], w_m[2] = {m_run[0], m_run[1]}, w_l[2] = {l_run[0], l_run[1]};
        uint32_t w_q[8 * KS];
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) {
#pragma unroll
          for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int r = 0; r < 16; ++r) w_o[(db * 2 + qb) * 16 + r] = o[db][qb][r];
#pragma unroll
          for (int ks = 0; ks < KS; ++ks) {
            const u32x4 raw = __builtin_bit_cast(u32x4, qf[qb][ks]);
#pragma unroll
            for (int e = 0; e < 4; ++e) w_q[(qb * KS + ks) * 4 + e] = raw[e];
          }
        }
        // ring stages as byte offsets: K of tile t in stage t % NSK, V in stage t % NSV
        uint32_t w_kcur = (c0 % NSK) * TL::kTileBytes, w_knext = ((c0 + 1) % NSK) * TL::kTileBytes;
        uint32_t w_vcur = (c0 % NSV) * TL::kTileBytes, w_vprev = ((c0 + NSV - 1) % NSV) * TL::kTileBytes;
        uint32_t w_pvoff = w_vcur + 2 * kVRowsOff16;   // the first step reads a landed stage (its P is zero)
        const uint32_t w_kdst = smem_base + wave * TL::kBlockPitch, w_vdst = smem_base + kVRing + wave * TL::kBlockPitch;
        uint32_t w_nt = full_tiles;
        // full tiles still to be requested (the ring holds c0 .. c0 + NSK - 1); with none
        // left the loop re-requests the last full tile, so the address must stay on it
        uint32_t w_nreal = full_end - c0 > NSK ? full_end - c0 - NSK : 0;
        const uint64_t ktile64 = static_cast<uint64_t>(kKeyTile * k_row_bytes), vtile64 = static_cast<uint64_t>(kKeyTile * v_row_bytes);
        const uint64_t krun64 = reinterpret_cast<uint64_t>(k_run) - (w_nreal ? 0 : ktile64), vrun64 = reinterpret_cast<uint64_t>(v_run) - (w_nreal ? 0 : vtile64);
        uint32_t w_krun_lo = static_cast<uint32_t>(krun64), w_krun_hi = static_cast<uint32_t>(krun64 >> 32);
        uint32_t w_vrun_lo = static_cast<uint32_t>(vrun64), w_vrun_hi = static_cast<uint32_t>(vrun64 >> 32);
        const uint32_t w_ktile_lo = static_cast<uint32_t>(ktile64), w_ktile_hi = static_cast<uint32_t>(ktile64 >> 32);
        const uint32_t w_vtile_lo = static_cast<uint32_t>(vtile64), w_vtile_hi = static_cast<uint32_t>(vtile64 >> 32);
        const uint32_t w_kstep_lo = static_cast<uint32_t>(k_step), w_kstep_hi = static_cast<uint32_t>(static_cast<uint64_t>(k_step) >> 32);
        const uint32_t w_vstep_lo = static_cast<uint32_t>(v_step), w_vstep_hi = static_cast<uint32_t>(static_cast<uint64_t>(v_step) >> 32);
        const uint32_t w_krd = k_rd, w_vrd = v_rd, w_koff = k_lane_off, w_voff = v_lane_off;
        const float w_c = c;
        // The statement names M0 among its clobbers (its tile requests set it): the compiler never keeps a
        // value of its own there, which is all its warning about reserved registers says, but it does merge
        // and hoist the M0 writes of its own requests around the statement and must see this one.
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
        if constexpr (D == 128 && std::is_same<T, __bf16>::value) FTA_WIDE_LOOP_128_BF16();
        else if constexpr (D == 128) FTA_WIDE_LOOP_128_F16();
        else if constexpr (std::is_same<T, __bf16>::value) FTA_WIDE_LOOP_64_BF16();
        else FTA_WIDE_LOOP_64_F16();
#pragma clang diagnostic pop
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) {
#pragma unroll
          for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int r = 0; r < 16; ++r) o[db][qb][r] = w_o[(db * 2 + qb) * 16 + r];
          m_run[qb] = w_m[qb];
          l_run[qb] = w_l[qb];
        }
      } else {
        for (int t = c0; t < full_end; ++t) sync_steady();   // the same barriers and loads as the loop
      }
      // Tiles requested past the last full one were stand-ins: the ragged tile, if any, goes out below.
      next_issue = full_end;
      k_slot = full_end % NSK;
      v_slot = full_end % NSV;
    }
    // phase C: the ragged last cache tile, half by half with the masked step
    if (cache_tiles > full_tiles) {
      const int t = full_end;
      if (full_tiles >= 1) sync_point(-1, t, t, ntiles);   // everybody is out of the pipeline: request the tile
      sync_point(t, t, t, ntiles);
      if (wave_active) {
        const int key0 = kv_start + (t - c0) * kKeyTile;
        float madd[32];
        gather_madd(std::false_type{}, key0, kv_end, madd);
        masked_half(h0, t, madd);
        if (key0 + 32 < kv_end) {
          gather_madd(std::false_type{}, key0 + 32, kv_end, madd);
          masked_half(h1, t, madd);
        }
      }
    }
    wait_vmcnt<0>();   // tiles requested past the end are still landing: they must not outlive the workgroup's LDS
    if (!wave_active) return;
  } else {
    // phase A: the tree tiles, one complete step each (scores, masked softmax, P.V twice)
    for (int u = 0; u < tree_tiles; ++u) {
      sync_point(u, u, u, ntiles);
      if (!wave_active) continue;
      load_mask(u * kKeyTile, mask_vals);   // in flight while the scores are computed
      qk_tile(u, sB);
      softmax_tile(std::true_type{}, sB, pA, true, u * kKeyTile, L, mask_vals);
      pv_with_residue(u, true, sB);
    }

    // phase B: fused iterations over the full cache tiles that have a successor
    const int fused_cnt = cache_tiles >= 1 ? min(full_tiles, cache_tiles - 1) : 0;
    int t = c0;
    bool cur_in_B = false;   // which buffer pair holds the current scores / previous P
    if (cache_tiles >= 1) {
      sync_point(c0, c0, c0, ntiles);
      if (wave_active) qk_tile(c0, sA);
    }
    if (fused_cnt >= 1) {
      sync_point(c0 + 1, c0 + 1, c0, ntiles);
      if (wave_active) fused(std::false_type{}, c0, sA, sB, pB, pA);
      t = c0 + 1;
      cur_in_B = true;
      for (; t + 1 < c0 + fused_cnt; t += 2) {
        sync_point(t + 1, t + 1, max(c0, t - 1), ntiles);
        if (wave_active) {
          apply_rescale();
          fused(std::true_type{}, t, sB, sA, pA, pB);
        }
        sync_point(t + 2, t + 2, max(c0, t), ntiles);
        if (wave_active) {
          apply_rescale();
          fused(std::true_type{}, t + 1, sA, sB, pB, pA);
        }
      }
      if (t < c0 + fused_cnt) {
        sync_point(t + 1, t + 1, max(c0, t - 1), ntiles);
        if (wave_active) {
          apply_rescale();
          fused(std::true_type{}, t, sB, sA, pA, pB);
        }
        ++t;
        cur_in_B = false;
      }
    }
    // canonical roles for the tail: current scores in sB, previous P in pA
    bool pv_pending = fused_cnt >= 1;   // P of tile t-1 has not been multiplied yet
    bool prv_masked = false;
    if (!cur_in_B) {
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) sB[kb][qb] = sA[kb][qb];
#pragma unroll
      for (int qb = 0; qb < QB; ++qb)
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) pA[qb][kk] = pB[qb][kk];
    }

    // phase C: the last cache tiles of the split, step by step (the last one may be ragged)
    for (; t < ntiles; ++t) {
      sync_point(t + 1 < ntiles ? t + 1 : -1, t + 1, max(c0, t - 1), ntiles);
      if (!wave_active) continue;
      if (pv_pending) pv_with_residue(t - 1, prv_masked, sA);
      const bool masked = t - c0 >= full_tiles || full_tile_is_heavy(sB);   // ragged, or a heavy key: the residue is kept
      if (masked) softmax_tile(std::true_type{}, sB, pA, false, kv_start + (t - c0) * kKeyTile, kv_end, mask_vals);
      else softmax_tile(std::false_type{}, sB, pA, false, kv_start + (t - c0) * kKeyTile, kv_end, mask_vals);
      // a masked tile leaves the rounding residue of P in sB: park it in sA, the scores of
      // tile t+1 go to sB
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) sA[kb][qb] = sB[kb][qb];
      if (t + 1 < ntiles) qk_tile(t + 1, sB);
      pv_pending = true;
      prv_masked = masked;
    }
    if (!wave_active) return;
    if (pv_pending) pv_with_residue(ntiles - 1, prv_masked, sA);
  }

  // ---- epilogue
  // One split (of the launch, or of this sequence when the merge runs in this kernel):
  // the normalised result goes straight to `out`. Otherwise the normalised partial and
  // its log-sum-exp go to the scratch buffers, to be merged by stage 2 or, with
  // counters, by whichever workgroup of the sequence finishes last (below).
  const bool merge_here = p.counters != nullptr;
  const bool direct = p.num_splits == 1 || (merge_here && S_b == 1);
  float lse_own[QB];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    const float l_tot = half_swap_sum(l_run[qb], lh);
    lse_own[qb] = l_tot > 0.f ? (m_run[qb] + fast_log2(l_tot)) * kLn2 : neg_inf();
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int r = 0; r < 16; ++r) o[db][qb][r] *= inv;
    if (!row_ok[qb]) continue;
    const int head = row_head[qb], i = row_i[qb];
    if (direct) {
      T* dst = static_cast<T*>(p.out) + b * p.out_stride[0] + head * p.out_stride[1] + i * p.out_stride[2];
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int rg = 0; rg < 4; ++rg) {
          typename M::Vec4 v4;
#pragma unroll
          for (int e = 0; e < 4; ++e) v4[e] = static_cast<T>(o[db][qb][rg * 4 + e]);
          *reinterpret_cast<typename M::Vec4*>(dst + db * 32 + rg * 8 + 4 * lh) = v4;
        }
    } else {
      float* dst = p.mid_o + b * p.mid_o_stride[0] + head * p.mid_o_stride[1] + split * p.mid_o_stride[2] + i * p.mid_o_stride[3];
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int rg = 0; rg < 4; ++rg) {
          f32x4 v4;
#pragma unroll
          for (int e = 0; e < 4; ++e) v4[e] = o[db][qb][rg * 4 + e];
          if (merge_here) store_b128_device(dst + db * 32 + rg * 8 + 4 * lh, v4);
          else *reinterpret_cast<f32x4*>(dst + db * 32 + rg * 8 + 4 * lh) = v4;
        }
      if (lh == 0) {
        float* lse_dst = p.mid_lse + b * p.mid_lse_stride[0] + head * p.mid_lse_stride[1] + split * p.mid_lse_stride[2] + i;
        if (merge_here) __hip_atomic_store(lse_dst, lse_own[qb], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        else *lse_dst = lse_own[qb];
      }
    }
  }

  // ---- merge inside this launch (flash_tree_attn.py:339-365 without a second kernel).
  // Every workgroup of a (sequence, unit, row block) bumps that group's counter once its
  // partial has been written through (device-scope stores, all acknowledged); the one
  // that sees S_b - 1 is the last, resets the counter for the next call and merges: its
  // own partial from registers, the others from scratch with device-scope loads. No
  // workgroup ever waits for another, and no cache is flushed or invalidated as a whole.
  if (merge_here && !direct) {
    __shared__ int s_last;
    wait_vmcnt<0>();      // this thread's partial stores are acknowledged ...
    __syncthreads();      // ... and so are those of every thread of the workgroup
    if (tid == 0) {
      int32_t* cnt = p.counters + (static_cast<int64_t>(b) * p.units + w.unit) * p.row_blocks + w.row_block;
      const int old = __hip_atomic_fetch_add(cnt, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      const int last = old == S_b - 1;
      if (last) __hip_atomic_store(cnt, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      s_last = last;
    }
    __syncthreads();
    if (!s_last) return;
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      if (!row_ok[qb]) continue;
      const int head = row_head[qb], i = row_i[qb];
      const float* lse_p = p.mid_lse + b * p.mid_lse_stride[0] + head * p.mid_lse_stride[1] + i;
      const float* mo = p.mid_o + b * p.mid_o_stride[0] + head * p.mid_o_stride[1] + i * p.mid_o_stride[3] + 4 * lh;
      // log-sum-exp of the other splits: the first four in one round trip, kept for the weights
      float lse_c[4];
#pragma unroll
      for (int s = 0; s < 4; ++s)
        lse_c[s] = (s < S_b && s != split) ? __hip_atomic_load(lse_p + s * p.mid_lse_stride[2], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                                           : neg_inf();
      float mx = fmaxf(fmaxf(lse_own[qb], fmaxf(lse_c[0], lse_c[1])), fmaxf(lse_c[2], lse_c[3]));
      for (int s = 4; s < S_b; ++s)
        if (s != split) mx = fmaxf(mx, __hip_atomic_load(lse_p + s * p.mid_lse_stride[2], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
      float wsum = 0.f;
      if (mx != neg_inf()) {
        const float w_own = fast_exp2((lse_own[qb] - mx) * kLog2e);
        wsum = w_own;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
          for (int r = 0; r < 16; ++r) o[db][qb][r] *= w_own;
        for (int s = 0; s < S_b; ++s) {
          if (s == split) continue;
          const float lse_s = s == 0 ? lse_c[0] : s == 1 ? lse_c[1] : s == 2 ? lse_c[2] : s == 3 ? lse_c[3]
                            : __hip_atomic_load(lse_p + s * p.mid_lse_stride[2], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          const float wgt = fast_exp2((lse_s - mx) * kLog2e);
          wsum += wgt;
          const float* src = mo + s * p.mid_o_stride[2];
          f32x4 part[DB][4];
#pragma unroll
          for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int rg = 0; rg < 4; ++rg) part[db][rg] = load_b128_device(src + db * 32 + rg * 8);
          wait_vmcnt<0>();
#pragma unroll
          for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int rg = 0; rg < 4; ++rg) settle(part[db][rg]);
#pragma unroll
          for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int rg = 0; rg < 4; ++rg)
#pragma unroll
              for (int e = 0; e < 4; ++e) o[db][qb][rg * 4 + e] += wgt * part[db][rg][e];
        }
      }
      const float inv = wsum > 0.f ? 1.f / wsum : 0.f;
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
    }
  }
}

template <typename T, int D, int QB, int NW, int NS, int MODE, bool PAGED>
int launch(const KernelParams& p, hipStream_t stream) {
  // K ring of NS stages (+ 1 pipelined) + V ring of NS (+ 2 pipelined, + 1 half-tile pipeline)
  constexpr int kSmem = (MODE == kPipelined ? 2 * NS + 3 : MODE == kWide ? 2 * NS + 1 : 2 * NS) * TileLayout<D>::kTileBytes;   // kPlain, kSplitKeys: 2 * NS
  static_assert(kSmem + 3 * 1024 <= 160 * 1024, "LDS budget (rings + the static arrays of item_by_order)");
  auto kern = stage1_mfma_kernel<T, D, QB, NW, NS, MODE, PAGED>;
  if (kSmem > 64 * 1024) {
    // Raising the dynamic-LDS limit is a driver call: once per kernel and device, not per launch.
    static thread_local int configured_device = -1;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return FTA_ERR_NO_DEVICE;
    if (configured_device != dev) {
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, kSmem) != hipSuccess)
        return FTA_ERR_LAUNCH;
      configured_device = dev;
    }
  }
  const int64_t grid = static_cast<int64_t>(p.bsz) * p.units * p.row_blocks * p.num_splits;
  if (grid <= 0 || grid > 0x7fffffffLL) return FTA_ERR_SHAPE;
  if (p.rows_per_wg != (MODE == kSplitKeys ? NW / 2 : NW) * 32 * QB) return FTA_ERR_SHAPE;   // the plan's row blocks are this kernel's
  return launch_checked(kern, dim3(static_cast<unsigned>(grid)), dim3(NW * 64), kSmem, stream, p);
}


}  // namespace
}  // namespace fta
