/*
 * fta.h - C ABI of the MI355X (gfx950) tree-attention decode library.
 *
 * The reference exposes this path as one Python function,
 *   flash_decoding_attention(q, k_cache, v_cache, current_k, current_v, mask,
 *                            kv_seq_len, block_size, max_seq_len_in_batch,
 *                            output, mid_output, mid_output_lse, sm_scale,
 *                            kv_group_num)            (flash_tree_attn.py:216-231)
 * which launches two Triton kernels and a dozen eager ops. This header is what a
 * binding for that function talks to: plain pointers, sizes and element strides,
 * no torch types. Every function returns 0 (FTA_OK) or a negative fta_status and
 * never throws, allocates device memory, or synchronises the device.
 */
#ifndef FTA_H_
#define FTA_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FTA_ABI_VERSION 3

typedef enum fta_status {
  FTA_OK = 0,
  FTA_ERR_NULL_POINTER = -1,      /* a required pointer is NULL */
  FTA_ERR_HEAD_DIM = -2,          /* head_dim not in {32,64,128,256}   (flash_tree_attn.py:263) */
  FTA_ERR_BLOCK_SIZE = -3,        /* block_size not in {16,32,64,128}  (flash_tree_attn.py:268) */
  FTA_ERR_CACHE_LEN_MISMATCH = -4,/* k_cache/v_cache lengths differ    (flash_tree_attn.py:264) */
  FTA_ERR_SCRATCH_TOO_SMALL = -5, /* mid_o/mid_lse hold fewer splits than planned (flash_tree_attn.py:286-291) */
  FTA_ERR_DTYPE = -6,             /* unknown dtype / length dtype enum */
  FTA_ERR_SHAPE = -7,             /* non-positive size, Hq != Hkv*G, current_k heads not Hkv or Hq */
  FTA_ERR_STRIDE = -8,            /* negative stride, or rows not 16-byte aligned for the vector path */
  FTA_ERR_UNSUPPORTED = -9,       /* combination no kernel is instantiated for */
  FTA_ERR_LAUNCH = -10,           /* HIP reported a launch error */
  FTA_ERR_NO_DEVICE = -11         /* no gfx950 device is visible to HIP */
} fta_status;

typedef enum fta_dtype { FTA_F32 = 0, FTA_F16 = 1, FTA_BF16 = 2 } fta_dtype;
typedef enum fta_len_dtype { FTA_I32 = 0, FTA_I64 = 1 } fta_len_dtype;
/* Form of the tree mask. The reference adds a float tensor to the tree logits
 * (flash_tree_attn.py:368); a draft tree only ever needs "attend / do not attend", which
 * packs into one 64-bit word per query row and 64 tree positions. */
typedef enum fta_mask_kind {
  FTA_MASK_ADDITIVE_F32 = 0, /* float32, added to the tree logits (0 = attend, -inf = blocked, any other bias) */
  FTA_MASK_PACKED_U64 = 1    /* uint64 [.., q_len, ceil(q_len/64)]: bit (j % 64) of word j / 64 set = row attends tree key j */
} fta_mask_kind;

/* Which stage-1 kernel a plan selects. */
typedef enum fta_kernel {
  FTA_KERNEL_SHUFFLE = 0,  /* wavefront-shuffle reductions: any dtype / head_dim / q_len / sign of sm_scale */
  FTA_KERNEL_MFMA = 1,     /* MFMA tiles: f16/bf16, head_dim 64/128/256, sm_scale > 0; any number of rows */
  FTA_KERNEL_MFMA_WIDE = 2,/* only as fta_args.force_kernel: the MFMA kernel with 64 query rows per wave and the
                              hand-scheduled half-tile loop, for units of more than 128 rows on contiguous caches,
                              head_dim 64/128. A plan reports it as FTA_KERNEL_MFMA with mfma_loop = 1. Not the library's
                              choice anywhere: slower than the default loop where it was timed, and bf16 rows that a few
                              keys carry can leave atol 2e-3 / rtol 1e-2 in it (the other loops compensate for that). */
  FTA_KERNEL_MFMA_SPLIT_KEYS = 3 /* only as fta_args.force_kernel: the MFMA kernel for units of at most 64 query rows,
                              head_dim 64/128, with two waves per 32-row block that each take half of a tile's keys
                              (all four waves of a workgroup compute). A plan reports it as FTA_KERNEL_MFMA with
                              rows_per_wg = 64 and mfma_loop = 2. */
} fta_kernel;

/*
 * One call of the path. All strides are in ELEMENTS of the tensor they index;
 * the innermost (head_dim, and mask column) stride must be 1.
 * Shapes (reference docstring, flash_tree_attn.py:235-246):
 *   q         [bsz, num_q_heads, q_len, head_dim]
 *   k_cache   [bsz, num_kv_heads, cache_len, head_dim]   (same for v_cache)
 *   cur_k     [bsz, cur_heads, q_len, head_dim]          cur_heads = num_kv_heads or num_q_heads
 *   mask      float32, additive (flash_tree_attn.py:368); strides may be 0 to broadcast
 *             over batch and/or head, i.e. [q_len,q_len] .. [bsz,num_q_heads,q_len,q_len];
 *             or, with mask_kind FTA_MASK_PACKED_U64, uint64 [.., q_len, ceil(q_len/64)]
 *             (8 bytes per row and 64 tree keys instead of 256; strides in uint64 words)
 *   kv_seq_len[bsz] int32 or int64 (flash_tree_attn.py:434 passes int64)
 *   out       [bsz, num_q_heads, q_len, head_dim], dtype of q: the FINAL result
 *   mid_o     float32 [bsz, num_q_heads, mid_splits, q_len, head_dim]  (flash_tree_attn.py:276-279)
 *   mid_lse   float32 [bsz, num_q_heads, mid_splits, q_len]            (flash_tree_attn.py:280-281)
 * Paged caches (the layout the reference's kernel comments and docstring still describe,
 * flash_tree_attn.py:17-18,233, although its code addresses one contiguous cache per
 * sequence, :72-73): with block_table given, k_cache / v_cache are page pools
 *   [num_pages, num_kv_heads, page_size, head_dim]   (k_stride = page, head, position in page)
 * and position j of sequence b lives in page block_table[b, j / page_size] at row
 * j % page_size. cache_len is then the logical capacity per sequence
 * (<= pages per sequence * page_size) and bounds kv_seq_len as before.
 * mid_o / mid_lse are scratch; they may be NULL when the plan has num_splits == 1.
 *   counters  int32 [counter_elems], optional. When given (and the plan reports
 *             counter_elems > 0), fta_decode runs ONE launch: the workgroup that
 *             finishes a sequence's last split merges the partials itself, which
 *             replaces the second kernel of flash_tree_attn.py:339-365 and the gap
 *             between the two launches. Contract: all zero on entry; the kernel leaves
 *             them all zero again, so one buffer zeroed once serves every later call on
 *             the same stream; calls that may overlap in time need buffers of their
 *             own. A launch that fails, or a kernel that does not run to its end (a
 *             device fault, a reset), may leave counts behind: zero the buffer again
 *             before its next use, or no workgroup of a later call ever sees the last
 *             arrival and `out` stays unwritten, without an error. The buffer must stay
 *             allocated until every launch that was given it has finished; a captured
 *             graph holds its address for as long as the graph is replayed, and replays
 *             must not overlap eager calls on the same buffer. NULL keeps the two-launch
 *             path.
 */
typedef struct fta_args {
  const void* q;
  const void* k_cache;
  const void* v_cache;
  const void* cur_k;
  const void* cur_v;
  const void* mask;         /* float32 or uint64 words, see mask_kind */
  const void* kv_seq_len;
  void* out;
  float* mid_o;
  float* mid_lse;
  int32_t* counters;
  const int32_t* block_table; /* NULL = contiguous caches; else int32 [bsz, pages per sequence], see below */

  int32_t bsz;
  int32_t num_q_heads;
  int32_t num_kv_heads;
  int32_t cur_heads;
  int32_t q_len;
  int32_t head_dim;
  int32_t cache_len;        /* k_cache.size(2) */
  int32_t v_cache_len;      /* v_cache.size(2), must equal cache_len */
  int32_t block_size;       /* the reference's split granularity (flash_tree_attn.py:268) */
  int32_t max_seq_len_hint; /* max_seq_len_in_batch: an upper bound of kv_seq_len that sizes the grid and the scratch, or
                               0 = cache_len. How the keys are cut into chunks follows the real lengths (fta_plan_out) */
  int32_t mid_splits;       /* size(2) of mid_o / mid_lse, 0 when they are NULL */
  int32_t dtype;            /* fta_dtype of q/k/v/cur/out */
  int32_t len_dtype;        /* fta_len_dtype of kv_seq_len */
  int32_t force_splits;     /* 0 = heuristic; >0 pins the split count (tuning, tests) */
  int32_t force_kernel;     /* -1 = heuristic; else an fta_kernel (FTA_ERR_UNSUPPORTED where that kernel cannot run the call) */
  int32_t counter_elems;    /* int32 elements behind `counters`, 0 when it is NULL */
  int32_t mask_kind;        /* fta_mask_kind of `mask` */
  int32_t page_size;        /* positions per page, one of 16, 32, 64, 128; ignored without block_table */
  float sm_scale;

  int64_t q_stride[3];      /* batch, head, row */
  int64_t k_stride[3];      /* batch, head, position */
  int64_t v_stride[3];
  int64_t ck_stride[3];     /* batch, head, row */
  int64_t cv_stride[3];
  int64_t mask_stride[3];   /* batch, head, row (column / word stride is 1), in elements of the mask's type */
  int64_t out_stride[3];    /* batch, head, row */
  int64_t mid_o_stride[4];  /* batch, head, split, row */
  int64_t mid_lse_stride[3];/* batch, head, split */
  int64_t block_table_stride; /* batch stride of block_table */
} fta_args;

#define FTA_LEN_BUCKETS 16

/* What the split heuristic decided for one fta_args (pure host arithmetic). */
typedef struct fta_plan_out {
  int32_t kernel;         /* fta_kernel */
  int32_t num_splits;     /* grid extent along the KV sequence; 1 = single pass, no scratch, no stage 2 */
  int32_t chunk;          /* keys per split for a batch at the length cap; a multiple of block_size and of the kernel's key tile */
  int32_t rows_per_group; /* kv_group_num * q_len: query rows that share one K/V stream */
  int32_t rows_per_wg;    /* query rows one workgroup holds */
  int32_t row_blocks;     /* ceil(rows_per_group / rows_per_wg) */
  int32_t num_workgroups; /* stage-1 grid size */
  int32_t counter_elems;  /* int32 counters the single-launch path needs; 0 = this plan has no such path */
  int32_t single_launch;  /* 1 where the single-launch path is expected to be the faster one (two splits, one
                             round of workgroups: the last workgroup of a sequence merges alone, which does
                             not pay for more) */
  int32_t mfma_loop;      /* MFMA kernel: 0 = 32-row waves (4 per 128-row workgroup, 8 per 256-row one), 1 = 256-row workgroups of
                             4 waves x 64 rows (half-tile loop), 2 = 64-row workgroups, two waves per 32-row block (key halves) */
  int64_t mid_o_elems;    /* float32 elements a dense mid_o for this plan needs */
  int64_t mid_lse_elems;
  /* Keys per split by the batch's longest sequence: the kernels read the lengths, find the first i
   * with max(kv_seq_len) <= len_bound[i] (the last entry if none) and cut every sequence into chunks
   * of chunk_by_len[i] keys, so that a length cap far above the real lengths (a cache allocated for
   * the longest admissible context, a page table's full width) does not leave most splits empty.
   * len_bound ascends to the cap; chunk_by_len[FTA_LEN_BUCKETS - 1] == chunk. Sequence b then fills
   * min(num_splits, max(1, ceil(kv_seq_len[b] / that chunk))) split slots of mid_o / mid_lse. */
  int32_t len_bound[FTA_LEN_BUCKETS];
  int32_t chunk_by_len[FTA_LEN_BUCKETS];
} fta_plan_out;

/* ABI version of the loaded library (== FTA_ABI_VERSION it was built with). */
int fta_abi_version(void);

/* Static, human-readable text for a status code. */
const char* fta_strerror(int status);

/* Argument checks of flash_tree_attn.py:263-268,286-291 plus the stride/dtype
 * contract of this library. Pure host code: callable without a GPU; pointers are
 * only compared against NULL, never dereferenced. */
int fta_validate(const fta_args* args);

/* The split-count heuristic that replaces "one split per block_size keys"
 * (flash_tree_attn.py:266-274, :293-299). Pure host code. `num_cus` is the number
 * of compute units to fill (256 on MI355X); pass 0 to use that default. Does not
 * look at kv_seq_len values (no host sync, unlike flash_tree_attn.py:272). Scratch that is
 * already in the arguments (mid_o, mid_lse, mid_splits) and holds fewer slots than the
 * heuristic would take bounds its split count (a caller of the reference sizes it from the
 * batch's longest sequence); scratch sized from this function's own answer changes nothing,
 * so fta_decode, which plans from the arguments it is given, runs the plan reported here. */
int fta_plan(const fta_args* args, int num_cus, fta_plan_out* plan);

/* Runs the whole path (stage 1 with the tree block folded in, then the LSE merge
 * when the plan has more than one split: inside the same launch when `counters`
 * is given, as a second kernel otherwise) on `hip_stream` (a hipStream_t; NULL is
 * the default stream). Replaces flash_tree_attn.py:293-376. Asynchronous. */
int fta_decode(const fta_args* args, void* hip_stream);

/* The two halves of fta_decode, for callers that place something between them: a
 * deployment that shards the KV sequence over devices runs stage 1 on each shard,
 * exchanges the fp32 partials (mid_o, mid_lse) and runs stage 2 on the gathered set;
 * a profiler times them separately. fta_decode_stage1 replaces flash_tree_attn.py:
 * 295-334 and :367-373 (with one split it writes `out` directly and stage 2 is a
 * no-op); fta_decode_stage2 replaces flash_tree_attn.py:339-365. */
int fta_decode_stage1(const fta_args* args, void* hip_stream);
int fta_decode_stage2(const fta_args* args, void* hip_stream);

/*
 * Accepted-path KV append: the step that follows this op in a speculative-decoding loop
 * (the reference leaves it to the caller: README.md:63-64 "kv cache management"). For
 * every sequence b and a < accept_len[b]:
 *     k_cache[b, h, T_b + a, :] = cur_k[b, h, accept_idx[b, a], :]      (same for v)
 * with T_b = kv_seq_len[b], then kv_seq_len_out[b] = T_b + accept_len[b]. Rows that would
 * land past cache_len are dropped and the new length is clamped to cache_len (there is
 * no host sync to report it). accept_len is clamped to [0, max_accept]; an accept_idx
 * outside [0, q_len) drops that row's copy but still counts it. Strides in elements,
 * inner stride 1, rows 16-byte aligned, as for fta_args. kv_seq_len_out may alias
 * kv_seq_len (in-place update; then the lengths are written by a second, one-block
 * launch after the copies have read them).
 */
typedef struct fta_append_args {
  void* k_cache;             /* [bsz, num_kv_heads, cache_len, head_dim] */
  void* v_cache;
  const void* cur_k;         /* [bsz, num_kv_heads, q_len, head_dim] */
  const void* cur_v;
  const int32_t* accept_idx; /* [bsz, max_accept] tree positions of the accepted path, in order */
  const void* accept_len;    /* [bsz], len_dtype */
  const void* kv_seq_len;    /* [bsz], len_dtype */
  void* kv_seq_len_out;      /* [bsz], len_dtype */
  const int32_t* block_table;/* NULL = contiguous caches; else int32 [bsz, pages per sequence] as in fta_args:
                                k_cache / v_cache are page pools, k_stride = (page, head, position in page) */

  int32_t bsz;
  int32_t num_kv_heads;
  int32_t q_len;
  int32_t head_dim;
  int32_t cache_len;         /* capacity per sequence (paged: <= pages per sequence * page_size) */
  int32_t max_accept;
  int32_t dtype;             /* fta_dtype */
  int32_t len_dtype;         /* fta_len_dtype of accept_len, kv_seq_len and kv_seq_len_out */
  int32_t page_size;         /* 16, 32, 64 or 128; ignored without block_table */
  int32_t reserved;

  int64_t k_stride[3];       /* batch, head, position */
  int64_t v_stride[3];
  int64_t ck_stride[3];      /* batch, head, row */
  int64_t cv_stride[3];
  int64_t accept_idx_stride; /* batch stride of accept_idx */
  int64_t block_table_stride;/* batch stride of block_table */
} fta_append_args;

/* Validates, then launches on `hip_stream`. Asynchronous; allocates nothing. */
int fta_append_kv(const fta_append_args* args, void* hip_stream);

/* Number of compute units of the current HIP device, or a negative fta_status. */
int fta_device_cus(void);

#ifdef __cplusplus
}
#endif
#endif /* FTA_H_ */
