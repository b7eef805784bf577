// Accepted-path KV append: copies the accepted tree rows of current_k / current_v to
// the end of each sequence's cache and advances kv_seq_len. The reference has no code
// for it (README.md:63-64 lists cache management as the caller's job); it is the step
// that follows the tree-attention call in a speculative-decoding loop.
//
// Pure data movement, tiny (accepted rows x kv heads x 2 x head_dim elements): one
// thread moves 16 bytes, a workgroup of 256 threads covers 256 such pieces of the
// flattened (sequence, accepted row, head, K|V, 16-byte piece) index space, so a whole
// call is a handful of workgroups and launch-bound.
#include <hip/hip_runtime.h>

#include <algorithm>

#include "fta_device.h"

namespace fta {
namespace {

struct AppendParams {
  char* k; char* v;
  const char* ck; const char* cv;
  const int32_t* idx;
  const int32_t* table;  // null = contiguous caches
  const void* acc_len; const void* lens; void* lens_out;
  int32_t bsz, heads, q_len, cache_len, max_accept, len_is_i64;
  int32_t row_bytes;     // head_dim * element size
  int32_t write_lens;    // 1: this launch also writes the new lengths (out does not alias in)
  int64_t k_stride[3], v_stride[3], ck_stride[3], cv_stride[3];   // in BYTES
  int64_t idx_stride, table_stride;
  int32_t page_shift;
};

__device__ __forceinline__ int clamp_i64(int64_t v, int lo, int hi) {
  return static_cast<int>(v < lo ? lo : (v > hi ? hi : v));
}

__device__ __forceinline__ void store_len(void* out, int is_i64, int b, int v) {
  if (is_i64) static_cast<int64_t*>(out)[b] = v; else static_cast<int32_t*>(out)[b] = v;
}

__global__ void __launch_bounds__(256) append_kv_kernel(const AppendParams p) {
  const int pieces = p.row_bytes / 16;
  const int64_t per_row = static_cast<int64_t>(p.heads) * 2 * pieces;
  const int64_t per_seq = per_row * p.max_accept;
  const int64_t gid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (p.write_lens && gid < p.bsz) {
    const int b = static_cast<int>(gid);
    const int t = clamp_i64(load_len(p.lens, p.len_is_i64, b), 0, p.cache_len);
    const int n = clamp_i64(load_len(p.acc_len, p.len_is_i64, b), 0, p.max_accept);
    store_len(p.lens_out, p.len_is_i64, b, min(t + n, p.cache_len));
  }
  if (gid >= per_seq * p.bsz) return;
  const int b = static_cast<int>(gid / per_seq);
  int64_t r = gid % per_seq;
  const int a = static_cast<int>(r / per_row); r %= per_row;
  const int h = static_cast<int>(r / (2 * pieces)); r %= 2 * pieces;
  const int is_v = static_cast<int>(r / pieces);
  const int piece = static_cast<int>(r % pieces);
  const int t = clamp_i64(load_len(p.lens, p.len_is_i64, b), 0, p.cache_len);
  const int n = clamp_i64(load_len(p.acc_len, p.len_is_i64, b), 0, p.max_accept);
  if (a >= n || t + a >= p.cache_len) return;
  const int src_row = p.idx[b * p.idx_stride + a];
  if (src_row < 0 || src_row >= p.q_len) return;
  const char* src = is_v ? p.cv + b * p.cv_stride[0] + h * p.cv_stride[1] + src_row * p.cv_stride[2]
                         : p.ck + b * p.ck_stride[0] + h * p.ck_stride[1] + src_row * p.ck_stride[2];
  int64_t outer = b, pos = t + a;   // contiguous: [batch, head, position]
  if (p.table) {                     // paged: [page, head, position in page]
    outer = p.table[b * p.table_stride + (pos >> p.page_shift)];
    pos &= (1 << p.page_shift) - 1;
  }
  char* dst = is_v ? p.v + outer * p.v_stride[0] + h * p.v_stride[1] + pos * p.v_stride[2]
                   : p.k + outer * p.k_stride[0] + h * p.k_stride[1] + pos * p.k_stride[2];
  *reinterpret_cast<u32x4*>(dst + piece * 16) = *reinterpret_cast<const u32x4*>(src + piece * 16);
}

// In-place length update, launched after the copies (which read the old lengths).
__global__ void __launch_bounds__(256) append_len_kernel(const AppendParams p) {
  const int b = blockIdx.x * blockDim.x + threadIdx.x;
  if (b >= p.bsz) return;
  const int t = clamp_i64(load_len(p.lens, p.len_is_i64, b), 0, p.cache_len);
  const int n = clamp_i64(load_len(p.acc_len, p.len_is_i64, b), 0, p.max_accept);
  store_len(p.lens_out, p.len_is_i64, b, min(t + n, p.cache_len));
}

}  // namespace
}  // namespace fta

extern "C" int fta_append_kv(const fta_append_args* args, void* hip_stream) {
  using namespace fta;
  if (!args) return FTA_ERR_NULL_POINTER;
  const fta_append_args& a = *args;
  if (!a.k_cache || !a.v_cache || !a.cur_k || !a.cur_v || !a.accept_idx || !a.accept_len || !a.kv_seq_len || !a.kv_seq_len_out)
    return FTA_ERR_NULL_POINTER;
  if (a.dtype != FTA_F32 && a.dtype != FTA_F16 && a.dtype != FTA_BF16) return FTA_ERR_DTYPE;
  if (a.len_dtype != FTA_I32 && a.len_dtype != FTA_I64) return FTA_ERR_DTYPE;
  if (a.head_dim != 32 && a.head_dim != 64 && a.head_dim != 128 && a.head_dim != 256) return FTA_ERR_HEAD_DIM;
  if (a.bsz <= 0 || a.num_kv_heads <= 0 || a.q_len <= 0 || a.cache_len < 0 || a.max_accept < 0 || a.accept_idx_stride < 0)
    return FTA_ERR_SHAPE;
  if (a.block_table) {
    if (a.page_size != 16 && a.page_size != 32 && a.page_size != 64 && a.page_size != 128) return FTA_ERR_BLOCK_SIZE;
    if (a.block_table_stride < 0 || a.block_table_stride * a.page_size < a.cache_len) return FTA_ERR_SHAPE;
  }
  const int es = a.dtype == FTA_F32 ? 4 : 2;
  const int vec = 16 / es;
  const int64_t* strides[] = {a.k_stride, a.v_stride, a.ck_stride, a.cv_stride};
  for (const int64_t* s : strides)
    for (int i = 0; i < 3; ++i)
      if (s[i] < 0 || s[i] % vec != 0) return FTA_ERR_STRIDE;
  const void* ptrs[] = {a.k_cache, a.v_cache, a.cur_k, a.cur_v};
  for (const void* ptr : ptrs)
    if (reinterpret_cast<uintptr_t>(ptr) % 16 != 0) return FTA_ERR_STRIDE;

  AppendParams p{};
  p.k = static_cast<char*>(a.k_cache); p.v = static_cast<char*>(a.v_cache);
  p.ck = static_cast<const char*>(a.cur_k); p.cv = static_cast<const char*>(a.cur_v);
  p.idx = a.accept_idx; p.acc_len = a.accept_len; p.lens = a.kv_seq_len; p.lens_out = a.kv_seq_len_out;
  p.bsz = a.bsz; p.heads = a.num_kv_heads; p.q_len = a.q_len; p.cache_len = a.cache_len; p.max_accept = a.max_accept;
  p.len_is_i64 = a.len_dtype == FTA_I64;
  p.row_bytes = a.head_dim * es;
  const bool in_place = a.kv_seq_len_out == a.kv_seq_len;
  p.write_lens = !in_place;
  for (int i = 0; i < 3; ++i) {
    p.k_stride[i] = a.k_stride[i] * es; p.v_stride[i] = a.v_stride[i] * es;
    p.ck_stride[i] = a.ck_stride[i] * es; p.cv_stride[i] = a.cv_stride[i] * es;
  }
  p.idx_stride = a.accept_idx_stride;
  p.table = a.block_table; p.table_stride = a.block_table_stride;
  p.page_shift = a.page_size == 16 ? 4 : a.page_size == 32 ? 5 : a.page_size == 64 ? 6 : 7;

  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return FTA_ERR_NO_DEVICE;
  hipStream_t stream = static_cast<hipStream_t>(hip_stream);
  const int64_t threads = std::max<int64_t>(static_cast<int64_t>(a.bsz) * a.max_accept * a.num_kv_heads * 2 * (p.row_bytes / 16), a.bsz);
  const int64_t grid = (threads + 255) / 256;
  if (grid > 0x7fffffffLL) return FTA_ERR_SHAPE;
  if (int st = fta::launch_checked(append_kv_kernel, dim3(static_cast<unsigned>(grid)), dim3(256), 0, stream, p)) return st;
  if (in_place) return fta::launch_checked(append_len_kernel, dim3((a.bsz + 255) / 256), dim3(256), 0, stream, p);
  return FTA_OK;
}
