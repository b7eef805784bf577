// Stage 1, MFMA variant: the instantiations for workgroups of 32-row waves (plain loop and
// 8-wave pipelined loop) and the entry point that picks an instantiation. The kernel itself
// is the template in stage1_mfma_kernel.h; the 64-row-wave instantiations are compiled in
// stage1_mfma_wide.hip.
#include "stage1_mfma_kernel.h"

namespace fta {
namespace {

int dtype_of(_Float16) { return FTA_F16; }
int dtype_of(__bf16) { return FTA_BF16; }

template <typename T, bool PAGED>
int launch_t(const KernelParams& p, int head_dim, hipStream_t stream) {
  if (p.rows_per_wg == 256) {
    // 4 waves x 64 rows with the half-tile pipeline (stage1_mfma_wide.hip), or
    // 8 waves x 32 rows, pipelined over whole tiles, K requested 3 tiles ahead into 4 stages / V ring 5; one workgroup per CU either way
    if (p.wide_loop && !PAGED) return launch_stage1_mfma_wide(p, dtype_of(T{}), head_dim, stream);
    if (head_dim == 128) return launch<T, 128, 1, 8, 3, kPipelined, PAGED>(p, stream);
    if (head_dim == 64) return launch<T, 64, 1, 8, 3, kPipelined, PAGED>(p, stream);
  } else if (p.rows_per_wg == 128) {  // 4 waves, plain, two workgroups per CU, K and V rings of 2
    if (head_dim == 128) return launch<T, 128, 1, 4, 2, kPlain, PAGED>(p, stream);
    if (head_dim == 64) return launch<T, 64, 1, 4, 2, kPlain, PAGED>(p, stream);
    if (head_dim == 256) return launch<T, 256, 1, 4, 2, kPlain, PAGED>(p, stream);   // 132 KB of rings: one workgroup per CU
  } else if (p.rows_per_wg == 64) {   // 4 waves, two per row block, each half of a tile's keys (stage1_mfma_splitkeys.hip)
    return launch_stage1_mfma_splitkeys(p, dtype_of(T{}), head_dim, stream);
  }
  return FTA_ERR_UNSUPPORTED;
}

}  // namespace

int launch_stage1_mfma(const KernelParams& p, int dtype, int head_dim, void* stream) {
  if (p.scale_log2 <= 0.f) return FTA_ERR_UNSUPPORTED;  // row max is taken before scaling
  // Loads address each K/V stream with 32-bit lane offsets.
  if (p.k_stride[2] * 2 * 8 > 0x7fffffffLL || p.v_stride[2] * 2 * 8 > 0x7fffffffLL) return FTA_ERR_UNSUPPORTED;
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case FTA_F16: return p.block_table ? launch_t<_Float16, true>(p, head_dim, s) : launch_t<_Float16, false>(p, head_dim, s);
    case FTA_BF16: return p.block_table ? launch_t<__bf16, true>(p, head_dim, s) : launch_t<__bf16, false>(p, head_dim, s);
    default: return FTA_ERR_UNSUPPORTED;
  }
}

}  // namespace fta
