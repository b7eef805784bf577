// Stage 1, MFMA variant: the instantiations for units of at most 64 query rows in which two
// waves share a 32-row block and each takes 32 of a tile's 64 keys (4 waves, rings of 2, two
// workgroups per CU like the plain loop). The kernel is the template in stage1_mfma_kernel.h.
#include "stage1_mfma_kernel.h"

namespace fta {
namespace {

template <typename T, bool PAGED>
int launch_splitkeys_t(const KernelParams& p, int head_dim, hipStream_t stream) {
  if (head_dim == 128) return launch<T, 128, 1, 4, 2, kSplitKeys, PAGED>(p, stream);
  if (head_dim == 64) return launch<T, 64, 1, 4, 2, kSplitKeys, PAGED>(p, stream);
  return FTA_ERR_UNSUPPORTED;
}

}  // namespace

int launch_stage1_mfma_splitkeys(const KernelParams& p, int dtype, int head_dim, void* stream) {
  if (p.rows_per_wg != 64) return FTA_ERR_UNSUPPORTED;
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case FTA_F16: return p.block_table ? launch_splitkeys_t<_Float16, true>(p, head_dim, s) : launch_splitkeys_t<_Float16, false>(p, head_dim, s);
    case FTA_BF16: return p.block_table ? launch_splitkeys_t<__bf16, true>(p, head_dim, s) : launch_splitkeys_t<__bf16, false>(p, head_dim, s);
    default: return FTA_ERR_UNSUPPORTED;
  }
}

}  // namespace fta
