// Stage 1, MFMA variant: the instantiations with 64 query rows per wave (4 waves, one per
// SIMD, half-tile pipeline, K ring 4 / V ring 5) for units of more than 128 rows on contiguous caches. The kernel
// is the template in stage1_mfma_kernel.h.
#include "stage1_mfma_kernel.h"

namespace fta {
namespace {

template <typename T>
int launch_wide_t(const KernelParams& p, int head_dim, hipStream_t stream) {
  if (head_dim == 128) return launch<T, 128, 2, 4, 4, kWide, false>(p, stream);
  if (head_dim == 64) return launch<T, 64, 2, 4, 4, kWide, false>(p, stream);
  return FTA_ERR_UNSUPPORTED;
}

}  // namespace

int launch_stage1_mfma_wide(const KernelParams& p, int dtype, int head_dim, void* stream) {
  if (p.rows_per_wg != 256 || p.block_table) return FTA_ERR_UNSUPPORTED;   // contiguous caches only: the loop requests its tiles itself
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case FTA_F16: return launch_wide_t<_Float16>(p, head_dim, s);
    case FTA_BF16: return launch_wide_t<__bf16>(p, head_dim, s);
    default: return FTA_ERR_UNSUPPORTED;
  }
}

}  // namespace fta
