// The matrix-instruction kernels cannot run on host threads: in the host build they do not exist.
#include "fta_internal.h"
namespace fta {
int launch_stage1_mfma(const KernelParams&, int, int, void*) { return FTA_ERR_UNSUPPORTED; }
int launch_stage1_mfma_wide(const KernelParams&, int, int, void*) { return FTA_ERR_UNSUPPORTED; }
int launch_stage1_mfma_splitkeys(const KernelParams&, int, int, void*) { return FTA_ERR_UNSUPPORTED; }
}  // namespace fta
