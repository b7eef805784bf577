// The MFMA stage-1 kernel's translation unit for the host-thread harness: the product source, with the
// instruction wrappers of gfx950_ops.h replaced by the stand-ins of gfx950_ops_host.h (which must come
// first: it claims the include guards), key-halves instantiations included. The 64-row-wave instantiations are
// assembly and stay out.
#include "fta_device.h"
#include "gfx950_ops_host.h"

#include "stage1_mfma.hip"
#include "stage1_mfma_splitkeys.hip"

#ifndef FTA_HOST_WITH_WIDE_UNIT   // defined when stage1_mfma_wide_host.cpp is part of the build
namespace fta {
int launch_stage1_mfma_wide(const KernelParams&, int, int, void*) { return FTA_ERR_UNSUPPORTED; }
}  // namespace fta
#endif

// Switches the model of the direct global->LDS loads between launches: 0 = they land when issued, 1 = they land
// when a wait of their wave forces them to (gfx950_ops_host.h).
extern "C" void host_block_loads_land_late(int late) { host_block::loads_land_late() = late != 0; }
