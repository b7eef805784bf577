// The 64-row-wave instantiations of the MFMA stage-1 kernel for the host-thread harness: the product source, with
// the instruction wrappers replaced by gfx950_ops_host.h and the assembly statements of wide_loop_asm.inc replaced
// by calls of the interpreter in gfx950_asm_host.h on the same text (FTA_HOST_WIDE_LOOP_INC names the rendering).
// A translation unit of its own, next to stage1_mfma_host.cpp, as in the product.
#ifndef FTA_HOST_WIDE_LOOP_INC
#error "compile with -DFTA_HOST_WIDE_LOOP_INC=<rendering of the statements as interpreter calls>"
#endif
#include "fta_device.h"
#include "gfx950_ops_host.h"

#include "stage1_mfma_wide.hip"
