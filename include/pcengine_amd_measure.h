/* pcengine_amd, measurement build only (libpcengine_amd_measure.so: the same sources compiled with
 * -DPCE_MEASURE).  It exports everything pcengine_amd.h declares plus the switch below.  The product
 * library, libpcengine_amd.so, has no such switch: its forward entry points always run every stage
 * with the kernel the shape calls for.  No counterpart in the reference. */
#ifndef PCENGINE_AMD_MEASURE_H
#define PCENGINE_AMD_MEASURE_H

#include "pcengine_amd.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Bit i of the mask enables stage i of the forward entry points (0: centre GEMM or zero-fill,
 * 1: pair / tile kernel, 2: convert, scatter or row sum, 3: gather), so that a benchmark can time one
 * kernel of a dataflow alone.  Higher bits choose between kernel families for A/B measurements:
 * 4 = the deferred-scatter forms with a pair-driven row sum (cleared: centre GEMM with the partial-row
 * sum in its epilogue), 5 = the pipelined tile kernel for wide fp16 layers (cleared: the single-stage
 * tile kernel), 6 = pair tiles and centre GEMM of a wide deferred-scatter layer in one launch (cleared:
 * two launches), 9 = the pipelined output-stationary kernel for wide fp16 layers of few tiles (cleared:
 * the single-stage tile kernel), 10 = output rows may leave with the non-temporal hint (cleared: never),
 * 11 = ... only where the output tensor is 16 MiB or more (cleared, with 10 set: always), 12 = the
 * three-kind form of the ordered dataflow on clouds it is meant for and its stream workgroups as the plain
 * GEMM of narrow fp16 layers (cleared: the kernel that visits every row through the order; the tile
 * kernel).  Default: all bits set.  Process-wide and unsynchronised: one thread,
 * measurement runs only. */
void pce_set_stage_mask(uint32_t mask);

#ifdef __cplusplus
}
#endif
#endif /* PCENGINE_AMD_MEASURE_H */
