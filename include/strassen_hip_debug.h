/* strassen_hip_debug.h -- test and profiling hooks of libstrassen_hip.so.  Not part of the
 * drop-in boundary (strassen_hip.h); none of them has a counterpart in the reference.  The two
 * switches are process-wide: every public entry point reads them once when it is called, so a
 * change never affects a call that is already running, but it does affect other threads' later
 * calls.  Not for production code. */
#ifndef STRASSEN_HIP_DEBUG_H
#define STRASSEN_HIP_DEBUG_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Runs the 16-bit transposing LDS read on a 64 x 4 grid of 16-bit values (value = 4 * lane +
 * element) and writes what each lane received to out[64 * 4] (uint16, device memory).  Used by
 * the tests to pin the lane mapping the kernels rely on. */
int sthip_debug_transpose_read(void* out, void* stream);

/* Selects which stages of the pipelined paths later calls run (bit 0 = quadrant-sum pre-pass,
 * bit 1 = grouped GEMM, bit 2 = recombination pass; bit 3 lets two-level calls run as one
 * 49-product launch instead of the host recursion; bit 4 runs large one-level 16-bit Strassen
 * calls as ONE launch whose workgroups are the sums, the product tiles and the recombination --
 * same bits, slower than the three launches on MI355X, hence off by default; bit 5 makes the
 * 256 x 256 kernel launch one workgroup per tile instead of one per CU that walks the tiles --
 * same bits, slower; default 15) and returns the previous mask.
 * With mask 2 the GEMM re-uses the sums a previous call left in the same workspace, so the
 * dominant kernel can be timed alone. */
int sthip_debug_set_stages(int mask);

/* After a call that ran as ONE launch (bit 4 above) with this workspace and these sizes: waits for
 * `stream`, copies the launch's 16 dependency counters to counters[] (host memory; [0..2] finished
 * units of the three sums jobs, [8..14] finished tiles of the seven products, [15] workgroups whose
 * bounded wait for a producer expired) and returns counters[15], or a negative sthip_status.  The
 * one-launch form never hangs, at the price that a workgroup which gives up goes on with whatever
 * is in memory: when this returns anything but 0 the result of that call is undefined.  Its waits
 * end only if workgroups start in blockIdx order, which the hardware does today and HIP does not
 * promise; that, and being slower, is why the form stays behind a debug switch. */
int sthip_debug_one_launch_counters(const void* workspace, int64_t M, int64_t N, int64_t K,
                                    unsigned counters[16], void* stream);

/* Overrides the tile table for later calls where the shape allows the forced tile: "128x128",
 * "256x128" (kernels that recombine in registers), "128x128g", "256x256" (grouped products),
 * "64x64" (fp32: seven products side by side on small tiles, sums formed in the operand loads);
 * NULL or anything else = automatic.  Returns the previous setting as a code (0 = automatic).
 * The environment variable STHIP_FORCE_TILE gives the initial setting; it is read once, by the
 * first call into the library. */
int sthip_debug_force_tile(const char* tile);

#ifdef __cplusplus
}
#endif
#endif /* STRASSEN_HIP_DEBUG_H */
