/* libflh_hip -- entry points for tests and tuning runs only.  Not part of the product interface (include/flh_hip.h):
 * nothing here has a counterpart in the reference, and a serving process has no reason to call it. */
#ifndef FLH_HIP_TESTING_H
#define FLH_HIP_TESTING_H

#ifdef __cplusplus
extern "C" {
#endif

/* Overrides, PROCESS-WIDE, the tile (64, 128 or 256 rows; 0 = automatic) and the split of K inside a workgroup (1, 2 or
 * 4; 0 = automatic) that the GEMM entry points would choose from the shape.  Every variant gives the same bits; the tests
 * use this to reach all of them, a tuning run to compare them.  Combinations a kernel does not offer fall back to the
 * nearest one it does.  Not for use next to a running model: the setting is global to the process, and a second thread
 * that flips it changes the kernels the first one launches (same results, other timings).  Returns FLH_OK or
 * FLH_EINVAL (include/flh_hip.h). */
int flh_gemm_set_tuning(int tile, int k_split);

#ifdef __cplusplus
}
#endif
#endif
