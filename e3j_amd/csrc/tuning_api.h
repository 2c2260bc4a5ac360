/* Internal: launch-shape selection for tuning runs and for the tests that check that every
 * compiled launch shape gives the same results.  Not part of the public C ABI (include/e3j_amd.h);
 * the symbol is exported so that the in-tree tests reach it through ctypes.
 *
 * Selects which launch shape (channels per lane, waves per block, parts) of a signature's kernels
 * later calls use; 0 = default, unknown numbers = default.  Process-wide; may be called from any
 * thread while other threads launch (each launch reads the numbers once, atomically, and uses the
 * old or the new shape).  The environment variables E3J_AMD_FWD_VARIANT / E3J_AMD_BWD_VARIANT give
 * the initial values.  Results do not depend on it.  No counterpart in the reference, whose
 * launch shape is planned on the host per call (src/e3j/ops/convolution.py:178-208). */
#ifndef E3J_AMD_CSRC_TUNING_API_H_
#define E3J_AMD_CSRC_TUNING_API_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif
void e3j_amd_set_launch_variant(int32_t fwd_variant, int32_t bwd_variant);
#ifdef __cplusplus
}
#endif
#endif /* E3J_AMD_CSRC_TUNING_API_H_ */
