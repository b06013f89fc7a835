/*
 * egs_hip_testing.h -- switches for the library's own test-suite.  Not part of the drop-in boundary
 * (include/egs_hip.h): nothing here has a counterpart in the reference and production callers
 * never need it.
 */
#ifndef EGS_HIP_TESTING_H
#define EGS_HIP_TESTING_H

#ifdef __cplusplus
extern "C" {
#endif

/* Non-zero routes every later call of the process through the general tiled kernels, skipping the
 * specialised small-expert and direct-to-LDS kernels, so that both families can be checked against
 * the oracle on the same inputs (both must stay within the same tolerances).  Process-wide; the
 * test-suite sets and clears it around single-threaded test cases. */
void egs_testing_force_generic(int on);

#ifdef __cplusplus
}
#endif
#endif /* EGS_HIP_TESTING_H */
