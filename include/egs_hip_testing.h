/*
 * egs_hip_testing.h -- switches for the library's own test-suite.  Not part of the drop-in boundary
 * (include/egs_hip.h): nothing here has a counterpart in the reference and production callers
 * never need it.
 */
#ifndef EGS_HIP_TESTING_H
#define EGS_HIP_TESTING_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Non-zero routes every later call of the process through the general tiled kernels, skipping the
 * specialised small-expert and direct-to-LDS kernels, so that both families can be checked against
 * the oracle on the same inputs (both must stay within the same tolerances).  Process-wide; the
 * test-suite sets and clears it around single-threaded test cases. */
void egs_testing_force_generic(int on);

/* Which kernels did a call select?  _begin starts (and empties) a log kept for the calling thread; every kernel the
 * thread then launches through the library appends its name; _end copies the comma-separated names into `buf` (at most
 * n - 1 characters and a terminating 0), stops the log and returns the length of the full text.  Used by the benchmark
 * to name the kernels behind the launches it times, and by tests that assert which path a shape took. */
void egs_testing_launch_log_begin(void);
size_t egs_testing_launch_log_end(char *buf, size_t n);

#ifdef __cplusplus
}
#endif
#endif /* EGS_HIP_TESTING_H */
