/* libdeepshift_hip.so -- entry points for the library's own test-suite.
 *
 * Kept out of deepshift_hip.h on purpose: nothing here is part of the drop-in boundary, and a
 * production caller has no use for it.  No counterpart in the reference. */
#ifndef DEEPSHIFT_HIP_TEST_H
#define DEEPSHIFT_HIP_TEST_H

#ifdef __cplusplus
extern "C" {
#endif

/* Test hook: forces a launch variant of the compute entry points, process-wide, so that the
 * test-suite can run every kernel form on small shapes.  knob: "planes" (0 / 1: two-instruction /
 * shift-plane kernel), "split" (K split; shift-plane kernels: 0 = equal shares, 1 = one tile per
 * wave), "tile" (R * 100 + J of the two-instruction kernel), "cu" (0 / 4 / 8 waves per cooperative
 * workgroup), "notail", "wide" (1: the int8 fused launch keeps reductions longer than a chunk on the
 * widened tile buffer of eight-wave workgroups), "perm" (0: the int32 cooperative launch walks the pixel
 * tiles in image order); "chain_spin_us" (bound of a barrier wait of ds_linear_chain_f32 in
 * microseconds) and "chain_extra" (arrivals its barriers wait for beyond the grid, which never come: with
 * a small bound every workgroup gives up and exits, which is how the tests reach that path without
 * hanging anything).  knob == NULL clears every override.  Each knob is an atomic integer that an
 * entry point reads once per call, so a call sees either the old or the new value of a knob, never a
 * torn one; a thread that changes a knob changes the dispatch of every thread of the process, which
 * is why this header is not the production one.  The dispatch's own choice is the measured best. */
int ds_test_tune(const char *knob, int value);

/* q[i] = n[i] / d (and, uniform != 0, the same through the form the kernels use on wave-uniform
 * dividends) by the multiply-shift division with which every shift kernel turns flat indices into
 * (image, row, column) and share positions into tiles: the host derives the constants for the divisor,
 * the device applies them.  Device pointers, count elements, d >= 1; asynchronous on `stream` (a
 * hipStream_t, NULL = the default stream).  For the tests, which compare it with plain division over
 * divisors and dividends up to 2^32 - 1.  Returns 0 or a negative status. */
int ds_test_fast_div(const unsigned int *n, unsigned int *q, long count, unsigned int d, int uniform,
                     void *stream);

#ifdef __cplusplus
}
#endif
#endif /* DEEPSHIFT_HIP_TEST_H */
