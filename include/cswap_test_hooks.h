/* cswap_test_hooks.h -- entry points that exist for the library's own tests only.
 *
 * They are exported by libcswap_hip.so but are not part of its interface: they
 * force failure paths that cannot be provoked from outside, or expose a host-side
 * calculation so that it can be checked for parts this build never runs on.
 * Nothing here has a counterpart in the reference.  Do not call them from
 * production code: their effect is process-wide.
 */
#ifndef CSWAP_TEST_HOOKS_H
#define CSWAP_TEST_HOOKS_H

#ifdef __cplusplus
extern "C" {
#endif

/* The single-pass ZVC kernels wait, bounded, for status words of other workgroups.
 * spin_limit: how many times in all a wavefront asks again before it gives up
 * (0 = the default, some tens of milliseconds' worth); skip_first: if not 0 the
 * count of the first tile is never published, so that everything after it waits in
 * vain.  (0, 0) restores normal operation. */
void cswap_zvc_debug_set_lookback(unsigned spin_limit, unsigned skip_first);

/* Data workgroups the pipeline kernel of cswap_zvc_compress_fused is launched with for a
 * tensor of `tiles` tiles on a part with `compute_units` compute units (the scanner's
 * workgroup comes on top).  Host only. */
int cswap_test_zvc_stream_groups(int tiles, int compute_units);

#ifdef __cplusplus
}
#endif
#endif
