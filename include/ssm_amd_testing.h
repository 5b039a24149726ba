/*
 * ssm_amd_testing.h - what a -DSSM_TEST_HOOKS build of the library adds to ssm_amd.h.
 *
 * The shipped library (libssm_amd.so) picks its kernels by shape and dtype alone and rejects a non-zero
 * `reserved` field.  The test suite also needs to run a chosen kernel where the library would pick another
 * (to compare two implementations of one operator on the same inputs) and to learn which kernel a call
 * took.  A second build of the same sources with -DSSM_TEST_HOOKS (libssm_amd_testhooks.so) reads the
 * `reserved` fields as the selectors below and exports one more function.  Nothing here has a counterpart
 * in the reference and nothing here is part of the backend's interface.
 *
 *   ssm_scan_fwd_args.reserved        0 = automatic; 100 * steps-per-lane + states-per-LDS-pass (408, 808, 816);
 *                                     1616, 2416, 3216, 4816 = 816 with two, three, four, six channels per wave;
 *                                     100000 + v = variant v of the kernel for grouped time-varying projections
 *                                     (131042: the row-per-wave kernel for projections constant in time)
 *   ssm_scan_bwd_args.reserved        1 = the general kernel also where a wave-per-row kernel applies (grouped
 *                                     projections, projections of their own per channel, or projections that are
 *                                     constant in time);
 *                                     2 = the wave-per-row kernel with its bounded wait for a neighbouring wave
 *                                     cut to nothing, so that every wave takes the give-up path (dB and dC
 *                                     come back as NaN; the kernel ends normally)
 *   ssm_dscan_bwd_args.reserved       non-zero = the general two-kernel path also where the one-pass kernel applies
 *   ssm_ssd_bmm_args.reserved,
 *   ssm_ssd_chunk_state_args.reserved,
 *   ssm_ssd_chunk_scan_args.reserved  non-zero = the one-thread-per-output kernel instead of a matrix-core kernel
 */
#ifndef SSM_AMD_TESTING_H
#define SSM_AMD_TESTING_H

#include "ssm_amd.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Which of the calls made by this thread since the last query ran a bf16 / fp16 matrix-core kernel:
 * bit 0 bmm_chunk, bit 1 chunk_state, bit 2 chunk_scan, bit 3 the one-pass ssm_ssd_combined_fwd.
 * Resets on read. */
int ssm_ssd_mfma_launches(void);

#ifdef __cplusplus
}
#endif
#endif /* SSM_AMD_TESTING_H */
