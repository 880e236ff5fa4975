/*
 * stingray_sampler_test.h -- test and measurement hooks of libstingray_sampler.so.
 *
 * Not part of the interface a managed binding attaches to (that is stingray_sampler.h) and without a
 * counterpart in the reference: these entry points let the parity tests reach single device routines
 * (the exp and running-sum arithmetic that Sampler.cs:298-313, 460-465 spell as scalar loops), force
 * rarely taken paths from the host, and read phase timestamps out of a profiling build.
 */
#ifndef STINGRAY_SAMPLER_TEST_H
#define STINGRAY_SAMPLER_TEST_H

#include "stingray_sampler.h"

#ifdef __cplusplus
extern "C" {
#endif

/* y[i] = the device's expf for x[i] (device pointers): must equal MathF.Exp bit for bit. */
SR_API int sr_selftest_expf(sr_ctx* ctx, const float* x_dev, float* y_dev, int64_t n);

/* Exact left-to-right fp32 sum of x_dev[0..n) starting from s0, as the scalar loop of Sampler.cs:460-465 computes
 * it; with a target that is not NaN also the first index whose running sum reaches it (-1 if none).  Device
 * pointers for x and both results. */
SR_API int sr_selftest_seqsum(sr_ctx* ctx, const float* x_dev, int32_t n, float s0, float target, float* out_sum_dev,
                              int32_t* out_idx_dev);

/* The same sum and search the way the full-vocabulary path prepares long rows: the whole device turns every 1,024 terms
 * into a record for the binade that an approximate prefix sum predicts, and one wave walks the records.  `skew`
 * multiplies the approximate sums (1 = as in production; other values make the predictions miss: the results must
 * not change).  out_sum_dev[2], out_idx_dev[2]: [0] the sum and the search from the states the sum left, [1] the
 * running sum and index of the walk that searches by itself.  n <= 1,048,576. */
SR_API int sr_selftest_segsum(sr_ctx* ctx, const float* x_dev, int32_t n, double skew, float target, float* out_sum_dev,
                              int32_t* out_idx_dev);

/* How many sr_batch_append_tokens calls on this batch rebuilt it instead of updating it in place. */
SR_API int sr_debug_append_rebuilds(const sr_batch* batch);
/* ... and how many rows such calls moved to the end of the batch's edit array because they had run out of room. */
SR_API int sr_debug_append_moves(const sr_batch* batch);

/* How often a row tail of the selection kernel polls its row's counter before it stops waiting for the row's other
 * chunks and selects the row from its logits alone, the way a row whose candidates overflow the kernel's lists is
 * selected (default 2^22, more than a second).  0 makes every row take that way: the results must not change. */
SR_API int sr_debug_set_spin_limit(sr_ctx* ctx, uint32_t polls);

/* How often a workgroup of the full-vocabulary path's pass over long rows polls its row's count (every workgroup of the
 * row leaves its segments' maxima and counts itself in) before it stops waiting, marks its segments and leaves them to
 * the last of the row's workgroups (default 2^15, tens of milliseconds).  0 makes every workgroup leave its segments;
 * 1 or 2 make some of them do so: the results must not change. */
SR_API int sr_debug_set_row_wait_limit(sr_ctx* ctx, uint32_t polls);

/* Profiling builds (-DSR_PROFILE) only, SR_ERR_UNSUPPORTED otherwise: phase timestamps (wall_clock64, 100 MHz) of
 * the selection kernel go to prof_dev[unit][16], one unit per chunk item and per row; NULL switches them off. */
SR_API int sr_debug_set_profile(sr_ctx* ctx, unsigned long long* prof_dev);

#ifdef __cplusplus
}
#endif
#endif /* STINGRAY_SAMPLER_TEST_H */
