/* Entry points that exist only so that tests can exercise two device building blocks in
 * isolation (the bit-faithful expf and the sequential-sum emulation).  Not part of the
 * drop-in surface; no reference counterpart. */
#ifndef ETS_TEST_HOOKS_H_
#define ETS_TEST_HOOKS_H_

#include "../../include/et_sampler.h"

#ifdef __cplusplus
extern "C" {
#endif

/* y[i] = expf(x[i]) as evaluated inside the sampler; DEVICE pointers. */
ETS_API ets_status ets_test_expf(const float* d_x, float* d_y, int64_t n, void* hip_stream);

/* s = s0; for i < n: s += a[i]; stop at the first i with s > threshold.  One workgroup;
 * DEVICE pointers; *d_stop = -1 when the threshold is never exceeded. */
ETS_API ets_status ets_test_seq_sum(const float* d_a, int32_t n, float s0, float threshold, float* d_sum,
                                    int32_t* d_stop, void* hip_stream);

#ifdef __cplusplus
}
#endif
#endif
