/* TEST AND MEASUREMENT HOOKS, not part of the drop-in surface (no reference counterpart): they exist
 * so that tests can exercise two device building blocks in isolation (the bit-faithful expf and the
 * sequential-sum emulation) and so that the benchmark can time what a launch and a plain read cost.
 * A product build may leave them out: nothing in include/ declares them. */
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

/* Measurement floors for the benchmark: an empty launch, and a kernel of `workgroups` workgroups
 * of 256 lanes that does nothing but read `bytes` bytes (16-byte aligned DEVICE pointer). */
ETS_API ets_status ets_test_empty_launch(void* hip_stream);
ETS_API ets_status ets_test_read_floor(const void* d_data, int64_t bytes, int32_t workgroups, uint32_t* d_out,
                                       void* hip_stream);

/* dst = src with 16-byte accesses (16-byte aligned DEVICE pointers, bytes a multiple of 16): the
 * transfer of known size that fetch and write counters of a profiler run are scaled by. */
ETS_API ets_status ets_test_copy_probe(const void* d_src, void* d_dst, int64_t bytes, void* hip_stream);

/* Phase clocks of the finish kernel of the several-workgroups-per-row path, four 64-bit words per
 * row (staging, ordered sum, draw, in ticks of the 100 MHz wall clock; then the candidate and
 * prepared-slot counts), filled when ETS_SPLIT_TIMERS was set before the handle's first stochastic
 * call.  HOST pointer. */
ETS_API ets_status ets_test_split_timers(ets_sampler* s, uint64_t* out, int32_t rows);

#ifdef __cplusplus
}
#endif
#endif
