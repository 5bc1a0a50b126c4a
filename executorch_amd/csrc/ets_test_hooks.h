/* TEST AND MEASUREMENT HOOKS, not part of the drop-in surface (no reference counterpart): they exist
 * so that tests can exercise two device building blocks in isolation (the bit-faithful expf and the
 * sequential-sum emulation) and so that the benchmark can time what a launch, a plain read and a
 * hand-over between workgroups cost.  They are built into a library of their own,
 * libet_sampler_hooks.so (csrc/ets_test_hooks.hip); libet_sampler.so does not export them and
 * nothing in include/ declares them. */
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

/* Round trips between workgroup 0 and workgroup `partner` (1 .. 15) of a 16-workgroup launch through
 * two words in device memory (`d_words`: 64 words, zeroed by the caller), every wait bounded by
 * `spin_limit` polls.  d_out[0] (zeroed by the caller): waits that ran out; d_out[1]: ticks of the
 * 100 MHz clock that workgroup 0 spent on `hops` round trips.  DEVICE pointers. */
ETS_API ets_status ets_test_signal_floor(uint32_t* d_words, int32_t hops, int32_t spin_limit, int32_t partner,
                                         uint32_t* d_out, void* hip_stream);

/* Which of the handle's lazily allocated device buffers exist: out[0] candidate scratch, out[1] the
 * work buffers of the several-workgroups-per-row path, out[2] the pattern histograms, out[3] the
 * per-row parameter staging (1: allocated).  A handle that has only served calls of
 * ets_sampler_sample_batch_static() has none of them.  HOST pointer to four int32. */
ETS_API ets_status ets_test_handle_buffers(const ets_sampler* s, int32_t* out);

/* The number of the next launch with pass 1 inside pass 2 on the handle's own work buffers (the word its
 * workgroups tag their hand-over with; waits for the device).  With `mark_unfinished` the handle is left as
 * if its last such launch had not been followed by its finish kernel: the next one must then be given a
 * number of its own first. */
ETS_API ets_status ets_test_fused_launch_number(ets_sampler* s, int32_t mark_unfinished, uint32_t* out);

/* Sets that word (waits for the device): for a test of the numbers coming round after 2^32 - 1 launches. */
ETS_API ets_status ets_test_set_fused_launch_number(ets_sampler* s, uint32_t value);

/* The message of the calling thread's last failed hook. */
ETS_API const char* ets_test_last_error(void);

/* Phase clocks of the finish kernel of the several-workgroups-per-row path, four 64-bit words per
 * row (staging, ordered sum, draw, in ticks of the 100 MHz wall clock; then the candidate and
 * prepared-slot counts), filled when libet_sampler.so was built with -DETS_PHASE_CLOCKS=1 (a
 * profiling build; the product build has no clocks in its kernels) and ETS_SPLIT_TIMERS was set before
 * the handle's first stochastic call.  HOST pointer. */
ETS_API ets_status ets_test_split_timers(ets_sampler* s, uint64_t* out, int32_t rows);

#ifdef __cplusplus
}
#endif
#endif
