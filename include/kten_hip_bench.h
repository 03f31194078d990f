/*
 * kten_hip_bench.h — measurement entry points of libkten_hip.so that have no counterpart in the
 * reference's backend contract (the reference has no timing facility). They are exported by the
 * same library as the entry points of kten_hip.h and are kept out of that header so that a host
 * binding the contract (the Kotlin HipRawTensor / HipTensorOperations pair) does not meet them:
 * only a benchmark or a profiler harness includes this file. The one metrics call the contract
 * does have, PlatformMetricsProvider.getMetrics
 * (kten-api/src/main/kotlin/eu/redbean/kten/api/tensor/operations/PlatformMetricsProvider.kt:3-6),
 * is kth_metrics in kten_hip.h.
 *
 * Blocking calls here: kth_timer_end, kth_timer_laps, kth_measure_copy, kth_profile_end.
 */
#ifndef KTEN_HIP_BENCH_H
#define KTEN_HIP_BENCH_H

#include "kten_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Device-side stopwatch on the internal stream (a HIP event pair), for benchmarks that
 * must time the stream the kernels run on. No counterpart in the reference, which has
 * no timing facility. kth_timer_end blocks until the second event completes. */
int kth_timer_begin(void);
int kth_timer_end(float* milliseconds);

/* Lap timing on the internal stream, for benchmarks that report the spread of a repeated step. No
 * counterpart in the reference. kth_timer_lap records a HIP event (nothing blocks); kth_timer_laps waits for
 * the last one, writes the time between consecutive laps (count = laps - 1; at most `capacity` values are
 * written) and the time from the first lap to the last, and forgets the laps. */
int kth_timer_lap(void);
int kth_timer_laps(float* milliseconds, int capacity, int* count, float* total_ms);

/* The device-to-device copy rate of this GPU, the practical ceiling a streaming kernel is measured against:
 * times `reps` copies of n_floats values (a multiple of 4) between two pool buffers, once with hipMemcpyAsync
 * and once with the library's own copy kernel, and returns the milliseconds per copy of each. Blocking; no
 * counterpart in the reference. */
int kth_measure_copy(uint64_t n_floats, int reps, float* memcpy_ms, float* kernel_ms);

/* Per-kernel device timing, for benchmarks that must attribute the time of a region to
 * the kernels in it. No counterpart in the reference. Between kth_profile_begin and
 * kth_profile_end every kernel launch carries its own start and stop events (the duration of
 * the dispatch itself, as a kernel trace shows it); kth_profile_end blocks until those
 * launches have finished. Afterwards
 * kth_profile_count gives the number of distinct kernels seen and kth_profile_entry the
 * name ("family<Op>"), launch count, algorithmic bytes and summed duration of one. */
int kth_profile_begin(void);
int kth_profile_end(void);
int kth_profile_count(int* count);
int kth_profile_entry(int index, char* name, size_t cap, uint64_t* launches, uint64_t* bytes, double* total_ms);

#ifdef __cplusplus
}
#endif
#endif /* KTEN_HIP_BENCH_H */
