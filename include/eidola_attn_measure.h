/* Measurement hooks of the paged sink-attention library.  They exist ONLY in the measurement
 * build of the library (libeidola_attn_measure.so, the same sources compiled with
 * -DEID_MEASURE); the serving library (libeidola_attn_hip.so) has neither these entry points nor
 * the process-wide state behind them.  bench.py loads the measurement build for its kernel
 * timing pass and its per-workgroup timelines; nothing else should.
 * Both hooks hold pointers the caller owns: the device buffer and the events must outlive the
 * setting (switch the hook off before freeing them). */
#ifndef EIDOLA_ATTN_MEASURE_H
#define EIDOLA_ATTN_MEASURE_H
#include "eidola_attn.h"
#ifdef __cplusplus
extern "C" {
#endif

/* Measurement aid, no counterpart in the reference and no part of a serving path: hands the
 * library a DEVICE buffer of `entries` records of 64 bytes (eight uint64).  From then on every
 * chunked-prefill launch of this process whose waves (four per workgroup) fit the buffer lets
 * wave w of workgroup b write record 4 b + w:
 * {start, end} in 100 MHz wall-clock ticks, {hardware id | work units << 32, XCC id}, and in
 * words 4..6 the prefill kernel's stamps before its first K/V fetch, after the first tile
 * has arrived and after its last chunk; records of waves without work stay as the caller
 * left them.  NULL switches it off (the default).
 * Process-wide and not thread-safe: set it with no eid_* call in flight. */
void eid_debug_set_timeline(void *device_buf, int64_t entries);

/* Measurement aid, no counterpart in the reference and no part of a serving path: two
 * hipEvent_t (created with timing enabled) that the next attention calls of this process attach
 * to the dispatch of every split-KV and prefill kernel they launch (not the merges, the plan
 * kernel or the short-span kernel): after the stream has drained, hipEventElapsedTime(start,
 * stop) is the duration of the LAST such kernel as a profiler reports it, without the gaps that
 * events recorded around a launch include.  Meant for calls with one such kernel (a decode
 * call; a ragged call whose sequences are of one class).  NULL, NULL switches it off (the
 * default).  Process-wide: set it with no eid_* call in flight. */
void eid_debug_set_kernel_events(void *start_event, void *stop_event);

/* Measurement aid: how an even split with the caller's partition size (desc.partition_size != 0)
 * stores its partials from now on.  1: one partial per partition of that size, all of them merged
 * by the merge kernel (what a workgroup per partition would do); 0: one partial per piece (the
 * consecutive partitions a workgroup holds of one sequence, merged in registers: the library's
 * way); -1: as the environment variable EID_STORE_EVERY_PARTITION said at the first call (the
 * default).  Process-wide. */
void eid_debug_set_store_every_partition(int32_t mode);

#ifdef __cplusplus
}
#endif
#endif /* EIDOLA_ATTN_MEASURE_H */
