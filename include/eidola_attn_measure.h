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
 * hipEvent_t (created with timing enabled) that the next eid_attn_decode calls of this process
 * attach to the split-KV kernel's own dispatch (bf16 cache, one row per sequence, more than one
 * partition in the plan, stream not capturing): after the
 * stream has drained, hipEventElapsedTime(start, stop) is that kernel's duration as a profiler
 * reports it, without the gaps that events recorded around a launch include.  Every such launch
 * overwrites both events.  NULL, NULL switches it off (the default).
 * Process-wide and not thread-safe: set it with no eid_* call in flight. */
void eid_debug_set_kernel_events(void *start_event, void *stop_event);

#ifdef __cplusplus
}
#endif
#endif /* EIDOLA_ATTN_MEASURE_H */
