/*
 * libbptattn — measurement and testing hooks (NOT part of the drop-in boundary of include/bptattn.h).
 *
 * These entry points carry process-global state (a flag, two event handles) and exist for benchmarks and tests only:
 * a product binding of the graph-attention path needs none of them.  They have no counterpart in the reference.
 */
#ifndef BPTATTN_MEASURE_H
#define BPTATTN_MEASURE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* 1: force the shape-generic kernels even where a specialised one exists (testing). Returns the old value. */
int bpt_set_force_generic(int on);

/* Measurement aid (no counterpart in the reference): while `which` is one of BPT_KERNEL_*, every launch
 * of that main kernel of the fused path is bracketed by hipEventRecord(start_event) / (stop_event) on
 * the launch stream, so a benchmark can time one kernel with HIP events; 0 switches it off. */
enum { BPT_KERNEL_NONE = 0, BPT_KERNEL_ATTN_FWD = 1, BPT_KERNEL_ATTN_BWD_DST = 2, BPT_KERNEL_ATTN_BWD_SRC = 3 };
int bpt_profile_kernel(int which, void *start_event, void *stop_event);

/* Measurement aid (no counterpart in the reference): launches a kernel in which waves_per_cu wavefronts per compute unit
 * (a multiple of 4, at most 64) each read `iters` batches of in_flight (2, 4 or 8) pseudo-random 1 KB rows of `region`
 * (region_bytes of device memory, 16-byte aligned), the access pattern of the attention kernels' neighbour-row gathers.
 * Timed with events by the caller, 256 * waves_per_cu * iters * in_flight KB / duration is the rate at which this GPU's
 * memory system feeds such gathers: the practical ceiling of these kernels (lower than the streaming bandwidth).
 * sink: one float of device memory (never written in practice). */
int bpt_gather_probe(const void *region, int64_t region_bytes, int waves_per_cu, int in_flight, int iters, float *sink, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* BPTATTN_MEASURE_H */
