/*
 * Measurement helpers that libmooncake_ep_hip.so exports beside its public C
 * ABI (include/mooncake_ep_hip.h).  They take no part in dispatch / combine and
 * are not for callers of the library: bench.py uses them to calibrate the
 * profiler's counters and to measure what the GPU's memory system gives the
 * read : write mixes of the data kernels.
 */
#ifndef MOONCAKE_EP_DEBUG_H
#define MOONCAKE_EP_DEBUG_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Plain device copy of `bytes` (multiple of 16) by a grid-stride kernel: the
 * known-size kernel the profiler's FETCH_SIZE / WRITE_SIZE readings are scaled
 * against. */
int mc_ep_debug_copy(uint64_t dst_ptr, uint64_t src_ptr, uint64_t bytes, uint64_t stream_ptr);

/* A synthetic stream of n = unit_bytes / 16 threads, one 16-byte unit each:
 *   kind 0 copy      reads n units, writes n units
 *        1 read      reads n units
 *        2 write     writes n units
 *        3 widen     reads n/2 units, writes n units        (the cast-back kernel's 1 : 2)
 *        4 gather8   reads 8 streams of n units, writes n   (the reduce kernel's 8 : 1)
 *        5 scatter8  reads 2n units, writes 8 streams of n  (the fp8 pack kernel's 1 : 4)
 * src / dst must hold what the kind reads / writes. */
int mc_ep_debug_stream(int kind, uint64_t dst_ptr, uint64_t src_ptr, uint64_t unit_bytes, uint64_t stream_ptr);

/* From now on the synthetic streams (mc_ep_debug_stream, _gather_rows, _scatter_rows) run at most this many
 * waves per CU (0, the default: as many as fit), so that a stream can be measured at the occupancy the
 * kernel it stands for is launched with. */
int mc_ep_debug_set_stream_occupancy(int waves_per_cu);

/* The reduce kernel's address pattern with nothing else: out_rows rows of
 * row_bytes (multiple of 1024), each the xor of 8 whole rows at computed,
 * scattered places of a [regions, region_rows, row_bytes] source of which the
 * first `used` rows of every region are read (the packed layout: a region per
 * expert, its valid rows at the start).  No index loads, no arithmetic. */
int mc_ep_debug_gather_rows(uint64_t dst_ptr, uint64_t src_ptr, int row_bytes, int64_t out_rows, int regions,
                            int64_t region_rows, int used, uint64_t stream_ptr);

/* The fp8 pack kernel's address pattern with nothing else: in_rows source rows
 * of 2 * row_bytes, read once, folded to row_bytes (multiple of 1024) and
 * written to 8 whole rows at computed, scattered places of a
 * [regions, region_rows, row_bytes] destination (the first `used` rows of every
 * region, each written once). */
int mc_ep_debug_scatter_rows(uint64_t dst_ptr, uint64_t src_ptr, int row_bytes, int64_t in_rows, int regions,
                             int64_t region_rows, int used, uint64_t stream_ptr);

#ifdef __cplusplus
}
#endif

#endif /* MOONCAKE_EP_DEBUG_H */
