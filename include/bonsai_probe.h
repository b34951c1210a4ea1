/*
 * C ABI of libbonsai_probe.so: measurement aids of the benchmarks for the MI355X (gfx950)
 * packed low-bit GEMV.  Not part of the drop-in surface and not loaded by the operators: the
 * reference has no counterpart.  No probe does arithmetic of the GEMV; each isolates one cost
 * of the machine (the bytes alone, a launch, a dependent launch, a hand-over between
 * workgroups) so that a measured kernel time can be put beside it.  All pointers are device
 * memory, all work is enqueued on `stream` (a hipStream_t passed as void*), nothing allocates
 * or synchronises.  Status codes as in bonsai_gemv.h: 0 ok, 1 bad argument, 2 launch error.
 */
#ifndef BONSAI_PROBE_H
#define BONSAI_PROBE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Reads `bytes` of device memory at `src` (16-byte aligned) exactly once with `workgroups`
 * workgroups of 256 threads and discards them.  persistent = 0: every thread requests its share
 * up front (at most eight 16-byte loads, else status 1) -- the launch shape of a layer-sized
 * GEMV; persistent = 1: workgroups loop with eight loads per lane in flight -- the shape of the
 * kernels for very long matrices.  `sink` is 4 writable device bytes (practically never
 * written). */
int bonsai_read_probe(const void *src, size_t bytes, int workgroups, int persistent, void *sink,
                      void *stream);

/* Enqueues `launches` launches of a kernel that does nothing: `workgroups` workgroups of
 * `threads` threads (a multiple of 64, at most 1024) with `lds_bytes` (at most 65536) of
 * dynamic LDS.  `sink` is 4 writable device bytes, never written. */
int bonsai_probe_empty_launches(int launches, int workgroups, int threads, int lds_bytes, void *sink,
                                void *stream);

/* Enqueues `launches` launches of a one-wave kernel that increments the 32-bit word at `word`:
 * every launch consumes what the previous one wrote. */
int bonsai_probe_chain_launches(int launches, void *word, void *stream);

/* One launch of `workgroups` persistent workgroups of 256 threads (at most four per CU, else
 * status 1) that pass `barriers` (1..1000) device-wide barriers through one arrival counter.
 * `state` is two 32-bit words the caller has zeroed: [0] the counter, [1] error flags, set to 1
 * when a wait ran into its spin limit (the workgroups then leave instead of waiting on: the
 * kernel always ends). */
int bonsai_probe_grid_barrier(int workgroups, int barriers, void *state, void *stream);

/* Enqueues `launches` launches of the "last arriver finishes" probe over `workgroups` workgroups
 * of 256 threads.  mode 0: every workgroup writes a record of `words` (1..64) 32-bit words and
 * ends; mode 1: it then
 * makes the record visible, bumps an arrival counter, and the workgroup that arrives last reads
 * all records, adds them into state[1] and resets the counter (no workgroup ever waits); mode 2:
 * one workgroup that only reads the records -- the separate launch that mode 1 would save.
 * `records` holds workgroups x words words, `state` two zeroed words.  time(mode 1) against
 * time(mode 0) + time(mode 2) is what fusing a consumer stage behind an arrival counter gains or
 * loses over launching it on its own. */
int bonsai_probe_last_arriver(int launches, int workgroups, int words, int mode, void *records,
                              void *state, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* BONSAI_PROBE_H */
