/*
 * apt_synth.h — synthetic-input helpers of libapt_hip.so (benchmark and test
 * support; no counterpart in the reference, which loads OGB datasets through
 * DGL, scripts/preprocess_dataset.py).
 */
#ifndef APT_SYNTH_H_
#define APT_SYNTH_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Fill the neighbour lists of rows [row_begin, row_begin + num_rows) of an
 * R-MAT graph over num_nodes ids whose row degrees are already fixed by indptr
 * (device int64[num_rows + 1]).  R-MAT factorises: given the
 * bits of the row id u, each bit of a neighbour is an independent Bernoulli
 * draw with P(1 | row bit 0) = b/(a+b) and P(1 | row bit 1) = d/(c+d), so the
 * neighbour in slot k of row u is drawn from Philox keyed by (seed, u, k) with
 * no sort or transpose.  Candidates >= num_nodes are redrawn.
 *   thr0, thr1   the two probabilities scaled to [0, 65536]
 *   indices      device int64[indptr[num_rows]] (output)
 */
int apt_synth_rmat_fill(const int64_t* indptr, int64_t num_rows, int64_t row_begin,
                        int64_t num_nodes, int64_t num_edges, int levels, uint64_t seed,
                        uint32_t thr0, uint32_t thr1, int64_t* indices, void* stream);

/* Plain device-to-device copy of `bytes` (multiple of 16) with a known
 * traffic of `bytes` read + `bytes` written: the reference point for scaling
 * the FETCH_SIZE / WRITE_SIZE hardware counters. */
int apt_synth_copy(const void* src, void* dst, int64_t bytes, void* stream);

/* Random-access probe: num_accesses accesses, one per work item, each to a
 * pseudo-random 4-byte word of `table` (device memory, table_bytes long).
 * The sampling and relabel kernels are bound by the number of such
 * transactions, not by bytes; the benchmark measures the GPU's rate for them
 * with this call and quotes the kernels against it.
 *   mode  0 load, 1 store, 2 atomicMin (result unused), 3 atomicMin (result
 *         used), 4 aligned 16-byte load, 5 a load and an atomicMin at two
 *         independent random places per work item
 *   salt  varies the address sequence between calls
 *   sink  device uint32[1] (never written in practice; keeps loads alive) */
int apt_synth_random_access(int mode, void* table, int64_t table_bytes, int64_t num_accesses,
                            uint32_t salt, void* sink, void* stream);

/* What a step between two dependent phases costs, two ways.
 * apt_synth_grid_barrier: one kernel of num_groups workgroups (256 threads) that
 *   run `phases` phases separated by a grid-wide barrier (arrival counter and
 *   generation word in device memory); in every phase a thread writes a word
 *   that another workgroup reads after the barrier.  The spin is bounded: if a
 *   workgroup gives up, state[128] counts it and the kernel ends.
 *   state  device uint32[192], all zero before the first call (arrivals at word
 *          0, generation at 64, failures at 128)
 *   buf    device uint32[num_groups * 256]
 *   num_groups is limited to half of what can be resident at once.
 * apt_synth_empty_launches: `count` launches of an empty kernel, each dependent
 *   on the one before by stream order. */
int apt_synth_grid_barrier(int num_groups, int phases, void* state, void* buf, void* stream);
int apt_synth_empty_launches(int count, void* buf, void* stream);

#ifdef __cplusplus
}
#endif
#endif
