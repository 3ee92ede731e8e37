/*
 * apt_synth.h — libapt_bench.so: synthetic inputs and measurement helpers for
 * the benchmark and the tests.  A library of its own, not part of the product
 * ABI (libapt_hip.so, apt_amd.h); no counterpart in the reference, which loads
 * OGB datasets through DGL (scripts/preprocess_dataset.py, scripts/load_data.py).
 * Every function returns 0 or an error code whose text apt_synth_last_error()
 * gives.
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

/* Turns a forward CSR (fwd_indptr int64[num_nodes + 1], fwd_indices) into the rows
 * of its symmetrised form with a self-loop per node, unsorted and with repeats:
 * row u = [u, the forward neighbours of u, every w with a forward edge w -> u]
 * (what dgl.add_self_loop + dgl.to_bidirected give before parallel edges are
 * merged; reference scripts/load_data.py:13-17).  The caller sizes the rows:
 *   indptr   device int64[num_nodes + 1], row u holding 1 + out-degree + in-degree
 *   cursor   device uint32[num_nodes], all zero (tickets of the reverse copies)
 *   out      device int64[indptr[num_nodes]]
 * The order of the reverse copies inside a row depends on scheduling; sort the
 * rows (and drop repeats) afterwards. */
int apt_synth_symmetrize_fill(const int64_t* fwd_indptr, const int64_t* fwd_indices, int64_t num_nodes,
                              int64_t num_fwd_edges, const int64_t* indptr, void* cursor, int64_t* out,
                              void* stream);

/* Text of the last error of this library on the calling thread. */
const char* apt_synth_last_error(void);

#ifdef __cplusplus
}
#endif
#endif
