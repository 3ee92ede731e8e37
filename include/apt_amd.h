/*
 * apt_amd.h — C ABI of the MI355X (gfx950) mini-batch construction library.
 *
 * One shared library (libapt_hip.so) implements these entry points with
 * hand-written HIP kernels.  Every pointer named "device" is device memory of
 * the GPU that is current when the call is made; `stream` is a hipStream_t
 * passed as void* (NULL = the default stream).  Nothing here allocates or
 * frees device memory: outputs and scratch come from the caller.  Calls are
 * asynchronous unless the comment says otherwise.
 *
 * Return value: 0 on success, a negative APT_E* code on failure; the message
 * for the calling thread's last failure is apt_last_error().  A failing call
 * launches nothing.
 *
 * Conventions shared with the reference (src/utils.h:14-21):
 *   ids and offsets are int64; ENCODE_ID(i) = -(i)-2 marks "row i of the
 *   second table" in a position map; -1 in a feature position map means
 *   "not present".  In id arrays a negative id is padding: it has no
 *   neighbours, is not relabelled and stays negative in outputs.
 *
 * What the host can check (null pointers, sizes, alignment, workspace) is
 * checked before anything is launched.  Values that live in device memory are
 * checked by the kernels where an entry point's comment says what happens to a
 * value out of range (ids and positions: treated as padding, counted as misses
 * or skipped); the CSR arrays of a graph (indptr non-decreasing and within
 * indices) and index arrays that address a caller's side table (weight_row,
 * eids) are taken on trust, as the reference takes all of its inputs.
 *
 * Each entry point cites the reference interface it replaces.
 */
#ifndef APT_AMD_H_
#define APT_AMD_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define APT_OK 0
#define APT_EINVAL (-1)  /* bad argument (null pointer, negative size, ...) */
#define APT_ELIMIT (-2)  /* size beyond what the entry point supports */
#define APT_EWORKSPACE (-3) /* workspace too small */
#define APT_EHIP (-4)    /* a HIP runtime call failed */

#define APT_MAX_HOPS 8

/* Filled by apt_minibatch_sample_deferred: the description of a batch's last
 * relabel pass, for apt_gather_rows_with_lookup or apt_minibatch_lookup to
 * carry out.  Host memory, opaque, valid while the batch's buffers are. */
typedef struct apt_pending_lookup {
  uint64_t opaque[64];
} apt_pending_lookup;
#define APT_MAX_BUCKETS 64 /* reference: MAX_NUM_DEVICES 33 (src/cuda/npc_kernel.h:13) */

const char* apt_last_error(void);
/* Raised whenever a struct of this header or a signature changes; a binding
 * compares apt_abi_version() of the library it loaded with the header it was
 * written against. */
#define APT_ABI_VERSION 2
int apt_abi_version(void);

/* Kernel-variant knobs for measurement (process-wide, not thread-safe, no
 * counterpart in the reference whose launch shapes are compile-time constants,
 * src/cuda/npc_kernel.h:10-14).  value 0 restores the default.
 *   "sample_lanes_per_row"   8|16|32|64 lanes of a wavefront per frontier row
 *   "sample_min_workgroups"  workgroups a sampling launch must have before a lane
 *                            group is given more than one row
 *   "sample_direct_rows"     1|2|4 rows a lane group of the sampler has in flight where the launch is
 *                            too small to give a group several rows through the LDS-staged path
 *   "gather_rows_in_flight"  1|2|4|8 rows a lane group loads before storing
 *   "gather_max_blocks"      cap on the gather grid (rows are strided over)
 *   "gather_vector_bytes"    2|4|8|16: widest load/store a lane of the gather uses
 *                            (16 = global_load_dwordx4 where alignment allows)
 *   "relabel_lds"            1 (default; 0 = off) apt_relabel handles inputs of up to 8192
 *                            items in one workgroup with its hash table in LDS (one launch)
 *                            instead of the passes over a table in device memory
 *   "gather_store_policy"    how the gather stores a row's 16-byte pieces: 0 (default; 0 here
 *                            is a value, not "default of the day") chosen per launch from
 *                            the bytes it writes (write-through up to 128 MB; beyond that
 *                            non-temporal except for the part written last, see
 *                            "gather_wt_tail_mib"), 1 non-temporal, 2 plain, 3 write-through
 *   "gather_wt_tail_mib"     with policy 0 and an output above 128 MB: how many MiB at the
 *                            end of the output are stored write-through (0 = default, 64;
 *                            1 = practically none)
 *   "minibatch_payload_bits" width of the id field of rank-table entries (0 = as
 *                            narrow as the plan allows); wider = fewer epochs
 *                            between table refills (used to test the refill)
 *   "minibatch_fuse_mark"    1 (default; note: 0 here also means "off", not
 *                            "default") the sampling kernel of apt_minibatch_sample
 *                            also does the rank-table lookup / bid of each id
 *   "block_fused_scan"       1 (default; 0 = off) apt_block_formats lets its place
 *                            and scatter workgroups add up the tile counts
 *                            themselves when there are few tiles; off = always
 *                            the separate scan launches of large inputs */
int apt_set_tuning(const char* key, int value);

/* A CSR (CSC in the reference's naming: row v lists the in-neighbours of v)
 * graph as the reference registers it with mix_cache_graphs
 * (src/cache_graphs.cc:12-49, src/state.h:18-23).
 *   indptr/indices        the "global" table (uva_* in the reference): row r
 *                         describes node row_begin + r, r in [0, num_rows).
 *   cached_indptr/indices optional second table (dev_* in the reference).
 *   adj_pos_map           optional int64[num_total_nodes]: >= 0 -> row of the
 *                         cached table, < -1 -> row -(p)-2 of the global
 *                         table.  NULL = identity (node v is global row
 *                         v - row_begin; nodes outside the range have no row
 *                         and degree 0).
 * All pointers are device memory. */
typedef struct apt_graph {
  const int64_t* indptr;
  const int64_t* indices;
  int64_t row_begin;
  int64_t num_rows;
  const int64_t* cached_indptr;
  const int64_t* cached_indices;
  int64_t num_cached_rows;
  const int64_t* adj_pos_map;
  int64_t num_total_nodes;
} apt_graph;

/* One hop of uniform neighbour sampling.
 * Replaces LocalSampleNeighbors / _CSRRowWiseSampleReplaceKernel
 * (src/cuda/npc_kernel.cu:248-316), op local_sample_one_layer
 * (src/sampling.cc:13-17).
 *
 *   frontier          device int64[num_frontier]
 *   num_frontier_dev  optional device int64[1]; when not NULL the kernel
 *                     processes min(*num_frontier_dev, num_frontier) rows and
 *                     the host value only sizes the launch
 *   replace != 0      the reference's semantics: every row with degree > 0
 *                     gets exactly `fanout` draws with replacement
 *   replace == 0      without replacement: min(fanout, degree) neighbours;
 *                     a row with degree <= fanout is copied whole, in CSR order
 *   rng_seed, hop     Philox4x32-10 key (rng_seed) and counter word; the draw
 *                     for output slot s of node v uses counter (v, hop, s), so
 *                     results do not depend on launch geometry
 *   out_neighbors     device int64[num_frontier * fanout], row-major, unused
 *                     slots hold -1 (the reference leaves them uninitialised)
 *   out_counts        optional device int64[num_frontier]
 *   out_total         optional device int64[1], incremented by the number of
 *                     sampled edges (caller clears it)
 */
int apt_sample_neighbors(const apt_graph* graph, const int64_t* frontier,
                         int64_t num_frontier, const int64_t* num_frontier_dev,
                         int fanout, int replace, uint64_t rng_seed, int hop,
                         int64_t* out_neighbors, int64_t* out_counts,
                         int64_t* out_total, void* stream);

/* Relabel to compact ids in first-occurrence order.
 * Replaces TensorRelabelCSC (src/cuda/relabel.cu:175-185), op relabel_csc
 * (src/relabel.cc:9-15).
 *
 *   unique   = distinct non-negative values of cat(seeds, neighbors) in order
 *              of first occurrence; device int64[num_seeds + num_neighbors]
 *              capacity, the first *num_unique entries are written
 *   relabeled[j] = position of neighbors[j] in unique (or neighbors[j] itself
 *              if negative); device int64[num_neighbors]
 *   num_seeds_dev      optional device int64[1] overriding num_seeds (<= it)
 *   neighbor_stride    when num_seeds_dev is given the neighbours considered
 *                      are the first *num_seeds_dev * neighbor_stride entries;
 *                      otherwise ignored
 *   num_unique_dev     device int64[1], receives the count
 *   num_unique_host    optional host int64*; when not NULL the call
 *                      synchronises the stream and stores the count there
 *   workspace          device scratch of at least
 *                      apt_relabel_workspace_bytes(num_seeds + num_neighbors)
 */
size_t apt_relabel_workspace_bytes(int64_t num_items);
int apt_relabel(const int64_t* seeds, int64_t num_seeds,
                const int64_t* num_seeds_dev, const int64_t* neighbors,
                int64_t num_neighbors, int64_t neighbor_stride,
                int64_t* unique, int64_t* relabeled, int64_t* num_unique_dev,
                int64_t* num_unique_host, void* workspace,
                size_t workspace_bytes, void* stream);

/* apt_relabel's result through a node-indexed rank table instead of a hash table,
 * for callers whose ids index a known range [0, rank_table_len) (the nodes of a
 * registered graph): no probing, no fill pass per call, and nodes already in the
 * batch cost one load.  Same reference interface as apt_relabel (relabel_csc,
 * src/relabel.cc:9-15, called once per hop by python/npc/sampler.py:187-203).
 *   rank_table    as in apt_minibatch_sample (apt_rank_table_bytes /
 *                 apt_rank_table_init), but a table of its own: entries are laid
 *                 out for up to apt_relabel_ranked_max_items() items per call
 *   num_seeds_dev, neighbor_stride   as in apt_relabel
 *   continued     0: a fresh relabel of cat(seeds, neighbors).
 *                 != 0: the caller vouches that seeds[0 .. num_seeds) is exactly
 *                 the unique list that the previous call on this table wrote
 *                 (same values, same order, no other call on the table since):
 *                 the table still holds their ids, so only the neighbours are
 *                 looked up or bid for.  The result is what a fresh call gives.
 *                 Bit 1 (values 2 and 3, for a fresh and a continued call): the
 *                 neighbours come from apt_sample_neighbors_bidding, which has
 *                 placed this call's bids already and left the slot states in
 *                 `relabeled` (in / out then); same table, same workspace, same
 *                 seeds, no other call on the table in between; num_neighbors > 0.
 *   unique        device int64[num_seeds + num_neighbors] capacity
 *   num_unique_dev   device int64[1], receives the number of unique ids
 *   num_outside_dev  device int64[1], incremented once per id that the table
 *                 cannot hold (>= rank_table_len); the caller clears it.  When
 *                 it is not zero afterwards the outputs are not a valid relabel
 *                 (such ids were treated as padding) and the caller falls back
 *                 to apt_relabel
 *   counts_host   optional host int64[2]; when not NULL the call synchronises
 *                 the stream and stores the two counters there
 *   workspace     apt_relabel_ranked_workspace_bytes(num_seeds + num_neighbors)
 *                 bytes, 16-byte aligned, zeroed once with
 *                 apt_minibatch_workspace_init (a larger one may be reused for
 *                 smaller calls; calls leave it ready for the next one)
 * Negative ids are padding, as in apt_relabel. */
int64_t apt_relabel_ranked_max_items(void);
size_t apt_relabel_ranked_workspace_bytes(int64_t num_items);
int apt_relabel_ranked(const int64_t* seeds, int64_t num_seeds, const int64_t* num_seeds_dev,
                       const int64_t* neighbors, int64_t num_neighbors, int64_t neighbor_stride,
                       int continued, void* rank_table,
                       int64_t rank_table_len, int64_t* unique, int64_t* relabeled,
                       int64_t* num_unique_dev, int64_t* num_outside_dev,
                       int64_t* counts_host, void* workspace,
                       size_t workspace_bytes, void* stream);

/* apt_sample_neighbors (src/sampling.cc:13-17) that places the rank-table bids of
 * the apt_relabel_ranked call that follows on the way (the reference's sampler
 * calls the two back to back per hop, python/npc/sampler.py:187-203): the
 * sampling kernel has every id in registers, and a bid placed there overlaps
 * with its own random reads.  Sampled ids are those of apt_sample_neighbors.
 *   fanout          at most 64
 *   continued       0: the frontier starts a batch (its rows bid for their nodes
 *                   too).  != 0: the frontier is the unique list the previous
 *                   apt_relabel_ranked on this table wrote, as for that call
 *   slot_states     device int64[num_frontier * fanout]: pass it as `relabeled`
 *                   to apt_relabel_ranked with bit 1 of `continued` set
 *   num_outside_dev optional device int64[1]: incremented per frontier id that
 *                   the table cannot hold (fresh calls; the caller clears it)
 *   workspace       the workspace of that apt_relabel_ranked call
 * A call that is not followed by its apt_relabel_ranked leaves bids of an
 * abandoned batch in the table: the next call on the table must then be a fresh
 * one (continued == 0), which ignores them; and, if the abandoned call was a
 * continued one, flags in the workspace that only its apt_relabel_ranked would
 * have consumed: the workspace is then cleared again with
 * apt_minibatch_workspace_init. */
int apt_sample_neighbors_bidding(const apt_graph* graph, const int64_t* frontier,
                                 int64_t num_frontier, const int64_t* num_frontier_dev,
                                 int fanout, int replace, uint64_t rng_seed, int hop,
                                 int64_t* out_neighbors, int64_t* out_counts,
                                 int64_t* out_total, int continued, void* rank_table,
                                 int64_t rank_table_len, int64_t* slot_states,
                                 int64_t* num_outside_dev, void* workspace,
                                 size_t workspace_bytes, void* stream);

/* apt_relabel without a workspace argument and without any allocation.
 * No counterpart in the reference.  It is for callers that cannot allocate:
 * code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc.  The scratch of the passes lives in a fixed device array inside
 * the library (about 44 MiB per GPU, held until the process ends), so
 *   - num_seeds + num_neighbors must not exceed apt_relabel_static_max_items()
 *     (2^21); larger calls fail with APT_ELIMIT and enqueue nothing;
 *   - every call on a GPU shares that GPU's array: calls that overlap on one
 *     GPU (different streams or threads) race; calls on one stream do not;
 *   - the first call on a device resolves the array's address (no allocation,
 *     but make it outside a graph capture).
 * Arguments and results as apt_relabel (no host copy of the count). */
int64_t apt_relabel_static_max_items(void);
int apt_relabel_static(const int64_t* seeds, int64_t num_seeds,
                       const int64_t* num_seeds_dev, const int64_t* neighbors,
                       int64_t num_neighbors, int64_t neighbor_stride,
                       int64_t* unique, int64_t* relabeled,
                       int64_t* num_unique_dev, void* stream);

/* Feature tables as the reference registers them with cache_feats_shared
 * (src/cache_feats.cc:14-61, src/state.h:10-16).
 *   local_table  [num_local_rows, local_dim] elements ("uva_feats")
 *   cache_table  [num_cache_rows, out_dim] elements ("dev_feats"), optional
 *   pos_map      optional int64[num_total_nodes]: >= 0 cache row, < -1 local
 *                row -(p)-2, -1 not present.  NULL = identity into
 *                local_table.
 *   col_offset   first column of local_table rows that is copied
 *                ("feat_dim_offset"); out_dim columns are copied
 *   elem_size    bytes per element: 4 (fp32, the reference) or 2 (bf16/fp16)
 */
typedef struct apt_feat_store {
  const void* local_table;
  int64_t num_local_rows;
  int64_t local_dim;
  const void* cache_table;
  int64_t num_cache_rows;
  const int64_t* pos_map;
  int64_t num_total_nodes;
  int64_t col_offset;
  int64_t out_dim;
  int elem_size;
} apt_feat_store;

/* Indexed feature gather: out[r, :] = row of node index[r].
 * Replaces IndexSelectAll / _CSRRowWiseLoadSubtensorAlignedAllKernel
 * (src/cuda/npc_kernel.cu:187-246), op load_subtensor
 * (src/load_subtensor.cc:19-40).
 *   index          device int64[num_index]
 *   num_index_dev  optional device int64[1] (as in apt_sample_neighbors)
 *   out            device [num_index, out_dim] elements
 *   miss_count     optional device int64[1], incremented once per requested
 *                  node that is not present (position -1, a negative id, or
 *                  an id/position out of range); such rows are zero-filled
 *                  (the reference reads out of bounds there)
 */
int apt_gather_rows(const apt_feat_store* store, const int64_t* index,
                    int64_t num_index, const int64_t* num_index_dev, void* out,
                    int64_t* miss_count, void* stream);

/* Measurement hook (no counterpart in the reference): the next gather / permute /
 * scatter launch made by the calling thread records start_event when its kernel
 * begins and stop_event when it ends (the events ride on the dispatch itself), so
 * hipEventElapsedTime gives the kernel's duration without the dispatch gaps that a
 * hipEventRecord bracket includes.  Both are hipEvent_t created by the caller;
 * one-shot; NULL, NULL cancels. */
int apt_time_next_gather(void* start_event, void* stop_event);
/* The same hook for the sampling kernel: the next sampling launch made by the
 * calling thread with hop index `hop` (apt_sample_neighbors, or that hop inside
 * apt_minibatch_sample) records the two events on its dispatch.  One-shot;
 * NULL, NULL cancels. */
int apt_time_next_sample(int hop, void* start_event, void* stop_event);

/* Row permutation of a dense [rows, dim] table, the on-GPU halves of
 * FeatShuffle (src/feat_shuffle.cc:9-30) and the row gather by inverse_idx in
 * front of it (python/npc/model/sage_model.py:67):
 *   unpack (fwd):  out[i, :] = in[perm[i], :], i < n   (index_select, :27);
 *                  a perm[i] outside [0, num_in_rows) yields a zero row
 *   pack   (bwd):  out[perm[i], :] = in[i, :], i < n   (index_select_backward
 *                  of a bijection, :14-16); rows of out that no perm[i] names
 *                  are left untouched, so the caller zero-fills out first when
 *                  perm is not onto -- or passes workspace
 *                  (apt_scatter_workspace_bytes(num_out_rows) bytes, 4-byte
 *                  aligned; NULL = none): the scatter then flags the rows it
 *                  writes and the library zeroes exactly the others, far cheaper
 *                  than a fill of wide rows; a perm[i] outside [0, num_out_rows)
 *                  is skipped. */
int apt_permute_rows(const void* in, int64_t num_in_rows, const int64_t* perm,
                     int64_t n, int64_t dim, int elem_size, void* out,
                     void* stream);
size_t apt_scatter_workspace_bytes(int64_t num_out_rows);
int apt_scatter_rows(const void* in, const int64_t* perm, int64_t n,
                     int64_t dim, int elem_size, void* out, int64_t num_out_rows,
                     void* workspace, size_t workspace_bytes, void* stream);

/* Stable bucketing of ids by owner.
 * Replaces ClusterAndPermute (src/cuda/npc_kernel.cu:318-382,434-470), the
 * local half of ShuffleSeeds (src/sampling.cc:159-175).
 *   owner(v): d = id_offset; while (d+1 < num_buckets && min_vids[d+1] <= v) ++d;
 *             if (d < node_beg || d >= node_end) d = rank;
 *   bucket_size[num_buckets], bucket_offset[num_buckets] (inclusive cumsum),
 *   sorted_ids[n] (ids grouped by bucket, input order kept inside a bucket —
 *   the reference's order inside a bucket is whatever its atomics produce),
 *   permutation[n] (slot of ids[i] in sorted_ids).
 *   n_dev        optional device int64[1] (as in apt_sample_neighbors); outputs
 *                beyond the actual count are not written
 *   min_vids     device int64[num_buckets + 1]
 *   workspace    device scratch, apt_bucket_workspace_bytes(n, num_buckets)
 */
size_t apt_bucket_workspace_bytes(int64_t n, int num_buckets);
int apt_cluster_permute(const int64_t* ids, int64_t n, const int64_t* n_dev,
                        const int64_t* min_vids,
                        int num_buckets, int64_t id_offset, int rank,
                        int node_beg, int node_end, int64_t* bucket_size,
                        int64_t* bucket_offset, int64_t* sorted_ids,
                        int64_t* permutation, void* workspace,
                        size_t workspace_bytes, void* stream);

/* Bucketing of feature requests into "present here" (bucket 0) and per remote
 * worker buckets.  Replaces MultiMachinesClusterAndPermute
 * (src/cuda/npc_kernel.cu:384-432,472-508), op cluster_reqs
 * (src/load_subtensor.cc:83-86).
 *   bucket(v) = feat_pos_map[v] != -1 ? 0 : remote_worker_map[owner(v)]
 *   with owner(v) the min_vids scan above started at 0 and no rank override.
 *   bucket_offset is optional (NULL to skip). */
int apt_cluster_reqs(const int64_t* ids, int64_t n, const int64_t* n_dev,
                     const int64_t* feat_pos_map,
                     int64_t num_total_nodes, const int64_t* remote_worker_map,
                     const int64_t* min_vids, int world_size,
                     int num_remote_workers, int64_t* bucket_size,
                     int64_t* bucket_offset, int64_t* sorted_ids,
                     int64_t* permutation, void* workspace,
                     size_t workspace_bytes, void* stream);

/* Whole multi-hop mini-batch in one call: for every hop, sample the current
 * frontier, relabel, and make the unique node list the next frontier.
 * Replaces the DP branch of MixedPSNeighborSampler.sample
 * (python/npc/sampler.py:187-203,358-364) with its per-hop
 * local_sample_one_layer + relabel_csc calls; results are identical to calling
 * apt_sample_neighbors (hop index = position in hop_fanouts) and apt_relabel
 * hop by hop.  Nothing is read back to the host.
 *
 *   hop_fanouts     host int[num_hops], from the seeds outward (the reference's
 *                   --fan_out list reversed, python/npc/sampler.py:191)
 *   rng_seed_dev    optional device uint64[1] overriding rng_seed (lets a
 *                   captured HIP graph be replayed with a new seed)
 *   rank_table      device scratch of apt_rank_table_bytes(rank_table_len) bytes,
 *                   256-byte aligned, rank_table_len > every node id of the
 *                   graph (4 bytes per node + a small state block); initialise
 *                   it once with apt_rank_table_init, after that it belongs to
 *                   the library: calls may follow each other on one stream
 *                   without any clearing in between.  A node id outside
 *                   [0, rank_table_len) is treated like padding (no edge, not
 *                   in the node list): a negative one appears unchanged in
 *                   relabeled[], except that the 2^32 + 2 most negative
 *                   values, which the driver uses for slot states, become -1.
 *   nodes           device int64[capacity(num_hops)]: the unique node list;
 *                   its first sizes[h] entries are the frontier of hop h and
 *                   the source nodes of hop h-1's block, its first
 *                   sizes[num_hops] entries the input nodes of the batch
 *   neighbors[h], relabeled[h]   host arrays of device int64[capacity(h) *
 *                   hop_fanouts[h]]: sampled ids (-1 padded) and their compact
 *                   ids (= index into nodes)
 *   counts[h]       optional (counts or counts[h] may be NULL) device
 *                   int64[capacity(h)]
 *   sizes           device int64[num_hops + 2]: sizes[h] = frontier rows
 *                   entering hop h (sizes[0] = batch), sizes[num_hops] = input
 *                   nodes, sizes[num_hops + 1] = sampled edges of the batch
 *   workspace       device scratch of apt_minibatch_workspace_bytes, zeroed once
 *                   with apt_minibatch_workspace_init before its first use (and
 *                   again after a call that failed half-way); calls leave it
 *                   ready for the next one
 *   capacity(h)     apt_minibatch_capacity: batch * prod_{i<h}(1 + fanout_i)
 */
size_t apt_rank_table_bytes(int64_t num_total_nodes);
int apt_rank_table_init(void* table, size_t table_bytes, void* stream);
size_t apt_minibatch_workspace_bytes(int64_t batch, const int* hop_fanouts, int num_hops);
int apt_minibatch_workspace_init(void* workspace, size_t workspace_bytes, void* stream);
int64_t apt_minibatch_capacity(int64_t batch, const int* hop_fanouts, int num_hops, int hop);
int apt_minibatch_sample(const apt_graph* graph, const int64_t* seeds, int64_t batch,
                         const int* hop_fanouts, int num_hops, int replace,
                         uint64_t rng_seed, const uint64_t* rng_seed_dev,
                         void* rank_table, int64_t rank_table_len, int64_t* nodes,
                         int64_t* const* neighbors, int64_t* const* relabeled,
                         int64_t* const* counts, int64_t* sizes, void* workspace,
                         size_t workspace_bytes, void* stream);

/* apt_minibatch_sample in two parts, for a caller that gathers the batch's
 * features right after sampling it (no counterpart in the reference, where
 * sampling and load_subtensor are separate operators, python/npc/sampler.py:
 * 187-203 and python/npc/ops.py load_subtensor).  The last pass of the relabel
 * (slots that lost the race for a node read the winner's id) needs only the
 * placing of the last hop's owners before it and nothing but relabeled[] after
 * it, and it waits on a few dependent random reads, while the gather is bound
 * by bandwidth: apt_minibatch_sample_deferred leaves that pass out and
 * describes it in *pending; apt_gather_rows_with_lookup runs it in the first
 * workgroups of the gather's own launch (same stream, no other launch between
 * the two calls may touch the batch's buffers), apt_minibatch_lookup runs it as
 * a launch of its own.  Until one of the two has run, relabeled[h] holds slot
 * states in some places; nodes, neighbors, counts and sizes are final.
 * Results are those of apt_minibatch_sample + apt_gather_rows, bit for bit. */
int apt_minibatch_sample_deferred(const apt_graph* graph, const int64_t* seeds, int64_t batch,
                                  const int* hop_fanouts, int num_hops, int replace,
                                  uint64_t rng_seed, const uint64_t* rng_seed_dev,
                                  void* rank_table, int64_t rank_table_len, int64_t* nodes,
                                  int64_t* const* neighbors, int64_t* const* relabeled,
                                  int64_t* const* counts, int64_t* sizes, void* workspace,
                                  size_t workspace_bytes, void* stream,
                                  apt_pending_lookup* pending);
int apt_minibatch_lookup(const apt_pending_lookup* pending, void* stream);
int apt_gather_rows_with_lookup(const apt_feat_store* store, const int64_t* index,
                                int64_t num_index, const int64_t* num_index_dev, void* out,
                                int64_t* miss_count, const apt_pending_lookup* pending,
                                void* stream);

/* Epoch driver: what a trainer's data loader does around the sampler, with the
 * per-batch host work done by a thread of this library instead of the caller's.
 * Replaces the loop `for input_nodes, output_nodes, blocks in dataloader:` +
 * load_subtensor of the reference's trainer (examples/train.py:84-94,139; the
 * dgl DataLoader is built in python/npc/utils/utils.py with batch size :425),
 * DP strategy: per batch MixedPSNeighborSampler.sample
 * (python/npc/sampler.py:187-203,358-364) and load_subtensor
 * (python/npc/ops.py:598-600).
 *
 * The caller provides num_slots sets of device buffers ("slots", what
 * apt_minibatch_sample and apt_gather_rows take, plus a HIP stream each) and,
 * per epoch, the seeds of all batches as one device array.  The driver's thread
 * enqueues batch i on slot i % num_slots: apt_minibatch_sample_deferred +
 * apt_gather_rows_with_lookup (no features: apt_minibatch_sample alone; a
 * partitioned store: apt_minibatch_sample, apt_cluster_reqs on the input nodes,
 * apt_gather_rows of bucket 0), then copies the batch's sizes to pinned host
 * memory and records an event.  num_slots batches are in flight at any time.
 * Batch i is built from seeds[i * batch, (i + 1) * batch) with rng seed
 * rng_seed0 + i and is bit-identical to what those calls give on their own.
 * With slots on four or more different streams the driver launches a batch's two
 * large kernels at half width (512 workgroups for sampling, 1024 for the gather),
 * so that the gather of one batch and the last-hop sampler of another are
 * resident together: 5 % more batches per second than full-width launches that
 * take turns; results do not depend on the launch shape.
 * Nothing here allocates device memory; pinned host memory for the sizes, the
 * events and the thread belong to the handle. */
#define APT_MAX_SLOTS 16
/* One hop's block in the formats a GNN layer consumes (apt_block_formats), buffers
 * sized for the hop's upper bounds; csr_* NULL: COO + CSC only. */
typedef struct apt_block_buffers {
  int64_t* coo_row;
  int64_t* coo_col;
  int64_t* csc_indptr;
  int64_t* csr_indptr;
  int64_t* csr_indices;
  int64_t* csr_eids;
  void* workspace;                    /* apt_block_workspace_bytes(capacity(h), fanout, capacity(h + 1), csr) */
  size_t workspace_bytes;
} apt_block_buffers;

typedef struct apt_batch_slot {
  void* stream;                       /* hipStream_t of this slot (not the default stream) */
  int64_t* nodes;                     /* as in apt_minibatch_sample, sized by apt_minibatch_capacity */
  int64_t* neighbors[APT_MAX_HOPS];
  int64_t* relabeled[APT_MAX_HOPS];
  int64_t* counts[APT_MAX_HOPS];      /* counts[0] == NULL: no counts */
  int64_t* sizes;                     /* device int64[num_hops + 2] */
  void* rank_table;                   /* a table per slot (apt_rank_table_init) */
  void* workspace;                    /* apt_minibatch_workspace_bytes, initialised once */
  size_t workspace_bytes;
  void* features;                     /* [capacity(num_hops), out_dim] elements, or NULL for no gather */
  int64_t* miss_count;                /* optional device int64[1], see apt_gather_rows */
  /* partitioned feature store only (apt_epoch_desc.has_requests), as in apt_cluster_reqs: */
  int64_t* request_sizes;             /* device int64[num_remote_workers] */
  int64_t* request_offsets;           /* optional */
  int64_t* request_ids;               /* device int64[capacity(num_hops)] */
  int64_t* request_perm;              /* device int64[capacity(num_hops)] */
  void* request_workspace;            /* apt_bucket_workspace_bytes(capacity(num_hops), num_remote_workers) */
  size_t request_workspace_bytes;
  /* block formats only (apt_epoch_desc.formats): */
  apt_block_buffers blocks[APT_MAX_HOPS];
  int64_t* block_edges;               /* device int64[num_hops]: receives every hop's edge count */
} apt_batch_slot;

typedef struct apt_epoch_desc {
  apt_graph graph;
  apt_feat_store store;               /* read only when the slots have feature buffers */
  int64_t batch;
  int num_hops;
  int hop_fanouts[APT_MAX_HOPS];      /* from the seeds outward */
  int replace;
  int64_t rank_table_len;
  int has_requests;                   /* != 0: bucket the input nodes (apt_cluster_reqs), gather bucket 0 */
  const int64_t* request_pos_map;     /* feat_pos_map of apt_cluster_reqs */
  int64_t request_num_total_nodes;
  const int64_t* remote_worker_map;
  const int64_t* min_vids;
  int world_size;
  int num_remote_workers;
  int formats;                        /* != 0: every hop's block is also emitted as COO + CSC (+ CSR where the
                                         slot's csr_* buffers are not NULL), python/npc/sampler.py:44-69,76-91 */
  int num_slots;
  apt_batch_slot slots[APT_MAX_SLOTS];
} apt_epoch_desc;

typedef struct apt_epoch apt_epoch;   /* opaque */

/* apt_epoch_create   copies *desc (the buffers it points to stay the caller's and
 *                    must outlive the handle), creates events, pinned memory and
 *                    the thread, for the GPU that is current.
 * apt_epoch_begin    starts an epoch of num_batches batches over seeds (device
 *                    int64[num_batches * batch], must stay valid until the epoch
 *                    ends); the slots' streams first wait for ready_event
 *                    (hipEvent_t, may be NULL: the seeds are already complete).
 *                    An epoch still in progress is ended first.
 * apt_epoch_next     blocks until the next batch (they come in order) is
 *                    complete on the GPU; *slot = the slot that holds it,
 *                    sizes_host[num_hops + 2] = its sizes as apt_minibatch_sample
 *                    defines them, followed, with formats, by num_hops more
 *                    entries, the blocks' edge counts (sizes_host then has
 *                    2 * num_hops + 2 entries); request_sizes_host
 *                    [num_remote_workers] (optional) the request buckets.  The slot's buffers are
 *                    the caller's to read until apt_epoch_release.
 * apt_epoch_release  the caller is done with the batch apt_epoch_next returned
 *                    last: work it has enqueued on consumer_stream so far is
 *                    waited for (by the slot's stream, not the host) before the
 *                    slot is reused for batch i + num_slots.  Must be called
 *                    before the next apt_epoch_next.
 * apt_epoch_end      drops what has not been enqueued, synchronises the slots'
 *                    streams; after it every buffer is quiescent.  Optional
 *                    after the last batch.
 * apt_epoch_destroy  apt_epoch_end, then stops the thread and frees the handle.
 * One consumer thread per handle.  A batch that could not be enqueued makes
 * apt_epoch_next return its error. */
int apt_epoch_create(const apt_epoch_desc* desc, apt_epoch** out);
int apt_epoch_begin(apt_epoch* epoch, const int64_t* seeds, int64_t num_batches, uint64_t rng_seed0,
                    void* ready_event);
int apt_epoch_next(apt_epoch* epoch, int* slot, int64_t* sizes_host, int64_t* request_sizes_host);
int apt_epoch_release(apt_epoch* epoch, void* consumer_stream);
int apt_epoch_end(apt_epoch* epoch);
int apt_epoch_destroy(apt_epoch* epoch);
/* Where the host's time went since the handle was created: what the driver's
 * thread spent enqueueing batches (what a batch costs the host), and what
 * apt_epoch_next spent waiting, first for the batch to be on its stream, then
 * for the GPU to finish it. */
typedef struct apt_epoch_cost {
  int64_t batches;              /* batches enqueued so far */
  double enqueue_seconds;       /* driver thread, inside the enqueue calls */
  double wait_enqueue_seconds;  /* apt_epoch_next, waiting for the driver thread */
  double wait_gpu_seconds;      /* apt_epoch_next, waiting for the batch's completion event */
  double release_seconds;       /* apt_epoch_release, asking the consumer's stream whether it is idle */
} apt_epoch_cost;
int apt_epoch_host_cost(apt_epoch* epoch, apt_epoch_cost* cost);

/* Cache construction (the callers of the registries).
 *   apt_count_ids        freq[ids[i]] += 1 for ids in [0, num_total_nodes): the
 *                        access counting of a dry run (examples/dryrun.py:86-92,
 *                        counter[nodes] += 1 per batch, done there on the host);
 *                        n_dev as in apt_sample_neighbors
 *   apt_csr_row_degrees  degrees[i] = degree of node rows[i] (0 when the node has
 *                        no row in [row_begin, row_begin + num_rows))
 *   apt_csr_copy_rows    the adjacency rows of the chosen nodes as a second CSR:
 *                        out_indices[out_indptr[i] + k] = k-th neighbour of rows[i],
 *                        with out_indptr the exclusive prefix sum of the degrees
 *                        (n + 1 entries, out_indptr[n] = num_out_edges) — what
 *                        python/npc/ops.py:370-384 builds with one slice per node
 *                        before mix_cache_graphs.
 * The cached feature table is apt_gather_rows on the chosen ids. */
int apt_count_ids(const int64_t* ids, int64_t n, const int64_t* n_dev, int64_t* freq,
                  int64_t num_total_nodes, void* stream);
int apt_csr_row_degrees(const int64_t* indptr, int64_t row_begin, int64_t num_rows,
                        const int64_t* rows, int64_t n, int64_t* degrees, void* stream);
int apt_csr_copy_rows(const int64_t* indptr, const int64_t* indices, int64_t row_begin,
                      const int64_t* rows, int64_t n, const int64_t* out_indptr,
                      int64_t num_out_edges, int64_t* out_indices, void* stream);

/* Virtual nodes of SP mode: the part of a destination's neighbourhood that one
 * owner holds.  Replaces MapSrcDsttoVir / MapSrctoVir (src/cuda/npc_kernel.cu:15-113,
 * called by SrcDsttoVir / SrcToVir, src/sampling.cc:19-50) and GetVirSendOffset /
 * GetVirSendOffsetWithDst (:115-183).  owner() is the rule of apt_cluster_permute
 * (min_vids, id_offset, rank, node_beg, node_end as there).
 *   apt_map_to_vir, dst != NULL: vir_nodes[num_dst + num_src],
 *       vir[i] = owner(dst[i]) * num_dst + i,
 *       vir[num_dst + j] = owner(src[j]) * num_dst + world_size * num_dst + j / fanout
 *   dst == NULL: vir_nodes[num_src], vir[j] = owner(src[j]) * num_dst + j / fanout
 *   apt_vir_send_offset: lower bounds of multiples of base (= num_dst) in the
 *       sorted virtual nodes and in their unique values:
 *       with_dst == 0: send_offset[2 * world_size + 1]; [k] = lower_bound(sorted, k * base),
 *           k = 0..world_size; [world_size + k] = lower_bound(unique, k * base), k = 1..world_size
 *       with_dst != 0: send_offset[3 * world_size + 1]; [k] = lower_bound(sorted, k * base),
 *           k = 0..2 * world_size; [2 * world_size + k] = lower_bound(unique,
 *           (world_size + k) * base), k = 1..world_size */
int apt_map_to_vir(const int64_t* dst, int64_t num_dst, const int64_t* src, int64_t num_src,
                   int fanout, const int64_t* min_vids, int world_size, int64_t id_offset, int rank,
                   int node_beg, int node_end, int64_t* vir_nodes, void* stream);
int apt_vir_send_offset(int world_size, int64_t base, const int64_t* sorted_nodes, int64_t num_sorted,
                        const int64_t* unique_nodes, int64_t num_unique, int with_dst,
                        int64_t* send_offset, void* stream);

/* Sparse formats of a sampled block.  The reference hands (row, col) of a hop to
 * DGL, which materialises COO, CSR and CSC (python/npc/sampler.py:59-69,76-91;
 * create_block_from_csc :44-56 takes a CSC as it is).  Input is the hop's
 * fixed-stride block: relabeled[d * fanout + k] = k-th source of destination d,
 * negative where d has fewer neighbours.
 *   coo_row, coo_col   int64[num_dst * fanout]: edges in destination-major order,
 *                      row = source, col = destination; *num_edges_dev of them
 *   csc_indptr         int64[num_dst + 1] over destinations (its indices are
 *                      coo_row, its edge ids 0..E-1)
 *   csr_indptr         int64[num_src + 1] over sources, or NULL for no CSR;
 *   csr_indices, csr_eids  int64[num_dst * fanout]: destination and COO position of
 *                      every edge grouped by source, edges of one source by
 *                      increasing edge id (deterministic)
 * num_dst / num_src are upper bounds when the real counts live on the device
 * (num_dst_dev as n_dev in apt_sample_neighbors; sources need no count): the
 * offsets of rows past the real counts equal the edge total, i.e. empty rows.
 * workspace: apt_block_workspace_bytes(num_dst, fanout, num_src, csr != NULL)
 * bytes of device scratch; 0 = sizes out of range. */
size_t apt_block_workspace_bytes(int64_t num_dst, int fanout, int64_t num_src, int want_csr);
int apt_block_formats(const int64_t* relabeled, int64_t num_dst, const int64_t* num_dst_dev,
                      int fanout, int64_t num_src, int64_t* coo_row, int64_t* coo_col,
                      int64_t* csc_indptr, int64_t* num_edges_dev, int64_t* csr_indptr,
                      int64_t* csr_indices, int64_t* csr_eids, void* workspace,
                      size_t workspace_bytes, void* stream);

/* Aggregation over the COO edges of sampled blocks (optional stage).
 * Replaces CopyUSum / CopyESum / UMulESum (src/spmm.cc:9-42, src/cuda/spmm.cu:8-148)
 * and UAddV / UMulV (src/sddmm.cc:9-31, src/cuda/sddmm.cu:8-103).
 *
 * Edge e belongs to segment k = last k with coo_offset[k] <= e (the reference
 * concatenates the blocks of several ranks; one segment = plain COO):
 *   apt_spmm_sum  out[output_offset[k] + col[e], :] += x_e, x_e =
 *                   mode 0 (copy_u)  input[input_offset[k] + row[e], :]
 *                   mode 1 (copy_e)  input[e, :]
 *                   mode 2 (u_mul_e) input[input_offset[k] + row[e], :] * edata[e, :]
 *                 (the reference's u_mul_e kernel adds instead of multiplying,
 *                 src/cuda/spmm.cu:78, and has no caller; the product is
 *                 implemented).  `out` is fp32 [num_out_rows, dim] and must be
 *                 zero on entry.  grouped_dev, optional (NULL = unknown): device
 *                 flag written by apt_coo_is_grouped; when it is set (and there
 *                 is one segment) every row that lies inside a wavefront's 64
 *                 edges is stored instead of added atomically, which is what a
 *                 sampled block's destination-major COO gets.
 *   apt_coo_is_grouped  *flag = 1 iff col is non-decreasing (edges with equal col
 *                 are then consecutive), else 0; flag is a device int.
 *   apt_sddmm     out[e, :] = lhs[lhs_offset[k] + row[e], :] (+|*) rhs[rhs_offset[k] + col[e], :]
 *                 op 0 = u_add_v, 1 = u_mul_v; out is fp32 [num_edges, dim].
 * elem_size 4 = fp32 inputs (the reference), 2 = bf16 inputs; accumulation and
 * outputs are fp32.  All pointers device memory; the offset arrays have
 * num_segments (+1 for coo_offset) entries and may be NULL for "all zero"
 * (not coo_offset). */
int apt_spmm_sum(int mode, const int64_t* coo_row, const int64_t* coo_col, int64_t num_edges,
                 const void* input, int64_t num_in_rows, const void* edata, int64_t dim,
                 int elem_size, const int64_t* coo_offset, const int64_t* input_offset,
                 const int64_t* output_offset, int num_segments, float* out,
                 int64_t num_out_rows, const int* grouped_dev, void* stream);
int apt_coo_is_grouped(const int64_t* coo_col, int64_t num_edges, int* flag, void* stream);
/* SpMM over a sampled block in the layout the sampler and relabel emit
 * (apt_sample_neighbors / apt_relabel / apt_minibatch_sample): destination i
 * owns slots [i * fanout, (i+1) * fanout) of `neighbors` (compact source ids,
 * negative = no edge).  out[i, :] = sum (mean != 0: mean over the valid slots)
 * of input[neighbors[slot], :].  Same result as apt_spmm_sum mode 0 on the
 * block's COO (reference CopyUSum + the division by the fanout that
 * python/npc/model/sageconv.py:173-174 does), without atomics or zero-fill.
 * num_dst_dev: optional device int64[1] (as in apt_sample_neighbors). */
int apt_spmm_block(const int64_t* neighbors, int64_t num_dst, const int64_t* num_dst_dev,
                   int fanout, const void* input, int64_t num_src, int64_t dim, int elem_size,
                   int mean, float* out, void* stream);
int apt_sddmm(int op, const int64_t* coo_row, const int64_t* coo_col, int64_t num_edges,
              const void* lhs, int64_t num_lhs_rows, const void* rhs, int64_t num_rhs_rows,
              int64_t dim, int elem_size, const int64_t* coo_offset, const int64_t* lhs_offset,
              const int64_t* rhs_offset, int num_segments, float* out, void* stream);

/* GATConv aggregation (optional stage).  The reference's GAT layer computes its
 * attention with DGL on the sampled block (python/npc/model/gatconv.py:116-126):
 * el = (ft * attn_l).sum(-1), er likewise on the destination rows,
 * e = LeakyReLU(el[src] + er[dst]), a = edge_softmax over the in-edges of a
 * destination, out[dst] = sum a * ft[src].
 *   apt_gat_scores  out[r, h] = sum_d x[r, h, d] * attn[h, d]; x is
 *                   [num_rows, heads, dim] fp32 or bf16, attn and out fp32
 *   apt_gat_block   the rest, fused, over the sampler's fixed-stride block
 *                   (neighbors / num_dst / num_dst_dev / fanout as in
 *                   apt_spmm_block): ft [num_src, heads, dim] fp32 or bf16,
 *                   el [num_src, heads], er [num_dst, heads] fp32,
 *                   out [num_dst, heads, dim] fp32 (zero rows for destinations
 *                   without neighbours); attn_out, optional (NULL = not wanted):
 *                   [num_dst * fanout, heads] fp32 attention weights, 0 in empty
 *                   slots.  fp32 accumulation, fixed summation order. */
int apt_gat_scores(const void* x, int64_t num_rows, int heads, int64_t dim, int elem_size,
                   const float* attn, float* out, void* stream);
int apt_gat_block(const int64_t* neighbors, int64_t num_dst, const int64_t* num_dst_dev, int fanout,
                  const void* ft, int64_t num_src, int heads, int64_t dim, int elem_size,
                  const float* el, const float* er, float negative_slope, float* out,
                  float* attn_out, void* stream);

/* Backward pass of apt_gat_block (no counterpart in the reference, whose GAT layer
 * gets its gradients from DGL's autograd).  Edge half, fanout <= 64 (a wavefront
 * per destination when heads is a power of two and heads * fanout <= 64, lane
 * groups or a wavefront per (destination, head) otherwise): from dOut
 * [num_dst, heads, dim] and the
 * forward's attention weights attn [num_dst * fanout, heads] it writes, in the
 * block's COO order (edge id = csc_indptr[d] + rank of the slot among d's edges,
 * see apt_block_formats), a_edge and dz_edge [E, heads] (attention weight;
 * gradient of the logit before LeakyReLU) and d_er [num_dst, heads] = sum of dz
 * over a destination's edges.  The source half is two sums over the edges of a
 * source, both by one apt_spmm_heads call over the block's CSR order: d ft with
 * head_weights = a_edge, d el as the second sum with head_weights2 = dz_edge.
 * apt_spmm_heads is also the backward of the plain block sum / mean
 * (head_weights NULL, heads 1).
 *   apt_spmm_heads  out[col[e], h, :] += head_weights[w(e), h] * input[row[e], h, :],
 *                   w(e) = weight_row[e] or e when weight_row is NULL (dim = heads *
 *                   head_dim features per row; out fp32, zero-filled by the caller;
 *                   one segment).  grouped != 0: the caller guarantees that edges
 *                   with equal col are consecutive (the block's CSR order); rows that
 *                   lie inside a wavefront's 64 edges are then stored without
 *                   atomics (deterministic but for rows that span more than two
 *                   ranges).  head_weights2 / out2
 *                   (both or neither): out2[col[e], h] += head_weights2[w(e), h], a
 *                   second, scalar sum per row and head in the same pass (d el of
 *                   the GAT backward); out2 fp32 [num_out_rows, heads], zero-filled.
 *                   head_weights may be NULL (all ones).  out_indptr, optional, grouped
 *                   only: int64[num_out_rows + 1], offsets of the output rows in the edge
 *                   list (the CSR offsets that go with col).  The library then zeroes
 *                   the rows it must (rows without edges, rows whose edges span two
 *                   wavefront ranges) itself and stores every other row whole: out and
 *                   out2 need not be initialised. */
int apt_gat_block_backward(const int64_t* neighbors, int64_t num_dst, int fanout, const void* ft,
                           int64_t num_src, int heads, int64_t dim, int elem_size, const float* el,
                           const float* er, float negative_slope, const float* attn,
                           const float* d_out, const int64_t* csc_indptr, float* a_edge,
                           float* dz_edge, float* d_er, void* stream);
int apt_spmm_heads(const int64_t* coo_row, const int64_t* coo_col, int64_t num_edges,
                   const void* input, int64_t num_in_rows, const float* head_weights,
                   const int64_t* weight_row, int heads, int64_t dim, int elem_size, int grouped,
                   float* out, int64_t num_out_rows, const float* head_weights2, float* out2,
                   const int64_t* out_indptr, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* APT_AMD_H_ */
