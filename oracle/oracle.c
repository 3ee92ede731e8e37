/*
 * oracle.c — CPU restatement of the mini-batch construction path.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker the HIP library is
 * compared against and the CPU baseline bench.py times; nothing in the
 * product (apt_amd/) links, loads or calls it.
 *
 * The reference (kaihaoma/APT) has no CPU implementation of sampling, relabel
 * or bucketing and its CUDA sources cannot be built here (curand, thrust, cub,
 * nccl, glog), so each function restates the semantics of the CUDA kernel it
 * cites.  What pins each function (none of them has a fixture in the
 * reference's tests, which cover NCCL collectives only):
 *   orc_philox4x32_10   Random123 known-answer vectors + a vector produced by
 *                       rocRAND's host implementation of the same generator.
 *   orc_sample_*        brute force over tiny graphs, closed form when
 *                       fanout >= degree (whole row, CSR order), invariants
 *                       (true neighbours, distinct positions, counts),
 *                       chi-square uniformity over positions and over subsets.
 *                       The reference's exact draws (XORWOW, constant seed) are
 *                       not reproduced: parity of draw values is unpinned and
 *                       not claimed.
 *   orc_relabel         numpy closed form (np.unique first-occurrence order), for the
 *                       one-thread and the threaded variant alike.
 *   orc_gather_rows     numpy fancy indexing through the position map.
 *   orc_cluster_*       numpy searchsorted + stable argsort closed form; the
 *                       inputs of tests/test_shuffle_seeds.cc:19-26.
 *   orc_permute/scatter numpy take / put.
 *   orc_gat_scores/_block  scipy.special.softmax on a dense adjacency, the mean
 *                       SpMM when all logits are equal, shift invariance.
 *   orc_map_to_vir, orc_vir_send_offset   numpy searchsorted closed forms.
 *   orc_block_formats   numpy nonzero / stable argsort / bincount + cumsum.
 *   orc_count_ids, orc_csr_select_rows   numpy bincount / concatenated slices.
 *   orc_spmm_csr        scipy.sparse CSR matrix x dense product (float64), per head
 *                       with the edge weights as the matrix data; empty rows are zero.
 *   orc_spmm_sum/sddmm  numpy closed forms (np.add.at over fancy-indexed rows,
 *                       in float64); a sum over a row of ones equals its
 *                       in-degree.
 *
 * Build: make -C oracle   (gcc -O3 -fopenmp -shared -fPIC)
 */
#include <stdint.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_ENCODE_ID(i) (-(i)-2) /* src/utils.h:17 */

static int g_threads = 1;

void orc_set_threads(int t) { g_threads = t > 0 ? t : 1; }
int orc_get_threads(void) { return g_threads; }
int orc_max_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* ------------------------------------------------------------------ */
/* Philox4x32-10 (Salmon et al., SC'11; Random123 philox.h).           */
/* ------------------------------------------------------------------ */
void orc_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2],
                       uint32_t out[4]) {
  uint32_t c0 = ctr[0], c1 = ctr[1], c2 = ctr[2], c3 = ctr[3];
  uint32_t k0 = key[0], k1 = key[1];
  for (int r = 0; r < 10; ++r) {
    uint64_t p0 = (uint64_t)0xD2511F53u * c0;
    uint64_t p1 = (uint64_t)0xCD9E8D57u * c2;
    uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0;
    uint32_t n1 = (uint32_t)p1;
    uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
    uint32_t n3 = (uint32_t)p0;
    c0 = n0; c1 = n1; c2 = n2; c3 = n3;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

/* 64 random bits for output slot `slot` of node `node` at hop `hop`. */
static inline uint64_t draw64(uint64_t rng_seed, int64_t node, int hop,
                              uint32_t slot) {
  uint32_t ctr[4] = {(uint32_t)(uint64_t)node, (uint32_t)((uint64_t)node >> 32),
                     (uint32_t)hop, slot};
  uint32_t key[2] = {(uint32_t)rng_seed, (uint32_t)(rng_seed >> 32)};
  uint32_t o[4];
  orc_philox4x32_10(ctr, key, o);
  return ((uint64_t)o[1] << 32) | o[0];
}

/* floor(r * n / 2^64): r uniform on [0,2^64) -> uniform on [0,n) up to a
 * bias of n/2^64. */
static inline uint64_t bounded(uint64_t r, uint64_t n) {
  return (uint64_t)(((unsigned __int128)r * n) >> 64);
}

uint64_t orc_draw64(uint64_t rng_seed, int64_t node, int hop, uint32_t slot) {
  return draw64(rng_seed, node, hop, slot);
}
uint64_t orc_bounded(uint64_t r, uint64_t n) { return bounded(r, n); }

/* ------------------------------------------------------------------ */
/* Sampling: src/cuda/npc_kernel.cu:248-286 (row resolution, deg rule, */
/* with-replacement draws) + the without-replacement mode.             */
/* ------------------------------------------------------------------ */
typedef struct orc_graph {
  const int64_t* indptr;
  const int64_t* indices;
  int64_t row_begin;
  int64_t num_rows;
  const int64_t* cached_indptr;
  const int64_t* cached_indices;
  int64_t num_cached_rows;
  const int64_t* adj_pos_map;
  int64_t num_total_nodes;
} orc_graph;

/* Resolve node v to (neighbour list, degree); npc_kernel.cu:263-276. */
static inline void resolve_row(const orc_graph* g, int64_t v,
                               const int64_t** nbrs, int64_t* deg) {
  *nbrs = NULL;
  *deg = 0;
  if (v < 0) return;
  if (g->adj_pos_map) {
    if (v >= g->num_total_nodes) return;
    int64_t pos = g->adj_pos_map[v];
    if (pos >= 0) {
      if (pos >= g->num_cached_rows) return;
      int64_t s = g->cached_indptr[pos];
      *deg = g->cached_indptr[pos + 1] - s;
      *nbrs = g->cached_indices + s;
    } else {
      int64_t row = ORC_ENCODE_ID(pos);
      if (row < 0 || row >= g->num_rows) return;
      int64_t s = g->indptr[row];
      *deg = g->indptr[row + 1] - s;
      *nbrs = g->indices + s;
    }
  } else {
    int64_t row = v - g->row_begin;
    if (row < 0 || row >= g->num_rows) return;
    int64_t s = g->indptr[row];
    *deg = g->indptr[row + 1] - s;
    *nbrs = g->indices + s;
  }
}

static int64_t sample_one(const orc_graph* g, int64_t v, int fanout,
                          int replace, uint64_t rng_seed, int hop,
                          int64_t* out) {
  const int64_t* nbrs;
  int64_t deg;
  resolve_row(g, v, &nbrs, &deg);
  int64_t cnt = 0;
  if (replace) {
    /* npc_kernel.cu:277-283: fanout independent draws when deg > 0 */
    if (deg > 0) {
      for (int s = 0; s < fanout; ++s)
        out[s] = nbrs[bounded(draw64(rng_seed, v, hop, (uint32_t)s),
                              (uint64_t)deg)];
      cnt = fanout;
    }
  } else if (deg <= fanout) {
    for (int64_t s = 0; s < deg; ++s) out[s] = nbrs[s];
    cnt = deg;
  } else {
    /* Floyd's subset sampling: for j = deg-k .. deg-1 draw t in [0, j];
     * take t unless already taken, then take j.  Uniform over k-subsets. */
    int64_t* picks = (int64_t*)malloc(sizeof(int64_t) * (size_t)fanout);
    for (int s = 0; s < fanout; ++s) {
      int64_t j = deg - fanout + s;
      int64_t t = (int64_t)bounded(draw64(rng_seed, v, hop, (uint32_t)s),
                                   (uint64_t)(j + 1));
      int taken = 0;
      for (int q = 0; q < s; ++q)
        if (picks[q] == t) { taken = 1; break; }
      picks[s] = taken ? j : t;
      out[s] = nbrs[picks[s]];
    }
    free(picks);
    cnt = fanout;
  }
  for (int64_t s = cnt; s < fanout; ++s) out[s] = -1;
  return cnt;
}

/* Also exposes the chosen positions (for uniformity tests). */
int64_t orc_sample_positions(int64_t deg, int fanout, int replace,
                             uint64_t rng_seed, int64_t node, int hop,
                             int64_t* out_pos) {
  int64_t* row = (int64_t*)malloc(sizeof(int64_t) * (size_t)(deg > 0 ? deg : 1));
  for (int64_t i = 0; i < deg; ++i) row[i] = i;
  int64_t indptr[2] = {0, deg};
  orc_graph g = {indptr, row, node, 1, NULL, NULL, 0, NULL, node + 1};
  int64_t c = sample_one(&g, node, fanout, replace, rng_seed, hop, out_pos);
  free(row);
  return c;
}

int64_t orc_sample_neighbors(const orc_graph* g, const int64_t* frontier,
                             int64_t n, int fanout, int replace,
                             uint64_t rng_seed, int hop, int64_t* out_neighbors,
                             int64_t* out_counts) {
  int64_t total = 0;
#pragma omp parallel for schedule(dynamic, 256) reduction(+ : total) \
    num_threads(g_threads)
  for (int64_t i = 0; i < n; ++i) {
    int64_t c = sample_one(g, frontier[i], fanout, replace, rng_seed, hop,
                           out_neighbors + i * fanout);
    if (out_counts) out_counts[i] = c;
    total += c;
  }
  return total;
}

/* ------------------------------------------------------------------ */
/* Relabel: src/cuda/relabel.cu:78-185.  unique = distinct values of   */
/* cat(seeds, neighbors) in first-occurrence order (the AtomicMin on    */
/* the item index, :12-24, makes the smallest index the owner; the     */
/* exclusive scan of owner flags, :100-116, orders them by index);     */
/* relabeled[j] = rank of neighbors[j] (:153-173).  Negative ids are    */
/* padding: skipped and passed through.                                */
/* ------------------------------------------------------------------ */
static inline uint64_t mix64(uint64_t x) {
  x ^= x >> 33; x *= 0xff51afd7ed558ccdULL;
  x ^= x >> 33; x *= 0xc4ceb9fe1a85ec53ULL;
  x ^= x >> 33;
  return x;
}

static int64_t relabel_serial(const int64_t* seeds, int64_t ns, const int64_t* neighbors,
                              int64_t nn, int64_t* unique, int64_t* relabeled) {
  int64_t items = ns + nn;
  uint64_t cap = 16;
  while (cap < (uint64_t)items * 2) cap <<= 1;
  int64_t* keys = (int64_t*)malloc(sizeof(int64_t) * cap);
  int64_t* vals = (int64_t*)malloc(sizeof(int64_t) * cap);
  memset(keys, 0xFF, sizeof(int64_t) * cap); /* -1 = empty */
  int64_t u = 0;
  for (int64_t i = 0; i < items; ++i) {
    int64_t k = i < ns ? seeds[i] : neighbors[i - ns];
    if (k < 0) {
      if (i >= ns) relabeled[i - ns] = k;
      continue;
    }
    uint64_t pos = mix64((uint64_t)k) & (cap - 1);
    while (keys[pos] != -1 && keys[pos] != k) pos = (pos + 1) & (cap - 1);
    if (keys[pos] == -1) {
      keys[pos] = k;
      vals[pos] = u;
      unique[u++] = k;
    }
    if (i >= ns) relabeled[i - ns] = vals[pos];
  }
  free(keys);
  free(vals);
  return u;
}

/* The same result on several threads, the way the reference's kernels get it
 * (relabel.cu:12-24,100-116): concurrent insert with a CAS on the key and an
 * atomic minimum on the item index, owners = items whose index is their key's
 * minimum, ranks = exclusive prefix of the owner flags in item order. */
static int64_t relabel_threads(const int64_t* seeds, int64_t ns, const int64_t* neighbors,
                               int64_t nn, int64_t* unique, int64_t* relabeled, int threads) {
  const int64_t items = ns + nn;
  uint64_t cap = 16;
  while (cap < (uint64_t)items * 2) cap <<= 1;
  int64_t* keys = (int64_t*)malloc(sizeof(int64_t) * cap);
  int64_t* minidx = (int64_t*)malloc(sizeof(int64_t) * cap);   /* later: the key's rank */
  uint32_t* slot_of = (uint32_t*)malloc(sizeof(uint32_t) * (size_t)(items > 0 ? items : 1));
  uint8_t* owner = (uint8_t*)malloc((size_t)(items > 0 ? items : 1));
  int64_t* part = (int64_t*)calloc((size_t)threads + 1, sizeof(int64_t));
  int64_t total = 0;
#pragma omp parallel num_threads(threads)
  {
#pragma omp for schedule(static)
    for (uint64_t q = 0; q < cap; ++q) {
      keys[q] = -1;
      minidx[q] = INT64_MAX;
    }
#pragma omp for schedule(static)
    for (int64_t i = 0; i < items; ++i) {
      const int64_t k = i < ns ? seeds[i] : neighbors[i - ns];
      if (k < 0) continue;
      uint64_t pos = mix64((uint64_t)k) & (cap - 1);
      for (;;) {
        int64_t cur = __atomic_load_n(&keys[pos], __ATOMIC_RELAXED);
        if (cur == -1) {
          int64_t expect = -1;
          if (__atomic_compare_exchange_n(&keys[pos], &expect, k, 0, __ATOMIC_RELAXED, __ATOMIC_RELAXED)) break;
          cur = expect;
        }
        if (cur == k) break;
        pos = (pos + 1) & (cap - 1);
      }
      int64_t seen = __atomic_load_n(&minidx[pos], __ATOMIC_RELAXED);
      while (seen > i && !__atomic_compare_exchange_n(&minidx[pos], &seen, i, 1, __ATOMIC_RELAXED, __ATOMIC_RELAXED)) {
      }
      slot_of[i] = (uint32_t)pos;
    }
    /* owners per thread chunk -> offsets -> ranks (static schedule: the same chunks both times) */
    const int t = omp_get_thread_num();
    int64_t mine = 0;
#pragma omp for schedule(static)
    for (int64_t i = 0; i < items; ++i) {
      const int64_t k = i < ns ? seeds[i] : neighbors[i - ns];
      owner[i] = k >= 0 && minidx[slot_of[i]] == i;
      mine += owner[i];
    }
    part[t + 1] = mine;
#pragma omp barrier
#pragma omp single
    {
      for (int q = 0; q < threads; ++q) part[q + 1] += part[q];
      total = part[threads];
    }
    int64_t rank = part[t];
#pragma omp for schedule(static)
    for (int64_t i = 0; i < items; ++i) {
      if (!owner[i]) continue;
      unique[rank] = i < ns ? seeds[i] : neighbors[i - ns];
      keys[slot_of[i]] = rank++;   /* the slot's key is no longer needed: it now holds the rank */
    }
#pragma omp for schedule(static)
    for (int64_t j = 0; j < nn; ++j) {
      const int64_t k = neighbors[j];
      relabeled[j] = k < 0 ? k : keys[slot_of[ns + j]];
    }
  }
  free(keys);
  free(minidx);
  free(slot_of);
  free(owner);
  free(part);
  return total;
}

int64_t orc_relabel(const int64_t* seeds, int64_t ns, const int64_t* neighbors,
                    int64_t nn, int64_t* unique, int64_t* relabeled) {
#ifdef _OPENMP
  if (g_threads > 1 && ns + nn >= 4096)
    return relabel_threads(seeds, ns, neighbors, nn, unique, relabeled, g_threads);
#endif
  return relabel_serial(seeds, ns, neighbors, nn, unique, relabeled);
}

/* ------------------------------------------------------------------ */
/* Feature gather: src/cuda/npc_kernel.cu:187-224 (addressing),         */
/* src/load_subtensor.cc:10-40.                                         */
/* ------------------------------------------------------------------ */
typedef struct orc_feat_store {
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
} orc_feat_store;

int64_t orc_gather_rows(const orc_feat_store* st, const int64_t* index,
                        int64_t n, void* out) {
  const size_t es = (size_t)st->elem_size;
  const size_t row_bytes = (size_t)st->out_dim * es;
  int64_t miss = 0;
#pragma omp parallel for schedule(static) reduction(+ : miss) \
    num_threads(g_threads)
  for (int64_t r = 0; r < n; ++r) {
    char* dst = (char*)out + (size_t)r * row_bytes;
    int64_t v = index[r];
    const char* src = NULL;
    if (v >= 0) {
      if (st->pos_map) {
        if (v < st->num_total_nodes) {
          int64_t p = st->pos_map[v];
          if (p < -1) { /* npc_kernel.cu:196-199: second table + column window */
            int64_t row = ORC_ENCODE_ID(p);
            if (row < st->num_local_rows)
              src = (const char*)st->local_table +
                    ((size_t)row * (size_t)st->local_dim +
                     (size_t)st->col_offset) * es;
          } else if (p >= 0 && p < st->num_cache_rows) { /* :202-204 */
            src = (const char*)st->cache_table + (size_t)p * row_bytes;
          }
        }
      } else if (v < st->num_local_rows) {
        src = (const char*)st->local_table +
              ((size_t)v * (size_t)st->local_dim + (size_t)st->col_offset) * es;
      }
    }
    if (src) {
      memcpy(dst, src, row_bytes);
    } else {
      memset(dst, 0, row_bytes);
      miss += 1;
    }
  }
  return miss;
}

/* src/feat_shuffle.cc:27 (unpack) and :14-16 (pack). */
void orc_permute_rows(const void* in, const int64_t* perm, int64_t n,
                      int64_t dim, int elem_size, void* out) {
  size_t rb = (size_t)dim * (size_t)elem_size;
#pragma omp parallel for schedule(static) num_threads(g_threads)
  for (int64_t i = 0; i < n; ++i)
    memcpy((char*)out + (size_t)i * rb, (const char*)in + (size_t)perm[i] * rb,
           rb);
}

void orc_scatter_rows(const void* in, const int64_t* perm, int64_t n,
                      int64_t dim, int elem_size, void* out) {
  size_t rb = (size_t)dim * (size_t)elem_size;
#pragma omp parallel for schedule(static) num_threads(g_threads)
  for (int64_t i = 0; i < n; ++i)
    memcpy((char*)out + (size_t)perm[i] * rb, (const char*)in + (size_t)i * rb,
           rb);
}

/* ------------------------------------------------------------------ */
/* Bucketing: src/cuda/npc_kernel.cu:318-382 (owner rule :333-342,      */
/* outputs :460-467).  Order inside a bucket = input order (one of the  */
/* orders the reference's atomic tickets can produce).                  */
/* ------------------------------------------------------------------ */
static inline int owner_of(int64_t v, const int64_t* min_vids, int nb,
                           int64_t start) {
  int64_t d = start;
  while (d + 1 < nb && min_vids[d + 1] <= v) ++d;
  return (int)d;
}

static void stable_place(const int64_t* ids, int64_t n, const int* bucket,
                         int nb, int64_t* bucket_size, int64_t* bucket_offset,
                         int64_t* sorted_ids, int64_t* permutation) {
  int64_t* cursor = (int64_t*)calloc((size_t)nb, sizeof(int64_t));
  for (int b = 0; b < nb; ++b) bucket_size[b] = 0;
  for (int64_t i = 0; i < n; ++i) bucket_size[bucket[i]] += 1;
  int64_t acc = 0;
  for (int b = 0; b < nb; ++b) {
    cursor[b] = acc;
    acc += bucket_size[b];
    if (bucket_offset) bucket_offset[b] = acc; /* inclusive cumsum, :460 */
  }
  for (int64_t i = 0; i < n; ++i) {
    int64_t dst = cursor[bucket[i]]++;
    sorted_ids[dst] = ids[i];
    permutation[i] = dst;
  }
  free(cursor);
}

void orc_cluster_permute(const int64_t* ids, int64_t n, const int64_t* min_vids,
                         int num_buckets, int64_t id_offset, int rank,
                         int node_beg, int node_end, int64_t* bucket_size,
                         int64_t* bucket_offset, int64_t* sorted_ids,
                         int64_t* permutation) {
  int* bucket = (int*)malloc(sizeof(int) * (size_t)(n > 0 ? n : 1));
  for (int64_t i = 0; i < n; ++i) {
    int d = owner_of(ids[i], min_vids, num_buckets, id_offset);
    if (d < node_beg || d >= node_end) d = rank; /* :340-342 */
    bucket[i] = d;
  }
  stable_place(ids, n, bucket, num_buckets, bucket_size, bucket_offset,
               sorted_ids, permutation);
  free(bucket);
}

/* src/cuda/npc_kernel.cu:384-432: bucket 0 = present here. */
void orc_cluster_reqs(const int64_t* ids, int64_t n, const int64_t* feat_pos_map,
                      int64_t num_total_nodes, const int64_t* remote_worker_map,
                      const int64_t* min_vids, int world_size,
                      int num_remote_workers, int64_t* bucket_size,
                      int64_t* bucket_offset, int64_t* sorted_ids,
                      int64_t* permutation) {
  int* bucket = (int*)malloc(sizeof(int) * (size_t)(n > 0 ? n : 1));
  for (int64_t i = 0; i < n; ++i) {
    int64_t v = ids[i];
    int d = 0;
    int present = (v >= 0 && v < num_total_nodes) ? feat_pos_map[v] != -1 : 0;
    if (!present)
      d = (int)remote_worker_map[owner_of(v, min_vids, world_size, 0)];
    bucket[i] = d;
  }
  stable_place(ids, n, bucket, num_remote_workers, bucket_size, bucket_offset,
               sorted_ids, permutation);
  free(bucket);
}

/* ------------------------------------------------------------------ */
/* Aggregation: src/cuda/spmm.cu:8-83 (COO SpMM; segment of an edge by  */
/* upper bound in coo_off, :21,:47,:72) and src/cuda/sddmm.cu:8-59.     */
/* Sums are accumulated in double and rounded once, so the result is    */
/* the correctly rounded reference for the 1e-5 tolerance; u_mul_e      */
/* multiplies (the reference adds, spmm.cu:78; no caller).              */
/* Pinned by numpy closed forms (np.add.at on fancy-indexed rows).      */
/* ------------------------------------------------------------------ */
static inline int seg_of(const int64_t* coo_off, int num_seg, int64_t e) {
  int k = 0;
  while (k + 1 < num_seg && coo_off[k + 1] <= e) ++k;
  return k;
}

void orc_spmm_sum(int mode, const int64_t* row, const int64_t* col, int64_t E, const float* in,
                  const float* edata, int64_t dim, const int64_t* coo_off, const int64_t* in_off,
                  const int64_t* out_off, int num_seg, float* out, int64_t num_out) {
  double* acc = (double*)calloc((size_t)(num_out > 0 ? num_out : 1) * (size_t)dim, sizeof(double));
  for (int64_t e = 0; e < E; ++e) {
    int k = seg_of(coo_off, num_seg, e);
    int64_t dst = (out_off ? out_off[k] : 0) + col[e];
    int64_t src = (in_off ? in_off[k] : 0) + row[e];
    for (int64_t d = 0; d < dim; ++d) {
      double v;
      if (mode == 1) v = in[e * dim + d];
      else if (mode == 2) v = (double)in[src * dim + d] * (double)edata[e * dim + d];
      else v = in[src * dim + d];
      acc[dst * dim + d] += v;
    }
  }
  for (int64_t i = 0; i < num_out * dim; ++i) out[i] = (float)acc[i];
  free(acc);
}

/* Row-owned SpMM over CSR, the backward direction of a block (the reference runs
 * its COO operator with the edges reversed, python/npc/model/sageconv.py:100-114):
 * out[r] = sum_e col_scale[idx[e]] * w[weid(e), head] * x[idx[e]], float64 accumulation. */
void orc_spmm_csr(const int64_t* indptr, const int64_t* indices, const int64_t* eids, int64_t num_rows,
                  const float* x, int64_t num_x_rows, int64_t dim, const float* col_scale, const float* w,
                  const float* w2, int heads, float* out, float* out2) {
  const int64_t hd = dim / heads;
#pragma omp parallel for schedule(dynamic, 256) num_threads(g_threads)
  for (int64_t r = 0; r < num_rows; ++r) {
    for (int64_t d = 0; d < dim; ++d) {
      double acc = 0.0;
      for (int64_t e = indptr[r]; e < indptr[r + 1]; ++e) {
        const int64_t j = indices[e];
        if (j < 0 || j >= num_x_rows) continue;
        const int64_t we = eids ? eids[e] : e;
        double f = col_scale ? (double)col_scale[j] : 1.0;
        if (w) f *= (double)w[we * heads + d / hd];
        acc += f * (double)x[j * dim + d];
      }
      out[r * dim + d] = (float)acc;
    }
    if (w2)
      for (int h = 0; h < heads; ++h) {
        double acc = 0.0;
        for (int64_t e = indptr[r]; e < indptr[r + 1]; ++e) {
          const int64_t j = indices[e];
          if (j < 0 || j >= num_x_rows) continue;
          acc += (double)w2[(eids ? eids[e] : e) * heads + h];
        }
        out2[r * heads + h] = (float)acc;
      }
  }
}

void orc_sddmm(int op, const int64_t* row, const int64_t* col, int64_t E, const float* lhs,
               const float* rhs, int64_t dim, const int64_t* coo_off, const int64_t* lhs_off,
               const int64_t* rhs_off, int num_seg, float* out) {
#pragma omp parallel for schedule(static) num_threads(g_threads)
  for (int64_t e = 0; e < E; ++e) {
    int k = seg_of(coo_off, num_seg, e);
    int64_t src = (lhs_off ? lhs_off[k] : 0) + row[e];
    int64_t dst = (rhs_off ? rhs_off[k] : 0) + col[e];
    for (int64_t d = 0; d < dim; ++d) {
      float a = lhs[src * dim + d], b = rhs[dst * dim + d];
      out[e * dim + d] = op == 0 ? a + b : a * b;
    }
  }
}

/* ------------------------------------------------------------------ */
/* Cache construction: access counting (examples/dryrun.py:90-92) and   */
/* the cached CSR of chosen rows (python/npc/ops.py:370-384).  Pinned   */
/* by numpy closed forms (bincount; concatenation of row slices).       */
/* ------------------------------------------------------------------ */
void orc_count_ids(const int64_t* ids, int64_t n, int64_t* freq, int64_t num_total) {
  for (int64_t i = 0; i < n; ++i)
    if (ids[i] >= 0 && ids[i] < num_total) freq[ids[i]] += 1;
}

/* out_indptr must hold n + 1 entries; returns the number of edges.  With
 * out_indices == NULL only the offsets are computed. */
int64_t orc_csr_select_rows(const int64_t* indptr, const int64_t* indices, int64_t row_begin,
                            int64_t num_rows, const int64_t* rows, int64_t n, int64_t* out_indptr,
                            int64_t* out_indices) {
  int64_t acc = 0;
  for (int64_t i = 0; i < n; ++i) {
    out_indptr[i] = acc;
    int64_t r = rows[i] - row_begin;
    if (r < 0 || r >= num_rows) continue;
    int64_t s = indptr[r], e = indptr[r + 1];
    if (out_indices)
      for (int64_t k = s; k < e; ++k) out_indices[acc + (k - s)] = indices[k];
    acc += e - s;
  }
  out_indptr[n] = acc;
  return acc;
}

/* ------------------------------------------------------------------ */
/* Sparse formats of a block (python/npc/sampler.py:59-69,76-91: DGL   */
/* builds coo/csr/csc from row = relabeled, col = dst).  Pinned by      */
/* numpy closed forms (nonzero, stable argsort, bincount + cumsum).     */
/* ------------------------------------------------------------------ */
/* Arrays hold num_dst * fanout entries (offsets num_dst + 1 / num_src + 1);
 * returns the number of edges.  csr_* may be NULL. */
int64_t orc_block_formats(const int64_t* relabeled, int64_t num_dst, int fanout, int64_t num_src,
                          int64_t* coo_row, int64_t* coo_col, int64_t* csc_indptr, int64_t* csr_indptr,
                          int64_t* csr_indices, int64_t* csr_eids) {
  int64_t e = 0;
  for (int64_t d = 0; d < num_dst; ++d) {
    csc_indptr[d] = e;
    for (int k = 0; k < fanout; ++k) {
      const int64_t v = relabeled[d * fanout + k];
      if (v < 0) continue;
      coo_row[e] = v;
      coo_col[e] = d;
      ++e;
    }
  }
  csc_indptr[num_dst] = e;
  if (!csr_indptr) return e;
  for (int64_t s = 0; s <= num_src; ++s) csr_indptr[s] = 0;
  for (int64_t i = 0; i < e; ++i) csr_indptr[coo_row[i] + 1] += 1;
  for (int64_t s = 0; s < num_src; ++s) csr_indptr[s + 1] += csr_indptr[s];
  int64_t* next = (int64_t*)malloc(sizeof(int64_t) * (size_t)(num_src > 0 ? num_src : 1));
  for (int64_t s = 0; s < num_src; ++s) next[s] = csr_indptr[s];
  for (int64_t i = 0; i < e; ++i) {   /* edge order = increasing edge id inside a source */
    const int64_t at = next[coo_row[i]]++;
    csr_indices[at] = coo_col[i];
    csr_eids[at] = i;
  }
  free(next);
  return e;
}

/* ------------------------------------------------------------------ */
/* GAT aggregation (python/npc/model/gatconv.py:116-126; the arithmetic */
/* is DGL's: u_add_v, LeakyReLU, edge_softmax, u_mul_e + sum).  Double   */
/* accumulation.  Pinned by scipy.special.softmax on a dense adjacency,  */
/* by the mean SpMM (all logits equal) and by shift invariance.          */
/* ------------------------------------------------------------------ */
void orc_gat_scores(const float* x, int64_t n, int heads, int64_t dim, const float* attn, float* out) {
  for (int64_t r = 0; r < n; ++r)
    for (int h = 0; h < heads; ++h) {
      double acc = 0.0;
      for (int64_t d = 0; d < dim; ++d) acc += (double)x[(r * heads + h) * dim + d] * (double)attn[h * dim + d];
      out[r * heads + h] = (float)acc;
    }
}

/* attn_out may be NULL */
void orc_gat_block(const int64_t* nbr, int64_t num_dst, int fanout, const float* ft, int64_t num_src, int heads,
                   int64_t dim, const float* el, const float* er, double slope, float* out, float* attn_out) {
  double* e = (double*)malloc(sizeof(double) * (size_t)(fanout > 0 ? fanout : 1));
  double* acc = (double*)malloc(sizeof(double) * (size_t)dim);
  for (int64_t i = 0; i < num_dst; ++i)
    for (int h = 0; h < heads; ++h) {
      double top = -INFINITY, denom = 0.0;
      for (int k = 0; k < fanout; ++k) {
        const int64_t s = nbr[i * fanout + k];
        if (s < 0 || s >= num_src) continue;
        double v = (double)el[s * heads + h] + (double)er[i * heads + h];
        if (v < 0) v *= slope;
        e[k] = v;
        if (v > top) top = v;
      }
      for (int k = 0; k < fanout; ++k) {
        const int64_t s = nbr[i * fanout + k];
        if (s < 0 || s >= num_src) continue;
        denom += exp(e[k] - top);
      }
      for (int64_t d = 0; d < dim; ++d) acc[d] = 0.0;
      for (int k = 0; k < fanout; ++k) {
        const int64_t s = nbr[i * fanout + k];
        double a = 0.0;
        if (s >= 0 && s < num_src) {
          a = exp(e[k] - top) / denom;
          for (int64_t d = 0; d < dim; ++d) acc[d] += a * (double)ft[(s * heads + h) * dim + d];
        }
        if (attn_out) attn_out[(i * fanout + k) * heads + h] = (float)a;
      }
      for (int64_t d = 0; d < dim; ++d) out[(i * heads + h) * dim + d] = (float)acc[d];
    }
  free(e);
  free(acc);
}

/* ------------------------------------------------------------------ */
/* Virtual nodes of SP mode (src/cuda/npc_kernel.cu:15-183).  Pinned by */
/* numpy searchsorted closed forms.                                     */
/* ------------------------------------------------------------------ */
static int64_t orc_owner(int64_t v, const int64_t* min_vids, int world, int64_t id_offset, int rank,
                         int node_beg, int node_end) {
  int64_t d = id_offset;
  while (d + 1 < world && min_vids[d + 1] <= v) ++d;   /* :41-43 */
  if (d < node_beg || d >= node_end) d = rank;          /* :45-47 */
  return d;
}

void orc_map_to_vir(const int64_t* dst, int64_t num_dst, const int64_t* src, int64_t num_src, int fanout,
                    const int64_t* min_vids, int world, int64_t id_offset, int rank, int node_beg,
                    int node_end, int64_t* vir) {
  int64_t lead = 0;
  if (dst) {
    lead = num_dst;
    for (int64_t i = 0; i < num_dst; ++i)
      vir[i] = orc_owner(dst[i], min_vids, world, id_offset, rank, node_beg, node_end) * num_dst + i;
  }
  for (int64_t j = 0; j < num_src; ++j)
    vir[lead + j] = orc_owner(src[j], min_vids, world, id_offset, rank, node_beg, node_end) * num_dst +
                    (dst ? (int64_t)world * num_dst : 0) + j / fanout;
}

static int64_t orc_lower_bound(const int64_t* a, int64_t n, int64_t want) {
  int64_t lo = 0, hi = n;
  while (lo < hi) {
    int64_t mid = lo + (hi - lo) / 2;
    if (a[mid] < want) lo = mid + 1; else hi = mid;
  }
  return lo;
}

void orc_vir_send_offset(int world, int64_t base, const int64_t* sorted, int64_t ns, const int64_t* uniq,
                         int64_t nu, int with_dst, int64_t* out) {
  const int a_count = (with_dst ? 2 : 1) * world + 1;
  const int b_first = with_dst ? world + 1 : 1;
  for (int k = 0; k < a_count; ++k) out[k] = orc_lower_bound(sorted, ns, (int64_t)k * base);
  for (int k = 0; k < world; ++k) out[a_count + k] = orc_lower_bound(uniq, nu, (int64_t)(b_first + k) * base);
}
