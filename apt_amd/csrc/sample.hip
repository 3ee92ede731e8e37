// Uniform neighbour sampling over CSR, one hop.
//
// Replaces _CSRRowWiseSampleReplaceKernel / LocalSampleNeighbors
// (reference src/cuda/npc_kernel.cu:248-316).  Differences by design:
//   * a lane group (8..64 lanes of a wave64, the smallest power of two that
//     holds the fanout) owns a frontier row, with several rows per group in
//     flight; the block first stages every row's (neighbour pointer,
//     degree, node) in LDS with one lane per row, so the dependent
//     frontier -> pos_map -> indptr loads of a whole tile are in flight
//     together instead of one chain per wave;
//   * draws come from Philox4x32-10 keyed by (rng_seed) with counter
//     (node, hop, slot) instead of a per-thread XORWOW state re-initialised on
//     every launch (:258-261), so outputs are launch-geometry independent;
//   * a without-replacement mode (Floyd's subset sampling, resolved across the
//     lanes of the group with shuffles);
//   * unused output slots are written as -1 (the reference leaves garbage for
//     degree-0 rows, :277).
#include <hip/hip_ext.h>

#include "common.hpp"
#include "rank_table.hpp"

namespace apt {

// One-shot measurement hook (apt_time_next_sample): the next sampling launch of
// this thread whose hop index matches records the two events on its dispatch.
static thread_local hipEvent_t t_sample_start = nullptr, t_sample_stop = nullptr;
static thread_local int t_sample_hop = -1;

struct SampleParams {
  apt_graph g;
  const int64_t* frontier;
  int64_t n;
  const int64_t* n_dev;
  int fanout;
  uint64_t seed;
  const uint64_t* seed_dev;  // overrides seed when not NULL
  int hop;
  int64_t* out;
  int64_t* counts;
  int64_t* total;
  int rows_per_group;
  int direct;  // every lane group resolves its own rows (no staging of the tile in LDS, no workgroup barrier)
  // Optional fusion with the rank-table relabel of the multi-hop driver: every
  // sampled id is looked up / bid for in the rank table right after it is loaded.
  RankTable table;       // entries == NULL: plain sampling
  int64_t* relabeled;    // [n * fanout]
  int first_hop;
  int64_t* outside;      // optional, first hop: counts the frontier ids the table cannot hold (>= table.len)
};

constexpr int kSampleBlock = 512;
constexpr int kMaxRowsPerGroup = 16;
constexpr int kSampleMinWorkgroups = 8192;
constexpr int kSamplePersistentBlocks = 8192;
constexpr int kMaxFanout = 1024;

// Resolve node v to its neighbour list (reference :263-276).  Ids or map
// entries that point outside the tables yield degree 0 instead of a fault.
__device__ __forceinline__ void resolve_row(const apt_graph& g, int64_t v,
                                            const int64_t*& nbrs, int64_t& deg) {
  nbrs = nullptr;
  deg = 0;
  if (v < 0) return;
  const int64_t* indptr = g.indptr;
  const int64_t* indices = g.indices;
  int64_t row;
  if (g.adj_pos_map != nullptr) {
    if (v >= g.num_total_nodes) return;
    const int64_t pos = g.adj_pos_map[v];
    if (pos >= 0) {
      if (pos >= g.num_cached_rows) return;
      indptr = g.cached_indptr;
      indices = g.cached_indices;
      row = pos;
    } else {
      row = -pos - 2;
      if (row < 0 || row >= g.num_rows) return;
    }
  } else {
    row = v - g.row_begin;
    if (row < 0 || row >= g.num_rows) return;
  }
  const int64_t s = indptr[row];
  const int64_t e = indptr[row + 1];
  deg = e - s;
  nbrs = indices + s;
}

// Position inside its row that lane `l` of a group reads for output slot `l`
// (fanout <= LPS), or -1 for an unused slot.  Every lane of the wave runs the
// same instruction stream: rows whose degree fits in the fanout feed the
// identity permutation through the Floyd resolution loop, which then never
// finds a collision.
template <int LPS, bool REPLACE>
__device__ __forceinline__ int64_t slot_position(int l, int fanout, int64_t deg, int64_t node,
                                                 uint64_t seed, int hop) {
  const uint64_t r = draw64(seed, node, hop, static_cast<uint32_t>(l));
  if (REPLACE) {
    // reference :277-283: fanout independent draws when the row is not empty
    return (l < fanout && deg > 0) ? static_cast<int64_t>(bounded(r, static_cast<uint64_t>(deg))) : -1;
  }
  // Floyd: slot i draws t in [0, j], j = deg - fanout + i, and takes t unless
  // an earlier slot already holds t, then it takes j.
  const bool big = deg > fanout;
  const int64_t j = big ? deg - fanout + l : l;
  int64_t tpos = -1 - l;  // lanes past the fanout never match a position
  if (l < fanout) tpos = big ? static_cast<int64_t>(bounded(r, static_cast<uint64_t>(j + 1))) : l;
  bool coll = false;
  for (int q = 0; q + 1 < fanout; ++q) {
    const int64_t pq = __shfl(coll ? j : tpos, q, LPS);
    if (l > q && tpos == pq) coll = true;
  }
  const int64_t pick = coll ? j : tpos;
  const int64_t cnt = big ? fanout : deg;
  return l < cnt ? pick : -1;
}

template <int LPS, bool REPLACE, int U>
__global__ __launch_bounds__(kSampleBlock) void sample_kernel(SampleParams p) {
  constexpr int G = kSampleBlock / LPS;  // lane groups per block
  constexpr int kMaxTile = G * kMaxRowsPerGroup;
  __shared__ const int64_t* s_nbrs[kMaxTile];
  __shared__ int64_t s_deg[kMaxTile];
  __shared__ int64_t s_node[kMaxTile];
  __shared__ unsigned long long s_total;
  extern __shared__ int64_t s_picks[];  // [G][fanout], only when fanout > LPS

  const int tid = threadIdx.x;
  const int grp = tid / LPS;
  const int l = tid % LPS;
  const int tile = G * p.rows_per_group;
  // What does not depend on the row count is read before it: the rng seed and the table's epoch, and, in a small
  // launch with a device-side count (the later hops of a batch: a chain of dependent round trips with a single
  // round of waves to hide them), the frontier entry of the first row this lane will work on, so that the
  // read that follows the count finds it in the cache.  frontier[] has p.n entries whatever the count says.
  const uint64_t seed = p.seed_dev != nullptr ? *p.seed_dev : p.seed;
  RankEpoch ep{0, 0, 0};
  if (p.table.entries != nullptr) ep = rank_epoch(p.table.state);
  int64_t touched = 0;
  if (p.n_dev != nullptr && gridDim.x <= 512) {
    const int64_t first = static_cast<int64_t>(blockIdx.x) * tile + (p.direct != 0 ? grp : tid);
    if (first < p.n) touched = p.frontier[first];
  }
  const int64_t n = actual_count(p.n, p.n_dev);
  asm volatile("" ::"v"(touched));  // keeps the early read; nothing uses its value
  if (static_cast<int64_t>(blockIdx.x) * tile >= n) return;  // block-uniform

  const int fanout = p.fanout;
  const bool probe = gridDim.x > 512;   // small launches bid without reading the entry first (rank_table_bid)
  int64_t my_total = 0;
  if (tid == 0) s_total = 0;
  // Stage 1 of a tile puts its rows into LDS, one lane per row, so the dependent
  // frontier -> (pos_map ->) indptr loads of the whole tile overlap.  With one
  // row per group there is nothing to overlap: every group resolves its own row
  // (its lanes read the same addresses) and no group waits for another.
  const bool direct = p.direct != 0;
  __syncthreads();
  // The grid may be smaller than the number of tiles (it is capped when the row
  // count is only known on the device): a workgroup strides over the tiles.
  for (int64_t tile_base = static_cast<int64_t>(blockIdx.x) * tile; tile_base < n;
       tile_base += static_cast<int64_t>(gridDim.x) * tile) {
  if (!direct) {
    for (int t = tid; t < tile; t += kSampleBlock) {
      const int64_t gi = tile_base + t;
      const int64_t* nbrs = nullptr;
      int64_t deg = 0, v = -1;
      if (gi < n) {
        v = p.frontier[gi];
        resolve_row(p.g, v, nbrs, deg);
      }
      s_nbrs[t] = nbrs;
      s_deg[t] = deg;
      s_node[t] = v;
    }
    __syncthreads();
  }

  // Stage 2: one lane group per row.
  if (fanout <= LPS) {
    // U rows per group in flight: positions first, then the loads, then the
    // stores.
    for (int s0 = 0; s0 < p.rows_per_group; s0 += U) {
      const int64_t* src[U];
      int64_t pos[U];
      int64_t gis[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int t = (s0 + u) * G + grp;
        gis[u] = (s0 + u) < p.rows_per_group ? tile_base + t : n;
        pos[u] = -1;
        src[u] = nullptr;
        if (gis[u] < n) {
          int64_t deg, node;
          if (direct) {
            node = p.frontier[gis[u]];
            resolve_row(p.g, node, src[u], deg);
          } else {
            deg = s_deg[t];
            node = s_node[t];
            src[u] = s_nbrs[t];
          }
          // First hop of the fused driver: the row's seed bids for its node with
          // its own index, like its neighbours below (seeds may repeat).
          if (p.first_hop != 0 && p.table.entries != nullptr && l == 0 && node >= 0) {
            if (node < p.table.len) atomicMin(&p.table.entries[node], ep.base + static_cast<uint32_t>(gis[u]));
            else if (p.outside != nullptr) atomicAdd(reinterpret_cast<unsigned long long*>(p.outside), 1ull);
          }
          pos[u] = slot_position<LPS, REPLACE>(l, fanout, deg, node, seed, p.hop);
          if (l == 0) {
            const int64_t cnt = REPLACE ? (deg > 0 ? fanout : 0) : (deg < fanout ? deg : fanout);
            if (p.counts != nullptr) p.counts[gis[u]] = cnt;
            my_total += cnt;
          }
        }
      }
      int64_t val[U];
#pragma unroll
      for (int u = 0; u < U; ++u) val[u] = pos[u] >= 0 ? src[u][pos[u]] : -1;
#pragma unroll
      for (int u = 0; u < U; ++u)
        if (gis[u] < n && l < fanout) p.out[gis[u] * fanout + l] = val[u];
      if (p.table.entries != nullptr) {
        int64_t rel[U];
#pragma unroll
        for (int u = 0; u < U; ++u)
          rel[u] = (gis[u] < n && l < fanout)
                       ? rank_table_bid(p.table, ep, p.first_hop != 0, val[u], n, gis[u] * fanout + l, probe)
                       : -1;
#pragma unroll
        for (int u = 0; u < U; ++u)
          if (gis[u] < n && l < fanout) p.relabeled[gis[u] * fanout + l] = rel[u];
      }
    }
  } else {
    // fanout wider than a group: slots are resolved LPS at a time and earlier
    // chunks' picks are kept in LDS (whole-wave groups only).
    for (int s = 0; s < p.rows_per_group; ++s) {
      const int t = s * G + grp;
      const int64_t gi = tile_base + t;
      if (gi >= n) break;  // group-uniform
      const int64_t* nbrs = s_nbrs[t];
      const int64_t deg = s_deg[t];
      const int64_t node = s_node[t];
      int64_t* o = p.out + gi * fanout;
      int64_t cnt;
      if (REPLACE) {
        for (int i = l; i < fanout; i += LPS) {
          int64_t val = -1;
          if (deg > 0)
            val = nbrs[bounded(draw64(seed, node, p.hop, static_cast<uint32_t>(i)),
                               static_cast<uint64_t>(deg))];
          o[i] = val;
        }
        cnt = deg > 0 ? fanout : 0;
      } else if (deg <= fanout) {
        for (int i = l; i < fanout; i += LPS) o[i] = i < deg ? nbrs[i] : -1;
        cnt = deg;
      } else {
        int64_t* picks = s_picks + static_cast<size_t>(grp) * fanout;
        for (int c0 = 0; c0 < fanout; c0 += LPS) {
          const int i = c0 + l;
          const bool active = i < fanout;
          const int64_t j = deg - fanout + i;
          int64_t tpos = -1 - l;
          if (active)
            tpos = static_cast<int64_t>(bounded(draw64(seed, node, p.hop, static_cast<uint32_t>(i)),
                                                static_cast<uint64_t>(j + 1)));
          bool coll = false;
          for (int q = 0; q < c0; ++q) coll |= (picks[q] == tpos);
          const int len = min(LPS, fanout - c0);
          for (int q = 0; q + 1 < len; ++q) {
            const int64_t pq = __shfl(coll ? j : tpos, q, LPS);
            if (l > q && tpos == pq) coll = true;
          }
          const int64_t pick = coll ? j : tpos;
          if (active) {
            o[i] = nbrs[pick];
            picks[i] = pick;
          }
          __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
          __builtin_amdgcn_wave_barrier();
        }
        cnt = fanout;
      }
      if (l == 0) {
        if (p.counts != nullptr) p.counts[gi] = cnt;
        my_total += cnt;
      }
    }
  }
  if (!direct) __syncthreads();  // the next tile overwrites the staged rows
  }  // tiles
  if (p.total != nullptr) {
    if (l == 0 && my_total != 0)
      atomicAdd(&s_total, static_cast<unsigned long long>(my_total));
    __syncthreads();
    if (tid == 0 && s_total != 0)
      atomicAdd(reinterpret_cast<unsigned long long*>(p.total), s_total);
  }
}

template <int LPS>
static int launch_sample(const SampleParams& p, bool replace, int64_t blocks, size_t dyn_lds,
                         hipStream_t st) {
  const dim3 grid(static_cast<unsigned>(blocks)), block(kSampleBlock);
  // rows of a group in flight at once: as many as it has, up to 4
  const int u = p.rows_per_group >= 4 ? 4 : (p.rows_per_group >= 2 ? 2 : 1);
  hipEvent_t ev0 = nullptr, ev1 = nullptr;
  if (t_sample_hop == p.hop && (t_sample_start != nullptr || t_sample_stop != nullptr)) {
    ev0 = t_sample_start;
    ev1 = t_sample_stop;
    t_sample_start = t_sample_stop = nullptr;
    t_sample_hop = -1;
  }
#define APT_SAMPLE_LAUNCH(RP, UU)                                                                       \
  if (ev0 != nullptr || ev1 != nullptr)                                                                 \
    hipExtLaunchKernelGGL((sample_kernel<LPS, RP, UU>), grid, block, dyn_lds, st, ev0, ev1, 0, p);      \
  else                                                                                                  \
    hipLaunchKernelGGL((sample_kernel<LPS, RP, UU>), grid, block, dyn_lds, st, p)
  if (replace) {
    if (u == 4) { APT_SAMPLE_LAUNCH(true, 4); }
    else if (u == 2) { APT_SAMPLE_LAUNCH(true, 2); }
    else { APT_SAMPLE_LAUNCH(true, 1); }
  } else {
    if (u == 4) { APT_SAMPLE_LAUNCH(false, 4); }
    else if (u == 2) { APT_SAMPLE_LAUNCH(false, 2); }
    else { APT_SAMPLE_LAUNCH(false, 1); }
  }
#undef APT_SAMPLE_LAUNCH
  APT_LAUNCH_CHECK("sample_kernel");
  return APT_OK;
}

int tuning_sample_lanes();
int tuning_sample_min_workgroups();  // 0 = default
int tuning_sample_max_blocks();      // 0 = default
int tuning_sample_direct_rows();     // 0 / 1 = one row per lane group in the unstaged shape

}  // namespace apt

namespace apt {

// Shared by apt_sample_neighbors and the fused mini-batch driver.
int sample_launch(const apt_graph* graph, const int64_t* frontier, int64_t num_frontier,
                  const int64_t* num_frontier_dev, int fanout, int replace, uint64_t rng_seed,
                  const uint64_t* rng_seed_dev, int hop, int64_t* out_neighbors, int64_t* out_counts,
                  int64_t* out_total, hipStream_t st, const char* who, const SampleMark* mark) {
  APT_REQUIRE(graph != nullptr, APT_EINVAL, "%s: graph is NULL", who);
  APT_REQUIRE(num_frontier >= 0, APT_EINVAL, "%s: num_frontier %lld < 0", who, (long long)num_frontier);
  APT_REQUIRE(fanout > 0, APT_EINVAL, "%s: fanout %d must be > 0", who, fanout);
  APT_REQUIRE(fanout <= kMaxFanout, APT_ELIMIT, "%s: fanout %d exceeds the supported maximum %d", who,
              fanout, kMaxFanout);
  APT_REQUIRE(graph->num_rows >= 0 && graph->indptr != nullptr &&
                  (graph->indices != nullptr || graph->num_rows == 0),
              APT_EINVAL, "%s: graph has no indptr/indices", who);
  if (graph->adj_pos_map != nullptr) {
    APT_REQUIRE(graph->num_total_nodes >= 0, APT_EINVAL,
                "%s: adj_pos_map given but num_total_nodes < 0", who);
    APT_REQUIRE(graph->num_cached_rows == 0 ||
                    (graph->cached_indptr != nullptr && graph->cached_indices != nullptr),
                APT_EINVAL, "%s: cached rows without cached tables", who);
  }
  if (num_frontier == 0) return APT_OK;
  APT_REQUIRE(frontier != nullptr && out_neighbors != nullptr, APT_EINVAL,
              "%s: frontier/out_neighbors is NULL", who);
  APT_REQUIRE(num_frontier <= (INT64_MAX / 8) / fanout, APT_ELIMIT,
              "%s: num_frontier * fanout overflows", who);

  SampleParams p;
  p.g = *graph;
  p.frontier = frontier;
  p.n = num_frontier;
  p.n_dev = num_frontier_dev;
  p.fanout = fanout;
  p.seed = rng_seed;
  p.seed_dev = rng_seed_dev;
  p.hop = hop;
  p.out = out_neighbors;
  p.counts = out_counts;
  p.total = out_total;
  p.table = RankTable{nullptr, 0, nullptr, nullptr};
  p.relabeled = nullptr;
  p.first_hop = 0;
  if (mark != nullptr) {
    APT_REQUIRE(fanout <= kWave, APT_EINVAL, "%s: fused relabel marking needs fanout <= %d", who, kWave);
    p.table = mark->table;
    p.relabeled = mark->relabeled;
    p.first_hop = mark->first_hop;
    p.outside = mark->outside;
  }

  // Lanes per frontier row: the smallest power of two that holds the fanout
  // (8..64).  One whole wavefront per row leaves most lanes idle at the usual
  // fanouts (5..25) and costs more workgroups for the same rows.
  int lps = tuning_sample_lanes();
  if (lps != 8 && lps != 16 && lps != 32 && lps != 64) {
    lps = 8;
    while (lps < fanout && lps < kWave) lps <<= 1;
  }
  if (!replace && fanout > lps) lps = kWave;  // chunked Floyd needs whole waves
  if (mark != nullptr)                          // marking lives in the one-chunk path
    while (lps < fanout) lps <<= 1;
  const int groups = kSampleBlock / lps;
  // Rows are serialised inside a group only beyond kSampleMinWorkgroups
  // workgroups.  In the mini-batch driver num_frontier is an upper bound about
  // 3-4x the real count and the workgroups past the real count exit at once,
  // so this leaves roughly 2-4 k working workgroups (9-18 per CU), measured
  // best for the random-access bound hop.
  int64_t min_wg = tuning_sample_min_workgroups();
  if (min_wg <= 0) min_wg = kSampleMinWorkgroups;
  int64_t rpg = num_frontier / (static_cast<int64_t>(groups) * min_wg);
  if (rpg < 1) rpg = 1;
  if (rpg > kMaxRowsPerGroup) rpg = kMaxRowsPerGroup;
  p.rows_per_group = static_cast<int>(rpg);
  p.direct = rpg == 1 && fanout <= lps;
  // Several rows per lane group in flight without the staging (knob sample_direct_rows, 2 or 4): the group
  // issues the dependent loads of its rows back to back, so that the index loads and rank-table reads of one
  // row overlap the atomics of another inside a group and not only between groups.
  const int direct_rows = tuning_sample_direct_rows();
  if (p.direct && (direct_rows == 2 || direct_rows == 4)) {
    rpg = direct_rows;
    p.rows_per_group = direct_rows;
  }
  const int64_t tile = static_cast<int64_t>(groups) * rpg;
  int64_t blocks = ceil_div(num_frontier, tile);
  // With a device-side count num_frontier is an upper bound: a capped grid that
  // strides over the tiles avoids dispatching workgroups that find nothing to do.
  int64_t max_blocks = tuning_sample_max_blocks();
  if (max_blocks <= 0) max_blocks = num_frontier_dev != nullptr ? kSamplePersistentBlocks : (1 << 20);
  if (blocks > max_blocks) blocks = max_blocks;
  APT_REQUIRE(blocks <= 0x7fffffffLL, APT_ELIMIT, "%s: %lld rows need too many workgroups", who,
              (long long)num_frontier);
  const size_t dyn = (!replace && fanout > lps) ? sizeof(int64_t) * groups * (size_t)fanout : 0;
  switch (lps) {
    case 8: return launch_sample<8>(p, replace != 0, blocks, dyn, st);
    case 16: return launch_sample<16>(p, replace != 0, blocks, dyn, st);
    case 32: return launch_sample<32>(p, replace != 0, blocks, dyn, st);
    default: return launch_sample<64>(p, replace != 0, blocks, dyn, st);
  }
}

}  // namespace apt

extern "C" int apt_sample_neighbors(const apt_graph* graph, const int64_t* frontier,
                                    int64_t num_frontier, const int64_t* num_frontier_dev,
                                    int fanout, int replace, uint64_t rng_seed, int hop,
                                    int64_t* out_neighbors, int64_t* out_counts,
                                    int64_t* out_total, void* stream) {
  return apt::sample_launch(graph, frontier, num_frontier, num_frontier_dev, fanout, replace,
                            rng_seed, nullptr, hop, out_neighbors, out_counts, out_total,
                            static_cast<hipStream_t>(stream), "apt_sample_neighbors", nullptr);
}

extern "C" int apt_time_next_sample(int hop, void* start_event, void* stop_event) {
  apt::t_sample_start = static_cast<hipEvent_t>(start_event);
  apt::t_sample_stop = static_cast<hipEvent_t>(stop_event);
  apt::t_sample_hop = (start_event != nullptr || stop_event != nullptr) ? hop : -1;
  return APT_OK;
}
