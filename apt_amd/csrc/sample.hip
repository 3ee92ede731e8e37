// Uniform neighbour sampling over CSR, one hop.
//
// Replaces _CSRRowWiseSampleReplaceKernel / LocalSampleNeighbors
// (reference src/cuda/npc_kernel.cu:248-316).  Differences by design:
//   * a lane group (8..64 lanes of a wave64, default one whole wavefront) owns
//     a frontier row; the block first stages every row's (neighbour pointer,
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
#include "common.hpp"

namespace apt {

struct SampleParams {
  apt_graph g;
  const int64_t* frontier;
  int64_t n;
  const int64_t* n_dev;
  int fanout;
  uint64_t seed;
  int hop;
  int64_t* out;
  int64_t* counts;
  int64_t* total;
  int rows_per_group;
};

constexpr int kSampleBlock = 256;
constexpr int kMaxRowsPerGroup = 16;
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

template <int LPS, bool REPLACE>
__global__ __launch_bounds__(kSampleBlock) void sample_kernel(SampleParams p) {
  constexpr int G = kSampleBlock / LPS;  // lane groups per block
  constexpr int kMaxTile = G * kMaxRowsPerGroup;
  __shared__ const int64_t* s_nbrs[kMaxTile];
  __shared__ int64_t s_deg[kMaxTile];
  __shared__ int64_t s_node[kMaxTile];
  __shared__ unsigned long long s_total;
  extern __shared__ int64_t s_picks[];  // [G][fanout], only when fanout > LPS

  const int64_t n = actual_count(p.n, p.n_dev);
  const int tile = G * p.rows_per_group;
  const int64_t tile_base = static_cast<int64_t>(blockIdx.x) * tile;
  if (tile_base >= n) return;  // block-uniform

  const int tid = threadIdx.x;
  if (tid == 0) s_total = 0;
  // Stage 1: one lane per row of the tile.
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

  // Stage 2: one lane group per row.
  const int grp = tid / LPS;
  const int l = tid % LPS;
  const int fanout = p.fanout;
  int64_t my_total = 0;
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
      // reference :277-283
      for (int i = l; i < fanout; i += LPS) {
        int64_t val = -1;
        if (deg > 0)
          val = nbrs[bounded(draw64(p.seed, node, p.hop, static_cast<uint32_t>(i)),
                             static_cast<uint64_t>(deg))];
        o[i] = val;
      }
      cnt = deg > 0 ? fanout : 0;
    } else if (deg <= fanout) {
      for (int i = l; i < fanout; i += LPS) o[i] = i < deg ? nbrs[i] : -1;
      cnt = deg;
    } else {
      // Floyd: slot i draws t in [0, j], j = deg - fanout + i, and takes t
      // unless an earlier slot already holds t, then it takes j.
      int64_t* picks = s_picks + static_cast<size_t>(grp) * fanout;
      for (int c0 = 0; c0 < fanout; c0 += LPS) {
        const int i = c0 + l;
        const bool active = i < fanout;
        const int64_t j = deg - fanout + i;
        int64_t tpos = -1 - l;  // inactive lanes never match a position
        if (active)
          tpos = static_cast<int64_t>(
              bounded(draw64(p.seed, node, p.hop, static_cast<uint32_t>(i)),
                      static_cast<uint64_t>(j + 1)));
        bool coll = false;
        if (LPS == kWave && c0 > 0) {
          for (int q = 0; q < c0; ++q) coll |= (picks[q] == tpos);
        }
        const int len = min(LPS, fanout - c0);
        for (int q = 0; q + 1 < len; ++q) {
          const int64_t mine = coll ? j : tpos;
          const int64_t pq = __shfl(mine, q, LPS);
          if (l > q && tpos == pq) coll = true;
        }
        const int64_t pick = coll ? j : tpos;
        if (active) o[i] = nbrs[pick];
        if (LPS == kWave && fanout > LPS) {
          if (active) picks[i] = pick;
          __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
          __builtin_amdgcn_wave_barrier();
        }
      }
      cnt = fanout;
    }
    if (l == 0) {
      if (p.counts != nullptr) p.counts[gi] = cnt;
      my_total += cnt;
    }
  }
  if (p.total != nullptr) {
    if (l == 0 && my_total != 0)
      atomicAdd(&s_total, static_cast<unsigned long long>(my_total));
    __syncthreads();
    if (tid == 0 && s_total != 0)
      atomicAdd(reinterpret_cast<unsigned long long*>(p.total), s_total);
  }
}

template <int LPS>
static int launch_sample(const SampleParams& p, bool replace, int64_t blocks,
                         size_t dyn_lds, hipStream_t st) {
  if (replace)
    hipLaunchKernelGGL((sample_kernel<LPS, true>), dim3(static_cast<unsigned>(blocks)),
                       dim3(kSampleBlock), dyn_lds, st, p);
  else
    hipLaunchKernelGGL((sample_kernel<LPS, false>), dim3(static_cast<unsigned>(blocks)),
                       dim3(kSampleBlock), dyn_lds, st, p);
  APT_LAUNCH_CHECK("sample_kernel");
  return APT_OK;
}

int tuning_sample_lanes();  // 0 = automatic

}  // namespace apt

extern "C" int apt_sample_neighbors(const apt_graph* graph, const int64_t* frontier,
                                    int64_t num_frontier,
                                    const int64_t* num_frontier_dev, int fanout,
                                    int replace, uint64_t rng_seed, int hop,
                                    int64_t* out_neighbors, int64_t* out_counts,
                                    int64_t* out_total, void* stream) {
  using namespace apt;
  APT_REQUIRE(graph != nullptr, APT_EINVAL, "apt_sample_neighbors: graph is NULL");
  APT_REQUIRE(num_frontier >= 0, APT_EINVAL,
              "apt_sample_neighbors: num_frontier %lld < 0", (long long)num_frontier);
  APT_REQUIRE(fanout > 0, APT_EINVAL, "apt_sample_neighbors: fanout %d must be > 0", fanout);
  APT_REQUIRE(fanout <= kMaxFanout, APT_ELIMIT,
              "apt_sample_neighbors: fanout %d exceeds the supported maximum %d", fanout,
              kMaxFanout);
  APT_REQUIRE(graph->num_rows >= 0 && graph->indptr != nullptr &&
                  (graph->indices != nullptr || graph->num_rows == 0),
              APT_EINVAL, "apt_sample_neighbors: graph has no indptr/indices");
  if (graph->adj_pos_map != nullptr) {
    APT_REQUIRE(graph->num_total_nodes >= 0, APT_EINVAL,
                "apt_sample_neighbors: adj_pos_map given but num_total_nodes < 0");
    APT_REQUIRE(graph->num_cached_rows == 0 ||
                    (graph->cached_indptr != nullptr && graph->cached_indices != nullptr),
                APT_EINVAL, "apt_sample_neighbors: cached rows without cached tables");
  }
  if (num_frontier == 0) return APT_OK;
  APT_REQUIRE(frontier != nullptr && out_neighbors != nullptr, APT_EINVAL,
              "apt_sample_neighbors: frontier/out_neighbors is NULL");
  APT_REQUIRE(num_frontier <= (INT64_MAX / 8) / fanout, APT_ELIMIT,
              "apt_sample_neighbors: num_frontier * fanout overflows");

  SampleParams p;
  p.g = *graph;
  p.frontier = frontier;
  p.n = num_frontier;
  p.n_dev = num_frontier_dev;
  p.fanout = fanout;
  p.seed = rng_seed;
  p.hop = hop;
  p.out = out_neighbors;
  p.counts = out_counts;
  p.total = out_total;

  int lps = tuning_sample_lanes();
  if (lps == 0) lps = kWave;  // one wavefront per frontier row
  if (lps != 8 && lps != 16 && lps != 32 && lps != 64) lps = kWave;
  if (!replace && fanout > lps) lps = kWave;  // chunked Floyd needs whole waves
  const int groups = kSampleBlock / lps;
  // Enough blocks to cover 256 CUs several times over before rows are
  // serialised inside a group.
  int64_t rpg = num_frontier / (static_cast<int64_t>(groups) * 4096);
  if (rpg < 1) rpg = 1;
  if (rpg > kMaxRowsPerGroup) rpg = kMaxRowsPerGroup;
  p.rows_per_group = static_cast<int>(rpg);
  const int64_t tile = static_cast<int64_t>(groups) * rpg;
  const int64_t blocks = ceil_div(num_frontier, tile);
  APT_REQUIRE(blocks <= 0x7fffffffLL, APT_ELIMIT,
              "apt_sample_neighbors: %lld rows need too many workgroups",
              (long long)num_frontier);
  const size_t dyn =
      (!replace && fanout > lps) ? sizeof(int64_t) * groups * (size_t)fanout : 0;
  hipStream_t st = static_cast<hipStream_t>(stream);
  switch (lps) {
    case 8: return launch_sample<8>(p, replace != 0, blocks, dyn, st);
    case 16: return launch_sample<16>(p, replace != 0, blocks, dyn, st);
    case 32: return launch_sample<32>(p, replace != 0, blocks, dyn, st);
    default: return launch_sample<64>(p, replace != 0, blocks, dyn, st);
  }
}
