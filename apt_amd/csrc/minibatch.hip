// Fused multi-hop mini-batch construction: sample -> relabel for every hop in
// one call, without host round trips.
//
// Counterpart of the DP branch of MixedPSNeighborSampler.sample (reference
// python/npc/sampler.py:187-203,358-364), which per hop calls
// local_sample_one_layer, relabel_csc (torch::cat + 3 hash passes + cub scan,
// src/cuda/relabel.cu:78-185) and reads the unique count back to the host.
//
// Relabel here uses a node-indexed rank table instead of a hash table: one
// uint32 per node of the graph, resident in HBM for the life of the process
// (444 MB for 111M nodes; a few per mille of 288 GB).  table[v] is 0xFFFFFFFF
// when v is not in the batch, otherwise the compact id of v.  Because the
// unique list of hop h is the unique list of hop h-1 followed by the new nodes
// in first-occurrence order (the order the reference's AtomicMin-on-index
// produces), the list only ever grows and ids never change:
//   * the frontier of hop h is nodes[0 : n_h], already marked with its ids;
//   * a sampled neighbour that is already in the batch is relabelled by one
//     load, with no atomic at all (hubs are almost always already there);
//   * the others race with atomicMin on (n_h + slot index); the smallest index
//     owns the node.  The atomic returns the bid it replaces, the bidder flags
//     that slot as displaced, so ownership is known without reading the table
//     again (rank_table.hpp); owners are ranked with ballots + a two-level
//     prefix, get id n_h + rank and are appended to the list.
// Random atomics are the scarcest resource on this GPU (~20 G/s against
// ~45 G/s random loads), which is why the table is indexed directly (no CAS
// to claim a slot, no probing) and why nodes already present never touch one.
// Nothing is ever cleared per batch: an entry is (epoch << P) | payload, P =
// bits needed for the largest id of the plan, and every call uses the next
// lower epoch, so the entries of earlier batches (larger epochs, or the
// all-ones fill) compare greater than anything the current batch writes and an
// atomicMin overrides them without being told.  The epoch lives in device
// memory next to the table (the first kernel of a batch advances it), so a
// captured HIP graph replays correctly; when the epochs run out (every
// 2^(32-P) - 1 calls) that kernel refills the table.
// On the last hop the owners' ids are not even written to the table: the few
// slots that lost a race fetch the id from an output slot instead: the one they
// saw ahead of them when they lost (rank_table.hpp), or, if that one was
// displaced itself, the winner's.
#include "common.hpp"
#include "rank_table.hpp"

namespace apt {


int sample_launch(const apt_graph* graph, const int64_t* frontier, int64_t num_frontier,
                  const int64_t* num_frontier_dev, int fanout, int replace, uint64_t rng_seed,
                  const uint64_t* rng_seed_dev, int hop, int64_t* out_neighbors, int64_t* out_counts,
                  int64_t* out_total, hipStream_t st, const char* who, const SampleMark* mark);

int tuning_fuse_mark();  // 1 (default) = mark inside the sampling kernel

constexpr int kMbBlock = 256;
constexpr int kMbIters = 4;
constexpr int kMbTile = kMbBlock * kMbIters;     // items per workgroup in count / place
constexpr int kMbWaves = kMbBlock / kWave;
constexpr uint32_t kEmpty = 0xFFFFFFFFu;
constexpr int kMaxHops = APT_MAX_HOPS;

struct HopParams {
  const int64_t* seeds;      // first hop: the caller's seeds; later hops: unused
  int64_t ns_cap;            // frontier rows, host-side upper bound
  const int64_t* ns_dev;     // actual frontier rows (NULL on the first hop)
  int64_t fanout;
  const int64_t* neighbors;  // [ns_cap * fanout], -1 padded
  int64_t* relabeled;        // [ns_cap * fanout]
  uint32_t* table;
  int64_t table_len;
  const uint32_t* state;     // [0] epoch, [1] payload bits (see mb_begin_kernel)
  int last;                  // last hop: ids are not written back to the table
  int64_t* nodes;            // growing unique list
  int64_t nodes_cap;         // its capacity: an id beyond it (counters corrupted by the caller) is dropped, not written
  int64_t* n_next;           // receives the size of the list after this hop
  uint64_t* flags;           // owner bit per item, one word per wavefront-load
  uint32_t* tile_cnt;
  uint8_t* displaced;        // per slot: a smaller bid took the node over (rank_table.hpp)
  int64_t nn_fixed;          // >= 0: the number of neighbour slots, where it is not rows x fanout (apt_relabel_ranked)
  int64_t* outside;          // optional: counts the ids that the table cannot hold (>= table_len)
  int mark_seeds;            // the marking pass of the first hop also lets the seeds bid (no pass of their own)
  const int64_t* prefix_src; // the marking pass of a later hop also copies these ns ids to the head of `nodes`
};

struct HopSizes {
  int64_t ns, nn;
};

__device__ __forceinline__ HopSizes hop_sizes(const HopParams& p) {
  HopSizes s;
  s.ns = actual_count(p.ns_cap, p.ns_dev);
  s.nn = p.nn_fixed >= 0 ? p.nn_fixed : s.ns * p.fanout;
  return s;
}

__device__ __forceinline__ bool in_table(const HopParams& p, int64_t v) {
  return v >= 0 && v < p.table_len;
}

// Epoch bookkeeping (state block behind the table entries):
//   [0] epoch of the latest batch  [1] payload bits  [3] finished-workgroup counter
// First kernel of every batch, a few workgroups: move to the next lower epoch,
// or, when the epochs are used up (or the table was last used with another
// payload width, or is new), refill the table with all-ones and start the
// numbering over.  Every workgroup reads the state before any of them can
// change it, because only the workgroup that finishes last writes.
constexpr int kBeginBlocks = 64;

__global__ __launch_bounds__(kMbBlock) void mb_begin_kernel(uint4* table, int64_t vecs, uint32_t* state,
                                                            uint32_t payload_bits, int64_t* sizes,
                                                            int num_sizes, int64_t batch) {
  // per-batch counters: sizes[0] = batch, the rest 0
  if (blockIdx.x == 0 && static_cast<int>(threadIdx.x) < num_sizes) sizes[threadIdx.x] = threadIdx.x == 0 ? batch : 0;
  const bool refill = state[1] != payload_bits || state[0] == 0;
  if (refill) {
    const uint4 ones = make_uint4(kEmpty, kEmpty, kEmpty, kEmpty);
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kMbBlock + threadIdx.x; i < vecs;
         i += static_cast<int64_t>(gridDim.x) * kMbBlock)
      table[i] = ones;
    __threadfence();
  }
  __syncthreads();
  if (threadIdx.x == 0 && atomicAdd(&state[3], 1u) == gridDim.x - 1) {
    state[3] = 0;
    if (refill) {
      state[0] = (1u << (32 - payload_bits)) - 2;  // the all-ones epoch is the fill value
      state[1] = payload_bits;
    } else {
      state[0] -= 1;
    }
  }
}

// First hop only: seeds may repeat, so they race like everything else; the
// smallest seed index owns the node.  (Also sets the per-batch counters, as the
// first kernel of the batch already has.)
__global__ __launch_bounds__(kMbBlock) void mb_mark_seeds_kernel(HopParams p, int64_t* sizes,
                                                                 int num_sizes) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kMbBlock + threadIdx.x;
  if (i < num_sizes) sizes[i] = i == 0 ? p.ns_cap : 0;
  if (i < actual_count(p.ns_cap, p.ns_dev)) {
    const int64_t v = p.seeds[i];
    if (in_table(p, v)) atomicMin(&p.table[v], table_base(p.state) + static_cast<uint32_t>(i));
    else if (p.outside != nullptr && v >= p.table_len)
      atomicAdd(reinterpret_cast<unsigned long long*>(p.outside), 1ull);
  }
}

// Stand-alone marking pass (fanouts wider than a wavefront, or the fusion into
// the sampling kernel switched off): the same per-slot step as in sample.hip.
template <bool FIRST>
__global__ __launch_bounds__(kMbBlock) void mb_mark_neighbors_kernel(HopParams p) {
  const HopSizes s = hop_sizes(p);
  const RankEpoch ep = rank_epoch(p.state);
  const RankTable t{p.table, p.table_len, p.state, p.displaced};
  const bool with_rows = FIRST ? p.mark_seeds != 0 : p.prefix_src != nullptr;
  const int64_t work = with_rows && s.ns > s.nn ? s.ns : s.nn;
  for (int64_t j = static_cast<int64_t>(blockIdx.x) * kMbBlock + threadIdx.x; j < work;
       j += static_cast<int64_t>(gridDim.x) * kMbBlock) {
    if (j < s.nn) {
      const int64_t v = p.neighbors[j];
      p.relabeled[j] = rank_table_bid(t, ep, FIRST, v, s.ns, j);
      if (p.outside != nullptr && v >= p.table_len) atomicAdd(reinterpret_cast<unsigned long long*>(p.outside), 1ull);
    }
    if (with_rows && j < s.ns) {
      if (FIRST) {
        const int64_t v = p.seeds[j];
        if (in_table(p, v)) atomicMin(&p.table[v], ep.base + static_cast<uint32_t>(j));
        else if (p.outside != nullptr && v >= p.table_len)
          atomicAdd(reinterpret_cast<unsigned long long*>(p.outside), 1ull);
      } else {
        p.nodes[j] = p.prefix_src[j];
      }
    }
  }
}

// Upper bound of a hop's neighbour slots as the host knows it: what the buffers hold whatever the device-side
// row count says.  Loads of per-slot arrays below this bound are safe before that count has arrived, which
// takes a memory round trip or two out of the start of the small kernels of a batch (they are chains of three
// to five such trips and little else).  Only launches of a few hundred workgroups do that: in a large launch
// the workgroups past the real count would fetch megabytes for nothing, and its many waves hide the trip anyway.
__device__ __forceinline__ int64_t slot_capacity(const HopParams& p) {
  return p.nn_fixed >= 0 ? p.nn_fixed : p.ns_cap * p.fanout;
}
constexpr unsigned kLoadAheadMaxBlocks = 512;

template <bool FIRST>
__global__ __launch_bounds__(kMbBlock) void mb_count_kernel(HopParams p) {
  const int64_t base = static_cast<int64_t>(blockIdx.x) * kMbTile;
  __shared__ uint32_t s_wave[kMbWaves];
  const int wave = threadIdx.x / kWave;
  uint32_t c = 0;
  if (FIRST) {
    // First hop: an item (seed or neighbour, its index is its bid) owns its node iff the table still holds its
    // bid.  The tile's ids, then its table entries, are requested together: two round trips for the tile, not
    // two per iteration.
    const HopSizes s = hop_sizes(p);
    const int64_t items = s.ns + s.nn;
    if (base >= items) return;
    const uint32_t tb = table_base(p.state);
    int64_t v[kMbIters];
    uint32_t held[kMbIters];
#pragma unroll
    for (int it = 0; it < kMbIters; ++it) {
      const int64_t i = base + it * kMbBlock + threadIdx.x;
      v[it] = i < items ? (i < s.ns ? p.seeds[i] : p.neighbors[i - s.ns]) : -1;
    }
#pragma unroll
    for (int it = 0; it < kMbIters; ++it) held[it] = in_table(p, v[it]) ? p.table[v[it]] : 0u;
#pragma unroll
    for (int it = 0; it < kMbIters; ++it) {
      const int64_t i = base + it * kMbBlock + threadIdx.x;
      const uint64_t m = ballot(in_table(p, v[it]) && held[it] == tb + static_cast<uint32_t>(i));
      if (lane_id() == 0) p.flags[(static_cast<int64_t>(blockIdx.x) * kMbIters + it) * kMbWaves + wave] = m;
      c += __popcll(m);
    }
  } else {
    // Later hops: the bidding itself settled ownership (rank_table.hpp): a slot owns its node iff it is
    // kSlotOwner and was never displaced; the flag is consumed so that the buffer is clean for the next hop.
    // Both arrays are read under the host's bound, before the row count is known.
    const bool ahead = gridDim.x <= kLoadAheadMaxBlocks;
    const int64_t cap = ahead ? slot_capacity(p) : 0;
    int64_t rel[kMbIters];
    uint8_t dis[kMbIters];
#pragma unroll
    for (int it = 0; it < kMbIters; ++it) {
      const int64_t i = base + it * kMbBlock + threadIdx.x;
      rel[it] = i < cap ? p.relabeled[i] : 0;
      dis[it] = i < cap ? p.displaced[i] : 0;
    }
    const HopSizes s = hop_sizes(p);
    const int64_t items = s.nn;
    if (base >= items) return;
    if (!ahead) {
#pragma unroll
      for (int it = 0; it < kMbIters; ++it) {
        const int64_t i = base + it * kMbBlock + threadIdx.x;
        rel[it] = i < items ? p.relabeled[i] : 0;
        dis[it] = i < items ? p.displaced[i] : 0;
      }
    }
#pragma unroll
    for (int it = 0; it < kMbIters; ++it) {
      const int64_t i = base + it * kMbBlock + threadIdx.x;
      const bool bid_in = i < items && rel[it] == kSlotOwner;
      if (bid_in && dis[it] != 0) p.displaced[i] = 0;
      const uint64_t m = ballot(bid_in && dis[it] == 0);
      if (lane_id() == 0) p.flags[(static_cast<int64_t>(blockIdx.x) * kMbIters + it) * kMbWaves + wave] = m;
      c += __popcll(m);
    }
  }
  if (lane_id() == 0) s_wave[wave] = c;
  __syncthreads();
  if (threadIdx.x == 0) {
    uint32_t t = 0;
    for (int w = 0; w < kMbWaves; ++w) t += s_wave[w];
    p.tile_cnt[blockIdx.x] = t;
  }
}

// Owners get id base + (number of owners before them), are appended to the
// node list and written into the table.
template <bool FIRST>
__global__ __launch_bounds__(kMbBlock) void mb_place_kernel(HopParams p) {
  const int64_t base = static_cast<int64_t>(blockIdx.x) * kMbTile;
  const int wave = threadIdx.x / kWave;
  const int lane = lane_id();
  // In a small launch, what does not depend on the hop's row count is requested before it: the owner counts
  // of the tiles before this one and this tile's owner bits (the count pass wrote both for every tile that has
  // items, and a tile without items leaves below before using them), and, on later hops, the tile's neighbour
  // ids.
  const bool ahead_ok = gridDim.x <= kLoadAheadMaxBlocks;
  int64_t part = 0;
  uint64_t mask[kMbIters][kMbWaves];
  int64_t ahead[kMbIters];
  auto load_tile = [&](int64_t cap) {
    for (int64_t b = threadIdx.x; b < blockIdx.x; b += kMbBlock) part += p.tile_cnt[b];
#pragma unroll
    for (int it = 0; it < kMbIters; ++it)
#pragma unroll
      for (int w = 0; w < kMbWaves; ++w)
        mask[it][w] = p.flags[(static_cast<int64_t>(blockIdx.x) * kMbIters + it) * kMbWaves + w];
    if (!FIRST) {
#pragma unroll
      for (int it = 0; it < kMbIters; ++it) {
        const int64_t i = base + it * kMbBlock + threadIdx.x;
        ahead[it] = i < cap ? p.neighbors[i] : -1;
      }
    }
  };
  if (ahead_ok) load_tile(slot_capacity(p));
  const HopSizes s = hop_sizes(p);
  const int64_t items = FIRST ? s.ns + s.nn : s.nn;
  if (FIRST) {   // the first hop's items: seeds, then neighbours (the row count is the host's, nothing to wait for)
#pragma unroll
    for (int it = 0; it < kMbIters; ++it) {
      const int64_t i = base + it * kMbBlock + threadIdx.x;
      ahead[it] = i < items ? (i < s.ns ? p.seeds[i] : p.neighbors[i - s.ns]) : -1;
    }
  }
  const int64_t first_id = FIRST ? 0 : s.ns;
  if (items == 0) {
    if (blockIdx.x == 0 && threadIdx.x == 0) *p.n_next = first_id;
    return;
  }
  if (base >= items) return;
  if (!ahead_ok) load_tile(items);
  const int64_t tiles = (items + kMbTile - 1) / kMbTile;
  __shared__ int64_t s_red[kMbWaves];
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) part += __shfl_down(part, off, kWave);
  if (lane == 0) s_red[wave] = part;
  __syncthreads();
  int64_t running = first_id;
  for (int w = 0; w < kMbWaves; ++w) running += s_red[w];
#pragma unroll
  for (int it = 0; it < kMbIters; ++it) {
    int64_t before = running;
#pragma unroll
    for (int w = 0; w < kMbWaves; ++w) {
      const int c = __popcll(mask[it][w]);
      if (w < wave) before += c;
      running += c;
    }
    uint64_t mine = 0;
#pragma unroll
    for (int w = 0; w < kMbWaves; ++w)
      if (w == wave) mine = mask[it][w];
    if ((mine >> lane) & 1) {
      const int64_t i = base + it * kMbBlock + threadIdx.x;
      const int64_t id = before + rank_below(mine);
      const int64_t v = ahead[it];
      if (FIRST) {
        if (i >= s.ns) p.relabeled[i - s.ns] = id;
      } else {
        p.relabeled[i] = id;
      }
      if (id < p.nodes_cap) {
        p.nodes[id] = v;
        if (!p.last) p.table[v] = table_base(p.state) + static_cast<uint32_t>(id);
      }
    }
  }
  if (blockIdx.x == tiles - 1 && threadIdx.x == 0) *p.n_next = running;
}

// Slots that lost the ownership race read the winner's id (all hops at once).
__global__ __launch_bounds__(kLookupBlock) void mb_lookup_kernel(LookupParams p) { lookup_block(p, blockIdx.x); }

__global__ void mb_zero_state_kernel(uint32_t* state) { state[threadIdx.x] = 0; }

__global__ void mb_zero_sizes_kernel(int64_t* sizes, int n) {
  if (static_cast<int>(threadIdx.x) < n) sizes[threadIdx.x] = 0;
}

__global__ __launch_bounds__(kMbBlock) void mb_zero_kernel(uint4* p, int64_t vecs) {
  const uint4 z = make_uint4(0, 0, 0, 0);
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kMbBlock + threadIdx.x; i < vecs;
       i += static_cast<int64_t>(gridDim.x) * kMbBlock)
    p[i] = z;
}

__global__ __launch_bounds__(kMbBlock) void mb_fill_table_kernel(uint4* table, int64_t vecs) {
  const uint4 ones = make_uint4(kEmpty, kEmpty, kEmpty, kEmpty);
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kMbBlock + threadIdx.x; i < vecs;
       i += static_cast<int64_t>(gridDim.x) * kMbBlock)
    table[i] = ones;
}

static size_t mb_align(size_t x) { return (x + 255) / 256 * 256; }

struct MbLayout {
  size_t flags_off, tile_off, displaced_off, total;
  int64_t caps[kMaxHops + 1];
  int64_t max_items;
  uint32_t payload_bits;  // ids and bids of the plan are < 2^payload_bits
};

int tuning_payload_bits();  // 0 = as few as the plan needs

static size_t table_state_offset(int64_t table_len) {
  return (static_cast<size_t>(table_len) * sizeof(uint32_t) + 255) / 256 * 256;
}

static bool mb_layout(int64_t batch, const int* fanouts, int num_hops, MbLayout& L) {
  L.caps[0] = batch;
  L.max_items = 1;
  for (int h = 0; h < num_hops; ++h) {
    if (fanouts[h] <= 0) return false;
    const int64_t f = fanouts[h];
    if (L.caps[h] > (int64_t{1} << 31) / (1 + f)) return false;  // ids and bids are 32-bit
    L.caps[h + 1] = L.caps[h] * (1 + f);
    const int64_t items = h == 0 ? L.caps[h] * (1 + f) : L.caps[h] * f;
    if (items > L.max_items) L.max_items = items;
  }
  L.payload_bits = 1;
  while ((int64_t{1} << L.payload_bits) < L.caps[num_hops] + 1) ++L.payload_bits;
  if (tuning_payload_bits() > static_cast<int>(L.payload_bits) && tuning_payload_bits() <= 31)
    L.payload_bits = static_cast<uint32_t>(tuning_payload_bits());
  const int64_t tiles = ceil_div(L.max_items, kMbTile);
  size_t off = 0;
  L.flags_off = off; off = mb_align(off + sizeof(uint64_t) * tiles * kMbIters * kMbWaves);
  L.tile_off = off;  off = mb_align(off + sizeof(uint32_t) * tiles);
  L.displaced_off = off; off = mb_align(off + static_cast<size_t>(L.max_items));
  L.total = off;
  return true;
}

}  // namespace apt

extern "C" size_t apt_rank_table_bytes(int64_t num_total_nodes) {
  if (num_total_nodes < 0 || num_total_nodes >= (int64_t{1} << 32) - 1) return 0;
  return apt::table_state_offset(num_total_nodes) + 256;  // entries + epoch state
}

extern "C" int apt_rank_table_init(void* table, size_t table_bytes, void* stream) {
  using namespace apt;
  APT_REQUIRE(table != nullptr && table_bytes >= 256 && table_bytes % 256 == 0 &&
                  (reinterpret_cast<uintptr_t>(table) & 255) == 0,
              APT_EINVAL, "apt_rank_table_init: table must be 256-byte aligned and sized by "
                          "apt_rank_table_bytes");
  // entries all-ones; the trailing state block all-zero (epoch 0 = "start over")
  hipLaunchKernelGGL(mb_zero_state_kernel, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream),
                     reinterpret_cast<uint32_t*>(static_cast<char*>(table) + table_bytes - 256));
  APT_LAUNCH_CHECK("mb_zero_state_kernel");
  if (table_bytes == 256) return APT_OK;
  const int64_t vecs = static_cast<int64_t>((table_bytes - 256) / 16);
  const unsigned blocks = static_cast<unsigned>(std::min<int64_t>(ceil_div(vecs, kMbBlock), 16384));
  hipLaunchKernelGGL(mb_fill_table_kernel, dim3(blocks), dim3(kMbBlock), 0,
                     static_cast<hipStream_t>(stream), static_cast<uint4*>(table), vecs);
  APT_LAUNCH_CHECK("mb_fill_table_kernel");
  return APT_OK;
}

extern "C" size_t apt_minibatch_workspace_bytes(int64_t batch, const int* hop_fanouts, int num_hops) {
  apt::MbLayout L;
  if (batch < 0 || hop_fanouts == nullptr || num_hops < 1 || num_hops > apt::kMaxHops) return 0;
  if (!apt::mb_layout(batch, hop_fanouts, num_hops, L)) return 0;
  return L.total;
}

extern "C" int apt_minibatch_workspace_init(void* workspace, size_t workspace_bytes, void* stream) {
  using namespace apt;
  APT_REQUIRE(workspace != nullptr && workspace_bytes % 16 == 0 &&
                  (reinterpret_cast<uintptr_t>(workspace) & 15) == 0,
              APT_EINVAL, "apt_minibatch_workspace_init: workspace must be 16-byte aligned and sized");
  if (workspace_bytes == 0) return APT_OK;
  const int64_t vecs = static_cast<int64_t>(workspace_bytes / 16);
  hipLaunchKernelGGL(mb_zero_kernel, dim3(static_cast<unsigned>(std::min<int64_t>(ceil_div(vecs, kMbBlock), 4096))),
                     dim3(kMbBlock), 0, static_cast<hipStream_t>(stream), static_cast<uint4*>(workspace), vecs);
  APT_LAUNCH_CHECK("mb_zero_kernel");
  return APT_OK;
}

extern "C" int64_t apt_minibatch_capacity(int64_t batch, const int* hop_fanouts, int num_hops, int hop) {
  apt::MbLayout L;
  if (batch < 0 || hop_fanouts == nullptr || num_hops < 1 || num_hops > apt::kMaxHops) return -1;
  if (hop < 0 || hop > num_hops || !apt::mb_layout(batch, hop_fanouts, num_hops, L)) return -1;
  return L.caps[hop];
}

namespace apt {
static int minibatch_sample(const apt_graph* graph, const int64_t* seeds, int64_t batch,
                            const int* hop_fanouts, int num_hops, int replace, uint64_t rng_seed,
                            const uint64_t* rng_seed_dev, void* rank_table, int64_t rank_table_len,
                            int64_t* nodes, int64_t* const* neighbors, int64_t* const* relabeled,
                            int64_t* const* counts, int64_t* sizes, void* workspace,
                            size_t workspace_bytes, void* stream, PendingLookup* defer) {
  if (defer != nullptr) {
    defer->magic = kPendingMagic;
    defer->blocks = 0;
  }
  APT_REQUIRE(graph != nullptr, APT_EINVAL, "apt_minibatch_sample: graph is NULL");
  APT_REQUIRE(batch >= 0, APT_EINVAL, "apt_minibatch_sample: batch %lld < 0", (long long)batch);
  APT_REQUIRE(hop_fanouts != nullptr && num_hops >= 1 && num_hops <= kMaxHops, APT_ELIMIT,
              "apt_minibatch_sample: num_hops %d outside [1, %d]", num_hops, kMaxHops);
  MbLayout L;
  APT_REQUIRE(mb_layout(batch, hop_fanouts, num_hops, L), APT_ELIMIT,
              "apt_minibatch_sample: fanouts must be > 0 and batch * prod(1 + fanout) < 2^31");
  APT_REQUIRE(rank_table != nullptr && rank_table_len > 0 && rank_table_len < (int64_t{1} << 32) - 1,
              APT_EINVAL, "apt_minibatch_sample: rank table missing or too long");
  APT_REQUIRE(sizes != nullptr && neighbors != nullptr && relabeled != nullptr, APT_EINVAL,
              "apt_minibatch_sample: sizes/neighbors/relabeled is NULL");
  APT_REQUIRE(batch == 0 || (seeds != nullptr && nodes != nullptr), APT_EINVAL,
              "apt_minibatch_sample: seeds/nodes is NULL");
  APT_REQUIRE(workspace != nullptr && workspace_bytes >= L.total, APT_EWORKSPACE,
              "apt_minibatch_sample: workspace of %zu bytes, %zu needed", workspace_bytes, L.total);
  for (int h = 0; h < num_hops; ++h)
    APT_REQUIRE(batch == 0 || (neighbors[h] != nullptr && relabeled[h] != nullptr), APT_EINVAL,
                "apt_minibatch_sample: neighbors[%d]/relabeled[%d] is NULL", h, h);
  hipStream_t st = static_cast<hipStream_t>(stream);
  char* ws = static_cast<char*>(workspace);
  int64_t* total = sizes + num_hops + 1;

  uint32_t* state = reinterpret_cast<uint32_t*>(static_cast<char*>(rank_table) +
                                                table_state_offset(rank_table_len));
  if (batch == 0) {
    hipLaunchKernelGGL(mb_zero_sizes_kernel, dim3(1), dim3(64), 0, st, sizes, num_hops + 2);
    APT_LAUNCH_CHECK("mb_zero_sizes_kernel");
    return APT_OK;
  }
  {
    // next epoch; refills only when the epochs are used up (or the table is new)
    const int64_t vecs = static_cast<int64_t>(table_state_offset(rank_table_len) / 16);
    hipLaunchKernelGGL(mb_begin_kernel, dim3(kBeginBlocks), dim3(kMbBlock), 0, st,
                       static_cast<uint4*>(rank_table), vecs, state, L.payload_bits, sizes, num_hops + 2, batch);
    APT_LAUNCH_CHECK("mb_begin_kernel");
  }

  HopParams hp{};
  hp.nn_fixed = -1;
  hp.outside = nullptr;
  hp.mark_seeds = 0;
  hp.prefix_src = nullptr;
  hp.table = static_cast<uint32_t*>(rank_table);
  hp.table_len = rank_table_len;
  hp.state = state;
  hp.nodes = nodes;
  hp.nodes_cap = L.caps[num_hops];
  hp.flags = reinterpret_cast<uint64_t*>(ws + L.flags_off);
  hp.tile_cnt = reinterpret_cast<uint32_t*>(ws + L.tile_off);
  hp.displaced = reinterpret_cast<uint8_t*>(ws + L.displaced_off);
  hp.seeds = seeds;
  hp.ns_cap = batch;
  hp.ns_dev = nullptr;

  // First-hop seeds bid for their nodes: inside the sampling kernel when it does
  // the marking, else in a pass of their own.
  if (!(hop_fanouts[0] <= kWave && tuning_fuse_mark() != 0)) {
    const int64_t work = std::max<int64_t>(batch, num_hops + 2);
    hipLaunchKernelGGL(mb_mark_seeds_kernel, dim3(static_cast<unsigned>(ceil_div(work, kMbBlock))),
                       dim3(kMbBlock), 0, st, hp, sizes, num_hops + 2);
    APT_LAUNCH_CHECK("mb_mark_seeds_kernel");
  }
  auto grid_for = [](int64_t n, int64_t per_block, int64_t cap) {
    return dim3(static_cast<unsigned>(std::max<int64_t>(1, std::min<int64_t>(ceil_div(n, per_block), cap))));
  };
  for (int h = 0; h < num_hops; ++h) {
    const int64_t ns_cap = L.caps[h];
    const int64_t f = hop_fanouts[h];
    const int64_t nn_cap = ns_cap * f;
    const int64_t* frontier = h == 0 ? seeds : nodes;
    const int64_t* ns_dev = h == 0 ? nullptr : sizes + h;
    // The sampling kernel looks every id up in the rank table as soon as it has
    // loaded it (fanouts up to one wavefront); otherwise a separate pass does.
    const bool fuse = f <= kWave && tuning_fuse_mark() != 0;
    SampleMark mark{RankTable{static_cast<uint32_t*>(rank_table), rank_table_len, state, hp.displaced},
                    relabeled[h], h == 0 ? 1 : 0};
    int rc = sample_launch(graph, frontier, ns_cap, ns_dev, static_cast<int>(f), replace, rng_seed,
                           rng_seed_dev, h, neighbors[h], counts != nullptr ? counts[h] : nullptr,
                           total, st, "apt_minibatch_sample", fuse ? &mark : nullptr);
    if (rc != APT_OK) return rc;
    hp.ns_cap = ns_cap;
    hp.ns_dev = ns_dev;
    hp.fanout = f;
    hp.neighbors = neighbors[h];
    hp.relabeled = relabeled[h];
    hp.n_next = sizes + h + 1;
    hp.last = (h == num_hops - 1 && h > 0) ? 1 : 0;
    const int64_t items_cap = h == 0 ? ns_cap + nn_cap : nn_cap;
    const dim3 tiles = grid_for(items_cap, kMbTile, int64_t{1} << 30);
    const dim3 flat = grid_for(nn_cap, kMbBlock, 1 << 16);
    if (h == 0) {
      if (!fuse) {
        hipLaunchKernelGGL(mb_mark_neighbors_kernel<true>, flat, dim3(kMbBlock), 0, st, hp);
        APT_LAUNCH_CHECK("mb_mark_neighbors_kernel");
      }
      hipLaunchKernelGGL(mb_count_kernel<true>, tiles, dim3(kMbBlock), 0, st, hp);
      APT_LAUNCH_CHECK("mb_count_kernel");
      hipLaunchKernelGGL(mb_place_kernel<true>, tiles, dim3(kMbBlock), 0, st, hp);
      APT_LAUNCH_CHECK("mb_place_kernel");
    } else {
      if (!fuse) {
        hipLaunchKernelGGL(mb_mark_neighbors_kernel<false>, flat, dim3(kMbBlock), 0, st, hp);
        APT_LAUNCH_CHECK("mb_mark_neighbors_kernel");
      }
      hipLaunchKernelGGL(mb_count_kernel<false>, tiles, dim3(kMbBlock), 0, st, hp);
      APT_LAUNCH_CHECK("mb_count_kernel");
      hipLaunchKernelGGL(mb_place_kernel<false>, tiles, dim3(kMbBlock), 0, st, hp);
      APT_LAUNCH_CHECK("mb_place_kernel");
    }
  }
  LookupParams lp{};
  lp.num_hops = num_hops;
  lp.table = static_cast<const uint32_t*>(rank_table);
  lp.state = state;
  lp.last_is_bid = num_hops > 1 ? 1 : 0;
  int64_t nblocks = 0;
  for (int h = 0; h < num_hops; ++h) {
    lp.block_begin[h] = nblocks;
    lp.neighbors[h] = neighbors[h];
    lp.relabeled[h] = relabeled[h];
    lp.ns_dev[h] = h == 0 ? nullptr : sizes + h;
    lp.ns_cap[h] = L.caps[h];
    lp.fanout[h] = hop_fanouts[h];
    nblocks += std::max<int64_t>(1, std::min<int64_t>(ceil_div(L.caps[h] * hop_fanouts[h], kMbBlock), 2048));
  }
  lp.block_begin[num_hops] = nblocks;
  if (defer != nullptr) {  // the caller runs the pass: with the gather, or through apt_minibatch_lookup
    defer->blocks = static_cast<uint32_t>(nblocks);
    defer->lp = lp;
    return APT_OK;
  }
  hipLaunchKernelGGL(mb_lookup_kernel, dim3(static_cast<unsigned>(nblocks)), dim3(kLookupBlock), 0, st, lp);
  APT_LAUNCH_CHECK("mb_lookup_kernel");
  return APT_OK;
}
}  // namespace apt



extern "C" int apt_minibatch_sample(const apt_graph* graph, const int64_t* seeds, int64_t batch,
                                    const int* hop_fanouts, int num_hops, int replace,
                                    uint64_t rng_seed, const uint64_t* rng_seed_dev,
                                    void* rank_table, int64_t rank_table_len, int64_t* nodes,
                                    int64_t* const* neighbors, int64_t* const* relabeled,
                                    int64_t* const* counts, int64_t* sizes, void* workspace,
                                    size_t workspace_bytes, void* stream) {
  return apt::minibatch_sample(graph, seeds, batch, hop_fanouts, num_hops, replace, rng_seed, rng_seed_dev,
                               rank_table, rank_table_len, nodes, neighbors, relabeled, counts, sizes,
                               workspace, workspace_bytes, stream, nullptr);
}

extern "C" int apt_minibatch_sample_deferred(const apt_graph* graph, const int64_t* seeds, int64_t batch,
                                             const int* hop_fanouts, int num_hops, int replace,
                                             uint64_t rng_seed, const uint64_t* rng_seed_dev,
                                             void* rank_table, int64_t rank_table_len, int64_t* nodes,
                                             int64_t* const* neighbors, int64_t* const* relabeled,
                                             int64_t* const* counts, int64_t* sizes, void* workspace,
                                             size_t workspace_bytes, void* stream,
                                             apt_pending_lookup* pending) {
  APT_REQUIRE(pending != nullptr, APT_EINVAL, "apt_minibatch_sample_deferred: pending is NULL");
  return apt::minibatch_sample(graph, seeds, batch, hop_fanouts, num_hops, replace, rng_seed, rng_seed_dev,
                               rank_table, rank_table_len, nodes, neighbors, relabeled, counts, sizes,
                               workspace, workspace_bytes, stream,
                               reinterpret_cast<apt::PendingLookup*>(pending));
}

extern "C" int apt_minibatch_lookup(const apt_pending_lookup* pending, void* stream) {
  using namespace apt;
  const PendingLookup* q = reinterpret_cast<const PendingLookup*>(pending);
  APT_REQUIRE(q != nullptr && q->magic == kPendingMagic, APT_EINVAL,
              "apt_minibatch_lookup: pending was not filled by apt_minibatch_sample_deferred");
  if (q->blocks == 0) return APT_OK;
  hipLaunchKernelGGL(mb_lookup_kernel, dim3(q->blocks), dim3(kLookupBlock), 0, static_cast<hipStream_t>(stream),
                     q->lp);
  APT_LAUNCH_CHECK("mb_lookup_kernel");
  return APT_OK;
}

// ---------------------------------------------------------------------------
// apt_relabel_ranked: apt_relabel's result through a node-indexed rank table
// instead of a hash table, for ids that index a registered graph.  It is one hop
// of the driver above called on its own (reference python/npc/sampler.py:187-203
// calls relabel_csc once per hop, src/relabel.cc:9-15):
//   a fresh call     seeds and neighbours bid with their positions (the first-hop
//                    path: ownership is read back from the table);
//   a continued call the seeds are exactly the unique list the previous call
//                    returned, so the table still holds their ids: a neighbour
//                    already in the batch costs one load, the others bid with an
//                    atomicMin that settles ownership (the later-hop path).
namespace apt {
constexpr uint32_t kRankedPayloadBits = 24;  // fixed, so that calls of any size share a table without refills
constexpr int64_t kRankedMaxItems = (int64_t{1} << kRankedPayloadBits) - 2;

struct RankedLayout {
  size_t flags_off, tile_off, displaced_off, total;
};
static RankedLayout ranked_layout(int64_t items) {
  RankedLayout L;
  const int64_t tiles = ceil_div(std::max<int64_t>(items, 1), kMbTile);
  size_t off = 0;
  L.flags_off = off; off = mb_align(off + sizeof(uint64_t) * tiles * kMbIters * kMbWaves);
  L.tile_off = off;  off = mb_align(off + sizeof(uint32_t) * tiles);
  L.displaced_off = off; off = mb_align(off + static_cast<size_t>(std::max<int64_t>(items, 1)));
  L.total = off;
  return L;
}
}  // namespace apt

extern "C" int64_t apt_relabel_ranked_max_items(void) { return apt::kRankedMaxItems; }

extern "C" size_t apt_relabel_ranked_workspace_bytes(int64_t num_items) {
  if (num_items < 0 || num_items > apt::kRankedMaxItems) return 0;
  return apt::ranked_layout(num_items).total;
}

// apt_sample_neighbors with the bids of the apt_relabel_ranked call that follows placed on the way: the
// sampling kernel has every id in registers when it loads it, and a bid placed there overlaps with the kernel's
// own random reads instead of being a pass of its own over the ids.
extern "C" int apt_sample_neighbors_bidding(const apt_graph* graph, const int64_t* frontier, int64_t num_frontier,
                                            const int64_t* num_frontier_dev, int fanout, int replace,
                                            uint64_t rng_seed, int hop, int64_t* out_neighbors, int64_t* out_counts,
                                            int64_t* out_total, int continued, void* rank_table,
                                            int64_t rank_table_len, int64_t* slot_states, int64_t* num_outside_dev,
                                            void* workspace, size_t workspace_bytes, void* stream) {
  using namespace apt;
  APT_REQUIRE(fanout >= 1 && fanout <= kWave, APT_ELIMIT, "apt_sample_neighbors_bidding: fanout %d outside [1, %d]",
              fanout, kWave);
  APT_REQUIRE(num_frontier >= 0 && slot_states != nullptr, APT_EINVAL,
              "apt_sample_neighbors_bidding: negative size or slot_states is NULL");
  const int64_t items = num_frontier + num_frontier * fanout;
  APT_REQUIRE(items <= kRankedMaxItems, APT_ELIMIT,
              "apt_sample_neighbors_bidding: %lld items exceed the supported maximum %lld", (long long)items,
              (long long)kRankedMaxItems);
  APT_REQUIRE(rank_table != nullptr && rank_table_len > 0 && rank_table_len < (int64_t{1} << 32) - 1 &&
                  (reinterpret_cast<uintptr_t>(rank_table) & 255) == 0,
              APT_EINVAL, "apt_sample_neighbors_bidding: rank table missing, misaligned or too long");
  APT_REQUIRE(workspace != nullptr && workspace_bytes >= ranked_layout(items).total &&
                  (reinterpret_cast<uintptr_t>(workspace) & 15) == 0,
              APT_EWORKSPACE, "apt_sample_neighbors_bidding: workspace of %zu bytes, %zu needed (16-byte aligned)",
              workspace_bytes, ranked_layout(items).total);
  // the same layout as the apt_relabel_ranked call that will read the flags set here
  int64_t lo = items, hi = kRankedMaxItems;
  while (lo < hi) {
    const int64_t mid = lo + (hi - lo + 1) / 2;
    if (ranked_layout(mid).total <= workspace_bytes) lo = mid;
    else hi = mid - 1;
  }
  const RankedLayout L = ranked_layout(lo);
  hipStream_t st = static_cast<hipStream_t>(stream);
  uint32_t* state = reinterpret_cast<uint32_t*>(static_cast<char*>(rank_table) + table_state_offset(rank_table_len));
  if (continued == 0) {
    const int64_t vecs = static_cast<int64_t>(table_state_offset(rank_table_len) / 16);
    hipLaunchKernelGGL(mb_begin_kernel, dim3(kBeginBlocks), dim3(kMbBlock), 0, st, static_cast<uint4*>(rank_table), vecs,
                       state, kRankedPayloadBits, static_cast<int64_t*>(nullptr), 0, int64_t{0});
    APT_LAUNCH_CHECK("mb_begin_kernel");
  }
  SampleMark mark{RankTable{static_cast<uint32_t*>(rank_table), rank_table_len, state,
                            reinterpret_cast<uint8_t*>(static_cast<char*>(workspace) + L.displaced_off)},
                  slot_states, continued == 0 ? 1 : 0, num_outside_dev};
  return sample_launch(graph, frontier, num_frontier, num_frontier_dev, fanout, replace, rng_seed, nullptr, hop,
                       out_neighbors, out_counts, out_total, st, "apt_sample_neighbors_bidding", &mark);
}

extern "C" int apt_relabel_ranked(const int64_t* seeds, int64_t num_seeds, const int64_t* num_seeds_dev,
                                  const int64_t* neighbors, int64_t num_neighbors, int64_t neighbor_stride,
                                  int continued, void* rank_table, int64_t rank_table_len,
                                  int64_t* unique, int64_t* relabeled, int64_t* num_unique_dev, int64_t* num_outside_dev,
                                  int64_t* counts_host, void* workspace, size_t workspace_bytes, void* stream) {
  using namespace apt;
  APT_REQUIRE(num_seeds >= 0 && num_neighbors >= 0, APT_EINVAL, "apt_relabel_ranked: negative size");
  APT_REQUIRE(num_seeds_dev == nullptr || (neighbor_stride > 0 && num_seeds <= num_neighbors / neighbor_stride),
              APT_EINVAL, "apt_relabel_ranked: with num_seeds_dev, neighbors must hold num_seeds * neighbor_stride entries");
  const int64_t items = num_seeds + num_neighbors;
  APT_REQUIRE(items <= kRankedMaxItems, APT_ELIMIT, "apt_relabel_ranked: %lld items exceed the supported maximum %lld",
              (long long)items, (long long)kRankedMaxItems);
  APT_REQUIRE(rank_table != nullptr && rank_table_len > 0 && rank_table_len < (int64_t{1} << 32) - 1 &&
                  (reinterpret_cast<uintptr_t>(rank_table) & 255) == 0,
              APT_EINVAL, "apt_relabel_ranked: rank table missing, misaligned or too long");
  APT_REQUIRE(num_unique_dev != nullptr && num_outside_dev != nullptr, APT_EINVAL,
              "apt_relabel_ranked: num_unique_dev / num_outside_dev is NULL");
  APT_REQUIRE((num_seeds == 0 || seeds != nullptr) && (num_neighbors == 0 || (neighbors != nullptr && relabeled != nullptr)) &&
                  (items == 0 || unique != nullptr),
              APT_EINVAL, "apt_relabel_ranked: seeds / neighbors / unique / relabeled is NULL");
  APT_REQUIRE(workspace != nullptr && workspace_bytes >= ranked_layout(items).total &&
                  (reinterpret_cast<uintptr_t>(workspace) & 15) == 0,
              APT_EWORKSPACE, "apt_relabel_ranked: workspace of %zu bytes, %zu needed (16-byte aligned)", workspace_bytes,
              ranked_layout(items).total);
  // The parts of the workspace are laid out for the largest call it can hold, not for this call: the per-slot
  // flags must be all zero when a call starts (each call clears the ones it sets), so they must not share
  // their bytes with another call's tile counts.
  int64_t lo = items, hi = kRankedMaxItems;
  while (lo < hi) {
    const int64_t mid = lo + (hi - lo + 1) / 2;
    if (ranked_layout(mid).total <= workspace_bytes) lo = mid;
    else hi = mid - 1;
  }
  const RankedLayout L = ranked_layout(lo);
  hipStream_t st = static_cast<hipStream_t>(stream);
  char* ws = static_cast<char*>(workspace);
  uint32_t* state = reinterpret_cast<uint32_t*>(static_cast<char*>(rank_table) + table_state_offset(rank_table_len));
  auto grid_for = [](int64_t n, int64_t per_block, int64_t cap) {
    return dim3(static_cast<unsigned>(std::max<int64_t>(1, std::min<int64_t>(ceil_div(n, per_block), cap))));
  };
  HopParams hp{};
  hp.table = static_cast<uint32_t*>(rank_table);
  hp.table_len = rank_table_len;
  hp.state = state;
  hp.nodes = unique;
  hp.nodes_cap = items;
  hp.flags = reinterpret_cast<uint64_t*>(ws + L.flags_off);
  hp.tile_cnt = reinterpret_cast<uint32_t*>(ws + L.tile_off);
  hp.displaced = reinterpret_cast<uint8_t*>(ws + L.displaced_off);
  hp.seeds = seeds;
  hp.ns_cap = num_seeds;
  hp.ns_dev = num_seeds_dev;
  hp.fanout = num_seeds_dev != nullptr ? neighbor_stride : 1;
  hp.nn_fixed = num_seeds_dev != nullptr ? -1 : num_neighbors;   // device-side count: rows x stride slots
  hp.neighbors = neighbors;
  hp.relabeled = relabeled;
  hp.n_next = num_unique_dev;
  hp.outside = num_outside_dev;
  hp.last = 0;
  hp.mark_seeds = 1;
  hp.prefix_src = nullptr;
  const dim3 mark_grid = grid_for(std::max(num_neighbors, num_seeds), kMbBlock, 1 << 16);
  const bool marked = (continued & 2) != 0;   // apt_sample_neighbors_bidding has placed this call's bids
  continued &= 1;
  if (marked) {
    APT_REQUIRE(num_neighbors > 0, APT_EINVAL, "apt_relabel_ranked: a call whose bids are placed needs neighbours");
    const dim3 tiles = grid_for(continued ? num_neighbors : items, kMbTile, int64_t{1} << 30);
    if (continued != 0) {
      if (unique != seeds)
        APT_HIP(hipMemcpyAsync(unique, seeds, sizeof(int64_t) * static_cast<size_t>(num_seeds), hipMemcpyDeviceToDevice, st));
      hipLaunchKernelGGL(mb_count_kernel<false>, tiles, dim3(kMbBlock), 0, st, hp);
      APT_LAUNCH_CHECK("mb_count_kernel");
      hipLaunchKernelGGL(mb_place_kernel<false>, tiles, dim3(kMbBlock), 0, st, hp);
      APT_LAUNCH_CHECK("mb_place_kernel");
    } else {
      hipLaunchKernelGGL(mb_count_kernel<true>, tiles, dim3(kMbBlock), 0, st, hp);
      APT_LAUNCH_CHECK("mb_count_kernel");
      hipLaunchKernelGGL(mb_place_kernel<true>, tiles, dim3(kMbBlock), 0, st, hp);
      APT_LAUNCH_CHECK("mb_place_kernel");
    }
  } else if (continued == 0) {
    // a new batch of the table: next epoch (refill when they have run out); *num_unique_dev = num_seeds for now
    const int64_t vecs = static_cast<int64_t>(table_state_offset(rank_table_len) / 16);
    hipLaunchKernelGGL(mb_begin_kernel, dim3(kBeginBlocks), dim3(kMbBlock), 0, st, static_cast<uint4*>(rank_table), vecs,
                       state, kRankedPayloadBits, num_unique_dev, 1, num_seeds);
    APT_LAUNCH_CHECK("mb_begin_kernel");
    if (items > 0) {
      hipLaunchKernelGGL(mb_mark_neighbors_kernel<true>, mark_grid, dim3(kMbBlock), 0, st, hp);
      APT_LAUNCH_CHECK("mb_mark_neighbors_kernel");
      const dim3 tiles = grid_for(items, kMbTile, int64_t{1} << 30);
      hipLaunchKernelGGL(mb_count_kernel<true>, tiles, dim3(kMbBlock), 0, st, hp);
      APT_LAUNCH_CHECK("mb_count_kernel");
      hipLaunchKernelGGL(mb_place_kernel<true>, tiles, dim3(kMbBlock), 0, st, hp);
      APT_LAUNCH_CHECK("mb_place_kernel");
    }
  } else {
    // the seeds hold ids 0 .. num_seeds - 1 in the table's current epoch (the caller vouches for it); the marking
    // pass also copies them to the head of the unique list
    hp.prefix_src = unique != seeds ? seeds : nullptr;
    hipLaunchKernelGGL(mb_mark_neighbors_kernel<false>, mark_grid, dim3(kMbBlock), 0, st, hp);
    APT_LAUNCH_CHECK("mb_mark_neighbors_kernel");
    const dim3 tiles = grid_for(num_neighbors, kMbTile, int64_t{1} << 30);
    hipLaunchKernelGGL(mb_count_kernel<false>, tiles, dim3(kMbBlock), 0, st, hp);
    APT_LAUNCH_CHECK("mb_count_kernel");
    hipLaunchKernelGGL(mb_place_kernel<false>, tiles, dim3(kMbBlock), 0, st, hp);
    APT_LAUNCH_CHECK("mb_place_kernel");
  }
  if (num_neighbors > 0) {
    LookupParams lp{};
    lp.num_hops = 1;
    lp.table = static_cast<const uint32_t*>(rank_table);
    lp.state = state;
    lp.last_is_bid = 0;
    lp.block_begin[0] = 0;
    lp.neighbors[0] = neighbors;
    lp.relabeled[0] = relabeled;
    // the pass only needs the number of slots: rows x stride, or num_neighbors x 1
    lp.ns_dev[0] = num_seeds_dev;
    lp.ns_cap[0] = num_seeds_dev != nullptr ? num_seeds : num_neighbors;
    lp.fanout[0] = num_seeds_dev != nullptr ? neighbor_stride : 1;
    const int64_t nblocks = std::max<int64_t>(1, std::min<int64_t>(ceil_div(num_neighbors, kMbBlock), 2048));
    lp.block_begin[1] = nblocks;
    hipLaunchKernelGGL(mb_lookup_kernel, dim3(static_cast<unsigned>(nblocks)), dim3(kLookupBlock), 0, st, lp);
    APT_LAUNCH_CHECK("mb_lookup_kernel");
  }
  if (counts_host != nullptr) {
    if (num_outside_dev == num_unique_dev + 1) {  // neighbours in memory: one copy
      APT_HIP(hipMemcpyAsync(counts_host, num_unique_dev, 2 * sizeof(int64_t), hipMemcpyDeviceToHost, st));
    } else {
      APT_HIP(hipMemcpyAsync(counts_host, num_unique_dev, sizeof(int64_t), hipMemcpyDeviceToHost, st));
      APT_HIP(hipMemcpyAsync(counts_host + 1, num_outside_dev, sizeof(int64_t), hipMemcpyDeviceToHost, st));
    }
    APT_HIP(hipStreamSynchronize(st));
  }
  return APT_OK;
}
