// libnpc.so: the `npc` operator library for PyTorch-ROCm.
//
// Registers the hot-path operators under the names and C++ signatures the
// reference binds with TORCH_LIBRARY(npc, m) in src/pybind.cc:18-48, so that
// torch.ops.npc.<name>(...) keeps working.  Every operator is a thin host
// wrapper: it checks its tensors, allocates outputs with torch, and calls the
// C ABI of libapt_hip.so (include/apt_amd.h) on the current HIP stream.
// Operators whose reference implementation exchanges data with other GPUs
// over NCCL are registered too, and raise.
#include <ATen/hip/HIPEvent.h>
#include <c10/hip/HIPStream.h>
#include <torch/library.h>
#include <torch/torch.h>

#include <deque>
#include <memory>
#include <string>
#include <tuple>
#include <vector>

#include "../../include/apt_amd.h"

namespace npc {

using torch::Tensor;
using IdType = int64_t;  // reference src/utils.h:14

namespace {

struct State {  // counterpart of NPCState, reference src/state.h:32-63
  int64_t rank = 0, local_rank = 0, world_size = 1, node_size = 1;
  // graph (reference GraphStorage, state.h:18-23)
  bool has_graph = false;
  Tensor indptr, indices, cached_indptr, cached_indices, adj_pos_map;
  apt_graph graph{};
  // features (reference FeatStorage, state.h:10-16)
  bool has_feat = false;
  Tensor local_feats, cache_feats, feat_pos_map, cpu_feat_pos_map;
  bool identity_map = false;
  apt_feat_store feat{};
  // bucketing
  Tensor shuffle_min_vids, remote_worker_map;
  int64_t shuffle_id_offset = 0, num_remote_workers = 0;
  // sampling
  uint64_t rng_seed = 7777777;  // reference src/cuda/npc_kernel.cu:292
  int64_t sample_calls = 0;
  // How load_subtensor reports requested nodes that have no row here (the reference reads out of bounds):
  //   0 not at all (rows are zero-filled), 1 deferred (default): the miss counter travels to pinned host memory
  //   behind the gather and is looked at by the next operator call or by check_errors(), so no call waits for
  //   the GPU; 2 immediate: the call waits for its own counter and raises itself.
  int miss_check = 1;
  bool strict = true;   // feat_shuffle's pack checks permutations it did not produce itself
  struct PendingCheck {
    Tensor dev, host;
    std::shared_ptr<at::cuda::CUDAEvent> done;
  };
  std::deque<PendingCheck> pending_checks;
  // permutations handed out by shuffle_seeds / cluster_and_permute (kept alive, with their versions): bijections
  // by construction, which feat_shuffle's pack need not check
  std::deque<std::pair<Tensor, uint32_t>> own_permutations;
  // relabel_csc on a registered graph: a rank table of its own, a workspace that grows with the largest call, and
  // the unique list the last call returned (kept alive so that its address cannot be reused) with its version
  Tensor ranked_table, ranked_ws, ranked_counts, ranked_last;
  uint32_t ranked_last_version = 0;
  bool ranked_enabled = true;
  // A sampling operator call that has placed the bids of the relabel_csc call the reference's sampler makes
  // next (apt_sample_neighbors_bidding): its seeds and sampled ids (kept alive, with their versions) and the slot
  // states that call will take over.  A relabel_csc with other tensors finds abandoned bids in the table and
  // starts a fresh batch.
  struct RankedPending {
    bool valid = false, continued = false;
    Tensor seeds, neighbors, states;
    uint32_t seeds_version = 0, neighbors_version = 0;
  } ranked_pending;
  // pinned host words that the relabel operators read their counts into (a copy to pageable memory is staged)
  Tensor pinned_counts;
  // fused multi-hop driver: rank table of the registered graph, workspace of the last plan
  Tensor rank_table, mb_workspace;
  int64_t mb_batch = -1;
  std::vector<int64_t> mb_fanouts;
  // sample_blocks' output buffers (upper-bound sized).  Ring 0 (the default) = fresh tensors on every call,
  // as the reference's operators return them; set_block_buffer_ring(n) hands out n registry-owned sets in
  // turn instead: what call k returned is then overwritten by call k + n
  struct BlockBuffers {
    Tensor nodes, sizes, format_ws;
    std::vector<Tensor> nb, rl, ct, row, col, csc;
    bool formats = false;
  };
  std::vector<BlockBuffers> mb_ring;
  int64_t mb_ring_size = 0, mb_ring_pos = 0;
};

State& S() {
  // the C library found at run time must be the one this file's header describes
  static const bool abi_ok = [] {
    TORCH_CHECK(apt_abi_version() == APT_ABI_VERSION, "npc: libapt_hip.so has ABI version ", apt_abi_version(),
                ", libnpc.so was built against ", APT_ABI_VERSION);
    return true;
  }();
  (void)abi_ok;
  static State s;
  return s;
}

void check(int status) {
  TORCH_CHECK(status == APT_OK, "npc: ", apt_last_error(), " (status ", status, ")");
}

void* stream() { return static_cast<void*>(c10::hip::getCurrentHIPStream().stream()); }

c10::Device device() {
  TORCH_CHECK(torch::cuda::is_available(), "npc: no GPU; the operators have no CPU implementation");
  return c10::Device(c10::kCUDA, c10::hip::current_device());
}

Tensor ids_on_device(const Tensor& t, const char* name) {
  TORCH_CHECK(t.scalar_type() == torch::kInt64, "npc: ", name, " must be int64");
  TORCH_CHECK(t.dim() == 1, "npc: ", name, " must be 1-D");
  return t.to(device()).contiguous();
}

const int64_t* i64(const Tensor& t) { return t.defined() && t.numel() ? t.data_ptr<int64_t>() : nullptr; }

torch::TensorOptions i64_opts() { return torch::TensorOptions().dtype(torch::kInt64).device(device()); }

int64_t* pinned_counts() {
  auto& s = S();
  if (!s.pinned_counts.defined())
    s.pinned_counts = torch::zeros({4}, torch::TensorOptions().dtype(torch::kInt64).pinned_memory(true));
  return s.pinned_counts.data_ptr<int64_t>();
}

}  // namespace

// ---------------------------------------------------------------- registries
void SetTopology(IdType rank, IdType world_size, IdType node_size) {
  TORCH_CHECK(world_size >= 1 && world_size <= APT_MAX_BUCKETS && rank >= 0 && rank < world_size &&
                  node_size >= 1,
              "npc: bad topology");
  S().rank = rank;
  S().world_size = world_size;
  S().node_size = node_size;
  S().local_rank = rank % node_size;
}

void SetRngSeed(IdType seed) {
  S().rng_seed = static_cast<uint64_t>(seed);
  S().sample_calls = 0;
}

// Looks at the miss counters of earlier load_subtensor calls that have arrived (wait: all of them) and raises for
// the first that is not zero.
void PollChecks(bool wait) {
  auto& q = S().pending_checks;
  while (!q.empty()) {
    auto& p = q.front();
    if (wait) p.done->synchronize();
    else if (!p.done->query()) break;
    const int64_t m = p.host.data_ptr<int64_t>()[0];
    q.pop_front();
    TORCH_CHECK_INDEX(m == 0, "npc: load_subtensor (an earlier call): ", m,
                      " requested node(s) have no feature row on this GPU; their rows were zero-filled");
  }
}

void CheckErrors() { PollChecks(true); }

void SetStrict(bool strict) {
  S().strict = strict;
  S().miss_check = strict ? 1 : 0;
}

void SetMissCheck(std::string mode) {
  TORCH_CHECK(mode == "off" || mode == "deferred" || mode == "immediate",
              "npc: set_miss_check: 'off', 'deferred' or 'immediate'");
  PollChecks(true);
  S().miss_check = mode == "off" ? 0 : mode == "deferred" ? 1 : 2;
}

// relabel_csc goes through the registered graph's rank table where it can (default) or always through the
// hash table (false).
static void drop_pending_bids();
void SetRankedRelabel(bool enabled) {
  S().ranked_enabled = enabled;
  S().ranked_last = Tensor();
  drop_pending_bids();
}

// How many registry-owned sets of output buffers sample_blocks hands out in turn.  0 (the default) = fresh
// tensors on every call.  With n > 0 a call costs less (no allocation), but what call k returned is
// overwritten by call k + n whatever stream or consumer still holds it.
IdType BlockBufferRing() { return S().mb_ring_size; }

void SetBlockBufferRing(IdType sets) {
  TORCH_CHECK(sets >= 0 && sets <= 64, "npc: set_block_buffer_ring: 0..64 sets");
  S().mb_ring_size = sets;
  S().mb_ring.clear();
  S().mb_ring_pos = 0;
}

// reference src/cache_feats.cc:14-61
void CacheFeatsShared(IdType num_total_nodes, Tensor localnode_feats, Tensor cached_feats,
                      Tensor cached_idx, Tensor localnode_idx, IdType feat_dim_offset) {
  auto& s = S();
  TORCH_CHECK(localnode_feats.dim() == 2, "npc: localnode_feats must be [num_local, feat_dim]");
  TORCH_CHECK(localnode_feats.element_size() == 2 || localnode_feats.element_size() == 4,
              "npc: features must have 2- or 4-byte elements");
  const int64_t n_local = localnode_feats.size(0), feat_dim = localnode_feats.size(1);
  const int64_t n_cached = cached_feats.dim() == 2 ? cached_feats.size(0) : 0;
  auto local_idx = ids_on_device(localnode_idx, "localnode_idx");
  auto cache_idx = ids_on_device(cached_idx, "cached_idx");
  TORCH_CHECK(local_idx.numel() == n_local, "npc: localnode_idx must name every local row");
  TORCH_CHECK(cache_idx.numel() == n_cached, "npc: cached_idx must name every cached row");
  if (n_local)
    TORCH_CHECK(local_idx.min().item<int64_t>() >= 0 && local_idx.max().item<int64_t>() < num_total_nodes,
                "npc: localnode_idx out of range");
  if (n_cached)
    TORCH_CHECK(cache_idx.min().item<int64_t>() >= 0 && cache_idx.max().item<int64_t>() < num_total_nodes,
                "npc: cached_idx out of range");
  const int64_t rank_dim = n_cached ? cached_feats.size(1) : feat_dim - feat_dim_offset;
  TORCH_CHECK(feat_dim_offset >= 0 && feat_dim_offset + rank_dim <= feat_dim,
              "npc: feat_dim_offset + cached width exceeds the local feature width");
  s.local_feats = localnode_feats.to(device()).contiguous();
  auto pos = torch::full({num_total_nodes}, -1, i64_opts());  // FEAT_NOT_EXIST, src/utils.h:20
  pos.index_put_({local_idx}, -torch::arange(n_local, i64_opts()) - 2);  // ENCODE_ID, src/utils.h:17
  s.cpu_feat_pos_map = pos.cpu();  // without cache entries, src/cache_feats.cc:52
  s.cache_feats = Tensor();
  if (n_cached) {
    TORCH_CHECK(cached_feats.scalar_type() == localnode_feats.scalar_type(),
                "npc: cached_feats dtype differs from localnode_feats");
    s.cache_feats = cached_feats.to(device()).contiguous();
    pos.index_put_({cache_idx}, torch::arange(n_cached, i64_opts()));  // the cache wins, :53-55
  }
  s.feat_pos_map = pos;
  s.identity_map = n_cached == 0 && n_local == num_total_nodes &&
                   torch::equal(local_idx, torch::arange(n_local, i64_opts()));
  s.feat.local_table = s.local_feats.data_ptr();
  s.feat.num_local_rows = n_local;
  s.feat.local_dim = feat_dim;
  s.feat.cache_table = n_cached ? s.cache_feats.data_ptr() : nullptr;
  s.feat.num_cache_rows = n_cached;
  s.feat.pos_map = s.identity_map ? nullptr : pos.data_ptr<int64_t>();
  s.feat.num_total_nodes = num_total_nodes;
  s.feat.col_offset = feat_dim_offset;
  s.feat.out_dim = rank_dim;
  s.feat.elem_size = static_cast<int>(localnode_feats.element_size());
  s.has_feat = true;
}

// reference src/cache_graphs.cc:12-49
void MixCacheGraphs(IdType num_cached_nodes, Tensor cached_node_idx, Tensor cached_indptr,
                    Tensor cached_indices, Tensor global_indptr, Tensor global_indices) {
  auto& s = S();
  TORCH_CHECK(num_cached_nodes == cached_node_idx.numel(),
              "npc: num_cached_nodes != cached_node_idx.numel()");  // reference CHECK :19
  s.indptr = ids_on_device(global_indptr, "global_indptr");
  s.indices = ids_on_device(global_indices, "global_indices");
  const int64_t total = s.indptr.numel() - 1;
  TORCH_CHECK(total >= 0, "npc: global_indptr is empty");
  s.graph = apt_graph{};
  s.graph.indptr = s.indptr.data_ptr<int64_t>();
  s.graph.indices = i64(s.indices);
  s.graph.row_begin = 0;
  s.graph.num_rows = total;
  s.graph.num_total_nodes = total;
  s.rank_table = Tensor();
  s.ranked_table = Tensor();
  s.ranked_ws = Tensor();
  s.ranked_last = Tensor();
  s.ranked_pending = {};
  s.adj_pos_map = Tensor();
  if (num_cached_nodes > 0) {
    auto idx = ids_on_device(cached_node_idx, "cached_node_idx");
    s.cached_indptr = ids_on_device(cached_indptr, "cached_indptr");
    s.cached_indices = ids_on_device(cached_indices, "cached_indices");
    TORCH_CHECK(s.cached_indptr.numel() == num_cached_nodes + 1,
                "npc: cached_indptr must have num_cached_nodes + 1 entries");
    TORCH_CHECK(idx.min().item<int64_t>() >= 0 && idx.max().item<int64_t>() < total,
                "npc: cached_node_idx out of range");
    s.adj_pos_map = -torch::arange(total, i64_opts()) - 2;  // ENCODE_ID(v), :37-40
    s.adj_pos_map.index_put_({idx}, torch::arange(num_cached_nodes, i64_opts()));
    s.graph.cached_indptr = s.cached_indptr.data_ptr<int64_t>();
    s.graph.cached_indices = i64(s.cached_indices);
    s.graph.num_cached_rows = num_cached_nodes;
    s.graph.adj_pos_map = s.adj_pos_map.data_ptr<int64_t>();
  }
  s.has_graph = true;
}

// A contiguous-range partition: nodes outside [row_begin, row_begin + rows)
// have no adjacency.  No counterpart in the reference.
void RegisterGraphPartition(Tensor indptr, Tensor indices, IdType row_begin, IdType num_total_nodes) {
  auto& s = S();
  s.indptr = ids_on_device(indptr, "indptr");
  s.indices = ids_on_device(indices, "indices");
  TORCH_CHECK(s.indptr.numel() >= 1, "npc: indptr is empty");
  s.adj_pos_map = Tensor();
  s.graph = apt_graph{};
  s.graph.indptr = s.indptr.data_ptr<int64_t>();
  s.graph.indices = i64(s.indices);
  s.graph.row_begin = row_begin;
  s.graph.num_rows = s.indptr.numel() - 1;
  s.graph.num_total_nodes = num_total_nodes;
  s.rank_table = Tensor();
  s.ranked_table = Tensor();
  s.ranked_ws = Tensor();
  s.ranked_last = Tensor();
  s.ranked_pending = {};
  s.has_graph = true;
}

// reference src/core.cc:102-108
void RegisterMinVids(Tensor shuffle_min_vids, IdType shuffle_id_offset) {
  S().shuffle_min_vids = ids_on_device(shuffle_min_vids, "shuffle_min_vids");
  S().shuffle_id_offset = shuffle_id_offset;
}

// reference src/core.cc:110-125 (state only)
void RegisterMultiMachinesScheme(Tensor remote_worker_map, Tensor remote_worker_id) {
  S().remote_worker_map = ids_on_device(remote_worker_map, "remote_worker_map");
  S().num_remote_workers = remote_worker_id.numel();
}

// ---------------------------------------------------------------- hot path
static bool same_tensor(const Tensor& kept, uint32_t version, const Tensor& t) {
  return kept.defined() && kept.data_ptr() == t.data_ptr() && kept.numel() == t.numel() && version == t._version();
}

// Forgets bids that a sampling call placed for a relabel_csc call that did not come.  Those of a call that
// continued a batch have also set per-slot flags in the workspace, which only that relabel_csc would have
// consumed: the workspace is cleared.  (The bids themselves are harmless: the next call on the table starts a new
// batch.)
static void drop_pending_bids() {
  auto& s = S();
  if (s.ranked_pending.valid && s.ranked_pending.continued && s.ranked_ws.defined())
    check(apt_minibatch_workspace_init(s.ranked_ws.data_ptr(), static_cast<size_t>(s.ranked_ws.numel()), stream()));
  if (s.ranked_pending.valid && s.ranked_counts.defined()) s.ranked_counts.zero_();   // seeds it counted as outside
  s.ranked_pending = {};
}

// The rank table of the registered graph for relabel_csc (a table of its own) and a workspace for `items` items.
static bool ranked_resources(int64_t items) {
  auto& s = S();
  auto u8 = torch::TensorOptions().dtype(torch::kUInt8).device(device());
  if (!s.ranked_table.defined()) {
    const size_t bytes = apt_rank_table_bytes(s.graph.num_total_nodes);
    if (bytes == 0) return false;
    s.ranked_table = torch::empty({static_cast<int64_t>(bytes)}, u8);
    check(apt_rank_table_init(s.ranked_table.data_ptr(), bytes, stream()));
    s.ranked_counts = torch::zeros({2}, i64_opts());
    s.ranked_last = Tensor();
    s.ranked_pending = {};
  }
  const size_t need = apt_relabel_ranked_workspace_bytes(items);
  if (need == 0) return false;
  if (!s.ranked_ws.defined() || static_cast<size_t>(s.ranked_ws.numel()) < need) {
    // (a new workspace starts with clean flags; bids placed under the old one are abandoned)
    s.ranked_ws = torch::empty({static_cast<int64_t>(std::max<size_t>(need, 256) * 2)}, u8);
    check(apt_minibatch_workspace_init(s.ranked_ws.data_ptr(), static_cast<size_t>(s.ranked_ws.numel()), stream()));
    s.ranked_last = Tensor();
    s.ranked_pending = {};
  }
  return true;
}

// One hop of sampling.  Where the relabel_csc call that the reference's sampler makes next
// (python/npc/sampler.py:187-203) will go through the rank table, its bids are placed here, by the sampling kernel
// itself, and that call only ranks the owners.
static void sample_hop(const Tensor& f, IdType fanout, bool replace, uint64_t rng_seed, int hop, Tensor& out,
                       int64_t* counts) {
  auto& s = S();
  const int64_t n = f.numel(), items = n + n * fanout;
  if (s.ranked_enabled && fanout <= 64 && items > 8192 && items <= apt_relabel_ranked_max_items() &&
      s.graph.num_total_nodes > 0 && ranked_resources(items)) {
    // the batch continues if these seeds are the unique list the last relabel_csc returned and nothing has bid since
    const bool continued = !s.ranked_pending.valid && same_tensor(s.ranked_last, s.ranked_last_version, f);
    s.ranked_last = Tensor();
    drop_pending_bids();
    auto states = torch::empty({n * fanout}, i64_opts());
    check(apt_sample_neighbors_bidding(&s.graph, i64(f), n, nullptr, static_cast<int>(fanout), replace, rng_seed, hop,
                                       out.data_ptr<int64_t>(), counts, nullptr, continued ? 1 : 0,
                                       s.ranked_table.data_ptr(), s.graph.num_total_nodes, states.data_ptr<int64_t>(),
                                       s.ranked_counts.data_ptr<int64_t>() + 1, s.ranked_ws.data_ptr(),
                                       static_cast<size_t>(s.ranked_ws.numel()), stream()));
    auto& p = s.ranked_pending;
    p.valid = true;
    p.continued = continued;
    p.seeds = f;
    p.neighbors = out;
    p.states = states;
    p.seeds_version = f._version();
    p.neighbors_version = out._version();
    return;
  }
  check(apt_sample_neighbors(&s.graph, i64(f), n, nullptr, static_cast<int>(fanout), replace, rng_seed, hop,
                             out.data_ptr<int64_t>(), counts, nullptr, stream()));
}

std::tuple<Tensor, Tensor> SampleNeighbors(Tensor seeds, IdType fanout, bool replace, IdType rng_seed,
                                           IdType hop) {
  auto& s = S();
  TORCH_CHECK(s.has_graph, "npc: no graph registered (mix_cache_graphs)");
  TORCH_CHECK(fanout > 0, "npc: fanout must be > 0");
  auto f = ids_on_device(seeds, "seeds");
  auto out = torch::empty({f.numel() * fanout}, i64_opts());
  auto cnt = torch::empty({f.numel()}, i64_opts());
  sample_hop(f, fanout, replace, static_cast<uint64_t>(rng_seed), static_cast<int>(hop), out, cnt.data_ptr<int64_t>());
  return {out, cnt};
}

// The whole multi-hop loop of MixedPSNeighborSampler.sample, DP branch (reference
// python/npc/sampler.py:187-203,358-364: sample -> relabel -> frontier = unique, per
// hop) as one operator: every kernel of the batch is enqueued by one C call, the
// sizes stay on the device, and the host waits once, to cut the outputs to size.
// hop_fanouts: from the seeds outward.  Returns
//   [sizes (CPU int64[H + 2]: frontier rows entering each hop, input nodes, edges),
//    input_nodes, then per hop h: neighbors_h, relabeled_h, counts_h]
// with neighbors / relabeled in the fixed-stride layout [rows_h * fanout_h], -1 = no edge.
// The rank table and workspace live in the registry and are reused: calls must be
// ordered on one stream.
// with_formats: each hop's block is also emitted as COO + CSC before that one wait;
// appended per hop: coo_row_h, coo_col_h, csc_indptr_h (sizes then carries the hops'
// edge counts after its H + 2 entries).
std::vector<Tensor> SampleBlocks(Tensor seeds, std::vector<int64_t> hop_fanouts, bool replace, IdType rng_seed,
                                 bool with_formats) {
  auto& s = S();
  TORCH_CHECK(s.has_graph, "npc: no graph registered (mix_cache_graphs)");
  const int H = static_cast<int>(hop_fanouts.size());
  TORCH_CHECK(H >= 1 && H <= APT_MAX_HOPS, "npc: sample_blocks: 1..", APT_MAX_HOPS, " hops");
  auto sd = ids_on_device(seeds, "seeds");
  const int64_t B = sd.numel();
  TORCH_CHECK(B > 0, "npc: sample_blocks: no seeds");
  std::vector<int> fan(H);
  for (int h = 0; h < H; ++h) {
    TORCH_CHECK(hop_fanouts[h] > 0 && hop_fanouts[h] <= (1 << 20), "npc: sample_blocks: bad fanout");
    fan[h] = static_cast<int>(hop_fanouts[h]);
  }
  auto u8 = torch::TensorOptions().dtype(torch::kUInt8).device(device());
  if (!s.rank_table.defined()) {
    const size_t bytes = apt_rank_table_bytes(s.graph.num_total_nodes);
    TORCH_CHECK(bytes > 0, "npc: sample_blocks: graph too large for the rank table");
    s.rank_table = torch::empty({static_cast<int64_t>(bytes)}, u8);
    check(apt_rank_table_init(s.rank_table.data_ptr(), bytes, stream()));
  }
  if (s.mb_batch != B || s.mb_fanouts != hop_fanouts || !s.mb_workspace.defined()) {
    const size_t need = apt_minibatch_workspace_bytes(B, fan.data(), H);
    TORCH_CHECK(need > 0, "npc: sample_blocks: unsupported batch / fanouts");
    s.mb_workspace = torch::empty({static_cast<int64_t>(need)}, u8);
    check(apt_minibatch_workspace_init(s.mb_workspace.data_ptr(), need, stream()));
    s.mb_batch = B;
    s.mb_fanouts = hop_fanouts;
  }
  std::vector<int64_t> cap(H + 1);
  for (int h = 0; h <= H; ++h) {
    cap[h] = apt_minibatch_capacity(B, fan.data(), H, h);
    TORCH_CHECK(cap[h] > 0, "npc: sample_blocks: unsupported batch / fanouts");
  }
  // Output buffers at their upper bounds: a set of the ring (reused, see State::mb_ring) or fresh ones.
  State::BlockBuffers fresh;
  State::BlockBuffers* bufp = &fresh;
  if (s.mb_ring_size > 0) {
    if (static_cast<int64_t>(s.mb_ring.size()) != s.mb_ring_size) s.mb_ring.assign(s.mb_ring_size, State::BlockBuffers());
    bufp = &s.mb_ring[s.mb_ring_pos];
    s.mb_ring_pos = (s.mb_ring_pos + 1) % s.mb_ring_size;
  }
  State::BlockBuffers& b = *bufp;
  const bool fits = b.nodes.defined() && b.nodes.numel() == cap[H] && static_cast<int>(b.nb.size()) == H &&
                    b.sizes.numel() == H + 2 + (with_formats ? H : 0) && (!with_formats || b.formats) &&
                    [&] {
                      for (int h = 0; h < H; ++h)
                        if (b.nb[h].numel() != cap[h] * fan[h] || b.ct[h].numel() != cap[h]) return false;
                      return true;
                    }();
  if (!fits) {
    b = State::BlockBuffers();
    b.nodes = torch::empty({cap[H]}, i64_opts());
    b.sizes = torch::empty({H + 2 + (with_formats ? H : 0)}, i64_opts());
    b.nb.resize(H); b.rl.resize(H); b.ct.resize(H);
    for (int h = 0; h < H; ++h) {
      b.nb[h] = torch::empty({cap[h] * fan[h]}, i64_opts());
      b.rl[h] = torch::empty({cap[h] * fan[h]}, i64_opts());
      b.ct[h] = torch::empty({cap[h]}, i64_opts());
    }
    if (with_formats) {
      size_t need = 256;
      for (int h = 0; h < H; ++h) {
        const size_t bytes = apt_block_workspace_bytes(cap[h], fan[h], cap[h + 1], 0);
        TORCH_CHECK(bytes > 0, "npc: sample_blocks: block sizes out of range");
        need = std::max(need, bytes);
      }
      b.format_ws = torch::empty({static_cast<int64_t>(need)}, u8);   // the hops run one after the other
      b.row.resize(H); b.col.resize(H); b.csc.resize(H);
      for (int h = 0; h < H; ++h) {
        b.row[h] = torch::empty({cap[h] * fan[h]}, i64_opts());
        b.col[h] = torch::empty({cap[h] * fan[h]}, i64_opts());
        b.csc[h] = torch::empty({cap[h] + 1}, i64_opts());
      }
      b.formats = true;
    }
  }
  b.sizes.zero_();
  Tensor &nodes = b.nodes, &sizes = b.sizes;
  std::vector<Tensor>&nb = b.nb, &rl = b.rl, &ct = b.ct, &row = b.row, &col = b.col, &csc = b.csc;
  std::vector<int64_t*> nbp(H), rlp(H), ctp(H);
  for (int h = 0; h < H; ++h) {
    nbp[h] = nb[h].data_ptr<int64_t>();
    rlp[h] = rl[h].data_ptr<int64_t>();
    ctp[h] = ct[h].data_ptr<int64_t>();
  }
  const int rc = apt_minibatch_sample(&s.graph, i64(sd), B, fan.data(), H, replace ? 1 : 0,
                                      static_cast<uint64_t>(rng_seed), nullptr, s.rank_table.data_ptr(),
                                      s.graph.num_total_nodes, nodes.data_ptr<int64_t>(), nbp.data(), rlp.data(),
                                      ctp.data(), sizes.data_ptr<int64_t>(), s.mb_workspace.data_ptr(),
                                      static_cast<size_t>(s.mb_workspace.numel()), stream());
  if (rc != APT_OK) s.mb_workspace = Tensor();  // re-initialised by the next call
  check(rc);
  if (with_formats) {
    int64_t* dev_sizes = sizes.data_ptr<int64_t>();
    for (int h = 0; h < H; ++h)
      check(apt_block_formats(rlp[h], cap[h], dev_sizes + h, fan[h], cap[h + 1], row[h].data_ptr<int64_t>(),
                              col[h].data_ptr<int64_t>(), csc[h].data_ptr<int64_t>(), dev_sizes + H + 2 + h, nullptr,
                              nullptr, nullptr, b.format_ws.data_ptr(), static_cast<size_t>(b.format_ws.numel()),
                              stream()));
  }
  auto host = sizes.cpu();  // the one wait of the batch
  const int64_t* hs = host.data_ptr<int64_t>();
  std::vector<Tensor> out{host, nodes.narrow(0, 0, hs[H])};
  for (int h = 0; h < H; ++h) {
    out.push_back(nb[h].narrow(0, 0, hs[h] * fan[h]));
    out.push_back(rl[h].narrow(0, 0, hs[h] * fan[h]));
    out.push_back(ct[h].narrow(0, 0, hs[h]));
  }
  if (with_formats)
    for (int h = 0; h < H; ++h) {
      out.push_back(row[h].narrow(0, 0, hs[H + 2 + h]));
      out.push_back(col[h].narrow(0, 0, hs[H + 2 + h]));
      out.push_back(csc[h].narrow(0, 0, hs[h] + 1));
    }
  return out;
}

// COO / CSC / CSR of a fixed-stride block (what DGL derives from (row, col) in the
// reference, python/npc/sampler.py:59-69).  Returns [coo_row, coo_col, csc_indptr]
// (+ [csr_indptr, csr_indices, csr_eids] with want_csr), cut to the edge count.
std::vector<Tensor> BlockFormats(Tensor relabeled, IdType num_dst, IdType fanout, IdType num_src, bool want_csr) {
  auto rl = ids_on_device(relabeled, "relabeled");
  TORCH_CHECK(num_dst >= 0 && fanout > 0 && num_src >= 0, "npc: block_formats: bad shape");
  TORCH_CHECK(rl.numel() >= num_dst * fanout, "npc: block_formats: relabeled shorter than num_dst * fanout");
  const int64_t slots = num_dst * fanout;
  const size_t need = apt_block_workspace_bytes(num_dst, static_cast<int>(fanout), num_src, want_csr);
  TORCH_CHECK(need > 0 || slots == 0, "npc: block_formats: sizes out of range");
  auto ws = torch::empty({static_cast<int64_t>(std::max<size_t>(need, 256))},
                         torch::TensorOptions().dtype(torch::kUInt8).device(device()));
  auto row = torch::empty({slots}, i64_opts()), col = torch::empty({slots}, i64_opts());
  auto csc = torch::empty({num_dst + 1}, i64_opts()), edges = torch::zeros({1}, i64_opts());
  Tensor csr, ci, ce;
  if (want_csr) {
    csr = torch::empty({num_src + 1}, i64_opts());
    ci = torch::empty({slots}, i64_opts());
    ce = torch::empty({slots}, i64_opts());
  }
  check(apt_block_formats(i64(rl), num_dst, nullptr, static_cast<int>(fanout), num_src, row.data_ptr<int64_t>(),
                          col.data_ptr<int64_t>(), csc.data_ptr<int64_t>(), edges.data_ptr<int64_t>(),
                          want_csr ? csr.data_ptr<int64_t>() : nullptr, want_csr ? ci.data_ptr<int64_t>() : nullptr,
                          want_csr ? ce.data_ptr<int64_t>() : nullptr, ws.data_ptr(),
                          static_cast<size_t>(ws.numel()), stream()));
  const int64_t e = edges.item<int64_t>();
  std::vector<Tensor> out{row.narrow(0, 0, e), col.narrow(0, 0, e), csc};
  if (want_csr) {
    out.push_back(csr);
    out.push_back(ci.narrow(0, 0, e));
    out.push_back(ce.narrow(0, 0, e));
  }
  return out;
}

// reference src/sampling.cc:13-17
std::vector<Tensor> LocalSamplingNeibhorsOneLayer(Tensor seeds, IdType fanout) {
  auto& s = S();
  TORCH_CHECK(s.has_graph, "npc: no graph registered (mix_cache_graphs)");
  TORCH_CHECK(fanout > 0, "npc: fanout must be > 0");
  auto f = ids_on_device(seeds, "seeds");
  auto out = torch::empty({f.numel() * fanout}, i64_opts());
  sample_hop(f, fanout, true, s.rng_seed, static_cast<int>(s.sample_calls), out, nullptr);
  s.sample_calls += 1;
  return {f, out};
}

// relabel_csc through the rank table of the registered graph (apt_relabel_ranked).  The reference's sampler calls
// relabel_csc once per hop with seeds = the unique list of the hop before (python/npc/sampler.py:187-203): such a
// call continues the batch, its seeds are already in the table.  -> false when an id does not fit the table (the
// caller then takes the hash table).
static bool RelabelRanked(const Tensor& sd, const Tensor& nb, Tensor& unique, Tensor& relabeled) {
  auto& s = S();
  const int64_t items = sd.numel() + nb.numel();
  const int64_t len = s.graph.num_total_nodes;
  if (!ranked_resources(items)) return false;
  // bids placed by the sampling call for exactly these tensors?  Bids placed for others are abandoned: the table's
  // batch cannot be continued then.
  auto& p = s.ranked_pending;
  const bool marked = p.valid && nb.numel() > 0 && same_tensor(p.neighbors, p.neighbors_version, nb) &&
                      same_tensor(p.seeds, p.seeds_version, sd);
  const bool continued = marked ? p.continued
                                : !p.valid && same_tensor(s.ranked_last, s.ranked_last_version, sd);
  s.ranked_last = Tensor();
  unique = torch::empty({items}, i64_opts());
  relabeled = marked ? p.states : torch::empty({nb.numel()}, i64_opts());
  if (marked) s.ranked_pending = {};
  else drop_pending_bids();
  int64_t* host = pinned_counts();
  host[0] = host[1] = -1;
  // ranked_counts[1] counts ids beyond the graph; it is zero unless the previous call found some
  check(apt_relabel_ranked(i64(sd), sd.numel(), nullptr, i64(nb), nb.numel(), 0, (continued ? 1 : 0) | (marked ? 2 : 0),
                           s.ranked_table.data_ptr(), len,
                           unique.data_ptr<int64_t>(), nb.numel() ? relabeled.data_ptr<int64_t>() : nullptr,
                           s.ranked_counts.data_ptr<int64_t>(), s.ranked_counts.data_ptr<int64_t>() + 1, host,
                           s.ranked_ws.data_ptr(),
                           static_cast<size_t>(s.ranked_ws.numel()), stream()));
  if (host[1] != 0) {  // ids beyond the graph: not a valid relabel, and the table's batch is not continued
    s.ranked_counts.zero_();
    relabeled = Tensor();
    return false;
  }
  unique = unique.narrow(0, 0, host[0]);
  s.ranked_last = unique;
  s.ranked_last_version = unique._version();
  return true;
}

// reference src/relabel.cc:9-15
std::vector<Tensor> RelabelCSC(Tensor seeds, Tensor neighbors) {
  auto& s = S();
  auto sd = ids_on_device(seeds, "seeds");
  auto nb = ids_on_device(neighbors, "neighbors");
  const int64_t items = sd.numel() + nb.numel();
  // Small inputs: one workgroup with its table in LDS (inside apt_relabel).  Larger ones: the rank table of the
  // registered graph, if there is one and the ids fit it; else the hash table in device memory.
  if (s.has_graph && s.ranked_enabled && items > 8192 && items <= apt_relabel_ranked_max_items() &&
      s.graph.num_total_nodes > 0) {
    Tensor unique, relabeled;
    if (RelabelRanked(sd, nb, unique, relabeled)) return {unique, relabeled};
  }
  s.ranked_last = Tensor();
  if (s.ranked_pending.valid) {   // a sampling call has counted ids beyond the graph, or its bids are not used
    drop_pending_bids();
    if (s.ranked_counts.defined()) s.ranked_counts.zero_();
  }
  const size_t need = apt_relabel_workspace_bytes(items);
  TORCH_CHECK(need > 0, "npc: relabel_csc: ", items, " items exceed the supported maximum");
  auto ws = torch::empty({static_cast<int64_t>(need)}, torch::TensorOptions().dtype(torch::kUInt8).device(device()));
  auto unique = torch::empty({items}, i64_opts());
  auto relabeled = torch::empty({nb.numel()}, i64_opts());
  auto count = torch::empty({1}, i64_opts());
  int64_t* host_count = pinned_counts();
  *host_count = -1;
  check(apt_relabel(i64(sd), sd.numel(), nullptr, i64(nb), nb.numel(), 0, unique.data_ptr<int64_t>(),
                    relabeled.data_ptr<int64_t>(), count.data_ptr<int64_t>(), host_count,
                    ws.data_ptr(), need, stream()));
  return {unique.narrow(0, 0, *host_count), relabeled};
}

// reference src/load_subtensor.cc:19-40
Tensor LoadSubtensor(Tensor node_id) {
  auto& s = S();
  TORCH_CHECK(s.has_feat, "npc: no features registered (cache_feats_shared)");
  PollChecks(false);
  auto idx = ids_on_device(node_id, "node_id");
  auto out = torch::empty({idx.numel(), s.feat.out_dim}, s.local_feats.options());
  Tensor miss;
  if (s.miss_check != 0) miss = torch::zeros({1}, i64_opts());
  check(apt_gather_rows(&s.feat, i64(idx), idx.numel(), nullptr, out.data_ptr(),
                        s.miss_check != 0 ? miss.data_ptr<int64_t>() : nullptr, stream()));
  if (s.miss_check == 2) {
    const int64_t m = miss.item<int64_t>();
    TORCH_CHECK_INDEX(m == 0, "npc: load_subtensor: ", m,
                      " requested node(s) have no feature row on this GPU");
  } else if (s.miss_check == 1) {
    // the counter follows the gather to pinned host memory; nobody waits for it here
    State::PendingCheck p;
    p.dev = miss;
    p.host = torch::empty({1}, torch::TensorOptions().dtype(torch::kInt64).pinned_memory(true));
    p.host.copy_(miss, /*non_blocking=*/true);
    p.done = std::make_shared<at::cuda::CUDAEvent>();
    p.done->record();
    s.pending_checks.push_back(std::move(p));
    if (s.pending_checks.size() > 64) {   // a caller that never lets one arrive: wait for the oldest
      s.pending_checks.front().done->synchronize();
      PollChecks(false);
    }
  }
  return out;
}

// reference src/load_subtensor.cc:10-17: two index_selects, the result on the host
// as there.  The local table lives in HBM here, so the rows come from the GPU; the
// ids are checked on the host first (the map copy is a host tensor), where the
// reference's host index_select would raise: an id outside the map or without a
// local row never reaches a kernel.
Tensor CPULoadSubtensor(Tensor node_id) {
  auto& s = S();
  TORCH_CHECK(s.has_feat, "npc: no features registered (cache_feats_shared)");
  TORCH_CHECK(node_id.scalar_type() == torch::kInt64, "npc: node_id must be int64");
  auto ids = node_id.cpu().contiguous().view({-1});
  const int64_t total = s.cpu_feat_pos_map.numel();
  const int64_t* idp = ids.data_ptr<int64_t>();
  const int64_t* map = s.cpu_feat_pos_map.data_ptr<int64_t>();
  auto pos = torch::empty({ids.numel()}, torch::TensorOptions().dtype(torch::kInt64));
  int64_t* pp = pos.data_ptr<int64_t>();
  const int64_t n_local = s.local_feats.size(0);
  for (int64_t i = 0; i < ids.numel(); ++i) {
    const int64_t v = idp[i];
    TORCH_CHECK_INDEX(v >= 0 && v < total, "npc: cpu_load_subtensor: node id ", v, " at position ", i,
                      " is outside [0, ", total, ")");
    const int64_t row = -map[v] - 2;  // ENCODE_ID, src/utils.h:17
    TORCH_CHECK_INDEX(row >= 0 && row < n_local, "npc: cpu_load_subtensor: node ", v, " at position ", i,
                      " has no local feature row");
    pp[i] = row;
  }
  return s.local_feats.index_select(0, pos.to(s.local_feats.device())).cpu();
}

std::tuple<Tensor, Tensor, Tensor, Tensor> ClusterAndPermuteLocal(Tensor seeds) {
  auto& s = S();
  TORCH_CHECK(s.shuffle_min_vids.defined(), "npc: register_min_vids has not been called");
  TORCH_CHECK(s.shuffle_min_vids.numel() >= s.world_size + 1, "npc: min_vids shorter than world_size + 1");
  auto ids = ids_on_device(seeds, "seeds");
  const int W = static_cast<int>(s.world_size);
  const int node_beg = static_cast<int>(s.rank - (s.rank % s.node_size));  // src/sampling.cc:168-169
  auto size = torch::empty({W}, i64_opts()), offset = torch::empty({W}, i64_opts());
  auto sorted = torch::empty({ids.numel()}, i64_opts()), perm = torch::empty({ids.numel()}, i64_opts());
  const size_t need = apt_bucket_workspace_bytes(ids.numel(), W);
  TORCH_CHECK(need > 0, "npc: bucketing: unsupported size");
  auto ws = torch::empty({static_cast<int64_t>(need)}, torch::TensorOptions().dtype(torch::kUInt8).device(device()));
  check(apt_cluster_permute(i64(ids), ids.numel(), nullptr, s.shuffle_min_vids.data_ptr<int64_t>(), W,
                            s.shuffle_id_offset, static_cast<int>(s.rank), node_beg,
                            node_beg + static_cast<int>(s.node_size), size.data_ptr<int64_t>(),
                            offset.data_ptr<int64_t>(), sorted.data_ptr<int64_t>(),
                            perm.data_ptr<int64_t>(), ws.data_ptr(), need, stream()));
  auto& own = s.own_permutations;
  own.emplace_back(perm, perm._version());
  if (own.size() > 8) own.pop_front();
  return {size, offset, sorted, perm};
}

// reference src/sampling.cc:19-50: virtual nodes of SP mode (local arithmetic, no exchange)
static Tensor MapToVir(const char* who, IdType fanout, const Tensor* dst, IdType num_dst, Tensor src) {
  auto& s = S();
  TORCH_CHECK(s.shuffle_min_vids.defined(), "npc: ", who, ": register_min_vids has not been called");
  TORCH_CHECK(s.shuffle_min_vids.numel() >= s.world_size + 1, "npc: min_vids shorter than world_size + 1");
  TORCH_CHECK(fanout > 0, "npc: ", who, ": fanout must be > 0");
  auto sv = ids_on_device(src, "src");
  Tensor dv;
  if (dst != nullptr) {
    dv = ids_on_device(*dst, "dst");
    num_dst = dv.numel();
  }
  const int node_beg = static_cast<int>(s.rank - (s.rank % s.node_size));
  auto out = torch::empty({(dst != nullptr ? num_dst : 0) + sv.numel()}, i64_opts());
  check(apt_map_to_vir(dst != nullptr ? i64(dv) : nullptr, num_dst, i64(sv), sv.numel(), static_cast<int>(fanout),
                       s.shuffle_min_vids.data_ptr<int64_t>(), static_cast<int>(s.world_size),
                       s.shuffle_id_offset, static_cast<int>(s.rank), node_beg,
                       node_beg + static_cast<int>(s.node_size), out.data_ptr<int64_t>(), stream()));
  return out;
}
Tensor SrcDsttoVir(IdType fanout, Tensor dst, Tensor src) { return MapToVir("srcdst_to_vir", fanout, &dst, 0, src); }
Tensor SrcToVir(IdType fanout, IdType num_dst, Tensor src) {
  TORCH_CHECK(num_dst >= 0, "npc: src_to_vir: num_dst must be >= 0");
  return MapToVir("src_to_vir", fanout, nullptr, num_dst, src);
}

// reference src/sampling.cc:159-193; with one GPU both all-to-alls are identity copies
std::tuple<Tensor, Tensor, Tensor, Tensor> ShuffleSeeds(Tensor seeds) {
  TORCH_CHECK(S().world_size == 1,
              "npc: shuffle_seeds exchanges ids between GPUs; only world_size 1 is available "
              "(cluster_and_permute gives the local half)");
  auto r = ClusterAndPermuteLocal(seeds);
  auto off = std::get<1>(r).cpu();
  return {std::get<2>(r), std::get<3>(r), off.clone(), off};
}

// reference src/load_subtensor.cc:83-86
std::tuple<Tensor, Tensor, Tensor> ClusterReqs(Tensor node_id) {
  auto& s = S();
  TORCH_CHECK(s.has_feat && s.remote_worker_map.defined() && s.shuffle_min_vids.defined(),
              "npc: cluster_reqs needs cache_feats_shared, register_min_vids and "
              "register_multi_machines_scheme");
  TORCH_CHECK(s.shuffle_min_vids.numel() >= s.world_size + 1 && s.remote_worker_map.numel() >= s.world_size,
              "npc: min_vids / remote_worker_map shorter than world_size");
  auto ids = ids_on_device(node_id, "node_id");
  const int R = static_cast<int>(s.num_remote_workers);
  auto size = torch::empty({R}, i64_opts());
  auto sorted = torch::empty({ids.numel()}, i64_opts()), perm = torch::empty({ids.numel()}, i64_opts());
  const size_t need = apt_bucket_workspace_bytes(ids.numel(), R);
  TORCH_CHECK(need > 0, "npc: bucketing: unsupported size");
  auto ws = torch::empty({static_cast<int64_t>(need)}, torch::TensorOptions().dtype(torch::kUInt8).device(device()));
  check(apt_cluster_reqs(i64(ids), ids.numel(), nullptr, s.feat_pos_map.data_ptr<int64_t>(),
                         s.feat_pos_map.numel(), s.remote_worker_map.data_ptr<int64_t>(),
                         s.shuffle_min_vids.data_ptr<int64_t>(), static_cast<int>(s.world_size), R,
                         size.data_ptr<int64_t>(), nullptr, sorted.data_ptr<int64_t>(),
                         perm.data_ptr<int64_t>(), ws.data_ptr(), need, stream()));
  return {size, sorted, perm};
}

// reference src/feat_shuffle.cc:9-30 with one GPU
Tensor FeatShuffle(Tensor inputs, Tensor send_offset, Tensor recv_offset, Tensor permutation,
                   IdType feat_dim, IdType fwd_flag) {
  TORCH_CHECK(S().world_size == 1,
              "npc: feat_shuffle exchanges rows between GPUs; only world_size 1 is available");
  TORCH_CHECK(inputs.is_cuda() && (inputs.element_size() == 2 || inputs.element_size() == 4),
              "npc: feat_shuffle needs a GPU tensor with 2- or 4-byte elements");
  auto x = inputs.reshape({-1, feat_dim}).contiguous();
  auto perm = ids_on_device(permutation, "permutation");
  const int64_t n_out = recv_offset.index({-1}).item<int64_t>();
  if (fwd_flag) {
    TORCH_CHECK(x.size(0) == n_out, "npc: with one GPU the received row count equals the sent one");
    auto out = torch::empty({perm.numel(), feat_dim}, x.options());
    check(apt_permute_rows(x.data_ptr(), x.size(0), i64(perm), perm.numel(), feat_dim,
                           static_cast<int>(x.element_size()), out.data_ptr(), stream()));
    return out;
  }
  TORCH_CHECK(perm.numel() == x.size(0), "npc: permutation must name every input row");
  // rows that no permutation entry names (none when it is a bijection, as ShuffleSeeds makes it) are flagged by
  // the scatter and zeroed afterwards: cheaper than zero-filling the whole output first
  auto out = torch::empty({n_out, feat_dim}, x.options());
  auto ws = torch::empty({static_cast<int64_t>(apt_scatter_workspace_bytes(n_out))},
                         torch::TensorOptions().dtype(torch::kUInt8).device(device()));
  check(apt_scatter_rows(x.data_ptr(), i64(perm), perm.numel(), feat_dim, static_cast<int>(x.element_size()),
                         out.data_ptr(), n_out, ws.data_ptr(), static_cast<size_t>(ws.numel()), stream()));
  bool own = false;   // a permutation this library produced is a bijection onto [0, n): nothing to check
  for (const auto& p : S().own_permutations)
    own |= p.first.data_ptr() == perm.data_ptr() && p.first.numel() == perm.numel() && p.second == perm._version() &&
           perm.numel() == n_out;
  if (S().strict && !own) {
    // The reference's pack is index_select_backward (src/feat_shuffle.cc:14-16): rows named more than once
    // add up.  The scatter keeps one of them, which is the same thing only for a permutation without
    // repeats (what ShuffleSeeds produces).  The flags tell: as many rows named as entries <=> no repeats and
    // nothing out of range; otherwise the sum is formed the reference's way.
    const int64_t named = ws.narrow(0, 0, n_out).sum().item<int64_t>();
    if (named != perm.numel()) {
      TORCH_CHECK_INDEX(perm.numel() == 0 || (perm.min().item<int64_t>() >= 0 && perm.max().item<int64_t>() < n_out),
                        "npc: feat_shuffle: permutation entry outside [0, ", n_out, ")");
      out = torch::zeros({n_out, feat_dim}, x.options()).index_add_(0, perm, x);
    }
  }
  return out;
}

// ---------------------------------------------------------------- aggregation
namespace {

Tensor feat2d(const Tensor& t, const char* name) {
  TORCH_CHECK(t.is_cuda() && t.dim() == 2 &&
                  (t.scalar_type() == torch::kFloat32 || t.scalar_type() == torch::kBFloat16),
              "npc: ", name, " must be a 2-D fp32 or bf16 GPU tensor");
  return t.contiguous();
}

// out_num = output_offset[-1] is read on the host, as in the reference (src/spmm.cc:13).
Tensor spmm(int mode, Tensor coo_row, Tensor coo_col, Tensor input, const Tensor* edata, Tensor coo_offset,
            const Tensor* input_offset, Tensor output_offset) {
  auto row = ids_on_device(coo_row, "coo_row"), col = ids_on_device(coo_col, "coo_col");
  auto x = feat2d(input, "input");
  auto coo = ids_on_device(coo_offset, "coo_offset");
  auto oo = ids_on_device(output_offset, "output_offset");
  TORCH_CHECK(coo.numel() >= 2 && oo.numel() >= coo.numel() - 1 && row.numel() == col.numel(),
              "npc: spmm: bad offsets or edge lists");
  const int nseg = static_cast<int>(coo.numel() - 1);
  const int64_t out_num = oo.index({-1}).item<int64_t>();
  Tensor io, ed;
  if (input_offset) io = ids_on_device(*input_offset, "input_offset");
  if (edata) {
    ed = feat2d(*edata, "edata");
    TORCH_CHECK(ed.scalar_type() == x.scalar_type() && ed.size(0) == row.numel() && ed.size(1) == x.size(1),
                "npc: spmm: edata must be [E, dim] of the input dtype");
  }
  if (mode == 1) TORCH_CHECK(x.size(0) == row.numel(), "npc: spmm_copy_e_sum needs one input row per edge");
  auto out = torch::zeros({out_num, x.size(1)}, x.options().dtype(torch::kFloat32));
  // a block's COO is destination-major: found out on the device, rows inside a wavefront's edges skip the atomics
  auto grouped = torch::empty({1}, torch::TensorOptions().dtype(torch::kInt32).device(device()));
  check(apt_coo_is_grouped(i64(col), col.numel(), grouped.data_ptr<int>(), stream()));
  check(apt_spmm_sum(mode, i64(row), i64(col), row.numel(), x.data_ptr(), x.size(0),
                     edata ? ed.data_ptr() : nullptr, x.size(1), static_cast<int>(x.element_size()),
                     i64(coo), input_offset ? i64(io) : nullptr, i64(oo), nseg, out.data_ptr<float>(),
                     out_num, grouped.data_ptr<int>(), stream()));
  return out.to(x.scalar_type());
}

Tensor sddmm(int op, Tensor coo_row, Tensor coo_col, Tensor lhs, Tensor rhs, Tensor coo_offset,
             Tensor lhs_offset, Tensor rhs_offset) {
  auto row = ids_on_device(coo_row, "coo_row"), col = ids_on_device(coo_col, "coo_col");
  auto l = feat2d(lhs, "lhs"), r = feat2d(rhs, "rhs");
  TORCH_CHECK(l.scalar_type() == r.scalar_type() && l.size(1) == r.size(1) && row.numel() == col.numel(),
              "npc: sddmm: lhs/rhs mismatch");
  auto coo = ids_on_device(coo_offset, "coo_offset");
  auto lo = ids_on_device(lhs_offset, "lhs_offset"), ro = ids_on_device(rhs_offset, "rhs_offset");
  TORCH_CHECK(coo.numel() >= 2 && lo.numel() >= coo.numel() - 1 && ro.numel() >= coo.numel() - 1,
              "npc: sddmm: bad offsets");
  auto out = torch::empty({row.numel(), l.size(1)}, l.options().dtype(torch::kFloat32));
  check(apt_sddmm(op, i64(row), i64(col), row.numel(), l.data_ptr(), l.size(0), r.data_ptr(), r.size(0),
                  l.size(1), static_cast<int>(l.element_size()), i64(coo), i64(lo), i64(ro),
                  static_cast<int>(coo.numel() - 1), out.data_ptr<float>(), stream()));
  return out.to(l.scalar_type());
}

}  // namespace

// reference src/spmm.cc:9-42
Tensor CopyUSum(Tensor coo_row, Tensor coo_col, Tensor input, Tensor coo_offset, Tensor input_offset,
                Tensor output_offset) {
  return spmm(0, coo_row, coo_col, input, nullptr, coo_offset, &input_offset, output_offset);
}
Tensor CopyESum(Tensor coo_row, Tensor coo_col, Tensor input, Tensor coo_offset, Tensor output_offset) {
  return spmm(1, coo_row, coo_col, input, nullptr, coo_offset, nullptr, output_offset);
}
Tensor UMulESum(Tensor coo_row, Tensor coo_col, Tensor input, Tensor edata, Tensor coo_offset,
                Tensor input_offset, Tensor output_offset) {
  return spmm(2, coo_row, coo_col, input, &edata, coo_offset, &input_offset, output_offset);
}
// reference src/sddmm.cc:9-31
Tensor UAddV(Tensor coo_row, Tensor coo_col, Tensor lhs, Tensor rhs, Tensor coo_offset, Tensor lhs_offset,
             Tensor rhs_offset) {
  return sddmm(0, coo_row, coo_col, lhs, rhs, coo_offset, lhs_offset, rhs_offset);
}
Tensor UMulV(Tensor coo_row, Tensor coo_col, Tensor lhs, Tensor rhs, Tensor coo_offset, Tensor lhs_offset,
             Tensor rhs_offset) {
  return sddmm(1, coo_row, coo_col, lhs, rhs, coo_offset, lhs_offset, rhs_offset);
}

// ---------------------------------------------------------------- peers only
#define NPC_NEEDS_PEERS(name)                                                              \
  TORCH_CHECK(false, "npc." name " talks to other GPUs over NCCL in the reference; this " \
                     "library builds one GPU's share only")

Tensor NCCLGetUniqueId() { NPC_NEEDS_PEERS("nccl_get_unique_id"); }
void Initialize(IdType, IdType, IdType, Tensor, IdType) { NPC_NEEDS_PEERS("init"); }
void AlltoAll(Tensor, Tensor, Tensor, Tensor, IdType, IdType) { NPC_NEEDS_PEERS("alltoall"); }
Tensor CrossMachineLoadSubtensor(Tensor) { NPC_NEEDS_PEERS("crossmachine_load_subtensor"); }
std::vector<Tensor> NPSampleAndShuffle(Tensor, IdType) { NPC_NEEDS_PEERS("np_sample_and_shuffle"); }
std::vector<Tensor> SPSampleAndShuffle(IdType, Tensor, Tensor, Tensor, IdType) {
  NPC_NEEDS_PEERS("sp_sample_and_shuffle");
}
std::vector<Tensor> SPSampleShuffleSrc(Tensor) { NPC_NEEDS_PEERS("sp_sample_shuffle_src"); }
std::vector<Tensor> MPSampleShuffle(Tensor, Tensor, Tensor) { NPC_NEEDS_PEERS("mp_sample_shuffle"); }
Tensor SPFeatShuffle(Tensor, Tensor, Tensor, IdType, IdType, IdType) { NPC_NEEDS_PEERS("sp_feat_shuffle"); }
Tensor MPFeatShuffleFwd(Tensor, Tensor, Tensor, IdType) { NPC_NEEDS_PEERS("mp_feat_shuffle_fwd"); }
Tensor MPFeatShuffleBwd(Tensor, Tensor, Tensor, IdType) { NPC_NEEDS_PEERS("mp_feat_shuffle_bwd"); }

TORCH_LIBRARY(npc, m) {
  // same names and order as the reference's src/pybind.cc:18-48
  m.def("nccl_get_unique_id", &NCCLGetUniqueId)
      .def("init", &Initialize)
      .def("alltoall", &AlltoAll)
      .def("cache_feats_shared", &CacheFeatsShared)
      .def("mix_cache_graphs", &MixCacheGraphs)
      .def("register_min_vids", &RegisterMinVids)
      .def("register_multi_machines_scheme", &RegisterMultiMachinesScheme)
      .def("cpu_load_subtensor", &CPULoadSubtensor)
      .def("load_subtensor", &LoadSubtensor)
      .def("crossmachine_load_subtensor", &CrossMachineLoadSubtensor)
      .def("cluster_reqs", &ClusterReqs)
      .def("local_sample_one_layer", &LocalSamplingNeibhorsOneLayer)
      .def("srcdst_to_vir", &SrcDsttoVir)
      .def("src_to_vir", &SrcToVir)
      .def("np_sample_and_shuffle", &NPSampleAndShuffle)
      .def("sp_sample_and_shuffle", &SPSampleAndShuffle)
      .def("sp_sample_shuffle_src", &SPSampleShuffleSrc)
      .def("mp_sample_shuffle", &MPSampleShuffle)
      .def("feat_shuffle", &FeatShuffle)
      .def("sp_feat_shuffle", &SPFeatShuffle)
      .def("mp_feat_shuffle_fwd", &MPFeatShuffleFwd)
      .def("mp_feat_shuffle_bwd", &MPFeatShuffleBwd)
      .def("shuffle_seeds", &ShuffleSeeds)
      .def("relabel_csc", &RelabelCSC)
      .def("spmm_copy_u_sum", &CopyUSum)
      .def("spmm_copy_e_sum", &CopyESum)
      .def("spmm_u_mul_e_sum", &UMulESum)
      .def("sddmm_u_add_v", &UAddV)
      .def("sddmm_u_mul_v", &UMulV)
      // additions (no counterpart in the reference)
      .def("sample_neighbors", &SampleNeighbors)
      .def("sample_blocks", &SampleBlocks)
      .def("block_formats", &BlockFormats)
      .def("cluster_and_permute", &ClusterAndPermuteLocal)
      .def("register_graph_partition", &RegisterGraphPartition)
      .def("set_topology", &SetTopology)
      .def("set_rng_seed", &SetRngSeed)
      .def("set_strict", &SetStrict)
      .def("set_miss_check", &SetMissCheck)
      .def("check_errors", &CheckErrors)
      .def("set_ranked_relabel", &SetRankedRelabel)
      .def("set_block_buffer_ring", &SetBlockBufferRing)
      .def("block_buffer_ring", &BlockBufferRing);
}

}  // namespace npc
