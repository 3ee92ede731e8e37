// Stable bucketing of ids by owner ("cluster and permute").
//
// Replaces _CountDeviceVerticesKernel / _PermuteKernel / ClusterAndPermute and
// _CountMultiMachinesDeviceKernel / MultiMachinesClusterAndPermute (reference
// src/cuda/npc_kernel.cu:318-508).  The reference takes atomic tickets (shared
// memory, then global), so the order inside a bucket varies from run to run;
// here the rank of an id inside its bucket is computed from wave ballots and a
// per-bucket prefix over workgroups, so ids keep their input order (one of the
// orders the reference can produce) and the result is reproducible.
// Passes: classify + per-tile histogram -> per-bucket prefix over tiles ->
// place.
#include "common.hpp"

namespace apt {

constexpr int kBktBlock = 256;
constexpr int kBktIters = 4;
constexpr int kBktTile = kBktBlock * kBktIters;
constexpr int kBktWaves = kBktBlock / kWave;

struct BucketParams {
  const int64_t* ids;
  int64_t n;                 // host-side count (upper bound when n_dev != NULL)
  const int64_t* n_dev;
  const int64_t* min_vids;   // [world + 1]
  int world;                 // entries scanned in min_vids
  int num_buckets;           // output buckets
  int64_t id_offset;
  int rank, node_beg, node_end;
  const int64_t* feat_pos_map;       // non-null: request bucketing
  int64_t num_total_nodes;
  const int64_t* remote_worker_map;  // [world]
  uint8_t* bucket_of;        // [n]
  uint32_t* hist;            // [num_buckets][tiles]
  int64_t* totals;           // [num_buckets]
  int64_t tiles;
  int64_t* bucket_size;
  int64_t* bucket_offset;
  int64_t* sorted_ids;
  int64_t* permutation;
};

__global__ __launch_bounds__(kBktBlock) void bucket_classify_kernel(BucketParams p) {
  __shared__ int64_t s_min[APT_MAX_BUCKETS + 1];
  __shared__ int64_t s_map[APT_MAX_BUCKETS];
  __shared__ uint32_t s_hist[APT_MAX_BUCKETS];
  const int tid = threadIdx.x;
  if (tid <= p.world) s_min[tid] = p.min_vids[tid];
  if (p.feat_pos_map != nullptr && tid < p.world) s_map[tid] = p.remote_worker_map[tid];
  if (tid < APT_MAX_BUCKETS) s_hist[tid] = 0;
  __syncthreads();
  const int64_t n = actual_count(p.n, p.n_dev);
  const int64_t base = static_cast<int64_t>(blockIdx.x) * kBktTile;
  for (int it = 0; it < kBktIters; ++it) {
    const int64_t i = base + it * kBktBlock + tid;
    if (i < n) {
      const int64_t v = p.ids[i];
      int64_t d;
      if (p.feat_pos_map == nullptr) {
        // reference :331-342
        d = p.id_offset;
        while (d + 1 < p.world && s_min[d + 1] <= v) ++d;
        if (d < p.node_beg || d >= p.node_end) d = p.rank;
      } else {
        // reference :398-408
        d = 0;
        const bool present =
            (v >= 0 && v < p.num_total_nodes) ? p.feat_pos_map[v] != -1 : false;
        if (!present) {
          while (d + 1 < p.world && s_min[d + 1] <= v) ++d;
          d = s_map[d];
        }
      }
      // Out-of-range owners cannot index the histogram; fold them into the
      // last bucket rather than fault (arguments are validated on the host,
      // a bad remote_worker_map entry is data).
      if (d < 0 || d >= p.num_buckets) d = p.num_buckets - 1;
      p.bucket_of[i] = static_cast<uint8_t>(d);
      atomicAdd(&s_hist[d], 1u);
    }
  }
  __syncthreads();
  if (tid < p.num_buckets) p.hist[static_cast<int64_t>(tid) * p.tiles + blockIdx.x] = s_hist[tid];
}

// One workgroup per bucket: exclusive prefix of its histogram row over tiles.
__global__ __launch_bounds__(kBktBlock) void bucket_scan_kernel(BucketParams p) {
  __shared__ uint32_t s_wave[kBktWaves];
  uint32_t* row = p.hist + static_cast<int64_t>(blockIdx.x) * p.tiles;
  const int lane = lane_id();
  const int wave = threadIdx.x / kWave;
  int64_t carry = 0;
  for (int64_t c0 = 0; c0 < p.tiles; c0 += kBktBlock) {
    const int64_t i = c0 + threadIdx.x;
    const uint32_t x = i < p.tiles ? row[i] : 0u;
    uint32_t incl = x;
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
      const uint32_t y = __shfl_up(incl, off, kWave);
      if (lane >= off) incl += y;
    }
    if (lane == kWave - 1) s_wave[wave] = incl;
    __syncthreads();
    uint32_t before = 0, all = 0;
    for (int w = 0; w < kBktWaves; ++w) {
      if (w < wave) before += s_wave[w];
      all += s_wave[w];
    }
    // Offsets inside one bucket fit 32 bits only up to 2^32 ids per bucket;
    // the host rejects larger n.
    if (i < p.tiles) row[i] = static_cast<uint32_t>(carry) + before + incl - x;
    carry += all;
    __syncthreads();
  }
  if (threadIdx.x == 0) p.totals[blockIdx.x] = carry;
}

__global__ __launch_bounds__(kBktBlock) void bucket_place_kernel(BucketParams p) {
  __shared__ int64_t s_start[APT_MAX_BUCKETS];
  __shared__ uint32_t s_cnt[kBktIters * kBktWaves][APT_MAX_BUCKETS];
  const int tid = threadIdx.x;
  const int lane = lane_id();
  const int wave = tid / kWave;
  const int nb = p.num_buckets;
  const int64_t n = actual_count(p.n, p.n_dev);
  if (tid == 0) {
    int64_t acc = 0;
    for (int w = 0; w < nb; ++w) {
      const int64_t t = p.n > 0 ? p.totals[w] : 0;
      s_start[w] = acc;
      acc += t;
      if (blockIdx.x == 0) {
        p.bucket_size[w] = t;
        if (p.bucket_offset != nullptr) p.bucket_offset[w] = acc;  // inclusive, reference :460
      }
    }
  }
  const int64_t base = static_cast<int64_t>(blockIdx.x) * kBktTile;
  if (base >= n) return;  // block-uniform
  int mine[kBktIters];
  uint32_t rank_in_wave[kBktIters];
#pragma unroll
  for (int it = 0; it < kBktIters; ++it) {
    const int64_t i = base + it * kBktBlock + tid;
    mine[it] = i < n ? static_cast<int>(p.bucket_of[i]) : -1;
    rank_in_wave[it] = 0;
    for (int w = 0; w < nb; ++w) {
      const uint64_t m = ballot(mine[it] == w);
      if (mine[it] == w) rank_in_wave[it] = rank_below(m);
      if (lane == 0) s_cnt[it * kBktWaves + wave][w] = __popcll(m);
    }
  }
  __syncthreads();
  // Exclusive prefix over (iteration, wave) pairs, one thread per bucket.
  if (tid < nb) {
    uint32_t acc = 0;
    for (int k = 0; k < kBktIters * kBktWaves; ++k) {
      const uint32_t c = s_cnt[k][tid];
      s_cnt[k][tid] = acc;
      acc += c;
    }
  }
  __syncthreads();
#pragma unroll
  for (int it = 0; it < kBktIters; ++it) {
    const int64_t i = base + it * kBktBlock + tid;
    if (mine[it] >= 0) {
      const int w = mine[it];
      const int64_t dst = s_start[w] + p.hist[static_cast<int64_t>(w) * p.tiles + blockIdx.x] +
                          s_cnt[it * kBktWaves + wave][w] + rank_in_wave[it];
      p.sorted_ids[dst] = p.ids[i];
      p.permutation[i] = dst;
    }
  }
}

static size_t bucket_align(size_t x) { return (x + 255) / 256 * 256; }

struct BucketLayout {
  size_t bucket_of_off, hist_off, totals_off, total;
  int64_t tiles;
};

static BucketLayout bucket_layout(int64_t n, int num_buckets) {
  BucketLayout L;
  L.tiles = ceil_div(n > 0 ? n : 1, kBktTile);
  size_t off = 0;
  L.bucket_of_off = off; off = bucket_align(off + static_cast<size_t>(n > 0 ? n : 1));
  L.hist_off = off;      off = bucket_align(off + sizeof(uint32_t) * static_cast<size_t>(L.tiles) * num_buckets);
  L.totals_off = off;    off = bucket_align(off + sizeof(int64_t) * num_buckets);
  L.total = off;
  return L;
}

static int run_bucketing(BucketParams& p, void* workspace, size_t workspace_bytes,
                         hipStream_t st, const char* who) {
  const BucketLayout L = bucket_layout(p.n, p.num_buckets);
  APT_REQUIRE(workspace != nullptr && workspace_bytes >= L.total, APT_EWORKSPACE,
              "%s: workspace of %zu bytes, %zu needed", who, workspace_bytes, L.total);
  char* ws = static_cast<char*>(workspace);
  p.bucket_of = reinterpret_cast<uint8_t*>(ws + L.bucket_of_off);
  p.hist = reinterpret_cast<uint32_t*>(ws + L.hist_off);
  p.totals = reinterpret_cast<int64_t*>(ws + L.totals_off);
  p.tiles = L.tiles;
  const unsigned tiles = static_cast<unsigned>(L.tiles);
  if (p.n > 0) {
    hipLaunchKernelGGL(bucket_classify_kernel, dim3(tiles), dim3(kBktBlock), 0, st, p);
    APT_LAUNCH_CHECK("bucket_classify_kernel");
    hipLaunchKernelGGL(bucket_scan_kernel, dim3(p.num_buckets), dim3(kBktBlock), 0, st, p);
    APT_LAUNCH_CHECK("bucket_scan_kernel");
  }
  hipLaunchKernelGGL(bucket_place_kernel, dim3(tiles), dim3(kBktBlock), 0, st, p);
  APT_LAUNCH_CHECK("bucket_place_kernel");
  return APT_OK;
}

// ------------------------------------------------------------ virtual nodes
// SP mode groups the edges of a destination by the owner of their source:
// "virtual node" (owner, destination) stands for the part of a destination's
// neighbourhood that lives on one owner (reference src/cuda/npc_kernel.cu:15-113).
//   with dst:  vir[i]           = owner(dst[i]) * num_dst + i                          i < num_dst
//              vir[num_dst + j] = owner(src[j]) * num_dst + world * num_dst + j / fanout
//   without:   vir[j]           = owner(src[j]) * num_dst + j / fanout
// owner() is the bucketing rule of apt_cluster_permute.
struct VirParams {
  const int64_t* dst;        // NULL: sources only
  int64_t num_dst;
  const int64_t* src;
  int64_t num_src;
  int fanout;
  const int64_t* min_vids;
  int world;
  int64_t id_offset;
  int rank, node_beg, node_end;
  int64_t* vir;
};

__global__ __launch_bounds__(kBktBlock) void map_to_vir_kernel(VirParams p) {
  __shared__ int64_t s_min[APT_MAX_BUCKETS + 1];
  if (threadIdx.x <= p.world) s_min[threadIdx.x] = p.min_vids[threadIdx.x];
  __syncthreads();
  const int64_t lead = p.dst != nullptr ? p.num_dst : 0;
  const int64_t n = lead + p.num_src;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kBktBlock + threadIdx.x; i < n;
       i += static_cast<int64_t>(gridDim.x) * kBktBlock) {
    int64_t v, offset;
    if (i < lead) {
      v = p.dst[i];
      offset = i;
    } else {
      const int64_t j = i - lead;
      v = p.src[j];
      offset = (p.dst != nullptr ? static_cast<int64_t>(p.world) * p.num_dst : 0) + j / p.fanout;
    }
    int64_t d = p.id_offset;
    while (d + 1 < p.world && s_min[d + 1] <= v) ++d;
    if (d < p.node_beg || d >= p.node_end) d = p.rank;
    p.vir[i] = d * p.num_dst + offset;
  }
}

// out[k] = first position in sorted[0..n) whose value is >= (first + k) * base
// (thrust::lower_bound in GetVirSendOffset, reference :115-183).
__global__ void vir_lower_bound_kernel(const int64_t* __restrict__ sorted, int64_t n, int64_t base,
                                       int first, int count, int64_t* __restrict__ out) {
  const int k = blockIdx.x * blockDim.x + threadIdx.x;
  if (k >= count) return;
  const int64_t want = static_cast<int64_t>(first + k) * base;
  int64_t lo = 0, hi = n;
  while (lo < hi) {
    const int64_t mid = lo + (hi - lo) / 2;
    if (sorted[mid] < want) lo = mid + 1;
    else hi = mid;
  }
  out[k] = lo;
}

}  // namespace apt

extern "C" size_t apt_bucket_workspace_bytes(int64_t n, int num_buckets) {
  if (n < 0 || num_buckets < 1 || num_buckets > APT_MAX_BUCKETS) return 0;
  return apt::bucket_layout(n, num_buckets).total;
}

extern "C" int apt_cluster_permute(const int64_t* ids, int64_t n, const int64_t* n_dev,
                                   const int64_t* min_vids,
                                   int num_buckets, int64_t id_offset, int rank, int node_beg,
                                   int node_end, int64_t* bucket_size, int64_t* bucket_offset,
                                   int64_t* sorted_ids, int64_t* permutation, void* workspace,
                                   size_t workspace_bytes, void* stream) {
  using namespace apt;
  APT_REQUIRE(n >= 0, APT_EINVAL, "apt_cluster_permute: n %lld < 0", (long long)n);
  APT_REQUIRE(n <= 0xffffffffLL, APT_ELIMIT,
              "apt_cluster_permute: n %lld exceeds the supported maximum", (long long)n);
  APT_REQUIRE(num_buckets >= 1 && num_buckets <= APT_MAX_BUCKETS, APT_ELIMIT,
              "apt_cluster_permute: num_buckets %d outside [1, %d]", num_buckets,
              APT_MAX_BUCKETS);
  APT_REQUIRE(min_vids != nullptr && bucket_size != nullptr, APT_EINVAL,
              "apt_cluster_permute: min_vids/bucket_size is NULL");
  APT_REQUIRE(id_offset >= 0 && id_offset < num_buckets, APT_EINVAL,
              "apt_cluster_permute: id_offset %lld outside [0, %d)", (long long)id_offset,
              num_buckets);
  APT_REQUIRE(rank >= 0 && rank < num_buckets, APT_EINVAL,
              "apt_cluster_permute: rank %d outside [0, %d)", rank, num_buckets);
  APT_REQUIRE(n == 0 || (ids != nullptr && sorted_ids != nullptr && permutation != nullptr),
              APT_EINVAL, "apt_cluster_permute: ids/sorted_ids/permutation is NULL");
  BucketParams p{};
  p.ids = ids;
  p.n = n;
  p.n_dev = n_dev;
  p.min_vids = min_vids;
  p.world = num_buckets;
  p.num_buckets = num_buckets;
  p.id_offset = id_offset;
  p.rank = rank;
  p.node_beg = node_beg;
  p.node_end = node_end;
  p.feat_pos_map = nullptr;
  p.bucket_size = bucket_size;
  p.bucket_offset = bucket_offset;
  p.sorted_ids = sorted_ids;
  p.permutation = permutation;
  return run_bucketing(p, workspace, workspace_bytes, static_cast<hipStream_t>(stream),
                       "apt_cluster_permute");
}

extern "C" int apt_cluster_reqs(const int64_t* ids, int64_t n, const int64_t* n_dev,
                                const int64_t* feat_pos_map,
                                int64_t num_total_nodes, const int64_t* remote_worker_map,
                                const int64_t* min_vids, int world_size, int num_remote_workers,
                                int64_t* bucket_size, int64_t* bucket_offset,
                                int64_t* sorted_ids, int64_t* permutation, void* workspace,
                                size_t workspace_bytes, void* stream) {
  using namespace apt;
  APT_REQUIRE(n >= 0, APT_EINVAL, "apt_cluster_reqs: n %lld < 0", (long long)n);
  APT_REQUIRE(n <= 0xffffffffLL, APT_ELIMIT,
              "apt_cluster_reqs: n %lld exceeds the supported maximum", (long long)n);
  APT_REQUIRE(world_size >= 1 && world_size <= APT_MAX_BUCKETS, APT_ELIMIT,
              "apt_cluster_reqs: world_size %d outside [1, %d]", world_size, APT_MAX_BUCKETS);
  APT_REQUIRE(num_remote_workers >= 1 && num_remote_workers <= APT_MAX_BUCKETS, APT_ELIMIT,
              "apt_cluster_reqs: num_remote_workers %d outside [1, %d]", num_remote_workers,
              APT_MAX_BUCKETS);
  APT_REQUIRE(feat_pos_map != nullptr && remote_worker_map != nullptr && min_vids != nullptr &&
                  bucket_size != nullptr,
              APT_EINVAL, "apt_cluster_reqs: a map or bucket_size is NULL");
  APT_REQUIRE(num_total_nodes >= 0, APT_EINVAL, "apt_cluster_reqs: num_total_nodes < 0");
  APT_REQUIRE(n == 0 || (ids != nullptr && sorted_ids != nullptr && permutation != nullptr),
              APT_EINVAL, "apt_cluster_reqs: ids/sorted_ids/permutation is NULL");
  BucketParams p{};
  p.ids = ids;
  p.n = n;
  p.n_dev = n_dev;
  p.min_vids = min_vids;
  p.world = world_size;
  p.num_buckets = num_remote_workers;
  p.id_offset = 0;
  p.rank = 0;
  p.node_beg = 0;
  p.node_end = world_size;
  p.feat_pos_map = feat_pos_map;
  p.num_total_nodes = num_total_nodes;
  p.remote_worker_map = remote_worker_map;
  p.bucket_size = bucket_size;
  p.bucket_offset = bucket_offset;
  p.sorted_ids = sorted_ids;
  p.permutation = permutation;
  return run_bucketing(p, workspace, workspace_bytes, static_cast<hipStream_t>(stream),
                       "apt_cluster_reqs");
}

extern "C" int apt_map_to_vir(const int64_t* dst, int64_t num_dst, const int64_t* src, int64_t num_src,
                              int fanout, const int64_t* min_vids, int world_size, int64_t id_offset,
                              int rank, int node_beg, int node_end, int64_t* vir_nodes, void* stream) {
  using namespace apt;
  APT_REQUIRE(num_dst >= 0 && num_src >= 0 && fanout > 0, APT_EINVAL,
              "apt_map_to_vir: bad shape (num_dst %lld, num_src %lld, fanout %d)", (long long)num_dst,
              (long long)num_src, fanout);
  APT_REQUIRE(world_size >= 1 && world_size <= APT_MAX_BUCKETS, APT_ELIMIT,
              "apt_map_to_vir: world_size %d outside [1, %d]", world_size, APT_MAX_BUCKETS);
  APT_REQUIRE(id_offset >= 0 && id_offset < world_size && rank >= 0 && rank < world_size, APT_EINVAL,
              "apt_map_to_vir: id_offset / rank outside [0, %d)", world_size);
  const int64_t n = (dst != nullptr ? num_dst : 0) + num_src;
  if (n == 0) return APT_OK;
  APT_REQUIRE(min_vids != nullptr && vir_nodes != nullptr && (src != nullptr || num_src == 0), APT_EINVAL,
              "apt_map_to_vir: a pointer is NULL");
  VirParams p{dst, num_dst, src, num_src, fanout, min_vids, world_size, id_offset, rank, node_beg, node_end,
              vir_nodes};
  const unsigned blocks = static_cast<unsigned>(std::min<int64_t>(ceil_div(n, kBktBlock), 1 << 16));
  hipLaunchKernelGGL(map_to_vir_kernel, dim3(blocks), dim3(kBktBlock), 0, static_cast<hipStream_t>(stream), p);
  APT_LAUNCH_CHECK("map_to_vir_kernel");
  return APT_OK;
}

extern "C" int apt_vir_send_offset(int world_size, int64_t base, const int64_t* sorted_nodes,
                                   int64_t num_sorted, const int64_t* unique_nodes, int64_t num_unique,
                                   int with_dst, int64_t* send_offset, void* stream) {
  using namespace apt;
  APT_REQUIRE(world_size >= 1 && world_size <= APT_MAX_BUCKETS, APT_ELIMIT,
              "apt_vir_send_offset: world_size %d outside [1, %d]", world_size, APT_MAX_BUCKETS);
  APT_REQUIRE(num_sorted >= 0 && num_unique >= 0 && base >= 0, APT_EINVAL, "apt_vir_send_offset: negative size");
  APT_REQUIRE(send_offset != nullptr && (sorted_nodes != nullptr || num_sorted == 0) &&
                  (unique_nodes != nullptr || num_unique == 0),
              APT_EINVAL, "apt_vir_send_offset: a pointer is NULL");
  hipStream_t st = static_cast<hipStream_t>(stream);
  // boundaries of the sorted virtual nodes, then of the unique ones
  const int a_count = (with_dst ? 2 : 1) * world_size + 1;
  const int b_first = with_dst ? world_size + 1 : 1;
  hipLaunchKernelGGL(vir_lower_bound_kernel, dim3(1), dim3(256), 0, st, sorted_nodes, num_sorted, base, 0,
                     a_count, send_offset);
  APT_LAUNCH_CHECK("vir_lower_bound_kernel");
  hipLaunchKernelGGL(vir_lower_bound_kernel, dim3(1), dim3(256), 0, st, unique_nodes, num_unique, base, b_first,
                     world_size, send_offset + a_count);
  APT_LAUNCH_CHECK("vir_lower_bound_kernel");
  return APT_OK;
}
