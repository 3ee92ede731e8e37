// Relabel seeds + sampled neighbours to compact ids, first-occurrence order.
//
// Replaces RelabelHashmap / Unique<int64,true> / Relabel<int64> /
// TensorRelabelCSC (reference src/cuda/relabel.cu:7-185).  Same result
// (unique = distinct values of cat(seeds, neighbors) ordered by first
// occurrence; relabeled[j] = rank of neighbors[j]); different mechanics:
//   * no torch::cat: the item list is addressed as seeds ++ neighbors;
//   * one global open-addressing table (multiplicative hash, linear probing,
//     load <= 1/2) whose slot is remembered per item, so the later passes do
//     not probe again (the reference re-probes in each of its 3 passes);
//   * owner flags are compacted with wave ballots + popcounts and a two-level
//     block prefix (no spin-waiting between workgroups, no temp allocation)
//     instead of a device-wide cub scan over a materialised flag array;
//   * the count stays on the device unless the caller asks for it.
// Passes: fill -> insert -> count owners per block -> place owners -> relabel.
#include "common.hpp"

namespace apt {

constexpr int kRelBlock = 256;
constexpr int kRelItemsPerThread = 4;
constexpr int kRelTile = kRelBlock * kRelItemsPerThread;  // items per block in count/place
constexpr int64_t kRelMaxItems = (1LL << 30);

struct RelabelLayout {
  size_t keys_off, minidx_off, val_off, slot_off, blockcnt_off, total;
  uint64_t cap_max;
  int64_t blocks_max;
};

static inline uint64_t table_capacity(int64_t items) {
  uint64_t cap = 1024;
  while (cap < static_cast<uint64_t>(items) * 2) cap <<= 1;
  return cap;
}

static inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

static RelabelLayout relabel_layout(int64_t items) {
  RelabelLayout L;
  L.cap_max = table_capacity(items);
  L.blocks_max = ceil_div(items > 0 ? items : 1, kRelTile);
  size_t off = 0;
  L.keys_off = off;   off = align_up(off + L.cap_max * sizeof(int64_t), 256);
  // minidx directly follows keys so one fill covers both (all bytes 0xFF).
  L.minidx_off = off; off = align_up(off + L.cap_max * sizeof(uint32_t), 256);
  L.val_off = off;    off = align_up(off + L.cap_max * sizeof(uint32_t), 256);
  L.slot_off = off;   off = align_up(off + static_cast<size_t>(items > 0 ? items : 1) * sizeof(uint32_t), 256);
  L.blockcnt_off = off; off = align_up(off + static_cast<size_t>(L.blocks_max) * sizeof(uint32_t), 256);
  L.total = off;
  return L;
}

struct RelabelParams {
  const int64_t* seeds;
  int64_t ns;               // host-side (upper bound when ns_dev != NULL)
  const int64_t* ns_dev;
  const int64_t* neighbors;
  int64_t nn;               // host-side (upper bound)
  int64_t stride;           // neighbours per seed when ns_dev != NULL
  int64_t* keys;
  uint32_t* minidx;
  uint32_t* val;
  uint32_t* slot_of;
  uint32_t* block_cnt;
  int64_t* unique;
  int64_t* relabeled;
  int64_t* num_unique;
};

// Actual sizes (device-side seed count narrows both lists).
struct RelSizes {
  int64_t ns, nn, items;
  uint64_t mask;
  int shift;
};

__device__ __forceinline__ RelSizes rel_sizes(const RelabelParams& p) {
  RelSizes s;
  s.ns = p.ns;
  s.nn = p.nn;
  if (p.ns_dev != nullptr) {
    s.ns = actual_count(p.ns, p.ns_dev);
    const int64_t want = s.ns * p.stride;
    s.nn = want < p.nn ? want : p.nn;
  }
  s.items = s.ns + s.nn;
  uint64_t cap = 1024;
  int bits = 10;
  while (cap < static_cast<uint64_t>(s.items) * 2) { cap <<= 1; ++bits; }
  s.mask = cap - 1;
  s.shift = 64 - bits;
  return s;
}

__device__ __forceinline__ int64_t item_at(const RelabelParams& p, const RelSizes& s,
                                           int64_t i) {
  return i < s.ns ? p.seeds[i] : p.neighbors[i - s.ns];
}

__device__ __forceinline__ uint64_t hash_slot(int64_t key, const RelSizes& s) {
  return (static_cast<uint64_t>(key) * 0x9E3779B97F4A7C15ull) >> s.shift;
}

// keys := -1 and minidx := 0xFFFFFFFF, over the actual capacity only.
__global__ __launch_bounds__(kRelBlock) void relabel_fill_kernel(RelabelParams p) {
  const RelSizes s = rel_sizes(p);
  const uint64_t cap = s.mask + 1;
  // keys: cap * 8 bytes, minidx: cap * 4 bytes; both as 16-byte stores.
  const uint64_t key_vecs = cap / 2;      // 2 int64 per 16 B
  const uint64_t idx_vecs = cap / 4;      // 4 uint32 per 16 B
  const uint64_t total = key_vecs + idx_vecs;
  const uint4 ones = make_uint4(~0u, ~0u, ~0u, ~0u);
  uint4* kv = reinterpret_cast<uint4*>(p.keys);
  uint4* iv = reinterpret_cast<uint4*>(p.minidx);
  for (uint64_t i = static_cast<uint64_t>(blockIdx.x) * kRelBlock + threadIdx.x; i < total;
       i += static_cast<uint64_t>(gridDim.x) * kRelBlock) {
    if (i < key_vecs) kv[i] = ones;
    else iv[i - key_vecs] = ones;
  }
}

// Insert every item; the smallest item index per key wins (reference
// relabel.cu:12-24: CAS on the key, AtomicMin on the index).
__global__ __launch_bounds__(kRelBlock) void relabel_insert_kernel(RelabelParams p) {
  const RelSizes s = rel_sizes(p);
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kRelBlock + threadIdx.x; i < s.items;
       i += static_cast<int64_t>(gridDim.x) * kRelBlock) {
    const int64_t key = item_at(p, s, i);
    if (key < 0) continue;  // padding
    uint64_t slot = hash_slot(key, s);
    unsigned long long* keys = reinterpret_cast<unsigned long long*>(p.keys);
    while (true) {
      // Plain look first: repeated ids (hubs) mostly find their key in place
      // and skip the atomic.
      int64_t cur = __builtin_nontemporal_load(&p.keys[slot]);
      if (cur == -1)
        cur = static_cast<int64_t>(atomicCAS(&keys[slot], ~0ull, static_cast<unsigned long long>(key)));
      if (cur == -1 || cur == key) break;
      slot = (slot + 1) & s.mask;
    }
    const uint32_t me = static_cast<uint32_t>(i);
    // Indices only decrease, so a stale larger value costs one extra atomic
    // and a smaller one means this item cannot be the owner.
    if (__builtin_nontemporal_load(&p.minidx[slot]) > me) atomicMin(&p.minidx[slot], me);
    p.slot_of[i] = static_cast<uint32_t>(slot);
  }
}

__device__ __forceinline__ bool is_owner(const RelabelParams& p, const RelSizes& s, int64_t i) {
  if (i >= s.items) return false;
  if (item_at(p, s, i) < 0) return false;
  return p.minidx[p.slot_of[i]] == static_cast<uint32_t>(i);
}

// Owners per tile of kRelTile consecutive items.
__global__ __launch_bounds__(kRelBlock) void relabel_count_kernel(RelabelParams p) {
  const RelSizes s = rel_sizes(p);
  const int64_t base = static_cast<int64_t>(blockIdx.x) * kRelTile;
  if (base >= s.items) return;
  __shared__ uint32_t s_wave[kRelBlock / kWave];
  uint32_t c = 0;
#pragma unroll
  for (int it = 0; it < kRelItemsPerThread; ++it) {
    const bool own = is_owner(p, s, base + it * kRelBlock + threadIdx.x);
    c += __popcll(ballot(own));
  }
  if (lane_id() == 0) s_wave[threadIdx.x / kWave] = c;
  __syncthreads();
  if (threadIdx.x == 0) {
    uint32_t t = 0;
    for (int w = 0; w < kRelBlock / kWave; ++w) t += s_wave[w];
    p.block_cnt[blockIdx.x] = t;
  }
}

// Exclusive prefix of owner flags -> unique[] and the table's value column.
__global__ __launch_bounds__(kRelBlock) void relabel_place_kernel(RelabelParams p) {
  const RelSizes s = rel_sizes(p);
  const int64_t base = static_cast<int64_t>(blockIdx.x) * kRelTile;
  const int64_t tiles = (s.items + kRelTile - 1) / kRelTile;
  if (s.items == 0) {
    if (blockIdx.x == 0 && threadIdx.x == 0) *p.num_unique = 0;
    return;
  }
  if (base >= s.items) return;
  __shared__ int64_t s_red[kRelBlock / kWave];
  __shared__ uint32_t s_wcnt[kRelItemsPerThread][kRelBlock / kWave];
  const int wave = threadIdx.x / kWave;
  const int lane = lane_id();

  // Offset of this tile = owners in all earlier tiles.
  int64_t part = 0;
  for (int64_t b = threadIdx.x; b < blockIdx.x; b += kRelBlock) part += p.block_cnt[b];
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) part += __shfl_down(part, off, kWave);
  if (lane == 0) s_red[wave] = part;

  bool own[kRelItemsPerThread];
  uint64_t mask[kRelItemsPerThread];
#pragma unroll
  for (int it = 0; it < kRelItemsPerThread; ++it) {
    own[it] = is_owner(p, s, base + it * kRelBlock + threadIdx.x);
    mask[it] = ballot(own[it]);
    if (lane == 0) s_wcnt[it][wave] = __popcll(mask[it]);
  }
  __syncthreads();
  int64_t running = 0;
  for (int w = 0; w < kRelBlock / kWave; ++w) running += s_red[w];
#pragma unroll
  for (int it = 0; it < kRelItemsPerThread; ++it) {
    int64_t before = running;
    for (int w = 0; w < kRelBlock / kWave; ++w) {
      const uint32_t c = s_wcnt[it][w];
      if (w < wave) before += c;
      running += c;
    }
    if (own[it]) {
      const int64_t i = base + it * kRelBlock + threadIdx.x;
      const int64_t rank = before + rank_below(mask[it]);
      p.unique[rank] = item_at(p, s, i);
      p.val[p.slot_of[i]] = static_cast<uint32_t>(rank);
    }
  }
  if (blockIdx.x == tiles - 1 && threadIdx.x == 0) *p.num_unique = running;
}

// relabeled[j] = rank of neighbors[j] (reference relabel.cu:153-173).
__global__ __launch_bounds__(kRelBlock) void relabel_lookup_kernel(RelabelParams p) {
  const RelSizes s = rel_sizes(p);
  for (int64_t j = static_cast<int64_t>(blockIdx.x) * kRelBlock + threadIdx.x; j < s.nn;
       j += static_cast<int64_t>(gridDim.x) * kRelBlock) {
    const int64_t key = p.neighbors[j];
    p.relabeled[j] = key < 0 ? key : static_cast<int64_t>(p.val[p.slot_of[s.ns + j]]);
  }
}

}  // namespace apt

extern "C" size_t apt_relabel_workspace_bytes(int64_t num_items) {
  if (num_items < 0 || num_items > apt::kRelMaxItems) return 0;
  return apt::relabel_layout(num_items).total;
}

extern "C" int apt_relabel(const int64_t* seeds, int64_t num_seeds,
                           const int64_t* num_seeds_dev, const int64_t* neighbors,
                           int64_t num_neighbors, int64_t neighbor_stride,
                           int64_t* unique, int64_t* relabeled, int64_t* num_unique_dev,
                           int64_t* num_unique_host, void* workspace,
                           size_t workspace_bytes, void* stream) {
  using namespace apt;
  APT_REQUIRE(num_seeds >= 0 && num_neighbors >= 0, APT_EINVAL,
              "apt_relabel: negative size (%lld seeds, %lld neighbors)",
              (long long)num_seeds, (long long)num_neighbors);
  const int64_t items = num_seeds + num_neighbors;
  APT_REQUIRE(items <= kRelMaxItems, APT_ELIMIT,
              "apt_relabel: %lld items exceed the supported maximum %lld per call",
              (long long)items, (long long)kRelMaxItems);
  APT_REQUIRE(num_unique_dev != nullptr, APT_EINVAL, "apt_relabel: num_unique_dev is NULL");
  APT_REQUIRE(num_seeds == 0 || seeds != nullptr, APT_EINVAL, "apt_relabel: seeds is NULL");
  APT_REQUIRE(num_neighbors == 0 || (neighbors != nullptr && relabeled != nullptr), APT_EINVAL,
              "apt_relabel: neighbors/relabeled is NULL");
  APT_REQUIRE(items == 0 || unique != nullptr, APT_EINVAL, "apt_relabel: unique is NULL");
  APT_REQUIRE(num_seeds_dev == nullptr || neighbor_stride >= 0, APT_EINVAL,
              "apt_relabel: neighbor_stride %lld < 0", (long long)neighbor_stride);
  const RelabelLayout L = relabel_layout(items);
  APT_REQUIRE(workspace != nullptr && workspace_bytes >= L.total, APT_EWORKSPACE,
              "apt_relabel: workspace of %zu bytes, %zu needed", workspace_bytes, L.total);
  APT_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 15) == 0, APT_EINVAL,
              "apt_relabel: workspace must be 16-byte aligned");

  char* ws = static_cast<char*>(workspace);
  RelabelParams p;
  p.seeds = seeds;
  p.ns = num_seeds;
  p.ns_dev = num_seeds_dev;
  p.neighbors = neighbors;
  p.nn = num_neighbors;
  p.stride = neighbor_stride;
  p.keys = reinterpret_cast<int64_t*>(ws + L.keys_off);
  p.minidx = reinterpret_cast<uint32_t*>(ws + L.minidx_off);
  p.val = reinterpret_cast<uint32_t*>(ws + L.val_off);
  p.slot_of = reinterpret_cast<uint32_t*>(ws + L.slot_off);
  p.block_cnt = reinterpret_cast<uint32_t*>(ws + L.blockcnt_off);
  p.unique = unique;
  p.relabeled = relabeled;
  p.num_unique = num_unique_dev;

  hipStream_t st = static_cast<hipStream_t>(stream);
  const unsigned fill_blocks =
      static_cast<unsigned>(std::min<int64_t>(ceil_div((int64_t)(L.cap_max * 3 / 4), kRelBlock), 8192));
  const unsigned item_blocks =
      static_cast<unsigned>(std::min<int64_t>(ceil_div(items > 0 ? items : 1, kRelBlock), 65536));
  const unsigned tile_blocks = static_cast<unsigned>(L.blocks_max);

  hipLaunchKernelGGL(relabel_fill_kernel, dim3(fill_blocks), dim3(kRelBlock), 0, st, p);
  APT_LAUNCH_CHECK("relabel_fill_kernel");
  if (items > 0) {
    hipLaunchKernelGGL(relabel_insert_kernel, dim3(item_blocks), dim3(kRelBlock), 0, st, p);
    APT_LAUNCH_CHECK("relabel_insert_kernel");
    hipLaunchKernelGGL(relabel_count_kernel, dim3(tile_blocks), dim3(kRelBlock), 0, st, p);
    APT_LAUNCH_CHECK("relabel_count_kernel");
  }
  hipLaunchKernelGGL(relabel_place_kernel, dim3(tile_blocks), dim3(kRelBlock), 0, st, p);
  APT_LAUNCH_CHECK("relabel_place_kernel");
  if (num_neighbors > 0) {
    const unsigned nb =
        static_cast<unsigned>(std::min<int64_t>(ceil_div(num_neighbors, kRelBlock), 65536));
    hipLaunchKernelGGL(relabel_lookup_kernel, dim3(nb), dim3(kRelBlock), 0, st, p);
    APT_LAUNCH_CHECK("relabel_lookup_kernel");
  }
  if (num_unique_host != nullptr) {
    APT_HIP(hipMemcpyAsync(num_unique_host, num_unique_dev, sizeof(int64_t),
                           hipMemcpyDeviceToHost, st));
    APT_HIP(hipStreamSynchronize(st));
  }
  return APT_OK;
}
