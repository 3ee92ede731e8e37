// Relabel seeds + sampled neighbours to compact ids, first-occurrence order.
//
// Replaces RelabelHashmap / Unique<int64,true> / Relabel<int64> /
// TensorRelabelCSC (reference src/cuda/relabel.cu:7-185).  Same result
// (unique = distinct values of cat(seeds, neighbors) ordered by first
// occurrence; relabeled[j] = rank of neighbors[j]); different mechanics:
//   * no torch::cat: the item list is addressed as seeds ++ neighbors;
//   * one global open-addressing table (multiplicative hash, linear probing,
//     load <= 1/2) of 64-bit words (tag of the key, index of the key's first
//     item so far).  A new key costs one load and one CAS, a repeated key a
//     load and a look at the item the word points to; the reference (and a
//     key column + index column layout) pays a CAS on the key and an atomicMin
//     on the index for every item, and random atomics are the scarcest
//     resource here (~24 G/s against ~50 G/s for loads);
//   * who owns a key is settled inside the insert pass: a CAS that lowers a
//     word's index knows which item it displaced and flags it, so afterwards
//     "owner" = claimed or lowered a word and was never flagged, read from two
//     byte arrays in item order; the reference re-probes the table in each of
//     its 3 passes;
//   * owner flags are compacted with wave ballots + popcounts and a two-level
//     block prefix (no spin-waiting between workgroups, no temp allocation)
//     instead of a device-wide cub scan over a materialised flag array;
//   * the slot of every item is remembered, owners write their ids straight to
//     the output and into their slot, so only repeated keys go back to the table;
//   * the count stays on the device unless the caller asks for it.
// Passes: fill -> insert -> count owners per block -> place owners -> relabel.
#include <mutex>

#include "common.hpp"

namespace apt {

constexpr int kRelBlock = 256;
constexpr int kRelItemsPerThread = 4;
constexpr int kRelTile = kRelBlock * kRelItemsPerThread;  // items per block in count/place
constexpr int64_t kRelMaxItems = (1LL << 30);

struct RelabelLayout {
  size_t table_off, state_off, displaced_off, slot_off, blockcnt_off, total;
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
  L.table_off = off;  off = align_up(off + L.cap_max * sizeof(uint64_t), 256);
  // one byte per item each; separate arrays because different threads write them
  L.state_off = off;  off = align_up(off + static_cast<size_t>(items > 0 ? items : 1), 256);
  L.displaced_off = off; off = align_up(off + static_cast<size_t>(items > 0 ? items : 1), 256);
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
  unsigned long long* table;  // per slot: (tag << 32) | item index, later (tag << 32) | id
  uint8_t* state;             // per item, written by its own thread
  uint8_t* displaced;         // per item, written by the thread that took its key over
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

constexpr unsigned long long kEmptyWord = ~0ull;
constexpr uint8_t kItemPadding = 0;   // negative id: takes no part
constexpr uint8_t kItemFirst = 1;     // claimed or lowered its key's word: owner unless displaced later
constexpr uint8_t kItemRepeat = 2;    // an item with a smaller index holds the key

__device__ __forceinline__ uint32_t key_tag(int64_t key) {
  return static_cast<uint32_t>((static_cast<uint64_t>(key) * 0xD6E8FEB86659FD93ull) >> 32);
}

// table := empty, displaced := 0, over the actual sizes only.
__global__ __launch_bounds__(kRelBlock) void relabel_fill_kernel(RelabelParams p) {
  const RelSizes s = rel_sizes(p);
  const uint64_t table_vecs = (s.mask + 1) / 2;                                  // 2 words per 16 B
  const uint64_t flag_vecs = (static_cast<uint64_t>(s.items) + 15) / 16;         // the array is padded to 256 B
  const uint64_t total = table_vecs + flag_vecs;
  const uint4 ones = make_uint4(~0u, ~0u, ~0u, ~0u);
  const uint4 zero = make_uint4(0u, 0u, 0u, 0u);
  uint4* tv = reinterpret_cast<uint4*>(p.table);
  uint4* fv = reinterpret_cast<uint4*>(p.displaced);
  for (uint64_t i = static_cast<uint64_t>(blockIdx.x) * kRelBlock + threadIdx.x; i < total;
       i += static_cast<uint64_t>(gridDim.x) * kRelBlock) {
    if (i < table_vecs) tv[i] = ones;
    else fv[i - table_vecs] = zero;
  }
}

// Insert every item; the smallest item index per key ends up in the key's word
// (reference relabel.cu:12-24: CAS on the key, AtomicMin on the index).
__global__ __launch_bounds__(kRelBlock) void relabel_insert_kernel(RelabelParams p) {
  const RelSizes s = rel_sizes(p);
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kRelBlock + threadIdx.x; i < s.items;
       i += static_cast<int64_t>(gridDim.x) * kRelBlock) {
    const int64_t key = item_at(p, s, i);
    if (key < 0) {  // padding
      p.state[i] = kItemPadding;
      continue;
    }
    const uint32_t tag = key_tag(key);
    const unsigned long long mine = (static_cast<unsigned long long>(tag) << 32) | static_cast<uint32_t>(i);
    uint64_t slot = hash_slot(key, s);
    uint8_t state;
    // A read may be stale; it then shows the slot empty or its key with an
    // older, larger index, and the CAS that follows fails and returns the truth.
    unsigned long long w = __builtin_nontemporal_load(&p.table[slot]);
    while (true) {
      if (w == kEmptyWord) {
        w = atomicCAS(&p.table[slot], kEmptyWord, mine);
        if (w == kEmptyWord) {
          state = kItemFirst;
          break;
        }
      }
      const uint32_t other = static_cast<uint32_t>(w);
      if (static_cast<uint32_t>(w >> 32) == tag && item_at(p, s, other) == key) {
        if (other < static_cast<uint32_t>(i)) {
          state = kItemRepeat;
          break;
        }
        // the word points at a later item of this key: take it over
        const unsigned long long seen = atomicCAS(&p.table[slot], w, mine);
        if (seen == w) {
          p.displaced[other] = 1;
          state = kItemFirst;
          break;
        }
        w = seen;  // somebody else lowered it meanwhile: look again at the same slot
        continue;
      }
      slot = (slot + 1) & s.mask;
      w = __builtin_nontemporal_load(&p.table[slot]);
    }
    p.state[i] = state;
    p.slot_of[i] = static_cast<uint32_t>(slot);
  }
}

// Every lowering of a word is a CAS that flags the item it replaces, so the one
// item of a key that is never flagged is the one with the smallest index.
__device__ __forceinline__ bool is_owner(const RelabelParams& p, const RelSizes& s, int64_t i) {
  return i < s.items && p.state[i] == kItemFirst && p.displaced[i] == 0;
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

// Exclusive prefix of owner flags -> unique[], the owners' own outputs, and the
// id in the key's word for the repeats.
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
      if (i >= s.ns) p.relabeled[i - s.ns] = rank;
      // low half of the word: the id, for the key's other items
      reinterpret_cast<uint32_t*>(&p.table[p.slot_of[i]])[0] = static_cast<uint32_t>(rank);
    }
  }
  if (blockIdx.x == tiles - 1 && threadIdx.x == 0) *p.num_unique = running;
}

// relabeled[j] for the neighbours that are not the first item of their key
// (reference relabel.cu:153-173); padding passes through.
__global__ __launch_bounds__(kRelBlock) void relabel_lookup_kernel(RelabelParams p) {
  const RelSizes s = rel_sizes(p);
  for (int64_t j = static_cast<int64_t>(blockIdx.x) * kRelBlock + threadIdx.x; j < s.nn;
       j += static_cast<int64_t>(gridDim.x) * kRelBlock) {
    const int64_t i = s.ns + j;
    const uint8_t st = p.state[i];
    if (st == kItemPadding) p.relabeled[j] = p.neighbors[j];
    else if (st == kItemRepeat || p.displaced[i] != 0)
      p.relabeled[j] = static_cast<int64_t>(static_cast<uint32_t>(p.table[p.slot_of[i]]));
  }
}

// ---------------------------------------------------------------------------
// Small inputs (the first hop of a batch, hops of small batches): the whole
// relabel in one workgroup with the hash table in LDS, one launch instead of
// five and no global atomics.  The item keys are copied into LDS (64 KB for
// 8192 items); the table (2 slots per item, 4 bytes each: the index of the
// key's first item so far) takes another 64 KB.  A probe compares keys through
// the index a slot holds; claiming an empty slot is a CAS, lowering the index
// of a key that is already there an atomic minimum, both on LDS.  After a
// barrier an item owns its key iff its slot holds its own index; owners are
// ranked with ballots and a prefix over the workgroup's wavefronts, write their
// ids to the output and leave their rank in the slot for the key's other items.
constexpr int kLdsRelBlock = 1024;
constexpr int kLdsRelMaxItems = 8192;
constexpr int kLdsRelSlots = 2 * kLdsRelMaxItems;
constexpr int kLdsRelPerThread = kLdsRelMaxItems / kLdsRelBlock;
constexpr uint32_t kLdsEmpty = 0xFFFFFFFFu;
int tuning_relabel_lds();  // 1 (default) = inputs that fit take the LDS path

__global__ __launch_bounds__(kLdsRelBlock) void relabel_lds_kernel(RelabelParams p) {
  __shared__ int64_t s_key[kLdsRelMaxItems];
  __shared__ uint32_t s_table[kLdsRelSlots];
  __shared__ uint32_t s_wave[kLdsRelPerThread][kLdsRelBlock / kWave];
  const RelSizes s = rel_sizes(p);   // items <= kLdsRelMaxItems (the host checked the upper bounds)
  const int tid = threadIdx.x;
  const int lane = lane_id(), wave = tid / kWave;
  // Few values live per thread (a slot per item and a bit mask): keys are read back from LDS where needed,
  // so that nothing spills.  The keys are requested first, the table is cleared while they are on their way.
  {
    int64_t key[kLdsRelPerThread];
#pragma unroll
    for (int k = 0; k < kLdsRelPerThread; ++k) {
      const int i = k * kLdsRelBlock + tid;
      key[k] = i < s.items ? item_at(p, s, i) : -1;
    }
    uint4* t4 = reinterpret_cast<uint4*>(s_table);
    const uint4 ones = make_uint4(kLdsEmpty, kLdsEmpty, kLdsEmpty, kLdsEmpty);
#pragma unroll
    for (int q = 0; q < kLdsRelSlots / 4 / kLdsRelBlock; ++q) t4[q * kLdsRelBlock + tid] = ones;
#pragma unroll
    for (int k = 0; k < kLdsRelPerThread; ++k) s_key[k * kLdsRelBlock + tid] = key[k];
  }
  __syncthreads();
  // Insert: the smallest item index per key ends up in the key's slot (a CAS claims an empty slot, an atomic
  // minimum lowers the index of a key that is already there).
  uint32_t slot[kLdsRelPerThread];
#pragma unroll
  for (int k = 0; k < kLdsRelPerThread; ++k) {
    const uint32_t i = static_cast<uint32_t>(k * kLdsRelBlock + tid);
    const int64_t key = s_key[i];
    slot[k] = kLdsEmpty;
    if (key < 0) continue;  // padding (and the items past the end)
    uint32_t q = static_cast<uint32_t>((static_cast<uint64_t>(key) * 0x9E3779B97F4A7C15ull) >> 50);  // 14 bits
    uint32_t cur = atomicCAS(&s_table[q], kLdsEmpty, i);   // what the slot held before
    while (cur != kLdsEmpty) {
      if (s_key[cur] == key) {  // whichever item of this key holds the slot now
        if (cur > i) atomicMin(&s_table[q], i);
        break;
      }
      q = (q + 1) & (kLdsRelSlots - 1);
      cur = atomicCAS(&s_table[q], kLdsEmpty, i);
    }
    slot[k] = q;
  }
  __syncthreads();
  // owners, in item order: round k covers items [k * 1024, (k + 1) * 1024)
  uint32_t own = 0;
#pragma unroll
  for (int k = 0; k < kLdsRelPerThread; ++k) {
    const uint32_t i = static_cast<uint32_t>(k * kLdsRelBlock + tid);
    const bool mine = slot[k] != kLdsEmpty && s_table[slot[k]] == i;
    own |= (mine ? 1u : 0u) << k;
    const uint64_t m = ballot(mine);
    if (lane == 0) s_wave[k][wave] = static_cast<uint32_t>(__popcll(m));
  }
  __syncthreads();   // every ownership read of the table is done: owners now leave their rank in their slot
  uint32_t running = 0;
#pragma unroll
  for (int k = 0; k < kLdsRelPerThread; ++k) {
    uint32_t before = running;
#pragma unroll
    for (int w = 0; w < kLdsRelBlock / kWave; ++w) {
      const uint32_t c = s_wave[k][w];
      if (w < wave) before += c;
      running += c;
    }
    const bool mine = (own >> k) & 1;
    const uint64_t m = ballot(mine);
    if (mine) s_table[slot[k]] = before + static_cast<uint32_t>(rank_below(m));
  }
  __syncthreads();
#pragma unroll
  for (int k = 0; k < kLdsRelPerThread; ++k) {
    const int64_t i = static_cast<int64_t>(k) * kLdsRelBlock + tid;
    if (i >= s.items) continue;
    const int64_t key = s_key[i];
    const uint32_t r = key < 0 ? 0 : s_table[slot[k]];
    if ((own >> k) & 1) p.unique[r] = key;
    if (i >= s.ns) p.relabeled[i - s.ns] = key < 0 ? key : static_cast<int64_t>(r);
  }
  if (tid == 0) *p.num_unique = running;
}

}  // namespace apt

extern "C" size_t apt_relabel_workspace_bytes(int64_t num_items) {
  if (num_items < 0 || num_items > apt::kRelMaxItems) return 0;
  return apt::relabel_layout(num_items).total;
}

namespace apt {

// Validation shared by the two entry points.
static int relabel_check_args(const char* who, const int64_t* seeds, int64_t num_seeds,
                              const int64_t* num_seeds_dev, const int64_t* neighbors,
                              int64_t num_neighbors, int64_t neighbor_stride, const int64_t* unique,
                              const int64_t* relabeled, const int64_t* num_unique_dev, int64_t max_items) {
  APT_REQUIRE(num_seeds >= 0 && num_neighbors >= 0, APT_EINVAL,
              "%s: negative size (%lld seeds, %lld neighbors)", who,
              (long long)num_seeds, (long long)num_neighbors);
  // each size on its own first: their sum must not wrap
  APT_REQUIRE(num_seeds <= max_items && num_neighbors <= max_items && num_seeds + num_neighbors <= max_items,
              APT_ELIMIT, "%s: %lld seeds + %lld neighbors exceed the supported maximum of %lld items per call",
              who, (long long)num_seeds, (long long)num_neighbors, (long long)max_items);
  const int64_t items = num_seeds + num_neighbors;
  APT_REQUIRE(num_unique_dev != nullptr, APT_EINVAL, "%s: num_unique_dev is NULL", who);
  APT_REQUIRE(num_seeds == 0 || seeds != nullptr, APT_EINVAL, "%s: seeds is NULL", who);
  APT_REQUIRE(num_neighbors == 0 || (neighbors != nullptr && relabeled != nullptr), APT_EINVAL,
              "%s: neighbors/relabeled is NULL", who);
  APT_REQUIRE(items == 0 || unique != nullptr, APT_EINVAL, "%s: unique is NULL", who);
  APT_REQUIRE(num_seeds_dev == nullptr || neighbor_stride >= 0, APT_EINVAL,
              "%s: neighbor_stride %lld < 0", who, (long long)neighbor_stride);
  return APT_OK;
}

// The five passes on `st`; `ws` holds relabel_layout(num_seeds + num_neighbors).total bytes
// whose contents do not matter on entry (the fill pass sets what must start clean).
static int relabel_enqueue(const int64_t* seeds, int64_t num_seeds, const int64_t* num_seeds_dev,
                           const int64_t* neighbors, int64_t num_neighbors, int64_t neighbor_stride,
                           int64_t* unique, int64_t* relabeled, int64_t* num_unique_dev, char* ws,
                           hipStream_t st) {
  const int64_t items = num_seeds + num_neighbors;
  if (items <= kLdsRelMaxItems && tuning_relabel_lds() != 0) {
    // the whole input fits one workgroup's LDS: one launch, no workspace
    RelabelParams q{};
    q.seeds = seeds;
    q.ns = num_seeds;
    q.ns_dev = num_seeds_dev;
    q.neighbors = neighbors;
    q.nn = num_neighbors;
    q.stride = neighbor_stride;
    q.unique = unique;
    q.relabeled = relabeled;
    q.num_unique = num_unique_dev;
    hipLaunchKernelGGL(relabel_lds_kernel, dim3(1), dim3(kLdsRelBlock), 0, st, q);
    APT_LAUNCH_CHECK("relabel_lds_kernel");
    return APT_OK;
  }
  const RelabelLayout L = relabel_layout(items);
  RelabelParams p;
  p.seeds = seeds;
  p.ns = num_seeds;
  p.ns_dev = num_seeds_dev;
  p.neighbors = neighbors;
  p.nn = num_neighbors;
  p.stride = neighbor_stride;
  p.table = reinterpret_cast<unsigned long long*>(ws + L.table_off);
  p.state = reinterpret_cast<uint8_t*>(ws + L.state_off);
  p.displaced = reinterpret_cast<uint8_t*>(ws + L.displaced_off);
  p.slot_of = reinterpret_cast<uint32_t*>(ws + L.slot_off);
  p.block_cnt = reinterpret_cast<uint32_t*>(ws + L.blockcnt_off);
  p.unique = unique;
  p.relabeled = relabeled;
  p.num_unique = num_unique_dev;

  const unsigned fill_blocks =
      static_cast<unsigned>(std::min<int64_t>(ceil_div((int64_t)(L.cap_max / 2 + (items + 15) / 16), kRelBlock), 8192));
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
  return APT_OK;
}

}  // namespace apt

extern "C" int apt_relabel(const int64_t* seeds, int64_t num_seeds,
                           const int64_t* num_seeds_dev, const int64_t* neighbors,
                           int64_t num_neighbors, int64_t neighbor_stride,
                           int64_t* unique, int64_t* relabeled, int64_t* num_unique_dev,
                           int64_t* num_unique_host, void* workspace,
                           size_t workspace_bytes, void* stream) {
  using namespace apt;
  int rc = relabel_check_args("apt_relabel", seeds, num_seeds, num_seeds_dev, neighbors, num_neighbors,
                              neighbor_stride, unique, relabeled, num_unique_dev, kRelMaxItems);
  if (rc != APT_OK) return rc;
  const RelabelLayout L = relabel_layout(num_seeds + num_neighbors);
  APT_REQUIRE(workspace != nullptr && workspace_bytes >= L.total, APT_EWORKSPACE,
              "apt_relabel: workspace of %zu bytes, %zu needed", workspace_bytes, L.total);
  APT_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 15) == 0, APT_EINVAL,
              "apt_relabel: workspace must be 16-byte aligned");
  hipStream_t st = static_cast<hipStream_t>(stream);
  rc = relabel_enqueue(seeds, num_seeds, num_seeds_dev, neighbors, num_neighbors, neighbor_stride, unique,
                       relabeled, num_unique_dev, static_cast<char*>(workspace), st);
  if (rc != APT_OK) return rc;
  if (num_unique_host != nullptr) {
    APT_HIP(hipMemcpyAsync(num_unique_host, num_unique_dev, sizeof(int64_t),
                           hipMemcpyDeviceToHost, st));
    APT_HIP(hipStreamSynchronize(st));
  }
  return APT_OK;
}

// ---------------------------------------------------------------------------
// apt_relabel_static: the same passes with the scratch in a fixed device array
// of this library, for callers that cannot allocate (code under HIP graph
// capture, serving loops, harnesses that forbid hipMalloc).  One array per GPU,
// held until the process ends; every call on a GPU shares it, so calls that
// overlap on one GPU (two streams, two threads) race.  Its contents after a call
// are the last call's: nothing needs clearing between calls, because the fill
// pass of every call resets exactly what its own passes read.
namespace apt {

constexpr int64_t kRelStaticMaxItems = int64_t{1} << 21;  // seeds + neighbours per call
// relabel_layout(kRelStaticMaxItems).total: a table of 2^22 words (32 MiB), 6 bytes per item, 8 KiB of tile counts
constexpr size_t kRelStaticBytes = (size_t{1} << 22) * 8 + (size_t{1} << 21) * 6 + (size_t{1} << 21) / kRelTile * 4;

static __device__ __align__(256) unsigned char scratch[kRelStaticBytes];

constexpr int kRelMaxDevices = 64;
static std::mutex g_scratch_mu;
static void* g_scratch_ptr[kRelMaxDevices] = {};  // per device: that GPU's copy of the array

// Device address of the current GPU's array (resolved once per device, under the lock).
static int static_scratch(char** out) {
  int dev = -1;
  APT_HIP(hipGetDevice(&dev));
  APT_REQUIRE(dev >= 0 && dev < kRelMaxDevices, APT_ELIMIT, "apt_relabel_static: device %d outside [0, %d)", dev,
              kRelMaxDevices);
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  if (g_scratch_ptr[dev] == nullptr) {
    void* ptr = nullptr;
    APT_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    APT_REQUIRE(ptr != nullptr && (reinterpret_cast<uintptr_t>(ptr) & 255) == 0, APT_EHIP,
                "apt_relabel_static: the scratch array resolved to %p on device %d", ptr, dev);
    g_scratch_ptr[dev] = ptr;
  }
  *out = static_cast<char*>(g_scratch_ptr[dev]);
  return APT_OK;
}

}  // namespace apt

extern "C" int64_t apt_relabel_static_max_items(void) { return apt::kRelStaticMaxItems; }

extern "C" int apt_relabel_static(const int64_t* seeds, int64_t num_seeds, const int64_t* num_seeds_dev,
                                  const int64_t* neighbors, int64_t num_neighbors, int64_t neighbor_stride,
                                  int64_t* unique, int64_t* relabeled, int64_t* num_unique_dev, void* stream) {
  using namespace apt;
  static_assert(kRelStaticBytes % 256 == 0, "scratch size keeps the layout's alignment");
  int rc = relabel_check_args("apt_relabel_static", seeds, num_seeds, num_seeds_dev, neighbors, num_neighbors,
                              neighbor_stride, unique, relabeled, num_unique_dev, kRelStaticMaxItems);
  if (rc != APT_OK) return rc;
  APT_REQUIRE(relabel_layout(num_seeds + num_neighbors).total <= kRelStaticBytes, APT_ELIMIT,
              "apt_relabel_static: %lld items need more than the %zu bytes of fixed scratch",
              (long long)(num_seeds + num_neighbors), kRelStaticBytes);
  char* ws = nullptr;
  rc = static_scratch(&ws);
  if (rc != APT_OK) return rc;
  return relabel_enqueue(seeds, num_seeds, num_seeds_dev, neighbors, num_neighbors, neighbor_stride, unique,
                         relabeled, num_unique_dev, ws, static_cast<hipStream_t>(stream));
}
