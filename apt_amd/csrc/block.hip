// Sparse formats of a sampled block.
//
// A hop leaves a fixed-stride block: relabeled[d * fanout + k] is the k-th
// source of destination d, -1 where d has fewer than fanout neighbours.  The
// reference hands (row, col) to DGL, which materialises COO, CSR and CSC
// (python/npc/sampler.py:59-69,76-91; create_block_from_csc :44-56 takes a CSC
// directly).  Here the three formats are emitted on the GPU, with device-side
// sizes and no host round trip:
//   COO  edges in destination-major order: row[e] = source, col[e] = destination
//   CSC  csc_indptr over destinations; its indices are COO row, edge ids 0..E-1
//   CSR  csr_indptr over sources, csr_indices = destination, csr_eids = COO
//        position, edges of one source in increasing edge id
// COO/CSC are a stream compaction (count per tile -> place).  CSR is a stable
// least-significant-digit radix sort of (source, edge id) by source, 8 bits per
// pass (histogram per tile -> scatter); a workgroup ranks its tile with wave
// ballots, so equal keys keep their order and the result is reproducible (no
// atomic tickets).  A block of a mini-batch has few tiles, so the place and
// scatter workgroups add up the counts of the tiles before them themselves
// (a few KB from L2) instead of waiting for a scan kernel: every launch saved
// is worth more than the arithmetic here.  Large inputs take separate scan
// launches.
#include "common.hpp"

namespace apt {

constexpr int kFmtBlock = 256;
constexpr int kFmtWaves = kFmtBlock / kWave;
constexpr int kCompactIters = 8;
constexpr int kCompactTile = kFmtBlock * kCompactIters;  // slots per workgroup
constexpr int kSortBlock = kFmtBlock;
constexpr int kSortWaves = kSortBlock / kWave;
constexpr int kSortRounds = 16;
constexpr int kSortWaveItems = kWave * kSortRounds;       // consecutive items of one wave
constexpr int kSortTile = kSortWaveItems * kSortWaves;    // items per workgroup
constexpr int64_t kFusedCompactTiles = 8192;              // up to here a workgroup sums the tile counts itself
constexpr int64_t kFusedSortTiles = 32;
constexpr int kRadixBits = 8;
constexpr int kRadix = 1 << kRadixBits;
static_assert(kRadix == kSortBlock, "one thread per digit");
constexpr int kScanPerThread = 16;
constexpr int kScanChunk = kFmtBlock * kScanPerThread;    // elements per workgroup of the scan

// ------------------------------------------------------------------ scan
// Exclusive prefix sum of a uint32 array in place, at most kScanChunk^2
// elements: chunk sums -> scan of the sums (one workgroup) -> rescan + offset.
__device__ __forceinline__ int64_t ceil_div_dev(int64_t a, int64_t b) { return (a + b - 1) / b; }

__device__ __forceinline__ uint32_t block_exclusive(uint32_t x, uint32_t* s_wave, uint32_t& all) {
  const int lane = lane_id();
  const int wave = threadIdx.x / kWave;
  uint32_t incl = x;
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) {
    const uint32_t y = __shfl_up(incl, off, kWave);
    if (lane >= off) incl += y;
  }
  __syncthreads();  // s_wave may still be read by the previous call
  if (lane == kWave - 1) s_wave[wave] = incl;
  __syncthreads();
  uint32_t before = 0;
  all = 0;
#pragma unroll
  for (int w = 0; w < kFmtWaves; ++w) {
    const uint32_t c = s_wave[w];
    if (w < wave) before += c;
    all += c;
  }
  return before + incl - x;
}

__global__ __launch_bounds__(kFmtBlock) void scan_sums_kernel(const uint32_t* __restrict__ data, int64_t n,
                                                              uint32_t* __restrict__ sums) {
  __shared__ uint32_t s_wave[kFmtWaves];
  const int64_t base = static_cast<int64_t>(blockIdx.x) * kScanChunk;
  uint32_t acc = 0;
#pragma unroll
  for (int k = 0; k < kScanPerThread; ++k) {
    const int64_t i = base + k * kFmtBlock + threadIdx.x;
    if (i < n) acc += data[i];
  }
  uint32_t all;
  block_exclusive(acc, s_wave, all);
  if (threadIdx.x == 0) sums[blockIdx.x] = all;
}

// One workgroup: sums[0..m) -> exclusive prefix, m <= kScanChunk; the grand
// total goes to total_a / total_b (either may be NULL).
__global__ __launch_bounds__(kFmtBlock) void scan_top_kernel(uint32_t* sums, int64_t m, int64_t* total_a,
                                                             int64_t* total_b) {
  __shared__ uint32_t s_wave[kFmtWaves];
  uint32_t v[kScanPerThread];
  uint32_t acc = 0;
#pragma unroll
  for (int k = 0; k < kScanPerThread; ++k) {
    const int64_t i = static_cast<int64_t>(threadIdx.x) * kScanPerThread + k;
    v[k] = i < m ? sums[i] : 0u;
    acc += v[k];
  }
  uint32_t all;
  uint32_t run = block_exclusive(acc, s_wave, all);
#pragma unroll
  for (int k = 0; k < kScanPerThread; ++k) {
    const int64_t i = static_cast<int64_t>(threadIdx.x) * kScanPerThread + k;
    if (i < m) sums[i] = run;
    run += v[k];
  }
  if (threadIdx.x == 0) {
    if (total_a != nullptr) *total_a = all;
    if (total_b != nullptr) *total_b = all;
  }
}

__global__ __launch_bounds__(kFmtBlock) void scan_apply_kernel(uint32_t* data, int64_t n,
                                                               const uint32_t* __restrict__ sums) {
  __shared__ uint32_t s_wave[kFmtWaves];
  const int64_t base = static_cast<int64_t>(blockIdx.x) * kScanChunk +
                       static_cast<int64_t>(threadIdx.x) * kScanPerThread;
  uint32_t v[kScanPerThread];
  uint32_t acc = 0;
#pragma unroll
  for (int k = 0; k < kScanPerThread; ++k) {
    v[k] = base + k < n ? data[base + k] : 0u;
    acc += v[k];
  }
  uint32_t all;
  uint32_t run = sums[blockIdx.x] + block_exclusive(acc, s_wave, all);
#pragma unroll
  for (int k = 0; k < kScanPerThread; ++k) {
    if (base + k < n) data[base + k] = run;
    run += v[k];
  }
}

// data[0..n) -> exclusive prefix in place; sums: scratch of ceil(n / kScanChunk) entries.
static int exclusive_scan(uint32_t* data, int64_t n, uint32_t* sums, int64_t* total_a, int64_t* total_b,
                          hipStream_t st) {
  const int64_t chunks = ceil_div(n, kScanChunk);
  APT_REQUIRE(chunks <= kScanChunk, APT_ELIMIT, "block formats: %lld counters exceed the scan's range",
              static_cast<long long>(n));
  if (chunks <= 1) {
    hipLaunchKernelGGL(scan_top_kernel, dim3(1), dim3(kFmtBlock), 0, st, data, n, total_a, total_b);
    APT_LAUNCH_CHECK("scan_top_kernel");
    return APT_OK;
  }
  hipLaunchKernelGGL(scan_sums_kernel, dim3(static_cast<unsigned>(chunks)), dim3(kFmtBlock), 0, st, data, n,
                     sums);
  APT_LAUNCH_CHECK("scan_sums_kernel");
  hipLaunchKernelGGL(scan_top_kernel, dim3(1), dim3(kFmtBlock), 0, st, sums, chunks, total_a, total_b);
  APT_LAUNCH_CHECK("scan_top_kernel");
  hipLaunchKernelGGL(scan_apply_kernel, dim3(static_cast<unsigned>(chunks)), dim3(kFmtBlock), 0, st, data, n,
                     sums);
  APT_LAUNCH_CHECK("scan_apply_kernel");
  return APT_OK;
}

// ------------------------------------------------------------ COO + CSC
struct CompactParams {
  const int64_t* relabeled;
  int64_t num_dst;            // upper bound
  const int64_t* num_dst_dev;
  int fanout;
  uint32_t* tile_cnt;         // [tiles]; after a scan launch: the tile's first edge
  int64_t tiles;
  bool scanned;               // tile_cnt went through exclusive_scan
  int64_t* num_edges_dev;
  int64_t* coo_row;
  int64_t* coo_col;
  int64_t* csc_indptr;        // [num_dst + 1]
};

__global__ __launch_bounds__(kFmtBlock) void fmt_count_kernel(CompactParams p) {
  __shared__ uint32_t s_wave[kFmtWaves];
  const int64_t slots = actual_count(p.num_dst, p.num_dst_dev) * p.fanout;
  const int64_t base = static_cast<int64_t>(blockIdx.x) * kCompactTile;
  uint32_t c = 0;
#pragma unroll
  for (int it = 0; it < kCompactIters; ++it) {
    const int64_t s = base + it * kFmtBlock + threadIdx.x;
    if (s < slots && p.relabeled[s] >= 0) ++c;
  }
  uint32_t all;
  block_exclusive(c, s_wave, all);
  if (threadIdx.x == 0) p.tile_cnt[blockIdx.x] = all;
}

__global__ __launch_bounds__(kFmtBlock) void fmt_place_kernel(CompactParams p) {
  __shared__ uint32_t s_cnt[kCompactIters * kFmtWaves];
  const int lane = lane_id();
  const int wave = threadIdx.x / kWave;
  const int64_t slots = actual_count(p.num_dst, p.num_dst_dev) * p.fanout;
  const int64_t upper = p.num_dst * p.fanout;
  const int64_t base = static_cast<int64_t>(blockIdx.x) * kCompactTile;
  int64_t v[kCompactIters];
  uint32_t below[kCompactIters];
#pragma unroll
  for (int it = 0; it < kCompactIters; ++it) {   // the tile's slots are all requested before the first is looked at
    const int64_t s = base + it * kFmtBlock + threadIdx.x;
    v[it] = s < slots ? p.relabeled[s] : -1;
  }
#pragma unroll
  for (int it = 0; it < kCompactIters; ++it) {
    const uint64_t m = ballot(v[it] >= 0);
    below[it] = rank_below(m);
    if (lane == 0) s_cnt[it * kFmtWaves + wave] = __popcll(m);
  }
  uint32_t first = 0;
  if (p.scanned) {
    first = p.tile_cnt[blockIdx.x];
  } else {
    // edges of the tiles before this one, and of all tiles
    __shared__ uint32_t s_wave[kFmtWaves];
    const int64_t active = ceil_div_dev(slots, kCompactTile);
    uint32_t before = 0, total = 0;
    for (int64_t t = threadIdx.x; t < active; t += kFmtBlock) {
      const uint32_t c = p.tile_cnt[t];
      total += c;
      if (t < blockIdx.x) before += c;
    }
    uint32_t all_before, all_total;
    block_exclusive(before, s_wave, all_before);
    block_exclusive(total, s_wave, all_total);
    first = all_before;
    if (blockIdx.x == 0 && threadIdx.x == 0) {
      *p.num_edges_dev = all_total;
      p.csc_indptr[p.num_dst] = all_total;
    }
  }
  __syncthreads();
  static_assert(kCompactIters * kFmtWaves <= kWave, "one wavefront scans the tile's per-wave counts");
  if (wave == 0) {   // exclusive prefix of the (iteration, wave) counts, in the order the edges are numbered
    const uint32_t c = lane < kCompactIters * kFmtWaves ? s_cnt[lane] : 0u;
    uint32_t incl = c;
#pragma unroll
    for (int off = 1; off < kCompactIters * kFmtWaves; off <<= 1) {
      const uint32_t y = __shfl_up(incl, off, kWave);
      if (lane >= off) incl += y;
    }
    if (lane < kCompactIters * kFmtWaves) s_cnt[lane] = first + incl - c;
  }
  __syncthreads();
#pragma unroll
  for (int it = 0; it < kCompactIters; ++it) {
    const int64_t s = base + it * kFmtBlock + threadIdx.x;
    if (s >= upper) continue;
    const int64_t e = static_cast<int64_t>(s_cnt[it * kFmtWaves + wave]) + below[it];
    // (slot numbers fit 32 bits, fmt_sizes_ok: a 32-bit division, a fraction of the cost of a 64-bit one)
    const uint32_t fan = static_cast<uint32_t>(p.fanout);
    const uint32_t d = static_cast<uint32_t>(s) / fan;
    // Valid slots before the first slot of a destination = its CSC offset;
    // destinations past the device-side count get the edge total (empty rows).
    if (static_cast<uint32_t>(s) - d * fan == 0) p.csc_indptr[d] = e;
    if (v[it] >= 0) {
      p.coo_row[e] = v[it];
      p.coo_col[e] = d;
    }
  }
}

// ------------------------------------------------------------------- CSR
struct SortParams {
  const int64_t* coo_row;     // keys of the first pass
  const int64_t* coo_col;
  const int64_t* num_edges_dev;
  int64_t max_edges;
  const uint32_t* key_in;     // later passes
  const uint32_t* pay_in;
  uint32_t* key_out;
  uint32_t* pay_out;
  // fused: [tiles][kRadix] counts; else [kRadix][tiles], each digit's row scanned over tiles
  uint32_t* tile_hist;
  uint32_t* bin_total;        // [kRadix] (not fused)
  int64_t tiles;
  bool fused;
  int shift;
  int64_t* csr_indices;       // last pass
  int64_t* csr_eids;
};

template <bool FIRST>
__device__ __forceinline__ uint32_t sort_key(const SortParams& p, int64_t i) {
  return FIRST ? static_cast<uint32_t>(p.coo_row[i]) : p.key_in[i];
}

template <bool FIRST>
__global__ __launch_bounds__(kSortBlock) void radix_hist_kernel(SortParams p) {
  __shared__ uint32_t s_hist[kRadix];
  const int tid = threadIdx.x;
  s_hist[tid] = 0;
  __syncthreads();
  const int64_t n = actual_count(p.max_edges, p.num_edges_dev);
  const int64_t base = static_cast<int64_t>(blockIdx.x) * kSortTile;
  // all of a thread's keys are requested before the first is counted
  uint32_t key[kSortTile / kSortBlock];
#pragma unroll
  for (int k = 0; k < kSortTile / kSortBlock; ++k) {
    const int64_t i = base + k * kSortBlock + tid;
    key[k] = i < n ? sort_key<FIRST>(p, i) : 0u;
  }
#pragma unroll
  for (int k = 0; k < kSortTile / kSortBlock; ++k)
    if (base + k * kSortBlock + tid < n) atomicAdd(&s_hist[(key[k] >> p.shift) & (kRadix - 1)], 1u);
  __syncthreads();
  const int64_t at = p.fused ? static_cast<int64_t>(blockIdx.x) * kRadix + tid
                             : static_cast<int64_t>(tid) * p.tiles + blockIdx.x;
  p.tile_hist[at] = s_hist[tid];
}

// One workgroup per digit: exclusive prefix of its row of tile_hist over the tiles.
__global__ __launch_bounds__(kSortBlock) void radix_binscan_kernel(SortParams p) {
  __shared__ uint32_t s_wave[kSortWaves];
  uint32_t* row = p.tile_hist + static_cast<int64_t>(blockIdx.x) * p.tiles;
  const int64_t n = actual_count(p.max_edges, p.num_edges_dev);
  const int64_t active = ceil_div_dev(n, kSortTile);
  uint32_t carry = 0;
  for (int64_t c0 = 0; c0 < active; c0 += kSortBlock) {
    const int64_t i = c0 + threadIdx.x;
    const uint32_t x = i < active ? row[i] : 0u;
    uint32_t all;
    const uint32_t excl = block_exclusive(x, s_wave, all);
    if (i < active) row[i] = carry + excl;
    carry += all;
  }
  if (threadIdx.x == 0) p.bin_total[blockIdx.x] = carry;
}

template <bool FIRST, bool LAST>
__global__ __launch_bounds__(kSortBlock) void radix_scatter_kernel(SortParams p) {
  // s_pos[w][b]: next position, inside the tile's digit-sorted order, of digit b
  // for wave w.  A wave owns kSortWaveItems consecutive items, so walking waves
  // in order, and rounds in order inside a wave, keeps equal digits in input
  // order.  Items are first put into that order in LDS and then written out, so
  // that neighbouring lanes write neighbouring addresses (a digit's run).
  __shared__ uint32_t s_pos[kSortWaves][kRadix];
  __shared__ uint32_t s_delta[kRadix];     // output position = s_delta[digit] + position in the tile's order
  __shared__ uint32_t s_wave[kSortWaves];
  __shared__ uint32_t s_key[kSortTile];
  __shared__ uint32_t s_pay[kSortTile];
  const int tid = threadIdx.x;             // = digit in the per-digit steps
  const int lane = lane_id();
  const int wave = tid / kWave;
  const int64_t n = actual_count(p.max_edges, p.num_edges_dev);
  const int64_t tile_base = static_cast<int64_t>(blockIdx.x) * kSortTile;
  if (tile_base >= n) return;  // block-uniform
#pragma unroll
  for (int w = 0; w < kSortWaves; ++w) s_pos[w][tid] = 0;
  __syncthreads();
  const int64_t wave_base = tile_base + static_cast<int64_t>(wave) * kSortWaveItems;
  uint32_t key[kSortRounds], pay[kSortRounds];
#pragma unroll
  for (int r = 0; r < kSortRounds; ++r) {   // every load of the lane is requested before the first is used
    const int64_t i = wave_base + r * kWave + lane;
    key[r] = i < n ? sort_key<FIRST>(p, i) : 0u;
    pay[r] = FIRST ? static_cast<uint32_t>(i) : (i < n ? p.pay_in[i] : 0u);
  }
#pragma unroll
  for (int r = 0; r < kSortRounds; ++r)
    if (wave_base + r * kWave + lane < n) atomicAdd(&s_pos[wave][(key[r] >> p.shift) & (kRadix - 1)], 1u);
  // First output position of this tile's items of digit `tid`: items with a
  // smaller digit anywhere, plus items with the same digit in earlier tiles.
  uint32_t first;
  if (p.fused) {
    const int64_t active = ceil_div_dev(n, kSortTile);
    uint32_t before = 0, total = 0;
    for (int64_t t0 = 0; t0 < active; t0 += 8) {
      uint32_t c[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) c[u] = t0 + u < active ? p.tile_hist[(t0 + u) * kRadix + tid] : 0u;
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        total += c[u];
        if (t0 + u < blockIdx.x) before += c[u];
      }
    }
    uint32_t all;
    first = block_exclusive(total, s_wave, all) + before;
  } else {
    // tile_hist[digit][tile] already holds the prefix over tiles; bin_total the digit's count
    uint32_t all;
    first = block_exclusive(p.bin_total[tid], s_wave, all) +
            p.tile_hist[static_cast<int64_t>(tid) * p.tiles + blockIdx.x];
  }
  __syncthreads();
  uint32_t mine_total = 0;
#pragma unroll
  for (int w = 0; w < kSortWaves; ++w) mine_total += s_pos[w][tid];
  uint32_t all;
  uint32_t local = block_exclusive(mine_total, s_wave, all);   // digit's start inside the tile
  s_delta[tid] = first - local;
#pragma unroll
  for (int w = 0; w < kSortWaves; ++w) {
    const uint32_t c = s_pos[w][tid];
    s_pos[w][tid] = local;
    local += c;
  }
  __syncthreads();
  volatile uint32_t* mine = s_pos[wave];
#pragma unroll
  for (int r = 0; r < kSortRounds; ++r) {
    const int64_t i = wave_base + r * kWave + lane;
    const bool valid = i < n;
    const uint32_t d = valid ? (key[r] >> p.shift) & (kRadix - 1) : 0u;
    uint64_t peers = ballot(valid);
#pragma unroll
    for (int b = 0; b < kRadixBits; ++b) {
      const bool bit = (d >> b) & 1u;
      const uint64_t set = ballot(valid && bit);
      peers &= bit ? set : ~set;
    }
    const uint32_t rank = rank_below(peers);
    uint32_t pos = 0;
    if (valid) pos = mine[d] + rank;
    __builtin_amdgcn_wave_barrier();
    // the last lane of a digit's group moves the counter past the group
    if (valid && rank + 1 == static_cast<uint32_t>(__popcll(peers))) mine[d] = pos + 1;
    __builtin_amdgcn_wave_barrier();
    if (valid) {
      s_key[pos] = key[r];
      s_pay[pos] = pay[r];
    }
  }
  __syncthreads();
  const int count = static_cast<int>(min(static_cast<int64_t>(kSortTile), n - tile_base));
  // (in the last pass an item's destination is a dependent read: all of a thread's are requested before any store)
  int64_t col[LAST ? kSortRounds : 1];
  if (LAST) {
#pragma unroll
    for (int q = 0; q < kSortRounds; ++q) {
      const int j = q * kSortBlock + tid;
      col[q] = j < count ? p.coo_col[s_pay[j]] : 0;
    }
  }
#pragma unroll
  for (int q = 0; q < kSortRounds; ++q) {
    const int j = q * kSortBlock + tid;
    if (j >= count) break;
    const uint32_t k = s_key[j];
    const uint32_t v = s_pay[j];
    const uint32_t pos = s_delta[(k >> p.shift) & (kRadix - 1)] + j;
    if (LAST) {
      p.csr_eids[pos] = v;
      p.csr_indices[pos] = col[q];
    } else {
      p.pay_out[pos] = v;
    }
    p.key_out[pos] = k;
  }
}

// csr_indptr[s] = first position of a key >= s in the sorted keys, s in [0, num_src].
// Position e starts a run of its key k when the key before it, kp, is smaller: then e is the answer for every
// s in (kp, k].  One lane per position writes those entries itself when they are few (in a sampled block nearly
// every source has an edge, so the run before a key is one or two entries long); a longer stretch is filled by the
// whole wavefront.  Sources above the largest key get the edge total.  No searching: every offset is written
// once, from a coalesced read of the keys.
constexpr int kIndptrShortGap = 4;

__global__ __launch_bounds__(kFmtBlock) void csr_indptr_kernel(const uint32_t* __restrict__ keys,
                                                               const int64_t* num_edges_dev, int64_t max_edges,
                                                               int64_t num_src, int64_t* __restrict__ csr_indptr) {
  const int64_t n = actual_count(max_edges, num_edges_dev);
  const int64_t last = n > 0 ? static_cast<int64_t>(keys[n - 1]) : -1;
  const int lane = lane_id();
  const int64_t tid = static_cast<int64_t>(blockIdx.x) * kFmtBlock + threadIdx.x;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kFmtBlock;
  for (int64_t e0 = tid - lane; e0 < n; e0 += stride) {   // e0: the wavefront's first position (wave-uniform)
    const int64_t e = e0 + lane;
    int64_t k = -1, kp = -1;
    if (e < n) {
      k = static_cast<int64_t>(keys[e]);
      if (e > 0) kp = static_cast<int64_t>(keys[e - 1]);
      if (k > num_src) k = num_src;    // keys beyond the bound have no offset of their own
      if (kp > num_src) kp = num_src;
    }
    const int64_t gap = k - kp;        // entries (kp, k] hold e
    if (gap > 0 && gap <= kIndptrShortGap)
      for (int64_t t = kp + 1; t <= k; ++t) csr_indptr[t] = e;
    uint64_t wide = ballot(gap > kIndptrShortGap);
    while (wide != 0) {
      const int src = __ffsll(static_cast<long long>(wide)) - 1;
      wide &= wide - 1;
      const int64_t a = __shfl(kp, src, kWave) + 1, b = __shfl(k, src, kWave);
      for (int64_t t = a + lane; t <= b; t += kWave) csr_indptr[t] = e0 + src;
    }
  }
  for (int64_t t = last + 1 + tid; t <= num_src; t += stride) csr_indptr[t] = n;
}

// An empty block: offsets all zero.
__global__ __launch_bounds__(kFmtBlock) void fmt_zero_kernel(int64_t* a, int64_t na, int64_t* b, int64_t nb,
                                                             int64_t* c) {
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kFmtBlock + threadIdx.x; i < na || i < nb;
       i += static_cast<int64_t>(gridDim.x) * kFmtBlock) {
    if (a != nullptr && i < na) a[i] = 0;
    if (b != nullptr && i < nb) b[i] = 0;
  }
  if (c != nullptr && blockIdx.x == 0 && threadIdx.x == 0) *c = 0;
}

int tuning_block_fused_scan();  // 0 = always take the separate scan launches

static size_t fmt_align(size_t x) { return (x + 255) / 256 * 256; }

struct FmtLayout {
  int64_t slots, ctiles, stiles;
  size_t tile_cnt_off, sums_off, hist_off, bin_total_off, key_off[2], pay_off[2], total;
};

static FmtLayout fmt_layout(int64_t num_dst, int fanout, bool csr) {
  FmtLayout L;
  L.slots = num_dst * fanout;
  L.ctiles = ceil_div(L.slots > 0 ? L.slots : 1, kCompactTile);
  L.stiles = ceil_div(L.slots > 0 ? L.slots : 1, kSortTile);
  size_t off = 0;
  L.tile_cnt_off = off; off = fmt_align(off + sizeof(uint32_t) * static_cast<size_t>(L.ctiles));
  L.sums_off = off;     off = fmt_align(off + sizeof(uint32_t) * kScanChunk);
  L.hist_off = off;
  if (csr) {
    off = fmt_align(off + sizeof(uint32_t) * static_cast<size_t>(L.stiles) * kRadix);
    L.bin_total_off = off; off = fmt_align(off + sizeof(uint32_t) * kRadix);
    const size_t buf = sizeof(uint32_t) * static_cast<size_t>(L.slots > 0 ? L.slots : 1);
    for (int k = 0; k < 2; ++k) {
      L.key_off[k] = off; off = fmt_align(off + buf);
      L.pay_off[k] = off; off = fmt_align(off + buf);
    }
  }
  L.total = off;
  return L;
}

static bool fmt_sizes_ok(int64_t num_dst, int fanout, int64_t num_src) {
  return num_dst >= 0 && fanout >= 0 && num_src >= 0 && num_src <= 0xffffffffLL &&
         (fanout == 0 || num_dst <= 0x7fffffffLL / fanout);
}

}  // namespace apt

extern "C" size_t apt_block_workspace_bytes(int64_t num_dst, int fanout, int64_t num_src, int want_csr) {
  using namespace apt;
  if (!fmt_sizes_ok(num_dst, fanout, num_src)) return 0;
  return fmt_layout(num_dst, fanout, want_csr != 0).total;
}

extern "C" int apt_block_formats(const int64_t* relabeled, int64_t num_dst, const int64_t* num_dst_dev,
                                 int fanout, int64_t num_src, int64_t* coo_row, int64_t* coo_col,
                                 int64_t* csc_indptr, int64_t* num_edges_dev, int64_t* csr_indptr,
                                 int64_t* csr_indices, int64_t* csr_eids, void* workspace,
                                 size_t workspace_bytes, void* stream) {
  using namespace apt;
  APT_REQUIRE(fmt_sizes_ok(num_dst, fanout, num_src), APT_ELIMIT,
              "apt_block_formats: sizes out of range (num_dst %lld, fanout %d, num_src %lld)",
              static_cast<long long>(num_dst), fanout, static_cast<long long>(num_src));
  APT_REQUIRE(csc_indptr != nullptr && num_edges_dev != nullptr, APT_EINVAL,
              "apt_block_formats: csc_indptr / num_edges_dev is NULL");
  const bool csr = csr_indptr != nullptr;
  APT_REQUIRE(!csr || (csr_indices != nullptr && csr_eids != nullptr), APT_EINVAL,
              "apt_block_formats: csr_indices / csr_eids is NULL");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const FmtLayout L = fmt_layout(num_dst, fanout, csr);
  if (L.slots == 0) {
    const int64_t longest = std::max<int64_t>(num_dst + 1, csr ? num_src + 1 : 0);
    hipLaunchKernelGGL(fmt_zero_kernel, dim3(static_cast<unsigned>(std::min<int64_t>(ceil_div(longest, kFmtBlock), 4096))),
                       dim3(kFmtBlock), 0, st, csc_indptr, num_dst + 1, csr_indptr, csr ? num_src + 1 : 0,
                       num_edges_dev);
    APT_LAUNCH_CHECK("fmt_zero_kernel");
    return APT_OK;
  }
  APT_REQUIRE(relabeled != nullptr && coo_row != nullptr && coo_col != nullptr, APT_EINVAL,
              "apt_block_formats: relabeled / coo_row / coo_col is NULL");
  APT_REQUIRE(workspace != nullptr && workspace_bytes >= L.total, APT_EWORKSPACE,
              "apt_block_formats: workspace of %zu bytes, %zu needed", workspace_bytes, L.total);
  char* ws = static_cast<char*>(workspace);
  uint32_t* sums = reinterpret_cast<uint32_t*>(ws + L.sums_off);

  CompactParams c;
  c.relabeled = relabeled;
  c.num_dst = num_dst;
  c.num_dst_dev = num_dst_dev;
  c.fanout = fanout;
  c.tile_cnt = reinterpret_cast<uint32_t*>(ws + L.tile_cnt_off);
  c.coo_row = coo_row;
  c.coo_col = coo_col;
  c.csc_indptr = csc_indptr;
  c.tiles = L.ctiles;
  c.scanned = L.ctiles > kFusedCompactTiles || !tuning_block_fused_scan();
  c.num_edges_dev = num_edges_dev;
  const dim3 cgrid(static_cast<unsigned>(L.ctiles));
  hipLaunchKernelGGL(fmt_count_kernel, cgrid, dim3(kFmtBlock), 0, st, c);
  APT_LAUNCH_CHECK("fmt_count_kernel");
  // the edge total is also the last CSC offset
  if (c.scanned)
    if (int rc = exclusive_scan(c.tile_cnt, L.ctiles, sums, num_edges_dev, csc_indptr + num_dst, st)) return rc;
  hipLaunchKernelGGL(fmt_place_kernel, cgrid, dim3(kFmtBlock), 0, st, c);
  APT_LAUNCH_CHECK("fmt_place_kernel");
  if (!csr) return APT_OK;

  int bits = 1;
  while (bits < 32 && (1LL << bits) < num_src) ++bits;
  const int passes = (bits + kRadixBits - 1) / kRadixBits;
  SortParams s;
  s.coo_row = coo_row;
  s.coo_col = coo_col;
  s.num_edges_dev = num_edges_dev;
  s.max_edges = L.slots;
  s.tile_hist = reinterpret_cast<uint32_t*>(ws + L.hist_off);
  s.bin_total = reinterpret_cast<uint32_t*>(ws + L.bin_total_off);
  s.tiles = L.stiles;
  s.fused = L.stiles <= kFusedSortTiles && tuning_block_fused_scan();
  s.csr_indices = csr_indices;
  s.csr_eids = csr_eids;
  const dim3 sgrid(static_cast<unsigned>(L.stiles));
  for (int pass = 0; pass < passes; ++pass) {
    const bool first = pass == 0, last = pass == passes - 1;
    s.shift = pass * kRadixBits;
    s.key_in = first ? nullptr : reinterpret_cast<uint32_t*>(ws + L.key_off[(pass - 1) & 1]);
    s.pay_in = first ? nullptr : reinterpret_cast<uint32_t*>(ws + L.pay_off[(pass - 1) & 1]);
    s.key_out = reinterpret_cast<uint32_t*>(ws + L.key_off[pass & 1]);
    s.pay_out = reinterpret_cast<uint32_t*>(ws + L.pay_off[pass & 1]);
    if (first) hipLaunchKernelGGL(radix_hist_kernel<true>, sgrid, dim3(kSortBlock), 0, st, s);
    else hipLaunchKernelGGL(radix_hist_kernel<false>, sgrid, dim3(kSortBlock), 0, st, s);
    APT_LAUNCH_CHECK("radix_hist_kernel");
    if (!s.fused) {
      hipLaunchKernelGGL(radix_binscan_kernel, dim3(kRadix), dim3(kSortBlock), 0, st, s);
      APT_LAUNCH_CHECK("radix_binscan_kernel");
    }
    if (first && last) hipLaunchKernelGGL((radix_scatter_kernel<true, true>), sgrid, dim3(kSortBlock), 0, st, s);
    else if (first) hipLaunchKernelGGL((radix_scatter_kernel<true, false>), sgrid, dim3(kSortBlock), 0, st, s);
    else if (last) hipLaunchKernelGGL((radix_scatter_kernel<false, true>), sgrid, dim3(kSortBlock), 0, st, s);
    else hipLaunchKernelGGL((radix_scatter_kernel<false, false>), sgrid, dim3(kSortBlock), 0, st, s);
    APT_LAUNCH_CHECK("radix_scatter_kernel");
  }
  const uint32_t* sorted = reinterpret_cast<uint32_t*>(ws + L.key_off[(passes - 1) & 1]);
  const unsigned iblocks =
      static_cast<unsigned>(std::min<int64_t>(ceil_div(std::max<int64_t>(num_src + 1, L.slots), kFmtBlock), 4096));
  hipLaunchKernelGGL(csr_indptr_kernel, dim3(iblocks), dim3(kFmtBlock), 0, st, sorted, num_edges_dev, L.slots,
                     num_src, csr_indptr);
  APT_LAUNCH_CHECK("csr_indptr_kernel");
  return APT_OK;
}
