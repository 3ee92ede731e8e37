// libapt_bench.so: synthetic inputs and measurement helpers for the benchmark
// and the tests (R-MAT generator, symmetrisation, a plain copy kernel and a
// random-access probe).  Nothing here is on the reference's path and nothing of
// it is linked into libapt_hip.so.  See include/apt_synth.h.
#include "common.hpp"
#include "../../include/apt_synth.h"

namespace apt {

// This library keeps its own error text (libapt_hip.so is not loaded with it).
char* last_error_buf() {
  static thread_local char buf[512] = {0};
  return buf;
}

constexpr int kSynBlock = 256;
constexpr int kSynEdgesPerBlock = 4096;

// Last row r in [lo, hi] with indptr[r] <= e.
__device__ __forceinline__ int64_t row_of_edge(const int64_t* indptr, int64_t lo, int64_t hi,
                                               int64_t e) {
  while (lo < hi) {
    const int64_t mid = lo + (hi - lo + 1) / 2;
    if (indptr[mid] <= e) lo = mid;
    else hi = mid - 1;
  }
  return lo;
}

__global__ __launch_bounds__(kSynBlock) void rmat_fill_kernel(
    const int64_t* __restrict__ indptr, int64_t num_rows, int64_t row_begin, int64_t num_nodes,
    int64_t num_edges, int levels, uint64_t seed, uint32_t thr0, uint32_t thr1,
    int64_t* __restrict__ indices) {
  __shared__ int64_t s_lo, s_hi;
  const int64_t e0 = static_cast<int64_t>(blockIdx.x) * kSynEdgesPerBlock;
  if (e0 >= num_edges) return;
  const int64_t e1 = min(e0 + kSynEdgesPerBlock, num_edges) - 1;
  if (threadIdx.x == 0) s_lo = row_of_edge(indptr, 0, num_rows - 1, e0);
  if (threadIdx.x == 1) s_hi = row_of_edge(indptr, 0, num_rows - 1, e1);
  __syncthreads();
  const int64_t lo = s_lo, hi = s_hi;
  for (int64_t e = e0 + threadIdx.x; e <= e1; e += kSynBlock) {
    const int64_t u = row_begin + row_of_edge(indptr, lo, hi, e);
    // Slots are keyed by (row id, slot inside the row) so that a partition of
    // the rows generates exactly the rows of the whole graph.
    const uint64_t ekey = static_cast<uint64_t>(e - indptr[u - row_begin]);
    int64_t v = 0;
    for (uint32_t attempt = 0; attempt < 32; ++attempt) {
      v = 0;
      for (int l0 = 0; l0 < levels; l0 += 8) {
        uint32_t w[4];
        {
          uint32_t c0 = static_cast<uint32_t>(static_cast<uint64_t>(u));
          uint32_t c1 = static_cast<uint32_t>(static_cast<uint64_t>(u) >> 32) ^
                        (static_cast<uint32_t>(l0) << 16) ^ (attempt << 24);
          uint32_t c2 = static_cast<uint32_t>(ekey), c3 = static_cast<uint32_t>(ekey >> 32);
          uint32_t k0 = static_cast<uint32_t>(seed), k1 = static_cast<uint32_t>(seed >> 32);
#pragma unroll
          for (int r = 0; r < 10; ++r) {
            const uint32_t hi0 = __umulhi(0xD2511F53u, c0), lo0 = 0xD2511F53u * c0;
            const uint32_t hi1 = __umulhi(0xCD9E8D57u, c2), lo1 = 0xCD9E8D57u * c2;
            const uint32_t n0 = hi1 ^ c1 ^ k0, n2 = hi0 ^ c3 ^ k1;
            c0 = n0; c1 = lo1; c2 = n2; c3 = lo0;
            k0 += 0x9E3779B9u; k1 += 0xBB67AE85u;
          }
          w[0] = c0; w[1] = c1; w[2] = c2; w[3] = c3;
        }
        const int lim = min(8, levels - l0);
        for (int k = 0; k < lim; ++k) {
          const int bitpos = levels - 1 - (l0 + k);          // MSB first
          const uint32_t r16 = (w[k >> 1] >> ((k & 1) * 16)) & 0xFFFFu;
          const uint32_t thr = ((u >> bitpos) & 1) ? thr1 : thr0;
          v = (v << 1) | (r16 < thr ? 1 : 0);
        }
      }
      if (v < num_nodes) break;
    }
    if (v >= num_nodes) v %= num_nodes;
    indices[e] = v;
  }
}

// Rows of the symmetrised graph before sorting: row u = [u (self-loop), the forward
// neighbours of u, every w with a forward edge w -> u].  A workgroup owns 4096
// consecutive forward edges; the reverse copy of an edge takes the next free slot
// of its target's row (a ticket per row, so the order inside that part of a row
// depends on scheduling; the caller sorts the rows afterwards).
__global__ __launch_bounds__(kSynBlock) void symmetrize_fill_kernel(
    const int64_t* __restrict__ fwd_indptr, const int64_t* __restrict__ fwd_indices, int64_t num_nodes,
    int64_t num_fwd_edges, const int64_t* __restrict__ indptr, uint32_t* __restrict__ cursor,
    int64_t* __restrict__ out) {
  __shared__ int64_t s_lo, s_hi;
  const int64_t e0 = static_cast<int64_t>(blockIdx.x) * kSynEdgesPerBlock;
  if (e0 >= num_fwd_edges) return;
  const int64_t e1 = min(e0 + kSynEdgesPerBlock, num_fwd_edges) - 1;
  if (threadIdx.x == 0) s_lo = row_of_edge(fwd_indptr, 0, num_nodes - 1, e0);
  if (threadIdx.x == 1) s_hi = row_of_edge(fwd_indptr, 0, num_nodes - 1, e1);
  __syncthreads();
  const int64_t lo = s_lo, hi = s_hi;
  for (int64_t e = e0 + threadIdx.x; e <= e1; e += kSynBlock) {
    const int64_t u = row_of_edge(fwd_indptr, lo, hi, e);
    const int64_t v = fwd_indices[e];
    out[indptr[u] + 1 + (e - fwd_indptr[u])] = v;
    if (v < 0 || v >= num_nodes) continue;  // the generator never produces one
    const int64_t out_deg_v = fwd_indptr[v + 1] - fwd_indptr[v];
    const uint32_t ticket = atomicAdd(&cursor[v], 1u);
    const int64_t pos = indptr[v] + 1 + out_deg_v + ticket;
    if (pos < indptr[v + 1]) out[pos] = u;  // always, when indptr was sized from the same edges
  }
}

__global__ __launch_bounds__(kSynBlock) void self_loop_kernel(const int64_t* __restrict__ indptr,
                                                              int64_t num_nodes, int64_t* __restrict__ out) {
  for (int64_t u = static_cast<int64_t>(blockIdx.x) * kSynBlock + threadIdx.x; u < num_nodes;
       u += static_cast<int64_t>(gridDim.x) * kSynBlock)
    out[indptr[u]] = u;
}

// Plain streaming copy in 16-byte vectors: the known-size reference for
// scaling hardware traffic counters.
__global__ __launch_bounds__(kSynBlock) void copy_kernel(const uint4* __restrict__ src,
                                                         uint4* __restrict__ dst, int64_t vecs) {
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kSynBlock + threadIdx.x; i < vecs;
       i += static_cast<int64_t>(gridDim.x) * kSynBlock)
    dst[i] = src[i];
}

}  // namespace apt

namespace apt {

__device__ __forceinline__ uint64_t probe_mix(uint64_t x) {
  x *= 0x9E3779B97F4A7C15ull;
  x ^= x >> 32;
  x *= 0xD6E8FEB86659FD93ull;
  x ^= x >> 32;
  return x;
}

// One access per item to a pseudo-random word of a table: what bounds the
// sampling and relabel kernels (one transaction per sampled id), as opposed to
// bytes.  MODE 0 load, 1 store, 2 atomicMin without use of the result,
// 3 atomicMin whose result is used, 4 16-byte load, 5 a load and an atomicMin at two
// independent places (do the two kinds of access add up or overlap?).
template <int MODE>
__global__ __launch_bounds__(kSynBlock) void random_access_kernel(uint32_t* table, uint64_t words, int64_t n,
                                                                  uint32_t salt, uint32_t* sink) {
  uint32_t acc = 0;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kSynBlock + threadIdx.x; i < n;
       i += static_cast<int64_t>(gridDim.x) * kSynBlock) {
    const uint64_t w = probe_mix(static_cast<uint64_t>(i) + (static_cast<uint64_t>(salt) << 40)) % words;
    if (MODE == 0) acc += __builtin_nontemporal_load(&table[w]);
    else if (MODE == 1) table[w] = static_cast<uint32_t>(i);
    else if (MODE == 2) atomicMin(&table[w], static_cast<uint32_t>(i) | 0x80000000u);
    else if (MODE == 3) acc += atomicMin(&table[w], static_cast<uint32_t>(i) | 0x80000000u);
    else if (MODE == 5) {
      const uint64_t w2 = probe_mix(static_cast<uint64_t>(i) * 3 + 1 + (static_cast<uint64_t>(salt) << 40)) % words;
      acc += __builtin_nontemporal_load(&table[w]);
      atomicMin(&table[w2], static_cast<uint32_t>(i) | 0x80000000u);
    } else {
      const uint4 v = *reinterpret_cast<const uint4*>(&table[w & ~uint64_t{3}]);
      acc += v.x + v.w;
    }
  }
  if (acc == 0x12345679u) sink[0] = acc;  // keeps the loads alive
}

}  // namespace apt

extern "C" int apt_synth_random_access(int mode, void* table, int64_t table_bytes, int64_t num_accesses,
                                       uint32_t salt, void* sink, void* stream) {
  using namespace apt;
  APT_REQUIRE(mode >= 0 && mode <= 5, APT_EINVAL, "apt_synth_random_access: mode %d outside 0..5", mode);
  APT_REQUIRE(table != nullptr && sink != nullptr && table_bytes >= 16 && table_bytes % 16 == 0 &&
                  (reinterpret_cast<uintptr_t>(table) & 15) == 0,
              APT_EINVAL, "apt_synth_random_access: table must be 16-byte aligned, a multiple of 16 bytes long");
  APT_REQUIRE(num_accesses >= 0, APT_EINVAL, "apt_synth_random_access: num_accesses < 0");
  if (num_accesses == 0) return APT_OK;
  const uint64_t words = static_cast<uint64_t>(table_bytes) / 4;
  const dim3 grid(static_cast<unsigned>(std::min<int64_t>(ceil_div(num_accesses, kSynBlock), 16384))), block(kSynBlock);
  hipStream_t st = static_cast<hipStream_t>(stream);
  uint32_t* t = static_cast<uint32_t*>(table);
  uint32_t* sk = static_cast<uint32_t*>(sink);
  switch (mode) {
    case 0: hipLaunchKernelGGL(random_access_kernel<0>, grid, block, 0, st, t, words, num_accesses, salt, sk); break;
    case 1: hipLaunchKernelGGL(random_access_kernel<1>, grid, block, 0, st, t, words, num_accesses, salt, sk); break;
    case 2: hipLaunchKernelGGL(random_access_kernel<2>, grid, block, 0, st, t, words, num_accesses, salt, sk); break;
    case 3: hipLaunchKernelGGL(random_access_kernel<3>, grid, block, 0, st, t, words, num_accesses, salt, sk); break;
    case 5: hipLaunchKernelGGL(random_access_kernel<5>, grid, block, 0, st, t, words, num_accesses, salt, sk); break;
    default: hipLaunchKernelGGL(random_access_kernel<4>, grid, block, 0, st, t, words, num_accesses, salt, sk); break;
  }
  APT_LAUNCH_CHECK("random_access_kernel");
  return APT_OK;
}

extern "C" int apt_synth_copy(const void* src, void* dst, int64_t bytes, void* stream) {
  using namespace apt;
  APT_REQUIRE(bytes >= 0 && bytes % 16 == 0, APT_EINVAL, "apt_synth_copy: bytes must be a multiple of 16");
  if (bytes == 0) return APT_OK;
  APT_REQUIRE(src != nullptr && dst != nullptr &&
                  ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15) == 0,
              APT_EINVAL, "apt_synth_copy: src/dst must be 16-byte aligned");
  const int64_t vecs = bytes / 16;
  const unsigned blocks = static_cast<unsigned>(std::min<int64_t>(ceil_div(vecs, kSynBlock), 16384));
  hipLaunchKernelGGL(copy_kernel, dim3(blocks), dim3(kSynBlock), 0, static_cast<hipStream_t>(stream),
                     static_cast<const uint4*>(src), static_cast<uint4*>(dst), vecs);
  APT_LAUNCH_CHECK("copy_kernel");
  return APT_OK;
}

extern "C" int apt_synth_rmat_fill(const int64_t* indptr, int64_t num_rows, int64_t row_begin,
                                   int64_t num_nodes, int64_t num_edges, int levels, uint64_t seed,
                                   uint32_t thr0, uint32_t thr1, int64_t* indices, void* stream) {
  using namespace apt;
  APT_REQUIRE(num_nodes > 0 && num_edges >= 0 && num_rows > 0 && row_begin >= 0 &&
                  row_begin + num_rows <= num_nodes,
              APT_EINVAL, "apt_synth_rmat_fill: bad sizes");
  APT_REQUIRE(levels >= 1 && levels <= 40 && (num_nodes - 1) >> levels == 0, APT_EINVAL,
              "apt_synth_rmat_fill: %d levels do not cover %lld nodes", levels, (long long)num_nodes);
  APT_REQUIRE(thr0 <= 65536 && thr1 <= 65536, APT_EINVAL, "apt_synth_rmat_fill: bad thresholds");
  if (num_edges == 0) return APT_OK;
  APT_REQUIRE(indptr != nullptr && indices != nullptr, APT_EINVAL,
              "apt_synth_rmat_fill: indptr/indices is NULL");
  const int64_t blocks = ceil_div(num_edges, kSynEdgesPerBlock);
  APT_REQUIRE(blocks <= 0x7fffffffLL, APT_ELIMIT, "apt_synth_rmat_fill: too many edges");
  hipLaunchKernelGGL(rmat_fill_kernel, dim3(static_cast<unsigned>(blocks)), dim3(kSynBlock), 0,
                     static_cast<hipStream_t>(stream), indptr, num_rows, row_begin, num_nodes,
                     num_edges, levels, seed, thr0, thr1, indices);
  APT_LAUNCH_CHECK("rmat_fill_kernel");
  return APT_OK;
}

extern "C" int apt_synth_symmetrize_fill(const int64_t* fwd_indptr, const int64_t* fwd_indices, int64_t num_nodes,
                                         int64_t num_fwd_edges, const int64_t* indptr, void* cursor,
                                         int64_t* out, void* stream) {
  using namespace apt;
  APT_REQUIRE(num_nodes > 0 && num_fwd_edges >= 0, APT_EINVAL, "apt_synth_symmetrize_fill: bad sizes");
  APT_REQUIRE(fwd_indptr != nullptr && indptr != nullptr && cursor != nullptr && out != nullptr &&
                  (fwd_indices != nullptr || num_fwd_edges == 0),
              APT_EINVAL, "apt_synth_symmetrize_fill: a pointer is NULL");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const unsigned row_blocks = static_cast<unsigned>(std::min<int64_t>(ceil_div(num_nodes, kSynBlock), 16384));
  hipLaunchKernelGGL(self_loop_kernel, dim3(row_blocks), dim3(kSynBlock), 0, st, indptr, num_nodes, out);
  APT_LAUNCH_CHECK("self_loop_kernel");
  if (num_fwd_edges == 0) return APT_OK;
  const int64_t blocks = ceil_div(num_fwd_edges, kSynEdgesPerBlock);
  APT_REQUIRE(blocks <= 0x7fffffffLL, APT_ELIMIT, "apt_synth_symmetrize_fill: too many edges");
  hipLaunchKernelGGL(symmetrize_fill_kernel, dim3(static_cast<unsigned>(blocks)), dim3(kSynBlock), 0, st, fwd_indptr,
                     fwd_indices, num_nodes, num_fwd_edges, indptr, static_cast<uint32_t*>(cursor), out);
  APT_LAUNCH_CHECK("symmetrize_fill_kernel");
  return APT_OK;
}

extern "C" const char* apt_synth_last_error(void) { return apt::last_error_buf(); }
