// Building the GPU caches that the registries take: access counting during a
// dry run, and extraction of the adjacency rows of the chosen nodes into a
// second CSR.
//
// The reference counts accesses on the host (examples/dryrun.py:86-92:
// counter[nodes] += 1 per batch) and builds the cached CSR with one Python
// slice per cached node (python/npc/ops.py:370-384).  Here both are single
// kernels over device-resident arrays, with no host round trip, so a dry run
// can ride on the sampling pipeline.
#include "common.hpp"

namespace apt {

constexpr int kCacheBlock = 256;
constexpr int kCopyEdgesPerBlock = 4096;

// freq[ids[i]] += 1 for every valid id.
__global__ __launch_bounds__(kCacheBlock) void count_ids_kernel(const int64_t* __restrict__ ids,
                                                                int64_t n_host, const int64_t* n_dev,
                                                                int64_t* freq, int64_t num_total) {
  const int64_t n = actual_count(n_host, n_dev);
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kCacheBlock + threadIdx.x; i < n;
       i += static_cast<int64_t>(gridDim.x) * kCacheBlock) {
    const int64_t v = ids[i];
    if (v >= 0 && v < num_total)
      atomicAdd(reinterpret_cast<unsigned long long*>(&freq[v]), 1ull);
  }
}

// out_indptr[r] = sum of the degrees of rows[0..r), degree 0 for a row outside the table.
__global__ __launch_bounds__(kCacheBlock) void row_degree_kernel(const int64_t* __restrict__ indptr,
                                                                 int64_t row_begin, int64_t num_rows,
                                                                 const int64_t* __restrict__ rows,
                                                                 int64_t n, int64_t* __restrict__ deg) {
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kCacheBlock + threadIdx.x; i < n;
       i += static_cast<int64_t>(gridDim.x) * kCacheBlock) {
    const int64_t r = rows[i] - row_begin;
    deg[i] = (r >= 0 && r < num_rows) ? indptr[r + 1] - indptr[r] : 0;
  }
}

// Last row r in [lo, hi] with out_indptr[r] <= e.
__device__ __forceinline__ int64_t owner_row(const int64_t* out_indptr, int64_t lo, int64_t hi, int64_t e) {
  while (lo < hi) {
    const int64_t mid = lo + (hi - lo + 1) / 2;
    if (out_indptr[mid] <= e) lo = mid;
    else hi = mid - 1;
  }
  return lo;
}

// out_indices[out_indptr[i] + k] = indices[indptr[rows[i]] + k].  Work is split
// by output position, so a 2 M-edge hub row is copied by many workgroups.  A
// workgroup whose 4096 positions touch only a few rows (the usual case for hot
// rows) copies them segment by segment, each thread streaming 8-byte elements
// with nothing else to look up; one that spans many short rows finds every
// element's row by binary search.
constexpr int kCopySegRows = 16;

__global__ __launch_bounds__(kCacheBlock) void copy_rows_kernel(
    const int64_t* __restrict__ indptr, const int64_t* __restrict__ indices, int64_t row_begin,
    const int64_t* __restrict__ rows, int64_t n, const int64_t* __restrict__ out_indptr,
    int64_t* __restrict__ out_indices) {
  __shared__ int64_t s_lo, s_hi;
  __shared__ int64_t s_dst[kCopySegRows + 1], s_src[kCopySegRows];
  const int64_t total = out_indptr[n];
  const int64_t e0 = static_cast<int64_t>(blockIdx.x) * kCopyEdgesPerBlock;
  if (e0 >= total) return;
  const int64_t e1 = min(e0 + kCopyEdgesPerBlock, total) - 1;
  if (threadIdx.x == 0) s_lo = owner_row(out_indptr, 0, n - 1, e0);
  if (threadIdx.x == 1) s_hi = owner_row(out_indptr, 0, n - 1, e1);
  __syncthreads();
  const int64_t lo = s_lo, hi = s_hi;
  if (hi - lo < kCopySegRows) {
    const int nseg = static_cast<int>(hi - lo + 1);
    if (static_cast<int>(threadIdx.x) <= nseg) s_dst[threadIdx.x] = out_indptr[lo + threadIdx.x];
    if (static_cast<int>(threadIdx.x) < nseg) s_src[threadIdx.x] = indptr[rows[lo + threadIdx.x] - row_begin];
    __syncthreads();
    for (int k = 0; k < nseg; ++k) {
      const int64_t b = max(s_dst[k], e0), e = min(s_dst[k + 1], e1 + 1);
      const int64_t* src = indices + s_src[k] - s_dst[k];   // src[pos] is the element for output position pos
      for (int64_t pos = b + threadIdx.x; pos < e; pos += kCacheBlock)
        out_indices[pos] = __builtin_nontemporal_load(src + pos);
    }
    return;
  }
  for (int64_t e = e0 + threadIdx.x; e <= e1; e += kCacheBlock) {
    const int64_t i = owner_row(out_indptr, lo, hi, e);
    const int64_t r = rows[i] - row_begin;
    out_indices[e] = indices[indptr[r] + (e - out_indptr[i])];
  }
}

}  // namespace apt

extern "C" int apt_count_ids(const int64_t* ids, int64_t n, const int64_t* n_dev, int64_t* freq,
                             int64_t num_total_nodes, void* stream) {
  using namespace apt;
  APT_REQUIRE(n >= 0 && num_total_nodes >= 0, APT_EINVAL, "apt_count_ids: negative size");
  if (n == 0) return APT_OK;
  APT_REQUIRE(ids != nullptr && freq != nullptr, APT_EINVAL, "apt_count_ids: ids/freq is NULL");
  const unsigned blocks = static_cast<unsigned>(std::min<int64_t>(ceil_div(n, kCacheBlock), 8192));
  hipLaunchKernelGGL(count_ids_kernel, dim3(blocks), dim3(kCacheBlock), 0,
                     static_cast<hipStream_t>(stream), ids, n, n_dev, freq, num_total_nodes);
  APT_LAUNCH_CHECK("count_ids_kernel");
  return APT_OK;
}

extern "C" int apt_csr_row_degrees(const int64_t* indptr, int64_t row_begin, int64_t num_rows,
                                   const int64_t* rows, int64_t n, int64_t* degrees, void* stream) {
  using namespace apt;
  APT_REQUIRE(n >= 0 && num_rows >= 0, APT_EINVAL, "apt_csr_row_degrees: negative size");
  if (n == 0) return APT_OK;
  APT_REQUIRE(indptr != nullptr && rows != nullptr && degrees != nullptr, APT_EINVAL,
              "apt_csr_row_degrees: a pointer is NULL");
  const unsigned blocks = static_cast<unsigned>(std::min<int64_t>(ceil_div(n, kCacheBlock), 8192));
  hipLaunchKernelGGL(row_degree_kernel, dim3(blocks), dim3(kCacheBlock), 0,
                     static_cast<hipStream_t>(stream), indptr, row_begin, num_rows, rows, n, degrees);
  APT_LAUNCH_CHECK("row_degree_kernel");
  return APT_OK;
}

extern "C" int apt_csr_copy_rows(const int64_t* indptr, const int64_t* indices, int64_t row_begin,
                                 const int64_t* rows, int64_t n, const int64_t* out_indptr,
                                 int64_t num_out_edges, int64_t* out_indices, void* stream) {
  using namespace apt;
  APT_REQUIRE(n >= 0 && num_out_edges >= 0, APT_EINVAL, "apt_csr_copy_rows: negative size");
  if (n == 0 || num_out_edges == 0) return APT_OK;
  APT_REQUIRE(indptr != nullptr && indices != nullptr && rows != nullptr && out_indptr != nullptr &&
                  out_indices != nullptr,
              APT_EINVAL, "apt_csr_copy_rows: a pointer is NULL");
  const int64_t blocks = ceil_div(num_out_edges, kCopyEdgesPerBlock);
  APT_REQUIRE(blocks <= 0x7fffffffLL, APT_ELIMIT, "apt_csr_copy_rows: too many edges");
  hipLaunchKernelGGL(copy_rows_kernel, dim3(static_cast<unsigned>(blocks)), dim3(kCacheBlock), 0,
                     static_cast<hipStream_t>(stream), indptr, indices, row_begin, rows, n, out_indptr,
                     out_indices);
  APT_LAUNCH_CHECK("copy_rows_kernel");
  return APT_OK;
}
