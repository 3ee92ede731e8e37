// Aggregation on sampled blocks: SpMM (sum over in-edges) and SDDMM
// (per-edge element-wise combine) over COO.
//
// Replaces CopyUSumKernel / CopyESumKernel / UMulESumKernel (reference
// src/cuda/spmm.cu:8-148) and UAddVKernel / UMulVKernel (src/cuda/sddmm.cu:8-103).
// The reference launches a 2-D grid with one fp32 atomicAdd per (edge,
// feature) and a binary search of coo_off per edge.  Here a wavefront owns a
// run of consecutive edges and keeps the running sum of a destination row in
// registers; it touches memory only when the destination changes, so for the
// sampler's blocks (edges grouped by destination) a row is written by at most
// two wavefronts and the result does not depend on scheduling; for arbitrary
// edge order it degrades to the reference's atomic-per-edge behaviour.
// u_mul_e multiplies (the reference's kernel adds, src/cuda/spmm.cu:78, and
// has no caller).
#include "common.hpp"

namespace apt {

constexpr int kAggBlock = 256;
constexpr int kAggWaves = kAggBlock / kWave;
constexpr int kEdgesPerWave = 64;
constexpr int kMaxSegments = APT_MAX_BUCKETS + 1;

struct AggParams {
  const int64_t* row;       // source index per edge
  const int64_t* col;       // destination index per edge
  int64_t num_edges;
  const void* in;           // [*, D] (copy_u / u_mul_e / sddmm lhs) or [E, D] (copy_e)
  const void* edata;        // [E, D] (u_mul_e) / sddmm rhs [*, D]
  float* out;               // spmm: [num_out, D] fp32, zero-filled; sddmm: [E, D]
  const int64_t* coo_off;   // [num_seg + 1]
  const int64_t* in_off;    // [num_seg] or NULL
  const int64_t* out_off;   // [num_seg] (sddmm: rhs offsets) or NULL
  int num_seg;
  int64_t dim;
  int64_t num_in_rows, num_e_rows, num_out_rows;
  const float* head_w;      // MODE 3: [E, heads] scalar per edge and head
  const int64_t* head_w_row;  // MODE 3: row of head_w for edge e (NULL = e)
  const float* head_w2;     // MODE 3, optional: second [*, heads] table, summed per output row and head ...
  float* out2;              // ... into out2 [num_out, heads]
  int heads;
  int64_t head_dim;         // dim / heads
  int grouped;              // edges with equal col are consecutive: rows inside a wavefront's range are stored, not added
  const int* grouped_dev;   // the same as a device flag (apt_coo_is_grouped), or NULL
  const int64_t* out_indptr;  // grouped only, optional: offsets of the output rows in the edge list (CSR of col).
                              // Rows inside a wavefront's range are then recognised exactly, the rest (rows that
                              // span ranges, rows without edges) is zeroed by spmm_zero_rows_kernel: out need not be zero
};

template <typename T> __device__ __forceinline__ float to_float(T v);
template <> __device__ __forceinline__ float to_float<float>(float v) { return v; }
template <> __device__ __forceinline__ float to_float<uint16_t>(uint16_t v) {  // bf16 bits
  return __uint_as_float(static_cast<uint32_t>(v) << 16);
}

// Segment of edge e: last k with coo_off[k] <= e (reference: cub::UpperBound - 1).
__device__ __forceinline__ int segment_of(const int64_t* s_off, int num_seg, int64_t e) {
  int k = 0;
  while (k + 1 < num_seg && s_off[k + 1] <= e) ++k;
  return k;
}

template <typename T, int VEC> struct Pack;
template <> struct Pack<float, 4> { typedef float type __attribute__((ext_vector_type(4))); };
template <> struct Pack<float, 1> { typedef float type; };
template <> struct Pack<uint16_t, 4> { typedef uint16_t type __attribute__((ext_vector_type(4))); };
template <> struct Pack<uint16_t, 1> { typedef uint16_t type; };
template <> struct Pack<uint16_t, 8> { typedef uint16_t type __attribute__((ext_vector_type(8))); };

template <typename T, int VEC>
__device__ __forceinline__ void load_vec(const T* base, int64_t elem, float (&v)[VEC]) {
  using P = typename Pack<T, VEC>::type;
  const P raw = *reinterpret_cast<const P*>(base + elem);
  if constexpr (VEC == 1) {
    v[0] = to_float<T>(raw);
  } else {
#pragma unroll
    for (int i = 0; i < VEC; ++i) v[i] = to_float<T>(raw[i]);
  }
}

// MODE 0: copy_u  acc += in[in_off + src]
// MODE 1: copy_e  acc += in[e]
// MODE 2: u_mul_e acc += in[in_off + src] * edata[e]
// MODE 3: acc += in[in_off + src] * head_w[e, head of the feature] (VEC divides head_dim)
// A lane owns VEC consecutive features; kUnroll edges are loaded before they
// are accumulated.
// Value of a 64-bit variable in lane `src` of the wavefront (src is the same in all lanes).
__device__ __forceinline__ int64_t wave_read(int64_t v, int src) {
  const int lo = __builtin_amdgcn_readlane(static_cast<int>(v), src);
  const int hi = __builtin_amdgcn_readlane(static_cast<int>(v >> 32), src);
  return (static_cast<int64_t>(hi) << 32) | static_cast<uint32_t>(lo);
}

template <typename T, int MODE, int VEC>
__global__ __launch_bounds__(kAggBlock) void spmm_kernel(AggParams p) {
  constexpr int kUnroll = 4;
  __shared__ int64_t s_off[kMaxSegments + 1];
  __shared__ int64_t s_in[kMaxSegments], s_out[kMaxSegments];
  if (threadIdx.x <= p.num_seg) s_off[threadIdx.x] = p.coo_off != nullptr ? p.coo_off[threadIdx.x] : 0;  // NULL: one segment
  if (threadIdx.x < p.num_seg) {
    s_in[threadIdx.x] = p.in_off != nullptr ? p.in_off[threadIdx.x] : 0;
    s_out[threadIdx.x] = p.out_off != nullptr ? p.out_off[threadIdx.x] : 0;
  }
  __syncthreads();
  const int lane = threadIdx.x % kWave;
  const int64_t wave = static_cast<int64_t>(blockIdx.x) * kAggWaves + threadIdx.x / kWave;
  const int64_t e0 = wave * kEdgesPerWave;
  if (e0 >= p.num_edges) return;
  const int n = static_cast<int>(min(static_cast<int64_t>(kEdgesPerWave), p.num_edges - e0));
  const T* in = static_cast<const T*>(p.in);
  const T* ed = static_cast<const T*>(p.edata);
  // Lane i fetches what edge e0 + i needs (its rows, and where its weights are): three coalesced loads
  // for the wavefront's 64 edges; the edge loop below reads them lane by lane.
  int64_t my_dst = -1, my_src = -1, my_we = 0;
  if (lane < n) {
    const int64_t e = e0 + lane;
    const int k = segment_of(s_off, p.num_seg, e);
    my_dst = s_out[k] + p.col[e];
    if (MODE != 1) {
      my_src = s_in[k] + p.row[e];
      if (my_src >= p.num_in_rows) my_src = -1;
    }
    if (MODE == 3) my_we = p.head_w_row != nullptr ? p.head_w_row[e] : e;
  }
  const bool grouped = p.grouped || (p.grouped_dev != nullptr && *p.grouped_dev != 0);
  for (int64_t d0 = 0; d0 < p.dim; d0 += kWave * VEC) {
    const int64_t d = d0 + static_cast<int64_t>(lane) * VEC;
    const bool live = d < p.dim;
    const int64_t h = MODE == 3 ? d / p.head_dim : 0;
    float acc[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) acc[i] = 0.f;
    int64_t cur = -1;
    bool first_row = true;  // the row at the start of the range may have begun in the previous wavefront's range
    // MODE 3: the lane holding a head's first features also sums the second weight table
    const bool second = MODE == 3 && p.head_w2 != nullptr && live && d == h * p.head_dim;
    float acc2 = 0.f;
    auto flush = [&](bool last_row) {
      if (cur >= 0 && cur < p.num_out_rows && live) {
        bool inside = !first_row && !last_row;
        if (!inside && p.out_indptr != nullptr)   // the range's first or last row: does it begin and end in here?
          inside = p.out_indptr[cur] >= e0 && p.out_indptr[cur + 1] <= e0 + n;
        if (grouped && inside) {
#pragma unroll
          for (int i = 0; i < VEC; ++i) p.out[cur * p.dim + d + i] = acc[i];
          if (second) p.out2[cur * p.heads + h] = acc2;
        } else {
#pragma unroll
          for (int i = 0; i < VEC; ++i) atomicAdd(&p.out[cur * p.dim + d + i], acc[i]);
          if (second) atomicAdd(&p.out2[cur * p.heads + h], acc2);
        }
      }
      if (cur >= 0) first_row = false;
    };
    for (int i0 = 0; i0 < n; i0 += kUnroll) {
      float v[kUnroll][VEC];
      float v2[kUnroll];
      int64_t dst[kUnroll];
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        dst[u] = -1;
        v2[u] = 0.f;
#pragma unroll
        for (int i = 0; i < VEC; ++i) v[u][i] = 0.f;
        if (i0 + u < n) {
          dst[u] = wave_read(my_dst, i0 + u);
          if (MODE == 1) {
            if (live) load_vec<T, VEC>(in, (e0 + i0 + u) * p.dim + d, v[u]);
          } else {
            const int64_t src = wave_read(my_src, i0 + u);
            if (live && src >= 0) load_vec<T, VEC>(in, src * p.dim + d, v[u]);
            if (MODE == 2 && live) {
              float w[VEC];
              load_vec<T, VEC>(ed, (e0 + i0 + u) * p.dim + d, w);
#pragma unroll
              for (int i = 0; i < VEC; ++i) v[u][i] *= w[i];
            }
            if (MODE == 3) {
              const int64_t we = wave_read(my_we, i0 + u);
              if (live) {
                if (p.head_w != nullptr) {
                  const float w = p.head_w[we * p.heads + h];
#pragma unroll
                  for (int i = 0; i < VEC; ++i) v[u][i] *= w;
                }
                if (second) v2[u] = p.head_w2[we * p.heads + h];
              }
            }
          }
        }
      }
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        if (i0 + u < n) {
          if (dst[u] != cur) {
            flush(false);
#pragma unroll
            for (int i = 0; i < VEC; ++i) acc[i] = 0.f;
            acc2 = 0.f;
            cur = dst[u];
          }
#pragma unroll
          for (int i = 0; i < VEC; ++i) acc[i] += v[u][i];
          acc2 += v2[u];
        }
      }
    }
    flush(true);
  }
}

// Companion of spmm_kernel with out_indptr: zeroes the output rows that the main kernel does not store whole,
// i.e. rows without edges and rows whose edges lie in more than one wavefront range (those are added
// atomically).  A wavefront checks 64 rows with one coalesced pair of loads, then zeroes the flagged ones
// together, a row at a time.
__global__ __launch_bounds__(kAggBlock) void spmm_zero_rows_kernel(const int64_t* __restrict__ out_indptr,
                                                                   int64_t num_rows, int64_t dim, float* out,
                                                                   float* out2, int heads) {
  const int lane = threadIdx.x % kWave;
  for (int64_t base = (static_cast<int64_t>(blockIdx.x) * kAggWaves + threadIdx.x / kWave) * kWave; base < num_rows;
       base += static_cast<int64_t>(gridDim.x) * kAggWaves * kWave) {
    const int64_t r = base + lane;
    bool need = false;
    if (r < num_rows) {
      const int64_t lo = out_indptr[r], hi = out_indptr[r + 1];
      need = !(hi > lo && lo / kEdgesPerWave == (hi - 1) / kEdgesPerWave);   // else stored whole by one wavefront
    }
    uint64_t todo = ballot(need);
    while (todo != 0) {
      const int j = __ffsll(static_cast<long long>(todo)) - 1;
      todo &= todo - 1;
      float* row = out + (base + j) * dim;
      for (int64_t d = lane; d < dim; d += kWave) row[d] = 0.f;
      if (out2 != nullptr && lane < heads) out2[(base + j) * heads + lane] = 0.f;
    }
  }
}

// flag = 1 iff col is non-decreasing (then edges with equal col are consecutive).
__global__ void coo_grouped_init_kernel(int* flag) { *flag = 1; }

__global__ __launch_bounds__(kAggBlock) void coo_grouped_check_kernel(const int64_t* __restrict__ col, int64_t n,
                                                                      int* flag) {
  bool bad = false;
  for (int64_t e = static_cast<int64_t>(blockIdx.x) * kAggBlock + threadIdx.x; e + 1 < n;
       e += static_cast<int64_t>(gridDim.x) * kAggBlock)
    bad |= col[e] > col[e + 1];
  if (bad) *flag = 0;
}

// OP 0: lhs[src] + rhs[dst]; OP 1: lhs[src] * rhs[dst]  -> out[e]
template <typename T, int OP>
__global__ __launch_bounds__(kAggBlock) void sddmm_kernel(AggParams p) {
  __shared__ int64_t s_off[kMaxSegments + 1];
  __shared__ int64_t s_l[kMaxSegments], s_r[kMaxSegments];
  if (threadIdx.x <= p.num_seg) s_off[threadIdx.x] = p.coo_off != nullptr ? p.coo_off[threadIdx.x] : 0;  // NULL: one segment
  if (threadIdx.x < p.num_seg) {
    s_l[threadIdx.x] = p.in_off != nullptr ? p.in_off[threadIdx.x] : 0;
    s_r[threadIdx.x] = p.out_off != nullptr ? p.out_off[threadIdx.x] : 0;
  }
  __syncthreads();
  const T* lhs = static_cast<const T*>(p.in);
  const T* rhs = static_cast<const T*>(p.edata);
  const int lane = threadIdx.x % kWave;
  const int64_t waves = static_cast<int64_t>(gridDim.x) * kAggWaves;
  for (int64_t e = static_cast<int64_t>(blockIdx.x) * kAggWaves + threadIdx.x / kWave; e < p.num_edges;
       e += waves) {
    const int k = segment_of(s_off, p.num_seg, e);
    const int64_t src = s_l[k] + p.row[e];
    const int64_t dst = s_r[k] + p.col[e];
    const bool ok = src >= 0 && src < p.num_in_rows && dst >= 0 && dst < p.num_e_rows;
    for (int64_t d = lane; d < p.dim; d += kWave) {
      float v = 0.f;
      if (ok) {
        const float a = to_float<T>(lhs[src * p.dim + d]);
        const float b = to_float<T>(rhs[dst * p.dim + d]);
        v = OP == 0 ? a + b : a * b;
      }
      p.out[e * p.dim + d] = v;
    }
  }
}

// Fixed-stride ("ELL") SpMM over a sampled block as the sampler emits it:
// destination i owns slots [i*fanout, (i+1)*fanout) of `nbr`, negative = no
// edge.  A lane group owns a destination row, so there are no atomics, no
// zero-fill and the sum order is fixed.  LPR lanes x VEC features cover `dim`.
template <typename T, int VEC, int LPR>
__global__ __launch_bounds__(kAggBlock) void spmm_ell_kernel(const int64_t* __restrict__ nbr,
                                                             int64_t num_dst, const int64_t* num_dst_dev,
                                                             int fanout, const T* __restrict__ x,
                                                             int64_t num_src, int64_t dim,
                                                             float* __restrict__ out, int mean) {
  constexpr int kGroups = kAggBlock / LPR;
  constexpr int kUnroll = 5;
  const int64_t n = actual_count(num_dst, num_dst_dev);
  const int grp = threadIdx.x / LPR, l = threadIdx.x % LPR;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kGroups + grp; i < n;
       i += static_cast<int64_t>(gridDim.x) * kGroups) {
    const int64_t* ids = nbr + i * fanout;
    // lane s of the group fetches slot s's id (one coalesced load for the destination); the slot loop reads
    // it with a shuffle.  (Ids that do not fit 32 bits, or more slots than lanes: every lane loads them itself.)
    const bool shared_ids = fanout <= LPR && num_src <= 0x7fffffffLL;
    int my_id = -1;
    if (shared_ids && l < fanout) {
      const int64_t v = ids[l];
      my_id = (v >= 0 && v < num_src) ? static_cast<int>(v) : -1;
    }
    for (int64_t d0 = 0; d0 < dim; d0 += LPR * VEC) {   // every lane of the group stays in the loop (shuffles)
      const int64_t d = d0 + static_cast<int64_t>(l) * VEC;
      const bool live = d < dim;
      float acc[VEC];
#pragma unroll
      for (int k = 0; k < VEC; ++k) acc[k] = 0.f;
      int cnt = 0;
      for (int s0 = 0; s0 < fanout; s0 += kUnroll) {
        float v[kUnroll][VEC];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
#pragma unroll
          for (int k = 0; k < VEC; ++k) v[u][k] = 0.f;
          if (s0 + u < fanout) {
            const int64_t src = shared_ids ? static_cast<int64_t>(__shfl(my_id, s0 + u, LPR)) : ids[s0 + u];
            if (src >= 0 && src < num_src) {
              if (live) load_vec<T, VEC>(x, src * dim + d, v[u]);
              ++cnt;
            }
          }
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u)
#pragma unroll
          for (int k = 0; k < VEC; ++k) acc[k] += v[u][k];
      }
      const float scale = (mean && cnt > 0) ? 1.0f / static_cast<float>(cnt) : 1.0f;
      if (live) {
#pragma unroll
        for (int k = 0; k < VEC; ++k) out[i * dim + d + k] = acc[k] * scale;
      }
    }
  }
}

template <typename T, int VEC>
static void launch_ell(const int64_t* nbr, int64_t num_dst, const int64_t* num_dst_dev, int fanout,
                       const void* x, int64_t num_src, int64_t dim, float* out, int mean, hipStream_t st) {
  const int64_t per_row = ceil_div(dim, VEC);
  const T* xt = static_cast<const T*>(x);
#define APT_ELL(LPR)                                                                                 \
  hipLaunchKernelGGL((spmm_ell_kernel<T, VEC, LPR>),                                                  \
                     dim3(static_cast<unsigned>(std::min<int64_t>(ceil_div(num_dst, kAggBlock / LPR), 1 << 20))), \
                     dim3(kAggBlock), 0, st, nbr, num_dst, num_dst_dev, fanout, xt, num_src, dim, out, mean)
  if (per_row <= 8) APT_ELL(8);
  else if (per_row <= 16) APT_ELL(16);
  else if (per_row <= 32) APT_ELL(32);
  else APT_ELL(64);
#undef APT_ELL
}

// GAT attention logits: out[r, h] = sum_d x[r, h, d] * attn[h, d]
// (python/npc/model/gatconv.py:116-117: (feat * attn).sum(-1)).  A wavefront per
// (row, head); lanes stride over d and reduce with shuffles in a fixed order.
template <typename T>
__global__ __launch_bounds__(kAggBlock) void gat_scores_kernel(const T* __restrict__ x, int64_t num_rows,
                                                               int heads, int64_t dim,
                                                               const float* __restrict__ attn,
                                                               float* __restrict__ out) {
  const int lane = threadIdx.x % kWave;
  const int64_t items = num_rows * heads;
  for (int64_t it = static_cast<int64_t>(blockIdx.x) * kAggWaves + threadIdx.x / kWave; it < items;
       it += static_cast<int64_t>(gridDim.x) * kAggWaves) {
    const int h = static_cast<int>(it % heads);
    float acc = 0.f;
    for (int64_t d = lane; d < dim; d += kWave) acc += to_float<T>(x[it * dim + d]) * attn[h * dim + d];
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) acc += __shfl_down(acc, off, kWave);
    if (lane == 0) out[it] = acc;
  }
}

// The same for dim = VEC * LPH with LPH a power of two: LPH lanes per (row, head),
// VEC features per lane in one 16-byte load, xor-shuffle reduction inside the
// lane group.
template <typename T, int VEC, int LPH>
__global__ __launch_bounds__(kAggBlock) void gat_scores_vec_kernel(const T* __restrict__ x, int64_t items,
                                                                   int heads, const float* __restrict__ attn,
                                                                   float* __restrict__ out) {
  constexpr int kGroups = kAggBlock / LPH;
  constexpr int64_t dim = VEC * LPH;
  const int grp = threadIdx.x / LPH, l = threadIdx.x % LPH;
  for (int64_t it = static_cast<int64_t>(blockIdx.x) * kGroups + grp; it < items;
       it += static_cast<int64_t>(gridDim.x) * kGroups) {
    const int h = static_cast<int>(it % heads);
    float v[VEC];
    load_vec<T, VEC>(x, it * dim + l * VEC, v);
    float acc = 0.f;
#pragma unroll
    for (int q = 0; q < VEC; q += 4) {
      const float4 a = *reinterpret_cast<const float4*>(attn + h * dim + l * VEC + q);
      acc += v[q] * a.x + v[q + 1] * a.y + v[q + 2] * a.z + v[q + 3] * a.w;
    }
#pragma unroll
    for (int off = LPH / 2; off > 0; off >>= 1) acc += __shfl_xor(acc, off, kWave);
    if (l == 0) out[it] = acc;
  }
}

// GATConv aggregation over a fixed-stride block (gatconv.py:118-126, DGL's
// u_add_v -> LeakyReLU -> edge_softmax -> u_mul_e + sum): for destination i and
// head h, e_k = leaky(el[src_k, h] + er[i, h]) over the row's slots, a = softmax(e),
// out[i, h, :] = sum_k a_k * ft[src_k, h, :].  A lane group owns a destination
// row (all heads); the softmax runs online over the slots (running maximum,
// rescaled sum), so a row's features are read once and nothing is written but
// the result: no per-edge score, exponent or weight arrays, no atomics.
template <typename T, int VEC, int LPR>
__global__ __launch_bounds__(kAggBlock) void gat_ell_kernel(const int64_t* __restrict__ nbr, int64_t num_dst,
                                                            const int64_t* num_dst_dev, int fanout,
                                                            const T* __restrict__ ft, int64_t num_src,
                                                            int heads, int64_t dim,
                                                            const float* __restrict__ el,
                                                            const float* __restrict__ er, float slope,
                                                            float* __restrict__ out,
                                                            float* __restrict__ attn_out) {
  constexpr int kGroups = kAggBlock / LPR;
  constexpr int kUnroll = 5;
  const int64_t n = actual_count(num_dst, num_dst_dev);
  const int64_t row_len = static_cast<int64_t>(heads) * dim;
  const int grp = threadIdx.x / LPR, l = threadIdx.x % LPR;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kGroups + grp; i < n;
       i += static_cast<int64_t>(gridDim.x) * kGroups) {
    const int64_t* ids = nbr + i * fanout;
    for (int64_t d = static_cast<int64_t>(l) * VEC; d < row_len; d += LPR * VEC) {
      const int h = static_cast<int>(d / dim);   // VEC divides dim: a lane's features share a head
      const float er_i = er[i * heads + h];
      float acc[VEC];
#pragma unroll
      for (int k = 0; k < VEC; ++k) acc[k] = 0.f;
      float top = -INFINITY, denom = 0.f;
      for (int s0 = 0; s0 < fanout; s0 += kUnroll) {
        float v[kUnroll][VEC];
        float sc[kUnroll];
        bool ok[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
          ok[u] = false;
          sc[u] = 0.f;
#pragma unroll
          for (int k = 0; k < VEC; ++k) v[u][k] = 0.f;
          if (s0 + u < fanout) {
            const int64_t src = ids[s0 + u];
            if (src >= 0 && src < num_src) {
              ok[u] = true;
              sc[u] = el[src * heads + h];
              load_vec<T, VEC>(ft, src * row_len + d, v[u]);
            }
          }
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
          if (!ok[u]) continue;
          float e = sc[u] + er_i;
          e = e > 0.f ? e : e * slope;
          if (e > top) {
            const float shrink = expf(top - e);   // 0 on the first edge (top = -inf)
            denom *= shrink;
#pragma unroll
            for (int k = 0; k < VEC; ++k) acc[k] *= shrink;
            top = e;
          }
          const float w = expf(e - top);
          denom += w;
#pragma unroll
          for (int k = 0; k < VEC; ++k) acc[k] += w * v[u][k];
        }
      }
      const float inv = denom > 0.f ? 1.0f / denom : 0.f;
#pragma unroll
      for (int k = 0; k < VEC; ++k) out[i * row_len + d + k] = acc[k] * inv;
      // the lane that holds a head's first features also writes its attention weights
      if (attn_out != nullptr && d % dim == 0) {
        for (int s = 0; s < fanout; ++s) {
          const int64_t src = ids[s];
          float a = 0.f;
          if (src >= 0 && src < num_src) {
            float e = el[src * heads + h] + er_i;
            e = e > 0.f ? e : e * slope;
            a = expf(e - top) * inv;
          }
          attn_out[(i * fanout + s) * heads + h] = a;
        }
      }
    }
  }
}

// The same layer with a wavefront per destination and two lane layouts (needs
// heads and lph = dim / VEC to be powers of two, heads * lph <= 64 and
// heads * fanout <= 64).  Slot layout: lane j is (slot j / heads, head
// j % heads) and holds that slot's logit, so ids, el and the attention weights
// are one coalesced access each per destination and the softmax is three
// cross-lane reductions.  Feature layout: lane l holds VEC features of head
// l / lph and adds up the source rows, fetching each slot's weight from the slot
// layout with one shuffle.
template <typename T, int VEC>
__global__ __launch_bounds__(kAggBlock) void gat_ell_wave_kernel(
    const int64_t* __restrict__ nbr, int64_t num_dst, const int64_t* num_dst_dev, int fanout,
    const T* __restrict__ ft, int64_t num_src, int heads, int log2_heads, int64_t dim,
    const float* __restrict__ el, const float* __restrict__ er, float slope, float* __restrict__ out,
    float* __restrict__ attn_out) {
  constexpr int kUnroll = 5;
  const int64_t n = actual_count(num_dst, num_dst_dev);
  const int lane = threadIdx.x % kWave;
  const int lph = static_cast<int>(dim / VEC);
  const int64_t row_len = static_cast<int64_t>(heads) * dim;
  const bool live = lane < heads * lph;
  const int hf = live ? lane / lph : 0;
  const int64_t d = static_cast<int64_t>(lane) * VEC;
  const int k = lane >> log2_heads, hs = lane & (heads - 1);
  const bool slot = k < fanout;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kAggWaves + threadIdx.x / kWave; i < n;
       i += static_cast<int64_t>(gridDim.x) * kAggWaves) {
    const int64_t id = slot ? nbr[i * fanout + k] : -1;
    const bool valid = id >= 0 && id < num_src;
    float e = -INFINITY;
    if (valid) {
      e = el[id * heads + hs] + er[i * heads + hs];
      e = e > 0.f ? e : e * slope;
    }
    float top = e;
    for (int off = heads; off < kWave; off <<= 1) top = fmaxf(top, __shfl_xor(top, off, kWave));
    const float w = valid ? expf(e - top) : 0.f;
    float denom = w;
    for (int off = heads; off < kWave; off <<= 1) denom += __shfl_xor(denom, off, kWave);
    const float a = denom > 0.f ? w / denom : 0.f;
    if (attn_out != nullptr && slot) attn_out[(i * fanout + k) * heads + hs] = a;
    float acc[VEC];
#pragma unroll
    for (int q = 0; q < VEC; ++q) acc[q] = 0.f;
    for (int u0 = 0; u0 < fanout; u0 += kUnroll) {
      float v[kUnroll][VEC];
      float au[kUnroll];
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        au[u] = 0.f;
#pragma unroll
        for (int q = 0; q < VEC; ++q) v[u][q] = 0.f;
        if (u0 + u < fanout) {
          const int64_t src = wave_read(id, (u0 + u) << log2_heads);
          if (src >= 0 && src < num_src) {
            au[u] = __shfl(a, ((u0 + u) << log2_heads) + hf, kWave);
            if (live) load_vec<T, VEC>(ft, src * row_len + d, v[u]);
          }
        }
      }
#pragma unroll
      for (int u = 0; u < kUnroll; ++u)
#pragma unroll
        for (int q = 0; q < VEC; ++q) acc[q] += au[u] * v[u][q];
    }
    if (live) {
#pragma unroll
      for (int q = 0; q < VEC; ++q) out[i * row_len + d + q] = acc[q];
    }
  }
}

template <typename T, int VEC>
static bool launch_gat_wave(const int64_t* nbr, int64_t num_dst, const int64_t* num_dst_dev, int fanout,
                            const void* ft, int64_t num_src, int heads, int64_t dim, const float* el,
                            const float* er, float slope, float* out, float* attn_out, hipStream_t st) {
  if (dim % VEC != 0 || (heads & (heads - 1)) != 0 || heads * fanout > kWave) return false;
  const int64_t lph = dim / VEC;
  if ((lph & (lph - 1)) != 0 || heads * lph > kWave) return false;
  int log2_heads = 0;
  while ((1 << log2_heads) < heads) ++log2_heads;
  const unsigned blocks = static_cast<unsigned>(std::min<int64_t>(ceil_div(num_dst, kAggWaves), 1 << 20));
  hipLaunchKernelGGL((gat_ell_wave_kernel<T, VEC>), dim3(blocks), dim3(kAggBlock), 0, st, nbr, num_dst, num_dst_dev,
                     fanout, static_cast<const T*>(ft), num_src, heads, log2_heads, dim, el, er, slope, out, attn_out);
  return true;
}

template <typename T, int VEC>
static void launch_gat(const int64_t* nbr, int64_t num_dst, const int64_t* num_dst_dev, int fanout,
                       const void* ft, int64_t num_src, int heads, int64_t dim, const float* el,
                       const float* er, float slope, float* out, float* attn_out, hipStream_t st) {
  const int64_t per_row = ceil_div(static_cast<int64_t>(heads) * dim, VEC);
  const T* x = static_cast<const T*>(ft);
#define APT_GAT(LPR)                                                                                  \
  hipLaunchKernelGGL((gat_ell_kernel<T, VEC, LPR>),                                                   \
                     dim3(static_cast<unsigned>(std::min<int64_t>(ceil_div(num_dst, kAggBlock / LPR), 1 << 20))), \
                     dim3(kAggBlock), 0, st, nbr, num_dst, num_dst_dev, fanout, x, num_src, heads, dim, el, er, \
                     slope, out, attn_out)
  if (per_row <= 8) APT_GAT(8);
  else if (per_row <= 16) APT_GAT(16);
  else if (per_row <= 32) APT_GAT(32);
  else APT_GAT(64);
#undef APT_GAT
}

// Backward of gat_ell_kernel, edge half.  A wavefront per (destination, head):
// with a = softmax(e) and out = sum a_k ft[s_k],
//   g_k  = dOut . ft[s_k]                     (gradient wrt a_k)
//   de_k = a_k (g_k - sum_j a_j g_j)          (softmax)
//   dz_k = de_k * (z_k > 0 ? 1 : slope)       (LeakyReLU, z_k = el[s_k] + er[i])
// Lane k keeps slot k (fanout <= 64).  Written in the block's COO order (edge
// id = csc_indptr[i] + rank of the slot among the row's edges): the attention
// weight a and dz per edge and head, and der[i, h] = sum_k dz_k.  The source half
// (d ft[s] = sum a dOut[dst], d el[s] = sum dz) is a sum over the edges of a
// source and runs through the SpMM kernels on the block's CSR order.
template <typename T>
__global__ __launch_bounds__(kAggBlock) void gat_bwd_edge_kernel(
    const int64_t* __restrict__ nbr, int64_t num_dst, int fanout, const T* __restrict__ ft, int64_t num_src,
    int heads, int64_t dim, const float* __restrict__ el, const float* __restrict__ er, float slope,
    const float* __restrict__ attn, const float* __restrict__ d_out, const int64_t* __restrict__ csc_indptr,
    float* __restrict__ a_edge, float* __restrict__ dz_edge, float* __restrict__ d_er) {
  const int lane = threadIdx.x % kWave;
  const int64_t items = num_dst * heads;
  for (int64_t it = static_cast<int64_t>(blockIdx.x) * kAggWaves + threadIdx.x / kWave; it < items;
       it += static_cast<int64_t>(gridDim.x) * kAggWaves) {
    const int64_t i = it / heads;
    const int h = static_cast<int>(it % heads);
    const int64_t* ids = nbr + i * fanout;
    const int64_t mine = lane < fanout ? ids[lane] : -1;
    const bool valid = mine >= 0 && mine < num_src;
    float g = 0.f;   // lane k: dOut[i, h] . ft[s_k, h]
    for (int k = 0; k < fanout; ++k) {
      const int64_t src = __shfl(mine, k, kWave);
      if (src < 0 || src >= num_src) continue;   // wave-uniform
      float part = 0.f;
      for (int64_t d = lane; d < dim; d += kWave)
        part += d_out[it * dim + d] * to_float<T>(ft[(src * heads + h) * dim + d]);
#pragma unroll
      for (int off = kWave / 2; off > 0; off >>= 1) part += __shfl_xor(part, off, kWave);
      if (lane == k) g = part;
    }
    const float a = valid ? attn[(i * fanout + lane) * heads + h] : 0.f;
    float s = a * g;
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) s += __shfl_xor(s, off, kWave);
    float dz = 0.f;
    if (valid) {
      const float z = el[mine * heads + h] + er[it];
      dz = a * (g - s) * (z > 0.f ? 1.f : slope);
    }
    float sum_dz = dz;
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) sum_dz += __shfl_xor(sum_dz, off, kWave);
    const uint64_t m = ballot(valid);
    if (valid) {
      const int64_t e = csc_indptr[i] + rank_below(m);
      a_edge[e * heads + h] = a;
      dz_edge[e * heads + h] = dz;
    }
    if (lane == 0) d_er[it] = sum_dz;
  }
}

// The same on a lane group per destination row, for rows that fit one pass of
// the group: LPH = dim / VEC lanes per head (a power of two), heads * LPH <= G
// lanes.  The row's source features are read once, VEC per lane; the dot of a
// slot is reduced over the head's lanes with xor shuffles and parked in
// dz_edge until the row's sum is known.
template <typename T, int VEC, int G>
__global__ __launch_bounds__(kAggBlock) void gat_bwd_edge_group_kernel(
    const int64_t* __restrict__ nbr, int64_t num_dst, int fanout, const T* __restrict__ ft, int64_t num_src,
    int heads, int64_t dim, const float* __restrict__ el, const float* __restrict__ er, float slope,
    const float* __restrict__ attn, const float* __restrict__ d_out, const int64_t* __restrict__ csc_indptr,
    float* __restrict__ a_edge, float* __restrict__ dz_edge, float* __restrict__ d_er) {
  constexpr int kGroups = kAggBlock / G;
  constexpr int kUnroll = 5;
  const int lph = static_cast<int>(dim / VEC);
  const int64_t row_len = static_cast<int64_t>(heads) * dim;
  const int grp = threadIdx.x / G, l = threadIdx.x % G;
  const bool live = l < heads * lph;
  const int h = live ? l / lph : 0;
  const bool leader = live && l % lph == 0;
  const int64_t d = static_cast<int64_t>(l) * VEC;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kGroups + grp; i < num_dst;
       i += static_cast<int64_t>(gridDim.x) * kGroups) {
    const int64_t* ids = nbr + i * fanout;
    const int64_t e0 = csc_indptr[i];
    float go[VEC];
#pragma unroll
    for (int q = 0; q < VEC; ++q) go[q] = live ? d_out[i * row_len + d + q] : 0.f;
    float s = 0.f;
    int64_t e = e0;
    for (int k0 = 0; k0 < fanout; k0 += kUnroll) {
      float v[kUnroll][VEC];
      bool ok[kUnroll];
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        ok[u] = false;
#pragma unroll
        for (int q = 0; q < VEC; ++q) v[u][q] = 0.f;
        if (k0 + u < fanout) {
          const int64_t src = ids[k0 + u];
          if (src >= 0 && src < num_src) {
            ok[u] = true;
            if (live) load_vec<T, VEC>(ft, src * row_len + d, v[u]);
          }
        }
      }
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        if (!ok[u]) continue;  // group-uniform
        float part = 0.f;
#pragma unroll
        for (int q = 0; q < VEC; ++q) part += go[q] * v[u][q];
        for (int off = lph / 2; off > 0; off >>= 1) part += __shfl_xor(part, off, kWave);
        if (leader) {
          s += attn[(i * fanout + k0 + u) * heads + h] * part;
          dz_edge[e * heads + h] = part;
        }
        ++e;
      }
    }
    if (leader) {
      const float er_i = er[i * heads + h];
      float sum_dz = 0.f;
      e = e0;
      for (int k = 0; k < fanout; ++k) {
        const int64_t src = ids[k];
        if (src < 0 || src >= num_src) continue;
        const float a = attn[(i * fanout + k) * heads + h];
        const float z = el[src * heads + h] + er_i;
        const float dz = a * (dz_edge[e * heads + h] - s) * (z > 0.f ? 1.f : slope);
        a_edge[e * heads + h] = a;
        dz_edge[e * heads + h] = dz;
        sum_dz += dz;
        ++e;
      }
      d_er[i * heads + h] = sum_dz;
    }
  }
}

// The same edge half with a wavefront per destination and two lane layouts.
// Feature layout: lane l holds VEC features of head l / lph (as above).  Slot
// layout: lane j holds (slot j / heads, head j % heads), so everything that
// exists once per (slot, head) -- the neighbour id, the attention weight, el, the
// dot product, the logit gradient, the edge position -- is loaded, computed and
// stored by all lanes at once (three coalesced loads and two coalesced stores per
// destination instead of six accesses per slot and head by one lane in sixteen).
// Needs heads and lph to be powers of two, heads * lph <= 64 and
// heads * fanout <= 64.
template <typename T, int VEC>
__global__ __launch_bounds__(kAggBlock) void gat_bwd_edge_wave_kernel(
    const int64_t* __restrict__ nbr, int64_t num_dst, int fanout, const T* __restrict__ ft, int64_t num_src,
    int heads, int log2_heads, int64_t dim, const float* __restrict__ el, const float* __restrict__ er, float slope,
    const float* __restrict__ attn, const float* __restrict__ d_out, const int64_t* __restrict__ csc_indptr,
    float* __restrict__ a_edge, float* __restrict__ dz_edge, float* __restrict__ d_er) {
  constexpr int kUnroll = 5;
  const int lane = threadIdx.x % kWave;
  const int lph = static_cast<int>(dim / VEC);
  const int64_t row_len = static_cast<int64_t>(heads) * dim;
  const bool live = lane < heads * lph;
  const int64_t d = static_cast<int64_t>(lane) * VEC;
  const int k = lane >> log2_heads, hs = lane & (heads - 1);   // slot layout
  const bool slot = k < fanout;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kAggWaves + threadIdx.x / kWave; i < num_dst;
       i += static_cast<int64_t>(gridDim.x) * kAggWaves) {
    const int64_t id = slot ? nbr[i * fanout + k] : -1;
    const bool valid = id >= 0 && id < num_src;
    const float a = valid ? attn[(i * fanout + k) * heads + hs] : 0.f;
    const float z = valid ? el[id * heads + hs] + er[i * heads + hs] : 0.f;
    const int64_t e0 = csc_indptr[i];
    float go[VEC];
#pragma unroll
    for (int q = 0; q < VEC; ++q) go[q] = live ? d_out[i * row_len + d + q] : 0.f;
    float my_part = 0.f;   // slot layout: dOut[i, hs] . ft[id, hs]
    for (int u0 = 0; u0 < fanout; u0 += kUnroll) {
      float v[kUnroll][VEC];
      bool ok[kUnroll];
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        ok[u] = false;
#pragma unroll
        for (int q = 0; q < VEC; ++q) v[u][q] = 0.f;
        if (u0 + u < fanout) {
          const int64_t src = wave_read(id, (u0 + u) << log2_heads);
          if (src >= 0 && src < num_src) {
            ok[u] = true;
            if (live) load_vec<T, VEC>(ft, src * row_len + d, v[u]);
          }
        }
      }
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        if (!ok[u]) continue;  // the same in all lanes
        float part = 0.f;
#pragma unroll
        for (int q = 0; q < VEC; ++q) part += go[q] * v[u][q];
        for (int off = lph / 2; off > 0; off >>= 1) part += __shfl_xor(part, off, kWave);
        const float got = __shfl(part, hs * lph, kWave);   // the dot product of head hs
        if (k == u0 + u) my_part = got;
      }
    }
    // sums over the slots of a head: lanes j, j ^ heads, j ^ 2 heads, ...
    float s = a * my_part;
    for (int off = heads; off < kWave; off <<= 1) s += __shfl_xor(s, off, kWave);
    const float dz = a * (my_part - s) * (z > 0.f ? 1.f : slope);
    float sum_dz = dz;
    for (int off = heads; off < kWave; off <<= 1) sum_dz += __shfl_xor(sum_dz, off, kWave);
    // position of the slot's edge: e0 + number of valid slots before it
    const uint64_t vm = ballot(valid && hs == 0);
    const int first = k << log2_heads;
    const int rank = __popcll(vm & (first == 0 ? 0ull : (~0ull >> (kWave - first))));
    if (valid) {
      const int64_t e = e0 + rank;
      a_edge[e * heads + hs] = a;
      dz_edge[e * heads + hs] = dz;
    }
    if (lane < heads) d_er[i * heads + lane] = sum_dz;   // lanes 0 .. heads-1 are (slot 0, head lane)
  }
}

template <typename T, int VEC>
static bool launch_gat_bwd_wave(const int64_t* nbr, int64_t num_dst, int fanout, const void* ft, int64_t num_src,
                                int heads, int64_t dim, const float* el, const float* er, float slope,
                                const float* attn, const float* d_out, const int64_t* csc_indptr, float* a_edge,
                                float* dz_edge, float* d_er, hipStream_t st) {
  if (dim % VEC != 0 || (heads & (heads - 1)) != 0 || heads * fanout > kWave) return false;
  const int64_t lph = dim / VEC;
  if ((lph & (lph - 1)) != 0 || heads * lph > kWave) return false;
  if ((reinterpret_cast<uintptr_t>(ft) & 15) != 0) return false;
  int log2_heads = 0;
  while ((1 << log2_heads) < heads) ++log2_heads;
  const unsigned blocks = static_cast<unsigned>(std::min<int64_t>(ceil_div(num_dst, kAggWaves), 1 << 20));
  hipLaunchKernelGGL((gat_bwd_edge_wave_kernel<T, VEC>), dim3(blocks), dim3(kAggBlock), 0, st, nbr, num_dst, fanout,
                     static_cast<const T*>(ft), num_src, heads, log2_heads, dim, el, er, slope, attn, d_out,
                     csc_indptr, a_edge, dz_edge, d_er);
  return true;
}

template <typename T, int VEC>
static bool launch_gat_bwd_group(const int64_t* nbr, int64_t num_dst, int fanout, const void* ft, int64_t num_src,
                                 int heads, int64_t dim, const float* el, const float* er, float slope,
                                 const float* attn, const float* d_out, const int64_t* csc_indptr, float* a_edge,
                                 float* dz_edge, float* d_er, hipStream_t st) {
  if (dim % VEC != 0) return false;
  const int64_t lph = dim / VEC;
  if (lph > kWave || (lph & (lph - 1)) != 0 || heads * lph > kWave) return false;
  if ((reinterpret_cast<uintptr_t>(ft) & 15) != 0) return false;
  const int64_t lanes = heads * lph;
  const T* x = static_cast<const T*>(ft);
#define APT_GATB(G)                                                                                   \
  hipLaunchKernelGGL((gat_bwd_edge_group_kernel<T, VEC, G>),                                          \
                     dim3(static_cast<unsigned>(std::min<int64_t>(ceil_div(num_dst, kAggBlock / G), 1 << 20))), \
                     dim3(kAggBlock), 0, st, nbr, num_dst, fanout, x, num_src, heads, dim, el, er, slope, attn, \
                     d_out, csc_indptr, a_edge, dz_edge, d_er)
  if (lanes <= 8) APT_GATB(8);
  else if (lanes <= 16) APT_GATB(16);
  else if (lanes <= 32) APT_GATB(32);
  else APT_GATB(64);
#undef APT_GATB
  return true;
}

static int agg_check(const char* who, const int64_t* row, const int64_t* col, int64_t E, const void* in,
                     float* out, const int64_t* coo_off, int num_seg, int64_t dim, int elem_size) {
  APT_REQUIRE(E >= 0 && dim > 0, APT_EINVAL, "%s: bad shape (E %lld, dim %lld)", who, (long long)E,
              (long long)dim);
  APT_REQUIRE(elem_size == 2 || elem_size == 4, APT_EINVAL, "%s: elem_size %d (4 = fp32, 2 = bf16)", who,
              elem_size);
  APT_REQUIRE(num_seg >= 1 && num_seg <= kMaxSegments - 1, APT_ELIMIT, "%s: %d segments outside [1, %d]",
              who, num_seg, kMaxSegments - 1);
  APT_REQUIRE(coo_off != nullptr, APT_EINVAL, "%s: coo_offset is NULL", who);
  APT_REQUIRE(E == 0 || (row != nullptr && col != nullptr && in != nullptr && out != nullptr), APT_EINVAL,
              "%s: a tensor is NULL", who);
  return APT_OK;
}

}  // namespace apt

extern "C" int apt_spmm_sum(int mode, const int64_t* coo_row, const int64_t* coo_col, int64_t num_edges,
                            const void* input, int64_t num_in_rows, const void* edata, int64_t dim,
                            int elem_size, const int64_t* coo_offset, const int64_t* input_offset,
                            const int64_t* output_offset, int num_segments, float* out,
                            int64_t num_out_rows, const int* grouped_dev, void* stream) {
  using namespace apt;
  APT_REQUIRE(mode >= 0 && mode <= 2, APT_EINVAL, "apt_spmm_sum: mode %d (0 copy_u, 1 copy_e, 2 u_mul_e)", mode);
  int rc = agg_check("apt_spmm_sum", coo_row, coo_col, num_edges, input, out, coo_offset, num_segments, dim,
                     elem_size);
  if (rc != APT_OK) return rc;
  APT_REQUIRE(mode != 2 || edata != nullptr || num_edges == 0, APT_EINVAL, "apt_spmm_sum: edata is NULL");
  APT_REQUIRE(num_out_rows >= 0 && num_in_rows >= 0, APT_EINVAL, "apt_spmm_sum: negative row count");
  if (num_edges == 0) return APT_OK;
  AggParams p{};
  p.row = coo_row; p.col = coo_col; p.num_edges = num_edges; p.in = input; p.edata = edata; p.out = out;
  p.coo_off = coo_offset; p.in_off = input_offset; p.out_off = output_offset; p.num_seg = num_segments;
  p.dim = dim; p.num_in_rows = num_in_rows; p.num_e_rows = num_edges; p.num_out_rows = num_out_rows;
  // with several segments two segments may share output rows, so the flag only counts for plain COO
  p.grouped_dev = num_segments == 1 ? grouped_dev : nullptr;
  const int64_t waves = ceil_div(num_edges, kEdgesPerWave);
  const dim3 grid(static_cast<unsigned>(ceil_div(waves, kAggWaves))), block(kAggBlock);
  hipStream_t st = static_cast<hipStream_t>(stream);
  // 4 features per lane when rows are 4-element aligned
  const bool vec4 = dim % 4 == 0 && (reinterpret_cast<uintptr_t>(input) & 15) == 0 &&
                    (edata == nullptr || (reinterpret_cast<uintptr_t>(edata) & 15) == 0);
#define APT_SPMM_LAUNCH(T, V)                                                            \
  switch (mode) {                                                                         \
    case 0: hipLaunchKernelGGL((spmm_kernel<T, 0, V>), grid, block, 0, st, p); break;      \
    case 1: hipLaunchKernelGGL((spmm_kernel<T, 1, V>), grid, block, 0, st, p); break;      \
    default: hipLaunchKernelGGL((spmm_kernel<T, 2, V>), grid, block, 0, st, p); break;     \
  }
  if (elem_size == 4) {
    if (vec4) { APT_SPMM_LAUNCH(float, 4) } else { APT_SPMM_LAUNCH(float, 1) }
  } else {
    if (vec4) { APT_SPMM_LAUNCH(uint16_t, 4) } else { APT_SPMM_LAUNCH(uint16_t, 1) }
  }
#undef APT_SPMM_LAUNCH
  APT_LAUNCH_CHECK("spmm_kernel");
  return APT_OK;
}

extern "C" int apt_coo_is_grouped(const int64_t* coo_col, int64_t num_edges, int* flag, void* stream) {
  using namespace apt;
  APT_REQUIRE(num_edges >= 0 && flag != nullptr && (coo_col != nullptr || num_edges == 0), APT_EINVAL,
              "apt_coo_is_grouped: bad arguments");
  hipStream_t st = static_cast<hipStream_t>(stream);
  hipLaunchKernelGGL(coo_grouped_init_kernel, dim3(1), dim3(1), 0, st, flag);
  if (num_edges > 1) {
    const unsigned blocks = static_cast<unsigned>(std::min<int64_t>(ceil_div(num_edges, kAggBlock), 4096));
    hipLaunchKernelGGL(coo_grouped_check_kernel, dim3(blocks), dim3(kAggBlock), 0, st, coo_col, num_edges, flag);
  }
  APT_LAUNCH_CHECK("coo_grouped_check_kernel");
  return APT_OK;
}

extern "C" int apt_sddmm(int op, const int64_t* coo_row, const int64_t* coo_col, int64_t num_edges,
                         const void* lhs, int64_t num_lhs_rows, const void* rhs, int64_t num_rhs_rows,
                         int64_t dim, int elem_size, const int64_t* coo_offset, const int64_t* lhs_offset,
                         const int64_t* rhs_offset, int num_segments, float* out, void* stream) {
  using namespace apt;
  APT_REQUIRE(op == 0 || op == 1, APT_EINVAL, "apt_sddmm: op %d (0 u_add_v, 1 u_mul_v)", op);
  int rc = agg_check("apt_sddmm", coo_row, coo_col, num_edges, lhs, out, coo_offset, num_segments, dim,
                     elem_size);
  if (rc != APT_OK) return rc;
  APT_REQUIRE(rhs != nullptr || num_edges == 0, APT_EINVAL, "apt_sddmm: rhs is NULL");
  if (num_edges == 0) return APT_OK;
  AggParams p{};
  p.row = coo_row; p.col = coo_col; p.num_edges = num_edges; p.in = lhs; p.edata = rhs; p.out = out;
  p.coo_off = coo_offset; p.in_off = lhs_offset; p.out_off = rhs_offset; p.num_seg = num_segments;
  p.dim = dim; p.num_in_rows = num_lhs_rows; p.num_e_rows = num_rhs_rows; p.num_out_rows = 0;
  const dim3 grid(static_cast<unsigned>(std::min<int64_t>(ceil_div(num_edges, kAggWaves), 1 << 16))),
      block(kAggBlock);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (elem_size == 4) {
    if (op == 0) hipLaunchKernelGGL((sddmm_kernel<float, 0>), grid, block, 0, st, p);
    else hipLaunchKernelGGL((sddmm_kernel<float, 1>), grid, block, 0, st, p);
  } else {
    if (op == 0) hipLaunchKernelGGL((sddmm_kernel<uint16_t, 0>), grid, block, 0, st, p);
    else hipLaunchKernelGGL((sddmm_kernel<uint16_t, 1>), grid, block, 0, st, p);
  }
  APT_LAUNCH_CHECK("sddmm_kernel");
  return APT_OK;
}

extern "C" int apt_spmm_block(const int64_t* neighbors, int64_t num_dst, const int64_t* num_dst_dev,
                              int fanout, const void* input, int64_t num_src, int64_t dim, int elem_size,
                              int mean, float* out, void* stream) {
  using namespace apt;
  APT_REQUIRE(num_dst >= 0 && fanout > 0 && dim > 0 && num_src >= 0, APT_EINVAL,
              "apt_spmm_block: bad shape (num_dst %lld, fanout %d, dim %lld)", (long long)num_dst, fanout,
              (long long)dim);
  APT_REQUIRE(elem_size == 2 || elem_size == 4, APT_EINVAL, "apt_spmm_block: elem_size %d (4 = fp32, 2 = bf16)",
              elem_size);
  if (num_dst == 0) return APT_OK;
  APT_REQUIRE(neighbors != nullptr && out != nullptr && (input != nullptr || num_src == 0), APT_EINVAL,
              "apt_spmm_block: a tensor is NULL");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool vec4 = dim % 4 == 0 && (reinterpret_cast<uintptr_t>(input) & 15) == 0 &&
                    (reinterpret_cast<uintptr_t>(out) & 15) == 0;
  if (elem_size == 4) {
    if (vec4) launch_ell<float, 4>(neighbors, num_dst, num_dst_dev, fanout, input, num_src, dim, out, mean, st);
    else launch_ell<float, 1>(neighbors, num_dst, num_dst_dev, fanout, input, num_src, dim, out, mean, st);
  } else {
    if (vec4 && dim % 8 == 0) launch_ell<uint16_t, 8>(neighbors, num_dst, num_dst_dev, fanout, input, num_src, dim, out, mean, st);
    else if (vec4) launch_ell<uint16_t, 4>(neighbors, num_dst, num_dst_dev, fanout, input, num_src, dim, out, mean, st);
    else launch_ell<uint16_t, 1>(neighbors, num_dst, num_dst_dev, fanout, input, num_src, dim, out, mean, st);
  }
  APT_LAUNCH_CHECK("spmm_ell_kernel");
  return APT_OK;
}

extern "C" int apt_gat_scores(const void* x, int64_t num_rows, int heads, int64_t dim, int elem_size,
                              const float* attn, float* out, void* stream) {
  using namespace apt;
  APT_REQUIRE(num_rows >= 0 && heads > 0 && dim > 0, APT_EINVAL,
              "apt_gat_scores: bad shape (rows %lld, heads %d, dim %lld)", (long long)num_rows, heads,
              (long long)dim);
  APT_REQUIRE(elem_size == 2 || elem_size == 4, APT_EINVAL, "apt_gat_scores: elem_size %d (4 = fp32, 2 = bf16)",
              elem_size);
  if (num_rows == 0) return APT_OK;
  APT_REQUIRE(x != nullptr && attn != nullptr && out != nullptr, APT_EINVAL, "apt_gat_scores: a tensor is NULL");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int64_t items = num_rows * heads;
  const int vec = elem_size == 2 && dim % 8 == 0 ? 8 : 4;   // 16 bytes per lane
  const int64_t lph = dim / vec;
  if (dim % 4 == 0 && lph <= kWave && (lph & (lph - 1)) == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0 &&
      (reinterpret_cast<uintptr_t>(attn) & 15) == 0) {
#define APT_SCORES(T, V, LPH)                                                                           \
  hipLaunchKernelGGL((gat_scores_vec_kernel<T, V, LPH>),                                                \
                     dim3(static_cast<unsigned>(std::min<int64_t>(ceil_div(items, kAggBlock / LPH), 1 << 20))), \
                     dim3(kAggBlock), 0, st, static_cast<const T*>(x), items, heads, attn, out)
#define APT_SCORES_T(T, V)                               \
  switch (lph) {                                         \
    case 1: APT_SCORES(T, V, 1); break;                  \
    case 2: APT_SCORES(T, V, 2); break;                  \
    case 4: APT_SCORES(T, V, 4); break;                  \
    case 8: APT_SCORES(T, V, 8); break;                  \
    case 16: APT_SCORES(T, V, 16); break;                \
    case 32: APT_SCORES(T, V, 32); break;                \
    default: APT_SCORES(T, V, 64); break;                \
  }
    if (elem_size == 4) { APT_SCORES_T(float, 4) }
    else if (vec == 8) { APT_SCORES_T(uint16_t, 8) }
    else { APT_SCORES_T(uint16_t, 4) }
#undef APT_SCORES_T
#undef APT_SCORES
    APT_LAUNCH_CHECK("gat_scores_vec_kernel");
    return APT_OK;
  }
  const unsigned blocks = static_cast<unsigned>(std::min<int64_t>(ceil_div(items, kAggWaves), 1 << 20));
  if (elem_size == 4)
    hipLaunchKernelGGL(gat_scores_kernel<float>, dim3(blocks), dim3(kAggBlock), 0, st,
                       static_cast<const float*>(x), num_rows, heads, dim, attn, out);
  else
    hipLaunchKernelGGL(gat_scores_kernel<uint16_t>, dim3(blocks), dim3(kAggBlock), 0, st,
                       static_cast<const uint16_t*>(x), num_rows, heads, dim, attn, out);
  APT_LAUNCH_CHECK("gat_scores_kernel");
  return APT_OK;
}

extern "C" int apt_gat_block(const int64_t* neighbors, int64_t num_dst, const int64_t* num_dst_dev, int fanout,
                             const void* ft, int64_t num_src, int heads, int64_t dim, int elem_size,
                             const float* el, const float* er, float negative_slope, float* out,
                             float* attn_out, void* stream) {
  using namespace apt;
  APT_REQUIRE(num_dst >= 0 && fanout > 0 && heads > 0 && dim > 0 && num_src >= 0, APT_EINVAL,
              "apt_gat_block: bad shape (num_dst %lld, fanout %d, heads %d, dim %lld)", (long long)num_dst,
              fanout, heads, (long long)dim);
  APT_REQUIRE(elem_size == 2 || elem_size == 4, APT_EINVAL, "apt_gat_block: elem_size %d (4 = fp32, 2 = bf16)",
              elem_size);
  if (num_dst == 0) return APT_OK;
  APT_REQUIRE(neighbors != nullptr && out != nullptr && er != nullptr &&
                  ((ft != nullptr && el != nullptr) || num_src == 0),
              APT_EINVAL, "apt_gat_block: a tensor is NULL");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool vec4 = dim % 4 == 0 && (reinterpret_cast<uintptr_t>(ft) & 15) == 0 &&
                    (reinterpret_cast<uintptr_t>(out) & 15) == 0;
  if (vec4 && num_src > 0 &&
      (elem_size == 4 ? launch_gat_wave<float, 4>(neighbors, num_dst, num_dst_dev, fanout, ft, num_src, heads, dim, el,
                                                  er, negative_slope, out, attn_out, st)
                      : launch_gat_wave<uint16_t, 4>(neighbors, num_dst, num_dst_dev, fanout, ft, num_src, heads, dim,
                                                     el, er, negative_slope, out, attn_out, st))) {
    APT_LAUNCH_CHECK("gat_ell_wave_kernel");
    return APT_OK;
  }
  if (elem_size == 4) {
    if (vec4) launch_gat<float, 4>(neighbors, num_dst, num_dst_dev, fanout, ft, num_src, heads, dim, el, er, negative_slope, out, attn_out, st);
    else launch_gat<float, 1>(neighbors, num_dst, num_dst_dev, fanout, ft, num_src, heads, dim, el, er, negative_slope, out, attn_out, st);
  } else {
    if (vec4 && dim % 8 == 0) launch_gat<uint16_t, 8>(neighbors, num_dst, num_dst_dev, fanout, ft, num_src, heads, dim, el, er, negative_slope, out, attn_out, st);
    else if (vec4) launch_gat<uint16_t, 4>(neighbors, num_dst, num_dst_dev, fanout, ft, num_src, heads, dim, el, er, negative_slope, out, attn_out, st);
    else launch_gat<uint16_t, 1>(neighbors, num_dst, num_dst_dev, fanout, ft, num_src, heads, dim, el, er, negative_slope, out, attn_out, st);
  }
  APT_LAUNCH_CHECK("gat_ell_kernel");
  return APT_OK;
}

extern "C" int apt_spmm_heads(const int64_t* coo_row, const int64_t* coo_col, int64_t num_edges,
                              const void* input, int64_t num_in_rows, const float* head_weights,
                              const int64_t* weight_row, int heads, int64_t dim, int elem_size, int grouped,
                              float* out, int64_t num_out_rows, const float* head_weights2, float* out2,
                              const int64_t* out_indptr, void* stream) {
  using namespace apt;
  APT_REQUIRE(num_edges >= 0 && heads > 0 && dim > 0 && dim % heads == 0, APT_EINVAL,
              "apt_spmm_heads: bad shape (E %lld, heads %d, dim %lld)", (long long)num_edges, heads,
              (long long)dim);
  APT_REQUIRE(elem_size == 2 || elem_size == 4, APT_EINVAL, "apt_spmm_heads: elem_size %d (4 = fp32, 2 = bf16)",
              elem_size);
  APT_REQUIRE(num_out_rows >= 0 && num_in_rows >= 0, APT_EINVAL, "apt_spmm_heads: negative row count");
  APT_REQUIRE(out_indptr == nullptr || grouped != 0, APT_EINVAL, "apt_spmm_heads: out_indptr needs grouped edges");
  APT_REQUIRE(heads <= kWave || out2 == nullptr || out_indptr == nullptr, APT_ELIMIT,
              "apt_spmm_heads: out_indptr with a second sum supports at most 64 heads");
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (out_indptr != nullptr && num_out_rows > 0) {
    APT_REQUIRE(out != nullptr, APT_EINVAL, "apt_spmm_heads: out is NULL");
    const unsigned zb = static_cast<unsigned>(std::min<int64_t>(ceil_div(num_out_rows, kAggBlock), 1 << 20));
    hipLaunchKernelGGL(spmm_zero_rows_kernel, dim3(zb), dim3(kAggBlock), 0, st, out_indptr, num_out_rows, dim, out,
                       out2, heads);
    APT_LAUNCH_CHECK("spmm_zero_rows_kernel");
  }
  if (num_edges == 0) return APT_OK;
  APT_REQUIRE(coo_row != nullptr && coo_col != nullptr && input != nullptr && out != nullptr, APT_EINVAL,
              "apt_spmm_heads: a tensor is NULL");
  AggParams p{};
  p.row = coo_row; p.col = coo_col; p.num_edges = num_edges; p.in = input; p.out = out;
  p.num_seg = 1;  // no segment tables: every edge in segment 0, offsets 0
  p.coo_off = nullptr;
  p.dim = dim; p.num_in_rows = num_in_rows; p.num_e_rows = num_edges; p.num_out_rows = num_out_rows;
  p.head_w = head_weights; p.head_w_row = weight_row; p.heads = heads; p.head_dim = dim / heads;
  p.grouped = grouped != 0;
  p.out_indptr = out_indptr;
  APT_REQUIRE((head_weights2 == nullptr) == (out2 == nullptr), APT_EINVAL,
              "apt_spmm_heads: head_weights2 and out2 go together");
  p.head_w2 = head_weights2; p.out2 = out2;
  const int64_t waves = ceil_div(num_edges, kEdgesPerWave);
  const dim3 grid(static_cast<unsigned>(ceil_div(waves, kAggWaves))), block(kAggBlock);
  const bool vec4 = p.head_dim % 4 == 0 && (reinterpret_cast<uintptr_t>(input) & 15) == 0;
  if (elem_size == 4) {
    if (vec4) hipLaunchKernelGGL((spmm_kernel<float, 3, 4>), grid, block, 0, st, p);
    else hipLaunchKernelGGL((spmm_kernel<float, 3, 1>), grid, block, 0, st, p);
  } else {
    if (vec4) hipLaunchKernelGGL((spmm_kernel<uint16_t, 3, 4>), grid, block, 0, st, p);
    else hipLaunchKernelGGL((spmm_kernel<uint16_t, 3, 1>), grid, block, 0, st, p);
  }
  APT_LAUNCH_CHECK("spmm_kernel");
  return APT_OK;
}

extern "C" int apt_gat_block_backward(const int64_t* neighbors, int64_t num_dst, int fanout, const void* ft,
                                      int64_t num_src, int heads, int64_t dim, int elem_size, const float* el,
                                      const float* er, float negative_slope, const float* attn,
                                      const float* d_out, const int64_t* csc_indptr, float* a_edge,
                                      float* dz_edge, float* d_er, void* stream) {
  using namespace apt;
  APT_REQUIRE(num_dst >= 0 && fanout > 0 && fanout <= kWave && heads > 0 && dim > 0 && num_src >= 0, APT_EINVAL,
              "apt_gat_block_backward: bad shape (num_dst %lld, fanout %d (1..64), heads %d, dim %lld)",
              (long long)num_dst, fanout, heads, (long long)dim);
  APT_REQUIRE(elem_size == 2 || elem_size == 4, APT_EINVAL,
              "apt_gat_block_backward: elem_size %d (4 = fp32, 2 = bf16)", elem_size);
  if (num_dst == 0) return APT_OK;
  APT_REQUIRE(neighbors != nullptr && ft != nullptr && el != nullptr && er != nullptr && attn != nullptr &&
                  d_out != nullptr && csc_indptr != nullptr && a_edge != nullptr && dz_edge != nullptr &&
                  d_er != nullptr,
              APT_EINVAL, "apt_gat_block_backward: a tensor is NULL");
  const unsigned blocks =
      static_cast<unsigned>(std::min<int64_t>(ceil_div(num_dst * heads, kAggWaves), 1 << 20));
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool by_wave =
      elem_size == 4 ? launch_gat_bwd_wave<float, 4>(neighbors, num_dst, fanout, ft, num_src, heads, dim, el, er,
                                                     negative_slope, attn, d_out, csc_indptr, a_edge, dz_edge, d_er, st)
                     : launch_gat_bwd_wave<uint16_t, 4>(neighbors, num_dst, fanout, ft, num_src, heads, dim, el, er,
                                                        negative_slope, attn, d_out, csc_indptr, a_edge, dz_edge, d_er,
                                                        st);
  if (by_wave) {
    APT_LAUNCH_CHECK("gat_bwd_edge_wave_kernel");
    return APT_OK;
  }
  const bool grouped =
      elem_size == 4
          ? launch_gat_bwd_group<float, 4>(neighbors, num_dst, fanout, ft, num_src, heads, dim, el, er,
                                           negative_slope, attn, d_out, csc_indptr, a_edge, dz_edge, d_er, st)
          : (launch_gat_bwd_group<uint16_t, 8>(neighbors, num_dst, fanout, ft, num_src, heads, dim, el, er,
                                               negative_slope, attn, d_out, csc_indptr, a_edge, dz_edge, d_er, st) ||
             launch_gat_bwd_group<uint16_t, 4>(neighbors, num_dst, fanout, ft, num_src, heads, dim, el, er,
                                               negative_slope, attn, d_out, csc_indptr, a_edge, dz_edge, d_er, st));
  if (grouped) {
    APT_LAUNCH_CHECK("gat_bwd_edge_group_kernel");
    return APT_OK;
  }
  if (elem_size == 4)
    hipLaunchKernelGGL(gat_bwd_edge_kernel<float>, dim3(blocks), dim3(kAggBlock), 0, st, neighbors, num_dst,
                       fanout, static_cast<const float*>(ft), num_src, heads, dim, el, er, negative_slope, attn,
                       d_out, csc_indptr, a_edge, dz_edge, d_er);
  else
    hipLaunchKernelGGL(gat_bwd_edge_kernel<uint16_t>, dim3(blocks), dim3(kAggBlock), 0, st, neighbors, num_dst,
                       fanout, static_cast<const uint16_t*>(ft), num_src, heads, dim, el, er, negative_slope, attn,
                       d_out, csc_indptr, a_edge, dz_edge, d_er);
  APT_LAUNCH_CHECK("gat_bwd_edge_kernel");
  return APT_OK;
}
