// Indexed row gather from HBM-resident feature tables, and the row
// permute / scatter that FeatShuffle does on the GPU.
//
// Replaces _CSRRowWiseLoadSubtensorAlignedAllKernel / IndexSelectAll
// (reference src/cuda/npc_kernel.cu:187-246) and the index_select /
// index_select_backward halves of FeatShuffle (src/feat_shuffle.cc:14-16,27).
// The reference moves one 4-byte element per thread and reads
// feat_pos_map[index[row]] twice per thread; here a lane group owns a row,
// reads the id and the position once, and moves the row as 16-byte vectors
// (8/4/2-byte vectors when the row geometry is not 16-byte aligned), with
// several rows per group in flight.  Pure copy: results are bit-exact.
#include <hip/hip_ext.h>

#include "common.hpp"
#include "rank_table.hpp"

namespace apt {

constexpr int kGatherBlock = 256;
constexpr int kGatherPersistentBlocks = 16384;
constexpr int kGatherResidentBlocks = 2048;   // 256 CUs x 8 workgroups of 256 threads (if the runtime cannot be asked)

struct GatherParams {
  const char* local_table;
  int64_t num_local_rows;
  int64_t local_row_bytes;   // local_dim * elem_size
  int64_t col_offset_bytes;
  const char* cache_table;
  int64_t num_cache_rows;
  const int64_t* pos_map;
  int64_t num_total_nodes;
  int64_t out_row_bytes;
  const int64_t* index;
  int64_t n;
  const int64_t* n_dev;
  char* out;
  int64_t* miss_count;
  int scatter;               // 1: out[index[r]] = in[r] (pack); rows come from local_table
  int64_t num_out_rows;      // scatter only
  uint8_t* named;            // scatter only, optional: named[v] = 1 for every output row v that is written
  int store_policy;          // kStore* (apt_set_tuning gather_store_policy)
  int64_t wt_tail_bytes;     // kStoreAuto on a large output: the last bytes written go write-through
  int lookup_blocks;         // the first workgroups of the grid do a batch's pending relabel lookups instead
};

template <int V> struct VecT;
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
template <> struct VecT<16> { using type = u32x4_t; };
template <> struct VecT<8> { using type = u32x2_t; };
template <> struct VecT<4> { using type = uint32_t; };
template <> struct VecT<2> { using type = uint16_t; };

// Source address of the row for node v, or nullptr when it is not present
// (reference :196-205 for the two-table addressing).
__device__ __forceinline__ const char* source_row(const GatherParams& p, int64_t v) {
  if (v < 0) return nullptr;
  if (p.pos_map != nullptr) {
    if (v >= p.num_total_nodes) return nullptr;
    const int64_t pos = p.pos_map[v];
    if (pos < -1) {
      const int64_t row = -pos - 2;
      if (row >= p.num_local_rows) return nullptr;
      return p.local_table + row * p.local_row_bytes + p.col_offset_bytes;
    }
    if (pos < 0 || pos >= p.num_cache_rows) return nullptr;
    return p.cache_table + pos * p.out_row_bytes;
  }
  if (v >= p.num_local_rows) return nullptr;
  return p.local_table + v * p.local_row_bytes + p.col_offset_bytes;
}

// How a lane stores its 16 bytes of a gathered row.
//   write-through  the line goes on to the memory side as it is written instead
//                  of staying dirty in this XCD's L2 until the release at the
//                  end of the kernel writes the whole L2 back: the launch itself
//                  is 6-10 % shorter.  But the output then fills the memory-side
//                  cache, and what the next kernels of the batch kept there (the
//                  sampler's rank table) is gone: after a launch that writes
//                  185 MB the last hop's sampling kernel takes 84 instead of
//                  72 us and the batch is 3-4 % slower; after one that writes
//                  62 MB nothing is lost and the batch is 1-2 % faster.
//   non-temporal   streaming hint; the output does not displace anything.
//   plain          neither.
// kStoreAuto (shipped) decides per launch, on the device, from the rows it
// actually gathers: write-through while the output is at most half of the
// 256 MB memory-side cache; beyond that non-temporal, except for the 64 MB that
// the kernel writes last, which would otherwise be what the release at its end
// still has to write back.  That tail is a trade, not a gain: on a 185 MB output
// every 16 MB of it take 0.6 us off the launch and add about as much to the next
// batch's sampling kernel (70.2 -> 67.6 us and 71.4 -> 72.7 us at 64 MB); the
// batch is at its shortest between 48 and 64 MB (0.2119 against 0.2125 ms).
// Narrower vectors (row geometry not 16-byte aligned) have no write-through form
// and use non-temporal stores.
enum : int { kStoreAuto = 0, kStoreNonTemporal = 1, kStorePlain = 2, kStoreWriteThrough = 3 };
constexpr int64_t kWriteThroughMaxBytes = int64_t{128} << 20;
constexpr int64_t kWriteThroughTailMiB = 64;

template <int V>
__device__ __forceinline__ void store_row_vec(typename VecT<V>::type val, typename VecT<V>::type* dst, int policy) {
  if (V == 16 && policy == kStoreWriteThrough) {
    asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1" ::"v"(dst), "v"(val) : "memory");
  } else if (policy == kStorePlain) {
    *dst = val;
  } else {
    __builtin_nontemporal_store(val, dst);
  }
}

// LPR lanes per row, R rows per group per step, V bytes per lane access.
// A batch's pending relabel lookups (rank_table.hpp) can ride in the first
// workgroups of the grid: they wait on a few dependent random reads while the
// rest of the grid streams rows.
template <int V, int LPR, int R>
__device__ __forceinline__ void gather_rows_of_block(const GatherParams& p, int64_t block, int64_t num_blocks) {
  using Vec = typename VecT<V>::type;
  constexpr int kGroups = kGatherBlock / LPR;
  const int grp = threadIdx.x / LPR;
  const int l = threadIdx.x % LPR;
  const int64_t vec_per_row = p.out_row_bytes / V;
  const int64_t rows_per_block = static_cast<int64_t>(kGroups) * R;
  const int64_t stride = num_blocks * rows_per_block;
  int64_t base = block * rows_per_block;
  // The ids of a group's first rows are asked for before the device-side count has arrived: index[] has p.n
  // entries whatever the count says, so the two round trips overlap instead of following each other (a launch
  // of a few hundred thousand rows is a handful of iterations per group, and its first one starts on a cold
  // path).  Later iterations fetch their ids at the end of the iteration before.
  int64_t id[R];
#pragma unroll
  for (int k = 0; k < R; ++k) {
    const int64_t r = base + static_cast<int64_t>(k) * kGroups + grp;
    id[k] = r < p.n ? p.index[r] : -1;
  }
  const int64_t n = actual_count(p.n, p.n_dev);
  int launch_policy = p.store_policy;
  // rows from wt_from on are stored write-through: everything when the output is small, else the part the kernel
  // writes last
  int64_t wt_from = n;
  if (launch_policy == kStoreAuto) {
    launch_policy = kStoreNonTemporal;
    wt_from = n * p.out_row_bytes <= kWriteThroughMaxBytes ? 0 : n - p.wt_tail_bytes / p.out_row_bytes;
  }
  int64_t misses = 0;
  while (base < n) {
    const int policy = base >= wt_from ? kStoreWriteThrough : launch_policy;
    const char* src[R];
    char* dst[R];
#pragma unroll
    for (int k = 0; k < R; ++k) {
      const int64_t r = base + static_cast<int64_t>(k) * kGroups + grp;
      src[k] = nullptr;
      dst[k] = nullptr;
      if (r < n) {
        const int64_t v = id[k];
        if (p.scatter) {
          // pack: row r of the input goes to row index[r] of the output
          if (v >= 0 && v < p.num_out_rows) {
            src[k] = p.local_table + r * p.out_row_bytes;
            dst[k] = p.out + v * p.out_row_bytes;
            if (p.named != nullptr && l == 0) p.named[v] = 1;
          }
        } else {
          src[k] = source_row(p, v);
          dst[k] = p.out + r * p.out_row_bytes;
          if (src[k] == nullptr && l == 0) ++misses;
        }
      }
    }
    for (int64_t c = l; c < vec_per_row; c += LPR) {
      Vec val[R];
#pragma unroll
      for (int k = 0; k < R; ++k) {
        val[k] = Vec{};
        if (src[k] != nullptr)
          val[k] = __builtin_nontemporal_load(reinterpret_cast<const Vec*>(src[k]) + c);
      }
#pragma unroll
      for (int k = 0; k < R; ++k) {
        if (dst[k] != nullptr) store_row_vec<V>(val[k], reinterpret_cast<Vec*>(dst[k]) + c, policy);
      }
    }
    base += stride;
#pragma unroll
    for (int k = 0; k < R; ++k) {
      const int64_t r = base + static_cast<int64_t>(k) * kGroups + grp;
      if (r < n) id[k] = p.index[r];
    }
  }
  if (p.miss_count != nullptr && misses != 0)
    atomicAdd(reinterpret_cast<unsigned long long*>(p.miss_count),
              static_cast<unsigned long long>(misses));
}

template <int V, int LPR, int R>
__global__ __launch_bounds__(kGatherBlock) void gather_kernel(GatherParams p) {
  gather_rows_of_block<V, LPR, R>(p, blockIdx.x, gridDim.x);
}

// The gather with a batch's pending relabel lookups in its grid (16-byte vectors, two rows in flight): the
// grid's first workgroups do the lookup pass, whose dependent reads are then on their way while the rest stream
// rows.  The lookup blocks are numbered after the gather's and the workgroup ids rotated, rather than numbering
// them first and subtracting: written that way a launch of 235 k rows took 27 instead of 22 us.
template <int LPR>
__global__ __launch_bounds__(kGatherBlock) void gather_with_lookup_kernel(GatherParams p, LookupParams lp) {
  static_assert(kGatherBlock == kLookupBlock, "the lookup pass runs in workgroups of the gather's size");
  const int64_t num_blocks = static_cast<int64_t>(gridDim.x) - p.lookup_blocks;
  int64_t block = static_cast<int64_t>(blockIdx.x) + num_blocks;
  if (block >= static_cast<int64_t>(gridDim.x)) block -= gridDim.x;
  if (block >= num_blocks) {
    lookup_block(lp, block - num_blocks);
    return;
  }
  gather_rows_of_block<16, LPR, 2>(p, block, num_blocks);
}

static thread_local hipEvent_t t_gather_start = nullptr, t_gather_stop = nullptr;

// Takes the one-shot events off the thread at entry; rearm() hands them to the
// launch that follows.
struct TimingArm {
  hipEvent_t start, stop;
  TimingArm() : start(t_gather_start), stop(t_gather_stop) { t_gather_start = t_gather_stop = nullptr; }
  void rearm() const {
    t_gather_start = start;
    t_gather_stop = stop;
  }
};

int tuning_gather_rows();        // 0 = default
int tuning_gather_max_blocks();  // 0 = default
int tuning_gather_vector_bytes();  // 0 = as wide as alignment allows (16)
int tuning_gather_store_policy();
int tuning_gather_wt_tail_mib();  // 0 = kWriteThroughTailMiB

// How many workgroups of a kernel the GPU holds at once (asked once per kernel; 2048 for the plain gather of
// 16-byte vectors: 8 on each of 256 CUs).  The kernel is a template argument, not a function argument: all
// gather kernels have the same function type, and a cache per type would give every variant the figure of
// whichever was launched first.
template <auto Kernel>
static int64_t resident_blocks() {
  static const int64_t blocks = [] {
    int dev = 0, cus = 0, per_cu = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
        hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, Kernel, kGatherBlock, 0) != hipSuccess ||
        cus <= 0 || per_cu <= 0) {
      (void)hipGetLastError();
      return static_cast<int64_t>(kGatherResidentBlocks);
    }
    return static_cast<int64_t>(cus) * per_cu;
  }();
  return blocks;
}

// Grid of a gather launch.  With a device-side count the host size is only an
// upper bound: a capped grid that strides over the rows avoids dispatching
// workgroups that would find nothing to do.  Where the bound says the launch is
// a small one, the cap is what the CUs hold at once (`resident`): 23.7 against
// 24.4 us for the 235 k rows of a batch of 1024 (and 27 us when the cap is
// more than what they hold); for 725 k rows every cap from 2048 to 16384 gives
// the same 67 us.
static int64_t gather_blocks(const GatherParams& p, int groups, int R, int64_t resident) {
  int64_t max_blocks = tuning_gather_max_blocks();
  if (max_blocks <= 0)
    max_blocks = p.n_dev == nullptr                                    ? (1 << 20)
                 : p.n * p.out_row_bytes <= 5 * kWriteThroughMaxBytes ? resident
                                                                      : kGatherPersistentBlocks;
  return std::min(ceil_div(p.n, static_cast<int64_t>(groups) * R), max_blocks);
}

// Rows per lane group in flight: two (with the settings alternating inside one process on the batch's own
// launches, two are 1-3 % faster than one at a quarter of a million rows and at three quarters; four are slower).
static int gather_rows_in_flight() {
  const int R = tuning_gather_rows();
  return (R == 1 || R == 2 || R == 4 || R == 8) ? R : 2;
}

template <int V, int LPR>
static int launch_gather_r(const GatherParams& p, hipStream_t st) {
  const int R = gather_rows_in_flight();
  const int64_t resident = R == 1   ? resident_blocks<gather_kernel<V, LPR, 1>>()
                           : R == 2 ? resident_blocks<gather_kernel<V, LPR, 2>>()
                           : R == 8 ? resident_blocks<gather_kernel<V, LPR, 8>>()
                                    : resident_blocks<gather_kernel<V, LPR, 4>>();
  const dim3 grid(static_cast<unsigned>(gather_blocks(p, kGatherBlock / LPR, R, resident))), block(kGatherBlock);
  // One-shot measurement hook: the launch itself records the two events
  // (kernel begin / kernel end), see apt_time_next_gather.
  hipEvent_t ev0 = t_gather_start, ev1 = t_gather_stop;
  t_gather_start = t_gather_stop = nullptr;
#define APT_GATHER_LAUNCH(RR)                                                                        \
  if (ev0 != nullptr || ev1 != nullptr)                                                              \
    hipExtLaunchKernelGGL((gather_kernel<V, LPR, RR>), grid, block, 0, st, ev0, ev1, 0, p);          \
  else                                                                                               \
    hipLaunchKernelGGL((gather_kernel<V, LPR, RR>), grid, block, 0, st, p)
  switch (R) {
    case 1: APT_GATHER_LAUNCH(1); break;
    case 2: APT_GATHER_LAUNCH(2); break;
    case 8: APT_GATHER_LAUNCH(8); break;
    default: APT_GATHER_LAUNCH(4); break;
  }
#undef APT_GATHER_LAUNCH
  APT_LAUNCH_CHECK("gather_kernel");
  return APT_OK;
}

template <int V>
static int launch_gather_v(const GatherParams& p, hipStream_t st) {
  const int64_t vec_per_row = p.out_row_bytes / V;
  if (vec_per_row <= 8) return launch_gather_r<V, 8>(p, st);
  if (vec_per_row <= 16) return launch_gather_r<V, 16>(p, st);
  if (vec_per_row <= 32) return launch_gather_r<V, 32>(p, st);
  return launch_gather_r<V, 64>(p, st);
}

// Widest vector that every row start and the row length are multiples of.
static int vector_bytes(const GatherParams& p, int elem_size) {
  uintptr_t bits = reinterpret_cast<uintptr_t>(p.local_table) |
                   reinterpret_cast<uintptr_t>(p.out) |
                   static_cast<uintptr_t>(p.local_row_bytes) |
                   static_cast<uintptr_t>(p.col_offset_bytes) |
                   static_cast<uintptr_t>(p.out_row_bytes);
  if (p.cache_table != nullptr) bits |= reinterpret_cast<uintptr_t>(p.cache_table);
  int widest = tuning_gather_vector_bytes();
  if (widest != 2 && widest != 4 && widest != 8) widest = 16;
  for (int v = widest; v > elem_size; v >>= 1)
    if ((bits & (v - 1)) == 0) return v;
  return elem_size;
}

static int launch_gather(const GatherParams& p, int elem_size, hipStream_t st) {
  switch (vector_bytes(p, elem_size)) {
    case 16: return launch_gather_v<16>(p, st);
    case 8: return launch_gather_v<8>(p, st);
    case 4: return launch_gather_v<4>(p, st);
    default: return launch_gather_v<2>(p, st);
  }
}

// The gather with a pending lookup pass in its launch; false when this launch's geometry has no such kernel
// (rows not movable as 16-byte vectors, or a rows-in-flight setting other than two): the caller then runs the
// pass on its own.
template <int LPR>
static void launch_gather_with_lookup_r(GatherParams& p, const PendingLookup& lookup, hipStream_t st) {
  p.lookup_blocks = static_cast<int>(lookup.blocks);
  const int64_t resident = resident_blocks<gather_with_lookup_kernel<LPR>>();
  const dim3 grid(static_cast<unsigned>(gather_blocks(p, kGatherBlock / LPR, 2, resident) + p.lookup_blocks)),
      block(kGatherBlock);
  hipEvent_t ev0 = t_gather_start, ev1 = t_gather_stop;
  t_gather_start = t_gather_stop = nullptr;
  if (ev0 != nullptr || ev1 != nullptr)
    hipExtLaunchKernelGGL((gather_with_lookup_kernel<LPR>), grid, block, 0, st, ev0, ev1, 0, p, lookup.lp);
  else
    hipLaunchKernelGGL((gather_with_lookup_kernel<LPR>), grid, block, 0, st, p, lookup.lp);
}

static bool launch_gather_with_lookup(GatherParams& p, int elem_size, const PendingLookup& lookup, hipStream_t st) {
  if (lookup.blocks == 0 || vector_bytes(p, elem_size) != 16 || gather_rows_in_flight() != 2) return false;
  const int64_t vec_per_row = p.out_row_bytes / 16;
  if (vec_per_row <= 8) launch_gather_with_lookup_r<8>(p, lookup, st);
  else if (vec_per_row <= 16) launch_gather_with_lookup_r<16>(p, lookup, st);
  else if (vec_per_row <= 32) launch_gather_with_lookup_r<32>(p, lookup, st);
  else launch_gather_with_lookup_r<64>(p, lookup, st);
  return true;
}

}  // namespace apt

extern "C" int apt_minibatch_lookup(const apt_pending_lookup* pending, void* stream);

namespace apt {
static int gather_rows(const apt_feat_store* store, const int64_t* index, int64_t num_index,
                       const int64_t* num_index_dev, void* out, int64_t* miss_count, void* stream,
                       const apt_pending_lookup* pending) {
  const PendingLookup* lookup = reinterpret_cast<const PendingLookup*>(pending);
  APT_REQUIRE(lookup == nullptr || lookup->magic == kPendingMagic, APT_EINVAL,
              "apt_gather_rows_with_lookup: pending was not filled by apt_minibatch_sample_deferred");
  const TimingArm arm;  // a call that returns before its launch must not leave the events armed
  APT_REQUIRE(store != nullptr, APT_EINVAL, "apt_gather_rows: store is NULL");
  APT_REQUIRE(num_index >= 0, APT_EINVAL, "apt_gather_rows: num_index %lld < 0",
              (long long)num_index);
  APT_REQUIRE(store->elem_size == 2 || store->elem_size == 4, APT_EINVAL,
              "apt_gather_rows: elem_size %d (2 or 4 supported)", store->elem_size);
  APT_REQUIRE(store->out_dim > 0 && store->local_dim >= 0 && store->col_offset >= 0, APT_EINVAL,
              "apt_gather_rows: bad dims (local_dim %lld, col_offset %lld, out_dim %lld)",
              (long long)store->local_dim, (long long)store->col_offset,
              (long long)store->out_dim);
  APT_REQUIRE(store->num_local_rows == 0 ||
                  (store->local_table != nullptr &&
                   store->col_offset + store->out_dim <= store->local_dim),
              APT_EINVAL,
              "apt_gather_rows: column window [%lld, %lld) outside local_dim %lld",
              (long long)store->col_offset, (long long)(store->col_offset + store->out_dim),
              (long long)store->local_dim);
  APT_REQUIRE(store->num_cache_rows == 0 ||
                  (store->cache_table != nullptr && store->pos_map != nullptr),
              APT_EINVAL, "apt_gather_rows: cache rows need cache_table and pos_map");
  APT_REQUIRE(store->num_local_rows >= 0 && store->num_cache_rows >= 0, APT_EINVAL,
              "apt_gather_rows: negative row count");
  if (num_index == 0) return lookup != nullptr ? apt_minibatch_lookup(pending, stream) : APT_OK;
  APT_REQUIRE(index != nullptr && out != nullptr, APT_EINVAL,
              "apt_gather_rows: index/out is NULL");
  GatherParams p;
  p.local_table = static_cast<const char*>(store->local_table);
  p.num_local_rows = store->num_local_rows;
  p.local_row_bytes = store->local_dim * store->elem_size;
  p.col_offset_bytes = store->col_offset * store->elem_size;
  p.cache_table = store->num_cache_rows > 0 ? static_cast<const char*>(store->cache_table) : nullptr;
  p.num_cache_rows = store->num_cache_rows;
  p.pos_map = store->pos_map;
  p.num_total_nodes = store->num_total_nodes;
  p.out_row_bytes = store->out_dim * store->elem_size;
  p.index = index;
  p.n = num_index;
  p.n_dev = num_index_dev;
  p.out = static_cast<char*>(out);
  p.miss_count = miss_count;
  p.scatter = 0;
  p.num_out_rows = 0;
  p.named = nullptr;
  p.store_policy = tuning_gather_store_policy();
  p.wt_tail_bytes = (tuning_gather_wt_tail_mib() > 0 ? int64_t{tuning_gather_wt_tail_mib()} : kWriteThroughTailMiB) << 20;
  p.lookup_blocks = 0;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (lookup != nullptr) {
    arm.rearm();
    if (launch_gather_with_lookup(p, store->elem_size, *lookup, st)) {
      APT_LAUNCH_CHECK("gather_with_lookup_kernel");
      return APT_OK;
    }
    const TimingArm again;  // nothing was launched: the events stay for the plain launch below
    if (const int rc = apt_minibatch_lookup(pending, stream)) return rc;
    again.rearm();
    return launch_gather(p, store->elem_size, st);
  }
  arm.rearm();
  return launch_gather(p, store->elem_size, st);
}
}  // namespace apt

extern "C" int apt_gather_rows(const apt_feat_store* store, const int64_t* index,
                               int64_t num_index, const int64_t* num_index_dev, void* out,
                               int64_t* miss_count, void* stream) {
  return apt::gather_rows(store, index, num_index, num_index_dev, out, miss_count, stream, nullptr);
}

extern "C" int apt_gather_rows_with_lookup(const apt_feat_store* store, const int64_t* index,
                                           int64_t num_index, const int64_t* num_index_dev, void* out,
                                           int64_t* miss_count, const apt_pending_lookup* pending,
                                           void* stream) {
  APT_REQUIRE(pending != nullptr, APT_EINVAL, "apt_gather_rows_with_lookup: pending is NULL");
  return apt::gather_rows(store, index, num_index, num_index_dev, out, miss_count, stream, pending);
}

extern "C" int apt_time_next_gather(void* start_event, void* stop_event) {
  apt::t_gather_start = static_cast<hipEvent_t>(start_event);
  apt::t_gather_stop = static_cast<hipEvent_t>(stop_event);
  return APT_OK;
}

static int permute_common(const void* in, const int64_t* perm, int64_t n, int64_t dim,
                          int elem_size, void* out, int scatter, int64_t num_rows_other,
                          void* stream, const char* who, uint8_t* named = nullptr) {
  using namespace apt;
  const TimingArm arm;
  APT_REQUIRE(n >= 0 && dim > 0, APT_EINVAL, "%s: bad shape (n %lld, dim %lld)", who,
              (long long)n, (long long)dim);
  APT_REQUIRE(elem_size == 2 || elem_size == 4, APT_EINVAL, "%s: elem_size %d (2 or 4 supported)",
              who, elem_size);
  if (n == 0) return APT_OK;
  APT_REQUIRE(in != nullptr && perm != nullptr && out != nullptr, APT_EINVAL,
              "%s: in/perm/out is NULL", who);
  GatherParams p;
  p.local_table = static_cast<const char*>(in);
  p.num_local_rows = scatter ? n : num_rows_other;
  p.local_row_bytes = dim * elem_size;
  p.col_offset_bytes = 0;
  p.cache_table = nullptr;
  p.num_cache_rows = 0;
  p.pos_map = nullptr;
  p.num_total_nodes = 0;
  p.out_row_bytes = dim * elem_size;
  p.index = perm;
  p.n = n;
  p.n_dev = nullptr;
  p.out = static_cast<char*>(out);
  p.miss_count = nullptr;
  p.scatter = scatter;
  p.num_out_rows = scatter ? num_rows_other : 0;
  p.named = named;
  p.store_policy = tuning_gather_store_policy();
  p.wt_tail_bytes = (tuning_gather_wt_tail_mib() > 0 ? int64_t{tuning_gather_wt_tail_mib()} : kWriteThroughTailMiB) << 20;
  p.lookup_blocks = 0;
  arm.rearm();
  return launch_gather(p, elem_size, static_cast<hipStream_t>(stream));
}

extern "C" int apt_permute_rows(const void* in, int64_t num_in_rows, const int64_t* perm,
                                int64_t n, int64_t dim, int elem_size, void* out, void* stream) {
  APT_REQUIRE(num_in_rows >= 0, APT_EINVAL, "apt_permute_rows: num_in_rows %lld < 0",
              (long long)num_in_rows);
  return permute_common(in, perm, n, dim, elem_size, out, 0, num_in_rows, stream,
                        "apt_permute_rows");
}

namespace apt {

__global__ __launch_bounds__(kGatherBlock) void zero_words_kernel(uint32_t* w, int64_t n) {
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kGatherBlock + threadIdx.x; i < n;
       i += static_cast<int64_t>(gridDim.x) * kGatherBlock)
    w[i] = 0;
}

// rows whose flag is clear are zeroed, 16 lanes per row, 2 bytes per store (such rows are rare)
__global__ __launch_bounds__(kGatherBlock) void zero_unnamed_kernel(const uint8_t* __restrict__ named,
                                                                    int64_t num_rows, char* out, int64_t row_bytes) {
  constexpr int kLanes = 16;
  const int l = threadIdx.x % kLanes;
  for (int64_t r = (static_cast<int64_t>(blockIdx.x) * kGatherBlock + threadIdx.x) / kLanes; r < num_rows;
       r += static_cast<int64_t>(gridDim.x) * (kGatherBlock / kLanes)) {
    if (named[r] != 0) continue;
    uint16_t* row = reinterpret_cast<uint16_t*>(out + r * row_bytes);
    for (int64_t c = l; c < row_bytes / 2; c += kLanes) row[c] = 0;
  }
}

}  // namespace apt

extern "C" size_t apt_scatter_workspace_bytes(int64_t num_out_rows) {
  if (num_out_rows < 0) return 0;
  return (static_cast<size_t>(num_out_rows) + 3) / 4 * 4 + 4;
}

extern "C" int apt_scatter_rows(const void* in, const int64_t* perm, int64_t n, int64_t dim,
                                int elem_size, void* out, int64_t num_out_rows, void* workspace,
                                size_t workspace_bytes, void* stream) {
  using namespace apt;
  APT_REQUIRE(num_out_rows >= 0, APT_EINVAL, "apt_scatter_rows: num_out_rows %lld < 0",
              (long long)num_out_rows);
  if (workspace == nullptr)
    return permute_common(in, perm, n, dim, elem_size, out, 1, num_out_rows, stream, "apt_scatter_rows");
  // with scratch the library completes the output itself: a flag per output row, set by the scatter,
  // tells which rows nobody named; only those are zeroed
  APT_REQUIRE(workspace_bytes >= apt_scatter_workspace_bytes(num_out_rows) &&
                  (reinterpret_cast<uintptr_t>(workspace) & 3) == 0,
              APT_EWORKSPACE, "apt_scatter_rows: workspace too small or not 4-byte aligned "
                              "(see apt_scatter_workspace_bytes)");
  APT_REQUIRE(dim > 0 && (elem_size == 2 || elem_size == 4) && (out != nullptr || num_out_rows == 0), APT_EINVAL,
              "apt_scatter_rows: bad shape or out is NULL");
  if (num_out_rows == 0) return APT_OK;
  hipStream_t st = static_cast<hipStream_t>(stream);
  uint8_t* named = static_cast<uint8_t*>(workspace);
  const int64_t words = (num_out_rows + 3) / 4;
  auto blocks_for = [](int64_t items) {
    return dim3(static_cast<unsigned>(std::max<int64_t>(1, std::min<int64_t>(ceil_div(items, kGatherBlock), 4096))));
  };
  hipLaunchKernelGGL(zero_words_kernel, blocks_for(words), dim3(kGatherBlock), 0, st,
                     reinterpret_cast<uint32_t*>(named), words);
  APT_LAUNCH_CHECK("zero_words_kernel");
  const int rc = permute_common(in, perm, n, dim, elem_size, out, 1, num_out_rows, stream, "apt_scatter_rows", named);
  if (rc != APT_OK) return rc;
  hipLaunchKernelGGL(zero_unnamed_kernel, blocks_for(num_out_rows * 16), dim3(kGatherBlock), 0, st, named,
                     num_out_rows, static_cast<char*>(out), dim * elem_size);
  APT_LAUNCH_CHECK("zero_unnamed_kernel");
  return APT_OK;
}
