// Shared helpers of the gfx950 kernels: error reporting, Philox4x32-10,
// wave64 primitives.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <cstdarg>
#include <cstdio>

#include "../../include/apt_amd.h"

namespace apt {

constexpr int kWave = 64;  // CDNA wavefront width

// ---------------------------------------------------------------- errors
char* last_error_buf();
inline int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(last_error_buf(), 512, fmt, ap);
  va_end(ap);
  return code;
}

#define APT_REQUIRE(cond, code, ...)                \
  do {                                              \
    if (!(cond)) return ::apt::fail(code, __VA_ARGS__); \
  } while (0)

#define APT_HIP(call)                                                        \
  do {                                                                       \
    hipError_t e_ = (call);                                                  \
    if (e_ != hipSuccess)                                                    \
      return ::apt::fail(APT_EHIP, "%s failed: %s", #call, hipGetErrorString(e_)); \
  } while (0)

// Launch check: a failed launch leaves a sticky-free error we can read back.
#define APT_LAUNCH_CHECK(name)                                               \
  do {                                                                       \
    hipError_t e_ = hipGetLastError();                                       \
    if (e_ != hipSuccess)                                                    \
      return ::apt::fail(APT_EHIP, "launch of %s failed: %s", name,           \
                         hipGetErrorString(e_));                             \
  } while (0)

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// ---------------------------------------------------------------- Philox
// Philox4x32-10 (Salmon et al., SC'11).  Counter-based: the 128-bit counter is
// (node lo, node hi, hop, slot) and the 64-bit key is the caller's rng seed, so
// a draw depends only on what it is for, never on which lane computes it.
__device__ __forceinline__ void philox4x32_10(uint32_t c0, uint32_t c1,
                                              uint32_t c2, uint32_t c3,
                                              uint32_t k0, uint32_t k1,
                                              uint32_t& o0, uint32_t& o1) {
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    const uint32_t hi0 = __umulhi(0xD2511F53u, c0);
    const uint32_t lo0 = 0xD2511F53u * c0;
    const uint32_t hi1 = __umulhi(0xCD9E8D57u, c2);
    const uint32_t lo1 = 0xCD9E8D57u * c2;
    const uint32_t n0 = hi1 ^ c1 ^ k0;
    const uint32_t n2 = hi0 ^ c3 ^ k1;
    c0 = n0; c1 = lo1; c2 = n2; c3 = lo0;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  o0 = c0;
  o1 = c1;
}

__device__ __forceinline__ uint64_t draw64(uint64_t rng_seed, int64_t node,
                                           int hop, uint32_t slot) {
  uint32_t o0, o1;
  philox4x32_10(static_cast<uint32_t>(static_cast<uint64_t>(node)),
                static_cast<uint32_t>(static_cast<uint64_t>(node) >> 32),
                static_cast<uint32_t>(hop), slot,
                static_cast<uint32_t>(rng_seed),
                static_cast<uint32_t>(rng_seed >> 32), o0, o1);
  return (static_cast<uint64_t>(o1) << 32) | o0;
}

// floor(r * n / 2^64)
__device__ __forceinline__ uint64_t bounded(uint64_t r, uint64_t n) {
  return __umul64hi(r, n);
}

// ---------------------------------------------------------------- wave64
__device__ __forceinline__ int lane_id() {
  return __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
}

// Number of set bits of `mask` strictly below this lane.
__device__ __forceinline__ int rank_below(uint64_t mask) {
  return __builtin_amdgcn_mbcnt_hi(static_cast<uint32_t>(mask >> 32),
                                   __builtin_amdgcn_mbcnt_lo(static_cast<uint32_t>(mask), 0u));
}

__device__ __forceinline__ uint64_t ballot(bool p) { return __ballot(p); }

// Actual element count of a launch whose host-side size is only an upper
// bound: min(*n_dev, n_host) when a device-side count is supplied.
__device__ __forceinline__ int64_t actual_count(int64_t n_host,
                                                const int64_t* n_dev) {
  if (n_dev == nullptr) return n_host;
  const int64_t d = *n_dev;
  return d < n_host ? (d < 0 ? 0 : d) : n_host;
}

}  // namespace apt
