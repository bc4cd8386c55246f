// Shared helpers of libntship: status/error plumbing and wave64 device primitives (gfx950).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "nts_hip.h"

namespace nts {

constexpr int kWave = 64;            // CDNA wavefront width
constexpr uint32_t kNoSlot = 0xFFFFFFFFu;

// Records `msg` as the calling thread's last error and returns `code`.
int fail(int code, const char *msg);
int fail_hip(hipError_t err, const char *what);

#define NTS_HIP_TRY(expr)                                   \
  do {                                                      \
    hipError_t nts_err__ = (expr);                          \
    if (nts_err__ != hipSuccess) return ::nts::fail_hip(nts_err__, #expr); \
  } while (0)

// Launch check: hipGetLastError after a kernel launch.
#define NTS_LAUNCH_CHECK(name)                              \
  do {                                                      \
    hipError_t nts_err__ = hipGetLastError();               \
    if (nts_err__ != hipSuccess) return ::nts::fail_hip(nts_err__, name); \
  } while (0)

inline bool aligned_to(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

inline uint32_t ceil_div(uint64_t a, uint64_t b) { return static_cast<uint32_t>((a + b - 1) / b); }

#if defined(__HIPCC__)
// Value of `v` held by wavefront lane `lane` (lane must be wave-uniform); result is an SGPR.
__device__ __forceinline__ uint32_t wave_read(uint32_t v, uint32_t lane) {
  return static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(v), static_cast<int>(lane)));
}
__device__ __forceinline__ float wave_read(float v, uint32_t lane) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), static_cast<int>(lane)));
}
__device__ __forceinline__ uint32_t wave_first(uint32_t v) {
  return static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(v)));
}

// Largest r such that off[r] <= pos, searched in off[0 .. n] (off ascending, off[n] > pos): the row
// that owns edge position `pos`.
__device__ __forceinline__ uint32_t owner_of(const uint32_t *__restrict__ off, uint32_t n, uint32_t pos) {
  uint32_t lo = 0, hi = n;  // answer in [lo, hi)
  while (hi - lo > 1) {
    const uint32_t mid = lo + (hi - lo) / 2;
    if (off[mid] <= pos) lo = mid; else hi = mid;
  }
  return lo;
}

// Butterfly reductions over the `width` lanes of an aligned lane group (width = power of two <= 64).
template <int WIDTH>
__device__ __forceinline__ float group_max(float v) {
#pragma unroll
  for (int m = WIDTH / 2; m >= 1; m >>= 1) v = fmaxf(v, __shfl_xor(v, m, kWave));
  return v;
}
template <int WIDTH>
__device__ __forceinline__ float group_sum(float v) {
#pragma unroll
  for (int m = WIDTH / 2; m >= 1; m >>= 1) v += __shfl_xor(v, m, kWave);
  return v;
}
#endif

}  // namespace nts
