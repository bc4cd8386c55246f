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

// Named ranges around the entry points for a profiler's marker trace (rocTX).  Off unless the
// environment has NTS_TRACE_RANGES=1 when the first entry point runs; then the rocTX library is
// loaded at run time (the library itself does not link against it) and every traced entry point
// pushes its name on entry and pops it on return.
struct TraceApi {
  int (*push)(const char *);
  int (*pop)();
};
const TraceApi *trace_api();  // NULL when ranges are off or the rocTX library is not there
void count_trace_range();
long trace_ranges_emitted();
struct TraceRange {
  explicit TraceRange(const char *name) : api(trace_api()) {
    if (api) {
      api->push(name);
      count_trace_range();
    }
  }
  ~TraceRange() {
    if (api) api->pop();
  }
  TraceRange(const TraceRange &) = delete;
  TraceRange &operator=(const TraceRange &) = delete;
  const TraceApi *api;
};
#define NTS_TRACE_RANGE(name) ::nts::TraceRange nts_trace_range__(name)

// Stream-ordered scratch of the entry points that need device memory beyond their arguments
// (lists of hub rows, partial sums of calls without a plan).  It comes from a memory pool of the
// library's own, one per device, that keeps freed blocks instead of handing them back to the
// driver at every synchronisation (the default pool's behaviour, which makes each call pay for a
// fresh allocation): the pool holds on to the largest scratch any call has needed.
hipError_t scratch_alloc(void **ptr, size_t bytes, hipStream_t stream);
hipError_t scratch_free(void *ptr, hipStream_t stream);
hipError_t scratch_trim();  // gives the current device's unused scratch back to the driver
long scratch_alloc_count();  // scratch blocks handed out so far by this process

// A scratch block that is returned to the pool when its scope ends, whichever way the function is
// left (the error paths included); release() frees it early and reports the result.
struct ScratchBlock {
  void *ptr = nullptr;
  hipStream_t stream = nullptr;
  ScratchBlock() = default;
  ScratchBlock(const ScratchBlock &) = delete;
  ScratchBlock &operator=(const ScratchBlock &) = delete;
  hipError_t alloc(size_t bytes, hipStream_t s) {
    stream = s;
    return scratch_alloc(&ptr, bytes, s);
  }
  hipError_t release() {
    const hipError_t e = ptr ? scratch_free(ptr, stream) : hipSuccess;
    ptr = nullptr;
    return e;
  }
  ~ScratchBlock() {
    if (ptr) (void)scratch_free(ptr, stream);
  }
};

inline bool aligned_to(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

inline uint32_t ceil_div(uint64_t a, uint64_t b) { return static_cast<uint32_t>((a + b - 1) / b); }

// A count that kernels need: known on the host (`n` null, value = `cap`), or produced earlier in the
// same stream and read on the device -- the word `*n`, or `off[*n]` when `off` is set (an offsets
// array indexed by a live row count, i.e. an edge total).  Device values are clamped to the
// capacities the host sized grids and buffers for, so a kernel never indexes past them.
struct DevCount {
  uint32_t cap;
  const uint32_t *n;
  const uint32_t *off;
  uint32_t n_cap;
#if defined(__HIPCC__)
  __device__ __forceinline__ uint32_t get() const {
    if (!n) return cap;
    uint32_t v = *n;
    if (off) v = off[v < n_cap ? v : n_cap];
    return v < cap ? v : cap;
  }
#endif
};
inline DevCount host_count(uint32_t v) { return DevCount{v, nullptr, nullptr, 0}; }
inline DevCount device_count(const uint32_t *n, uint32_t cap) { return DevCount{cap, n, nullptr, 0}; }
inline DevCount device_edge_count(const uint32_t *off, const uint32_t *n, uint32_t n_cap, uint32_t cap) {
  return DevCount{cap, n, off, n_cap};
}

// A seed that is either a host value or a device word plus an offset (the batch builder keeps the
// batch's seed on the device, so that the same launches serve every batch).
struct DevSeed {
  const uint64_t *base;
  uint64_t add;
#if defined(__HIPCC__)
  __device__ __forceinline__ uint64_t get() const { return (base ? *base : 0ull) + add; }
#endif
};
inline DevSeed host_seed(uint64_t v) { return DevSeed{nullptr, v}; }
inline DevSeed device_seed(const uint64_t *base, uint64_t add) { return DevSeed{base, add}; }

// Distinct uniform positions of the neighbour pick: up to 64 inside lane groups with Floyd's algorithm,
// up to this many by a keyed permutation of the positions staged in LDS, above it by a radix select
// of keyed hashes (any fanout).
constexpr int32_t kWidestFanout = 1024;

// Steps of a sampled layer's construction with sizes that may live on the device (sampler.hip,
// layout.hip); the C entry points pass host counts, the batch builder device counts.
int hop_offsets(uint32_t *co, const uint32_t *graph_co, const uint32_t *dst, DevCount n, int32_t fanout, void *scan_tmp,
                size_t scan_tmp_bytes, hipStream_t stream);
int hop_neighbors(uint32_t *ri_global, const uint32_t *co, const uint32_t *graph_co, const uint32_t *graph_ri,
                  const uint32_t *dst, DevCount n, uint32_t edge_cap, int32_t fanout, DevSeed seed, uint32_t *mark_bits,
                  uint32_t *owner, hipStream_t stream);  // owner (nullable): [edge_cap] destination slot of every edge
size_t hop_scan_bytes(uint32_t n);
// fill_to > E: local[E .. fill_to) = fill_value (padding for a sort over a fixed capacity);
// n_source_copy / e_out (nullable) receive the source count again / the edge count.  marked: the
// bitmap at the start of `work` already holds the ids' bits (hop_neighbors wrote them).
int relabel_sources(uint32_t *source, uint32_t *n_source, uint32_t *n_source_copy, uint32_t *local,
                    const uint32_t *global_ids, DevCount E, uint32_t fill_to, uint32_t fill_value, uint32_t *e_out,
                    uint32_t V, void *work, bool marked, hipStream_t stream);
// Sorts sort_n keys of key_bits bits (sort_n = E.cap, padded entries sort last).  owner (nullable): the
// destination slot of every CSC edge, which the neighbour pick can record; without it the slots are
// searched for in co.  The sorted keys (the source of every CSR edge) stay at the start of `work`.
int csr_from_csc(uint32_t *ro, uint32_t *ci, uint32_t *perm, const uint32_t *co, const uint32_t *ri, DevCount Vd,
                 DevCount Vs, DevCount E, uint32_t sort_n, unsigned key_bits, void *work, const uint32_t *owner,
                 hipStream_t stream);
size_t csr_from_csc_bytes(uint32_t sort_n);
int gcn_edge_weights(float *ewf, float *ewb, const uint32_t *co, const uint32_t *ri, const uint32_t *ro,
                     const uint32_t *ci, DevCount Vd, DevCount Vs, uint32_t *clear, uint32_t clear_words,
                     const uint32_t *csc_owner, const uint32_t *csr_owner, hipStream_t stream);  // owners nullable

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

// Owners of the 64 consecutive edge positions base .. base + 63, one per lane, for a wavefront that
// walks a contiguous span of edges: a binary search per lane is ~log2(n) dependent loads per step,
// while consecutive edges belong to a handful of consecutive rows.  `d0` (wave-uniform) enters as
// any row with off[d0] <= base, e.g. the owner found for an earlier step, and leaves as the owner
// of `base`.  The wavefront reads the 64 offsets after d0 in one load; a lane's owner is d0 plus the
// number of those offsets that are <= its position (found with six shuffles).  Only a step that
// spans more than 64 rows (runs of empty rows) falls back to the search.  Lanes at or beyond
// off[n] return n.  All 64 lanes must call it.
__device__ __forceinline__ uint32_t owners_of_step(const uint32_t *__restrict__ off, uint32_t n, uint32_t base,
                                                   uint32_t &d0) {
  const uint32_t lane = threadIdx.x & (kWave - 1);
  const uint32_t total = off[n];
  uint32_t win;
  while (true) {
    const uint32_t idx = d0 + 1 + lane;
    win = off[idx < n ? idx : n];
    const uint32_t behind = __popcll(__ballot(win <= base));  // offsets of the window not beyond `base`
    if (behind == 0 || base >= total) break;
    d0 = behind < static_cast<uint32_t>(kWave) ? d0 + behind : owner_of(off, n, base);
  }
  const uint32_t e = base + lane;
  uint32_t pos = 0;
#pragma unroll
  for (uint32_t step = kWave / 2; step >= 1; step >>= 1) {
    const uint32_t v = __shfl(win, pos + step - 1, kWave);
    if (v <= e) pos += step;
  }
  const uint32_t last = __shfl(win, kWave - 1, kWave);
  if (e >= total) return n;
  return last <= e ? owner_of(off, n, e) : d0 + pos;
}

// Exclusive prefix of `mine` over the THREADS threads of a block, in thread order; *total = the sum.
template <int THREADS>
__device__ __forceinline__ uint32_t block_prefix(uint32_t mine, uint32_t *wave_sums, uint32_t *total) {
  const uint32_t lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  uint32_t incl = mine;
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    const uint32_t up = __shfl_up(incl, d, kWave);
    if (lane >= static_cast<uint32_t>(d)) incl += up;
  }
  __syncthreads();  // wave_sums may still be read from an earlier call
  if (lane == kWave - 1) wave_sums[wave] = incl;
  __syncthreads();
  uint32_t before = 0, all = 0;
#pragma unroll
  for (uint32_t w = 0; w < THREADS / kWave; ++w) {
    const uint32_t v = wave_sums[w];
    if (w < wave) before += v;
    all += v;
  }
  *total = all;
  return before + incl - mine;
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
