// Neighbour sampling of one hop on the device (the construction steps of Sampler::sample_one,
// core/ntsSampler.hpp:843-1106, over a whole-graph CSC resident in HBM):
//   init_co      prefix of min(in-degree, fanout) per destination      core/FullyRepGraph.hpp:199-209
//   the pick     all in-neighbours when fanout < 0 or fanout >= degree, otherwise `fanout` DISTINCT
//                positions of the destination's CSC segment, uniformly at random
// The reference draws positions with a per-thread mt19937 and iterates an unordered_set, so which
// neighbours it picks (and in which order) is implementation-defined; here positions come from a
// counter-based hash of (seed, destination slot) through Floyd's sampling and are emitted in
// ascending position order, which keeps source ids ascending inside a destination for graphs with
// sorted adjacency.  Results depend only on the arguments: the same seed gives the same sample.
#include <rocprim/device/device_scan.hpp>

#include "common.hpp"

namespace nts {
namespace {

constexpr int kMaxFanout = 64;  // distinct picks are kept in a per-thread array of this size

__device__ __forceinline__ uint64_t mix64(uint64_t z) {
  z += 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

__global__ __launch_bounds__(256) void hop_counts_kernel(uint32_t *__restrict__ counts,
                                                         const uint32_t *__restrict__ graph_co,
                                                         const uint32_t *__restrict__ dst, uint32_t n,
                                                         int32_t fanout) {
  const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i > n) return;
  if (i == n) {
    counts[n] = 0;  // the exclusive scan turns this last slot into the edge total
    return;
  }
  const uint32_t d = dst[i];
  const uint32_t deg = graph_co[d + 1] - graph_co[d];
  counts[i] = (fanout < 0 || deg < static_cast<uint32_t>(fanout)) ? deg : static_cast<uint32_t>(fanout);
}

// One thread per destination.
__global__ __launch_bounds__(256) void hop_pick_kernel(uint32_t *__restrict__ ri_out,
                                                       const uint32_t *__restrict__ co,
                                                       const uint32_t *__restrict__ graph_co,
                                                       const uint32_t *__restrict__ graph_ri,
                                                       const uint32_t *__restrict__ dst, uint32_t n, int32_t fanout,
                                                       uint64_t seed) {
  const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const uint32_t d = dst[i];
  const uint32_t base = graph_co[d];
  const uint32_t deg = graph_co[d + 1] - base;
  const uint32_t out = co[i];
  const uint32_t take = co[i + 1] - out;
  if (take == deg) {  // full neighbourhood, in CSC order
    for (uint32_t k = 0; k < deg; ++k) ri_out[out + k] = graph_ri[base + k];
    return;
  }
  uint64_t state = mix64(seed ^ (static_cast<uint64_t>(i) << 32) ^ d);
  if (take > kMaxFanout) {
    // Very large fanouts: a window of consecutive positions from a random start (distinct by
    // construction), emitted in ascending position order.
    const uint32_t start = static_cast<uint32_t>(state % deg);
    const uint32_t wrap = start + take > deg ? start + take - deg : 0;  // positions [0, wrap) belong to the window
    uint32_t k = 0;
    for (uint32_t p = 0; p < wrap; ++p) ri_out[out + k++] = graph_ri[base + p];
    for (uint32_t p = start; p < deg && k < take; ++p) ri_out[out + k++] = graph_ri[base + p];
    return;
  }
  // Floyd's algorithm: `take` distinct values from [0, deg), kept sorted by insertion.
  uint32_t pick[kMaxFanout];
  uint32_t m = 0;
  for (uint32_t j = deg - take; j < deg; ++j) {
    state = mix64(state);
    uint32_t t = static_cast<uint32_t>(state % (static_cast<uint64_t>(j) + 1));
    bool present = false;
    for (uint32_t q = 0; q < m; ++q) present = present || pick[q] == t;
    if (present) t = j;  // j cannot be present yet: every earlier value is < j
    uint32_t pos = m;
    while (pos > 0 && pick[pos - 1] > t) {
      pick[pos] = pick[pos - 1];
      --pos;
    }
    pick[pos] = t;
    ++m;
  }
  for (uint32_t k = 0; k < take; ++k) ri_out[out + k] = graph_ri[base + pick[k]];
}

hipError_t scan_bytes(uint32_t n, size_t *bytes) {
  size_t tmp = 0;
  uint32_t *nul = nullptr;
  hipError_t err = rocprim::exclusive_scan(nullptr, tmp, nul, nul, 0u, n ? n : 1u, rocprim::plus<uint32_t>(),
                                           static_cast<hipStream_t>(nullptr), false);
  *bytes = tmp;
  return err;
}

inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

}  // namespace
}  // namespace nts

using namespace nts;

extern "C" {

size_t nts_sample_hop_work_bytes(uint32_t n) {
  size_t tmp = 0;
  if (scan_bytes(n + 1, &tmp) != hipSuccess) return 0;
  return align_up((static_cast<size_t>(n) + 1) * sizeof(uint32_t), 256) + align_up(tmp, 256) + 256;
}

int nts_sample_hop_offsets(uint32_t *co, const uint32_t *graph_co, const uint32_t *dst, uint32_t n, int32_t fanout,
                           void *work, nts_stream_t stream) {
  if (!co) return fail(NTS_ERR_INVALID, "nts_sample_hop_offsets: null co");
  if (n == 0) return nts_memset_zero(co, sizeof(uint32_t), stream);
  if (!graph_co || !dst || !work) return fail(NTS_ERR_INVALID, "nts_sample_hop_offsets: null pointer");
  if (!aligned_to(work, 256)) return fail(NTS_ERR_INVALID, "nts_sample_hop_offsets: work must be 256-byte aligned");
  unsigned char *w = static_cast<unsigned char *>(work);
  uint32_t *counts = reinterpret_cast<uint32_t *>(w);
  const size_t arr = align_up((static_cast<size_t>(n) + 1) * sizeof(uint32_t), 256);
  size_t tmp = 0;
  NTS_HIP_TRY(scan_bytes(n + 1, &tmp));
  hipLaunchKernelGGL(hop_counts_kernel, dim3(ceil_div(static_cast<uint64_t>(n) + 1, 256)), dim3(256), 0, stream, counts,
                     graph_co, dst, n, fanout);
  NTS_LAUNCH_CHECK("hop_counts_kernel");
  NTS_HIP_TRY(rocprim::exclusive_scan(w + arr, tmp, counts, co, 0u, n + 1, rocprim::plus<uint32_t>(), stream, false));
  return NTS_OK;
}

int nts_sample_hop_neighbors(uint32_t *ri_global, const uint32_t *co, const uint32_t *graph_co,
                             const uint32_t *graph_ri, const uint32_t *dst, uint32_t n, int32_t fanout, uint64_t seed,
                             nts_stream_t stream) {
  if (n == 0) return NTS_OK;
  if (!ri_global || !co || !graph_co || !graph_ri || !dst)
    return fail(NTS_ERR_INVALID, "nts_sample_hop_neighbors: null pointer");
  hipLaunchKernelGGL(hop_pick_kernel, dim3(ceil_div(n, 256)), dim3(256), 0, stream, ri_global, co, graph_co, graph_ri,
                     dst, n, fanout, seed);
  NTS_LAUNCH_CHECK("hop_pick_kernel");
  return NTS_OK;
}

}  // extern "C"
