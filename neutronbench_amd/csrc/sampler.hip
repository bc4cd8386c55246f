// Neighbour sampling of one hop on the device (the construction steps of Sampler::sample_one,
// core/ntsSampler.hpp:843-1106, over a whole-graph CSC resident in HBM):
//   init_co      prefix of min(in-degree, fanout) per destination      core/FullyRepGraph.hpp:199-209
//   the pick     all in-neighbours when fanout < 0 or fanout >= degree, otherwise `fanout` DISTINCT
//                positions of the destination's CSC segment, uniformly at random
// The reference draws positions with a per-thread mt19937 and iterates an unordered_set, so which
// neighbours it picks (and in which order) is implementation-defined; here positions come from a
// counter-based hash of (seed, destination slot) through Floyd's sampling (fanouts up to 64) or a
// keyed permutation of the positions (up to 1,024) or the positions with the smallest keyed hashes (any
// larger fanout) and are emitted in ascending position order, which keeps source ids ascending inside a
// destination for graphs with sorted adjacency.  Results depend only on the arguments: the same seed gives the same sample.
#include <rocprim/device/device_scan.hpp>
#include <rocprim/iterator/counting_iterator.hpp>
#include <rocprim/iterator/transform_iterator.hpp>

#include "common.hpp"

namespace nts {
namespace {

constexpr int kMaxFanout = 64;  // distinct picks are resolved inside one wavefront

__device__ __forceinline__ uint64_t mix64(uint64_t z) {
  z += 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

// min(in-degree, fanout) of destination slot i; 0 from the live count on, so that an exclusive scan
// over cap + 1 slots leaves the edge total in every slot from the live count up.
struct HopCount {
  const uint32_t *graph_co;
  const uint32_t *dst;
  DevCount n;
  int32_t fanout;
  __device__ uint32_t operator()(uint32_t i) const {
    if (i >= n.get()) return 0;
    const uint32_t d = dst[i];
    const uint32_t deg = graph_co[d + 1] - graph_co[d];
    return (fanout < 0 || deg < static_cast<uint32_t>(fanout)) ? deg : static_cast<uint32_t>(fanout);
  }
};
using HopCountIterator = rocprim::transform_iterator<rocprim::counting_iterator<uint32_t>, HopCount, uint32_t>;
// Every input of this scan costs three dependent loads (live count, destination, its offsets), and a
// thread works through its items one after the other: with the library's default of 8 to 16 items
// per thread the scan of 4,097 slots took 26 us.  Two items per thread make it a matter of more
// blocks instead.
using HopScanConfig = rocprim::scan_config<256, 2, rocprim::block_load_method::block_load_transpose,
                                           rocprim::block_store_method::block_store_transpose,
                                           rocprim::block_scan_algorithm::using_warp_scan>;

// True if `pred` holds on any lane of the caller's aligned group of G lanes (all of them active).
template <int G>
__device__ __forceinline__ bool group_any(bool pred) {
  const uint64_t votes = __ballot(pred);
  if (G == kWave) return votes != 0;
  const uint32_t first = (threadIdx.x & (kWave - 1)) & ~static_cast<uint32_t>(G - 1);
  return ((votes >> first) & ((1ull << G) - 1ull)) != 0;
}

// Stores one sampled source id; with `mark` also sets its bit in the bitmap of sampled sources
// (integer OR: the result does not depend on the order), which saves the relabelling a pass; with
// `owner` also records the destination slot the edge belongs to, which saves the construction of the
// transposed structure a search per edge.
__device__ __forceinline__ void emit(uint32_t *__restrict__ ri_out, uint32_t *__restrict__ mark,
                                     uint32_t *__restrict__ owner, uint32_t pos, uint32_t g, uint32_t slot) {
  ri_out[pos] = g;
  if (owner) owner[pos] = slot;
  if (mark) atomicOr(&mark[g >> 5], 1u << (g & 31));
}

// A group of G lanes per destination (G = power of two >= the fanout, at most one wavefront).
//
// Floyd's algorithm draws `take` distinct positions of [0, deg): for j = deg-take .. deg-1 it draws
// t uniform in [0, j] and inserts t, or j when t is already in the set.  Lane l owns step
// j_l = deg-take+l: every lane advances the destination's hash chain to its own step and draws its
// t at the same time (the 64-bit modulo is the expensive part); the "already in the set" decisions,
// which depend on the earlier steps, are then resolved in `take` rounds of cross-lane shuffles
// without touching memory; finally every lane ranks its value among the group's (values are
// distinct) and copies one neighbour, so the sample comes out in ascending position order and the
// neighbour reads of a destination are one parallel access instead of a chain.
template <int G>
__global__ __launch_bounds__(256) void hop_pick_kernel(uint32_t *__restrict__ ri_out,
                                                       const uint32_t *__restrict__ co,
                                                       const uint32_t *__restrict__ graph_co,
                                                       const uint32_t *__restrict__ graph_ri,
                                                       const uint32_t *__restrict__ dst, DevCount n,
                                                       uint32_t edge_cap, int32_t fanout, DevSeed seed,
                                                       uint32_t *__restrict__ mark, uint32_t *__restrict__ owner) {
  const uint32_t i = (blockIdx.x * blockDim.x + threadIdx.x) / G;
  if (i >= n.get()) return;  // whole groups leave together
  const uint32_t gl = threadIdx.x & (G - 1);
  const uint32_t d = dst[i];
  const uint32_t base = graph_co[d];
  const uint32_t deg = graph_co[d + 1] - base;
  const uint32_t out = co[i];
  const uint32_t take = co[i + 1] - out;
  if (co[i + 1] > edge_cap) return;  // never past the edge array (a full-neighbourhood batch that repeats vertices)
  if (take == deg) {  // full neighbourhood, in CSC order
    for (uint32_t k = gl; k < deg; k += G) emit(ri_out, mark, owner, out + k, graph_ri[base + k], i);
    return;
  }
  const uint64_t state0 = mix64(seed.get() ^ (static_cast<uint64_t>(i) << 32) ^ d);
  if (take > kMaxFanout || take > G) return;  // fanouts above one wavefront: hop_pick_wide_kernel
  // Lane gl < take: step j = deg - take + gl, hash chain advanced gl + 1 times.
  uint64_t state = state0;
  for (uint32_t q = 0; q <= gl && q < take; ++q) state = mix64(state);
  const uint32_t j = deg - take + gl;
  const uint32_t t = gl < take ? static_cast<uint32_t>(state % (static_cast<uint64_t>(j) + 1)) : 0xFFFFFFFFu;
  uint32_t v = 0xFFFFFFFFu;  // this lane's inserted value, set in round gl
  for (uint32_t l = 0; l < take; ++l) {
    const uint32_t tl = __shfl(t, l, G);
    // lanes of earlier rounds that already hold tl (at most one); lanes >= l still hold the marker
    const bool present = group_any<G>(v == tl);
    if (gl == l) v = present ? j : tl;  // j cannot be present yet: every earlier value is < j
  }
  if (gl < take) {
    uint32_t rank = 0;
    for (uint32_t q = 0; q < take; ++q) rank += __shfl(v, q, G) < v ? 1u : 0u;
    emit(ri_out, mark, owner, out + rank, graph_ri[base + v], i);
  }
}

// Fanouts of 65 .. 1,024: one wavefront per destination.  The positions are the first `take` values of
// a keyed pseudo-random permutation of [0, deg): three rounds of (multiply by an odd constant, add a
// key, fold the high bits down) are a bijection on [0, 2^b) for the smallest 2^b >= deg, and values
// that land at or beyond deg are sent through the rounds again until they fall inside (cycle walking:
// still a bijection, on [0, deg)), so the picks are distinct by construction and spread over the whole
// neighbourhood.  They are staged in LDS, ranked, and emitted in ascending position order like the
// narrower fanouts.  Destinations with at most `fanout` neighbours were copied whole by hop_pick_kernel.
__global__ __launch_bounds__(256) void hop_pick_wide_kernel(uint32_t *__restrict__ ri_out,
                                                            const uint32_t *__restrict__ co,
                                                            const uint32_t *__restrict__ graph_co,
                                                            const uint32_t *__restrict__ graph_ri,
                                                            const uint32_t *__restrict__ dst, DevCount n,
                                                            uint32_t edge_cap, DevSeed seed,
                                                            uint32_t *__restrict__ mark, uint32_t *__restrict__ owner) {
  __shared__ uint32_t picked[4][kWidestFanout];
  const uint32_t lane = threadIdx.x & (kWave - 1);
  uint32_t *mine = picked[threadIdx.x / kWave];
  const uint32_t i = (blockIdx.x * blockDim.x + threadIdx.x) / kWave;
  if (i >= n.get()) return;  // whole wavefronts leave together
  const uint32_t d = dst[i];
  const uint32_t base = graph_co[d];
  const uint32_t deg = graph_co[d + 1] - base;
  const uint32_t out = co[i];
  const uint32_t take = co[i + 1] - out;
  if (co[i + 1] > edge_cap || take == deg || take <= static_cast<uint32_t>(kMaxFanout)) return;
  const uint64_t key = mix64(seed.get() ^ (static_cast<uint64_t>(i) << 32) ^ d);
  uint32_t bits = 1;
  while ((1ull << bits) < deg) ++bits;
  const uint32_t mask = bits >= 32 ? 0xFFFFFFFFu : (1u << bits) - 1u;
  const uint32_t k0 = static_cast<uint32_t>(key), k1 = static_cast<uint32_t>(key >> 32),
                 k2 = static_cast<uint32_t>(mix64(key));
  const uint32_t fold = bits > 1 ? bits / 2 : 1;
  auto rounds = [&](uint32_t x) {
    x = (x * 0x9E3779B1u + k0) & mask;
    x ^= x >> fold;
    x = (x * 0x85EBCA6Bu + k1) & mask;
    x ^= x >> fold;
    x = (x * 0xC2B2AE35u + k2) & mask;
    x ^= x >> fold;
    return x;
  };
  for (uint32_t k = lane; k < take; k += kWave) {
    uint32_t x = rounds(k);
    while (x >= deg) x = rounds(x);
    mine[k] = x;
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  for (uint32_t k = lane; k < take; k += kWave) {
    const uint32_t v = mine[k];
    uint32_t rank = 0;
    for (uint32_t q = 0; q < take; ++q) rank += mine[q] < v ? 1u : 0u;
    emit(ri_out, mark, owner, out + rank, graph_ri[base + v], i);
  }
}

// Fanouts above 1,024: one block per destination that has more neighbours than the fanout.  Every
// position p of the neighbourhood gets a 32-bit key hashed from (seed, destination slot, p); the
// sample is the `take` positions with the smallest keys -- a uniform subset without replacement,
// distinct by construction -- and ties at the largest chosen key are broken by position.  The take-th
// smallest key is found by a radix select (four passes over the positions, one byte of the key each,
// a 256-bin histogram in LDS; keys are recomputed, not stored), then one more pass copies the chosen
// neighbours in ascending position order, their output slots coming from a block-wide count of the
// chosen positions before them.  Any fanout and any degree; the work is five hashes per neighbour of
// the destinations that need it.  Blocks stride over the destinations.
__global__ __launch_bounds__(256) void hop_pick_select_kernel(uint32_t *__restrict__ ri_out,
                                                              const uint32_t *__restrict__ co,
                                                              const uint32_t *__restrict__ graph_co,
                                                              const uint32_t *__restrict__ graph_ri,
                                                              const uint32_t *__restrict__ dst, DevCount n,
                                                              uint32_t edge_cap, DevSeed seed,
                                                              uint32_t *__restrict__ mark,
                                                              uint32_t *__restrict__ owner) {
  __shared__ uint32_t hist[256];
  __shared__ uint32_t sh_prefix, sh_k, wave_less[4], wave_eq[4];
  const uint32_t lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const uint32_t live = n.get();
  for (uint32_t i = blockIdx.x; i < live; i += gridDim.x) {
    const uint32_t d = dst[i];
    const uint32_t base = graph_co[d];
    const uint32_t deg = graph_co[d + 1] - base;
    const uint32_t out = co[i];
    const uint32_t take = co[i + 1] - out;
    if (co[i + 1] > edge_cap || take == deg || take <= static_cast<uint32_t>(kWidestFanout)) continue;  // block-uniform
    const uint64_t key = mix64(seed.get() ^ (static_cast<uint64_t>(i) << 32) ^ d);
    auto key_of = [&](uint32_t p) { return static_cast<uint32_t>(mix64(key ^ (static_cast<uint64_t>(p) * 0x9E3779B97F4A7C15ull)) >> 32); };
    // radix select: the take-th smallest key (1-based rank k among the keys that share the prefix)
    if (threadIdx.x == 0) {
      sh_prefix = 0;
      sh_k = take;
    }
    for (int pass = 0; pass < 4; ++pass) {
      const uint32_t shift = 24 - 8 * pass;
      hist[threadIdx.x] = 0;
      __syncthreads();
      const uint32_t prefix = sh_prefix;
      for (uint32_t p = threadIdx.x; p < deg; p += 256) {
        const uint32_t h = key_of(p);
        if (pass == 0 || (h >> (shift + 8)) == prefix) atomicAdd(&hist[(h >> shift) & 255u], 1u);
      }
      __syncthreads();
      if (threadIdx.x == 0) {
        uint32_t k = sh_k, digit = 0;
        while (digit < 255u && hist[digit] < k) k -= hist[digit++];
        sh_k = k;
        sh_prefix = (prefix << 8) | digit;
      }
      __syncthreads();
    }
    const uint32_t threshold = sh_prefix, ties_wanted = sh_k;  // keys below are all chosen; of the equal ones the first few
    uint32_t less_before = 0, eq_before = 0;                   // chosen / tied positions before this chunk (block-uniform)
    for (uint32_t p0 = 0; p0 < deg; p0 += 256) {
      const uint32_t p = p0 + threadIdx.x;
      const uint32_t h = p < deg ? key_of(p) : 0xFFFFFFFFu;
      const bool less = p < deg && h < threshold, eq = p < deg && h == threshold;
      const uint64_t less_mask = __ballot(less), eq_mask = __ballot(eq);
      const uint64_t below = (1ull << lane) - 1ull;
      if (lane == 0) {
        wave_less[wave] = __popcll(less_mask);
        wave_eq[wave] = __popcll(eq_mask);
      }
      __syncthreads();
      uint32_t my_less = less_before + __popcll(less_mask & below), my_eq = eq_before + __popcll(eq_mask & below);
      uint32_t chunk_less = 0, chunk_eq = 0;
      for (uint32_t w = 0; w < 4; ++w) {
        if (w < wave) {
          my_less += wave_less[w];
          my_eq += wave_eq[w];
        }
        chunk_less += wave_less[w];
        chunk_eq += wave_eq[w];
      }
      // ties are taken in position order, so the number taken before this position is min(my_eq, wanted)
      const uint32_t ties_before = my_eq < ties_wanted ? my_eq : ties_wanted;
      if (less || (eq && my_eq < ties_wanted))
        emit(ri_out, mark, owner, out + my_less + ties_before, graph_ri[base + p], i);
      less_before += chunk_less;
      eq_before += chunk_eq;
      __syncthreads();
    }
  }
}

hipError_t scan_bytes(uint32_t n, size_t *bytes) {
  size_t tmp = 0;
  uint32_t *nul = nullptr;
  HopCountIterator in(rocprim::counting_iterator<uint32_t>(0u), HopCount{nullptr, nullptr, host_count(0), 0});
  hipError_t err = rocprim::exclusive_scan<HopScanConfig>(nullptr, tmp, in, nul, 0u, n ? n : 1u,
                                                          rocprim::plus<uint32_t>(), static_cast<hipStream_t>(nullptr),
                                                          false);
  *bytes = tmp;
  return err;
}

inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

}  // namespace

size_t hop_scan_bytes(uint32_t n) {
  size_t tmp = 0;
  return scan_bytes(n + 1, &tmp) == hipSuccess ? tmp : 0;
}

int hop_offsets(uint32_t *co, const uint32_t *graph_co, const uint32_t *dst, DevCount n, int32_t fanout, void *scan_tmp,
                size_t scan_tmp_bytes, hipStream_t stream) {
  // One scan whose input is computed on the fly; slot n.cap (count 0) receives the edge total.
  HopCountIterator in(rocprim::counting_iterator<uint32_t>(0u), HopCount{graph_co, dst, n, fanout});
  NTS_HIP_TRY(rocprim::exclusive_scan<HopScanConfig>(scan_tmp, scan_tmp_bytes, in, co, 0u, n.cap + 1,
                                                     rocprim::plus<uint32_t>(), stream, false));
  return NTS_OK;
}

int hop_neighbors(uint32_t *ri_global, const uint32_t *co, const uint32_t *graph_co, const uint32_t *graph_ri,
                  const uint32_t *dst, DevCount n, uint32_t edge_cap, int32_t fanout, DevSeed seed, uint32_t *mark_bits,
                  uint32_t *owner, hipStream_t stream) {
  // Lanes per destination: the fanout rounded up to a power of two (full neighbourhoods and
  // fanouts above one wavefront are strided copies, for which a quarter wavefront serves well).
  int g = 8;
  if (fanout > 0 && fanout <= kMaxFanout)
    while (g < fanout) g <<= 1;
  else
    g = 16;
  const dim3 grid(ceil_div(static_cast<uint64_t>(n.cap) * g, 256));
#define NTS_LAUNCH_PICK(G)                                                                                      \
  hipLaunchKernelGGL(hop_pick_kernel<G>, grid, dim3(256), 0, stream, ri_global, co, graph_co, graph_ri, dst, n, \
                     edge_cap, fanout, seed, mark_bits, owner)
  switch (g) {
    case 8: NTS_LAUNCH_PICK(8); break;
    case 16: NTS_LAUNCH_PICK(16); break;
    case 32: NTS_LAUNCH_PICK(32); break;
    default: NTS_LAUNCH_PICK(64); break;
  }
#undef NTS_LAUNCH_PICK
  NTS_LAUNCH_CHECK("hop_pick_kernel");
  if (fanout > kWidestFanout) {
    const uint32_t blocks = n.cap < 4096u ? n.cap : 4096u;
    hipLaunchKernelGGL(hop_pick_select_kernel, dim3(blocks ? blocks : 1u), dim3(256), 0, stream, ri_global, co, graph_co,
                       graph_ri, dst, n, edge_cap, seed, mark_bits, owner);
    NTS_LAUNCH_CHECK("hop_pick_select_kernel");
  } else if (fanout > kMaxFanout) {
    hipLaunchKernelGGL(hop_pick_wide_kernel, dim3(ceil_div(static_cast<uint64_t>(n.cap) * kWave, 256)), dim3(256), 0,
                       stream, ri_global, co, graph_co, graph_ri, dst, n, edge_cap, seed, mark_bits, owner);
    NTS_LAUNCH_CHECK("hop_pick_wide_kernel");
  }
  return NTS_OK;
}

}  // namespace nts

using namespace nts;

extern "C" {

size_t nts_sample_hop_work_bytes(uint32_t n) {
  size_t tmp = 0;
  if (scan_bytes(n + 1, &tmp) != hipSuccess) return 0;
  return align_up(tmp, 256) + 256;
}

int nts_sample_hop_offsets(uint32_t *co, const uint32_t *graph_co, const uint32_t *dst, uint32_t n, int32_t fanout,
                           void *work, nts_stream_t stream) {
  NTS_TRACE_RANGE("nts_sample_hop_offsets");
  if (!co) return fail(NTS_ERR_INVALID, "nts_sample_hop_offsets: null co");
  if (n == 0) return nts_memset_zero(co, sizeof(uint32_t), stream);
  if (!graph_co || !dst || !work) return fail(NTS_ERR_INVALID, "nts_sample_hop_offsets: null pointer");
  if (!aligned_to(work, 256)) return fail(NTS_ERR_INVALID, "nts_sample_hop_offsets: work must be 256-byte aligned");
  size_t tmp = 0;
  NTS_HIP_TRY(scan_bytes(n + 1, &tmp));
  return hop_offsets(co, graph_co, dst, host_count(n), fanout, work, tmp, stream);
}

int nts_sample_hop_neighbors(uint32_t *ri_global, const uint32_t *co, const uint32_t *graph_co,
                             const uint32_t *graph_ri, const uint32_t *dst, uint32_t n, int32_t fanout, uint64_t seed,
                             nts_stream_t stream) {
  NTS_TRACE_RANGE("nts_sample_hop_neighbors");
  if (n == 0) return NTS_OK;
  if (!ri_global || !co || !graph_co || !graph_ri || !dst)
    return fail(NTS_ERR_INVALID, "nts_sample_hop_neighbors: null pointer");
  return hop_neighbors(ri_global, co, graph_co, graph_ri, dst, host_count(n), 0xFFFFFFFFu, fanout, host_seed(seed), nullptr,
                       nullptr, stream);
}

}  // extern "C"
