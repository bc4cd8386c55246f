// Device-side construction of a sampled layer's transposed structure and GCN edge weights
// (sampCSC::generate_csr_from_csc, update_degree, compute_weight_forward / backward:
// core/coocsc.hpp:136-216, 243-309).  Integer results and weights are bit-exact with the host
// algorithms; everything is order-independent, so the outputs are deterministic.
#include <string.h>

#include <rocprim/device/device_radix_sort.hpp>
#include <rocprim/device/device_scan.hpp>
#include <rocprim/iterator/counting_iterator.hpp>
#include <rocprim/iterator/transform_iterator.hpp>

#include "common.hpp"

namespace nts {
namespace {

// ro[s] = number of sorted keys < s, for s in [0, Vs]; keys ascending, E of them.
__global__ __launch_bounds__(256) void offsets_from_sorted_kernel(uint32_t *__restrict__ ro,
                                                                  const uint32_t *__restrict__ keys, DevCount Vs,
                                                                  DevCount E) {
  const uint32_t s = blockIdx.x * blockDim.x + threadIdx.x;
  if (s > Vs.get()) return;
  uint32_t lo = 0, hi = E.get();  // first position whose key >= s
  while (lo < hi) {
    const uint32_t mid = lo + (hi - lo) / 2;
    if (keys[mid] < s) lo = mid + 1; else hi = mid;
  }
  ro[s] = lo;
}

// Both halves of the transposed structure from the sorted (source, CSC edge id) pairs in one launch:
// thread t writes ro[t] (as above) when t <= Vs, and ci[t] = the destination that owns CSC edge
// perm[t] when t < E.  perm may alias ci: each thread reads its own element before writing it.
// owner (nullable): the destination slot of every CSC edge; with it ci is a gather instead of a
// search, and ro comes from the places where the sorted keys change (thread t writes the offsets of
// the sources keys[t-1]+1 .. keys[t], a loop of one step when every source has an edge) instead of a
// search per source.
__global__ __launch_bounds__(256) void csr_finish_kernel(uint32_t *__restrict__ ro, uint32_t *ci,
                                                         const uint32_t *__restrict__ keys, const uint32_t *perm,
                                                         const uint32_t *__restrict__ co, DevCount Vd, DevCount Vs,
                                                         DevCount edges, const uint32_t *__restrict__ owner) {
  const uint32_t t = blockIdx.x * blockDim.x + threadIdx.x;
  const uint32_t E = edges.get();
  if (owner) {
    const uint32_t vs = Vs.get();
    if (E == 0) {
      if (t <= vs) ro[t] = 0;
      return;
    }
    if (t < E) {
      const uint32_t here = keys[t] < vs ? keys[t] : vs;
      const uint32_t from = t ? (keys[t - 1] < vs ? keys[t - 1] : vs) + 1 : 0u;
      for (uint32_t s = from; s <= here; ++s) ro[s] = t;
      if (t + 1 == E)
        for (uint32_t s = here + 1; s <= vs; ++s) ro[s] = E;
      ci[t] = owner[perm[t]];
    }
    return;
  }
  if (t <= Vs.get()) {
    uint32_t lo = 0, hi = E;
    while (lo < hi) {
      const uint32_t mid = lo + (hi - lo) / 2;
      if (keys[mid] < t) lo = mid + 1; else hi = mid;
    }
    ro[t] = lo;
  }
  if (t < E) ci[t] = owner_of(co, Vd.get(), perm[t]);
}

// 1 / ((float)sqrt((double)out_deg) * (float)sqrt((double)in_deg)) with every step rounded to
// nearest, as nts_norm_degree evaluates it on the host (core/ntsBaseOp.hpp:183-186).
__device__ __forceinline__ float norm_weight(uint32_t out_deg, uint32_t in_deg) {
  const float a = static_cast<float>(__dsqrt_rn(static_cast<double>(out_deg)));
  const float b = static_cast<float>(__dsqrt_rn(static_cast<double>(in_deg)));
  return __fdiv_rn(1.0f, __fmul_rn(a, b));
}

// blockIdx.y (+ first) = 0: CSC edges e, owner = destination, other end = ri[e] (a source)   -> ewf
//                        1: CSR edges k, owner = source, other end = ci[k] (a destination)    -> ewb
// The edge count is read on the device (own_off[n_own]); threads stride over the edges.  `clear`
// (nullable): `clear_words` words zeroed on the side for the caller's next step.  csc_owner / csr_owner
// (nullable): the owner of every CSC / CSR edge where the caller has them (the neighbour pick's record
// and the sorted keys of the transposition); without them the owner is searched for in the offsets.
__global__ __launch_bounds__(256) void edge_weights_kernel(float *__restrict__ ewf, float *__restrict__ ewb,
                                                           const uint32_t *__restrict__ co,
                                                           const uint32_t *__restrict__ ri,
                                                           const uint32_t *__restrict__ ro,
                                                           const uint32_t *__restrict__ ci, DevCount Vd, DevCount Vs,
                                                           int first, uint32_t *__restrict__ clear,
                                                           uint32_t clear_words,
                                                           const uint32_t *__restrict__ csc_owner,
                                                           const uint32_t *__restrict__ csr_owner) {
  const int which = first + static_cast<int>(blockIdx.y);
  const uint64_t stride = static_cast<uint64_t>(gridDim.x) * blockDim.x;
  const uint64_t start = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (clear && blockIdx.y == 0)
    for (uint64_t w = start; w < clear_words; w += stride) clear[w] = 0;
  const uint32_t *own_off = which == 0 ? co : ro;
  const uint32_t *other_off = which == 0 ? ro : co;
  const uint32_t *other_idx = which == 0 ? ri : ci;
  float *wout = which == 0 ? ewf : ewb;
  const uint32_t *known = which == 0 ? csc_owner : csr_owner;
  if (!wout) return;
  const uint32_t n_own = which == 0 ? Vd.get() : Vs.get();
  const uint32_t E = own_off[n_own];
  for (uint64_t e = start; e < E; e += stride) {
    const uint32_t o = known ? known[e] : owner_of(own_off, n_own, static_cast<uint32_t>(e));
    const uint32_t own_deg = own_off[o + 1] - own_off[o];
    const uint32_t t = other_idx[e];
    const uint32_t other_deg = other_off[t + 1] - other_off[t];
    wout[e] = which == 0 ? norm_weight(other_deg, own_deg) : norm_weight(own_deg, other_deg);
  }
}

// keys[e] = mirror ? mirror[ri[e]] : ri[e]
__global__ __launch_bounds__(256) void target_keys_kernel(uint32_t *__restrict__ keys, const uint32_t *__restrict__ ri,
                                                          const uint32_t *__restrict__ mirror, uint32_t E) {
  const uint32_t e = blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= E) return;
  const uint32_t s = ri[e];
  keys[e] = mirror ? mirror[s] : s;
}

// One wave per sorted position; only the first position of a run of equal keys works: it adds the
// run's edge rows in sorted (= ascending edge id) order into out[key].
__global__ __launch_bounds__(256) void add_runs_kernel(float *__restrict__ out, const float *__restrict__ msg,
                                                       const uint32_t *__restrict__ keys,
                                                       const uint32_t *__restrict__ perm, uint32_t E, uint32_t F) {
  const uint32_t k = blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
  if (k >= E) return;
  const uint32_t key = keys[k];
  if (k > 0 && keys[k - 1] == key) return;
  const uint32_t lane = threadIdx.x & (kWave - 1);
  uint32_t end = k + 1;
  while (end < E && keys[end] == key) ++end;
  for (uint32_t c = lane; c < F; c += kWave) {
    float a = 0.f;
    for (uint32_t j = k; j < end; ++j) a += msg[static_cast<size_t>(perm[j]) * F + c];
    out[static_cast<size_t>(key) * F + c] += a;
  }
}

// ---- sampled-source relabelling (bitmap of sampled global ids -> sorted list + local ids) --------

__global__ __launch_bounds__(256) void mark_bits_kernel(uint32_t *__restrict__ bits, const uint32_t *__restrict__ ids,
                                                        DevCount E) {
  const uint32_t e = blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= E.get()) return;
  const uint32_t g = ids[e];
  atomicOr(&bits[g >> 5], 1u << (g & 31));  // integer OR: the result does not depend on the order
}

struct WordPopcount {
  const uint32_t *bits;
  __device__ uint32_t operator()(uint32_t w) const { return __popc(bits[w]); }
};
using PopcountIterator = rocprim::transform_iterator<rocprim::counting_iterator<uint32_t>, WordPopcount, uint32_t>;

// Two independent uses of the bitmap and its per-word prefix in one launch.
// Threads [0, words): source[prefix[w] + rank] = 32*w + bit for every set bit of word w, ascending;
//   the last word also stores the total (twice when n_source_copy is set).
// Threads words + e: local[e] = rank of ids[e] among the set bits, for e < E; local[e] = fill_value
//   for E <= e < fill_to (padding for a sort over a fixed capacity); e_out (nullable) receives E.
__global__ __launch_bounds__(256) void expand_relabel_kernel(uint32_t *__restrict__ source,
                                                             uint32_t *__restrict__ n_source,
                                                             uint32_t *__restrict__ n_source_copy,
                                                             uint32_t *__restrict__ local,
                                                             const uint32_t *__restrict__ ids,
                                                             const uint32_t *__restrict__ bits,
                                                             const uint32_t *__restrict__ prefix, uint32_t words,
                                                             DevCount edges, uint32_t fill_to, uint32_t fill_value,
                                                             uint32_t *__restrict__ e_out) {
  const uint32_t t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t < words) {
    uint32_t word = bits[t];
    uint32_t pos = prefix[t];
    if (t + 1 == words) {
      *n_source = pos + __popc(word);
      if (n_source_copy) *n_source_copy = pos + __popc(word);
    }
    while (word) {
      const uint32_t b = __ffs(word) - 1;
      source[pos++] = (t << 5) + b;
      word &= word - 1;
    }
    return;
  }
  const uint32_t e = t - words;
  const uint32_t E = edges.get();
  if (e == 0 && e_out) *e_out = E;
  if (e >= E) {
    if (e < fill_to) local[e] = fill_value;
    return;
  }
  const uint32_t g = ids[e];
  const uint32_t w = g >> 5;
  local[e] = prefix[w] + __popc(bits[w] & ((1u << (g & 31)) - 1u));
}

hipError_t scan_temp_bytes(uint32_t words, size_t *bytes) {
  size_t tmp = 0;
  uint32_t *nul = nullptr;
  PopcountIterator in(rocprim::counting_iterator<uint32_t>(0u), WordPopcount{nullptr});
  hipError_t err = rocprim::exclusive_scan(nullptr, tmp, in, nul, 0u, words ? words : 1u, rocprim::plus<uint32_t>(),
                                           static_cast<hipStream_t>(nullptr), false);
  *bytes = tmp;
  return err;
}

inline unsigned bits_for(uint32_t n) {  // bits needed to represent values in [0, n)
  unsigned b = 1;
  while (b < 32 && (1ull << b) < n) ++b;
  return b;
}

inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

// ---- stable sort of a sampled hop's edges by local source ------------------------------------------
//
// generate_csr_from_csc is a stable counting sort of (local source, CSC edge id).  A sampled hop has
// 10^4 .. 10^6 edges and keys of 15 to 22 bits.  The library's device-wide radix sort spends ~24 us per
// eight-bit pass whatever the size and clears its histograms with memset nodes, which keeps a batch's
// construction out of a HIP graph.  This one is sized for hops: a least-significant-digit radix sort
// in ceil(key_bits / 10) passes of equal width, three launches per pass and no memset:
//   hop_sort_count    block b counts the digits of edges [2048 b, 2048 (b + 1)) in an LDS histogram and
//                     writes its column of the digit-major table counts[digit][block]
//   hop_sort_rows     one block per digit: exclusive scan of that digit's row over the blocks, and
//                     the digit's total
//   hop_sort_scatter  block b turns the totals into the digits' first positions, adds its entries of
//                     the table, ranks each of its 2,048 edges among the chunk's edges of the same
//                     digit (ballots inside a wavefront, per-wavefront histograms across them) and
//                     writes every edge to start[digit] + that rank
// Equal keys keep their order in every pass: the result is the stable order, bit for bit.  Only
// blocks below ceil(E / 2048) of the launched ceil(capacity / 2048) do anything.
constexpr int kHopSortThreads = 256;
constexpr int kHopSortItems = 8;
constexpr uint32_t kHopSortChunk = kHopSortThreads * kHopSortItems;  // 2,048 edges
constexpr unsigned kHopSortMaxDigitBits = 10;  // 11 (two passes for 22-bit keys) measured slower: 2,048-bin tables
constexpr uint32_t kHopSortMaxBins = 1u << kHopSortMaxDigitBits;

struct HopSortShape {
  uint32_t blocks;
  unsigned passes;
  unsigned digit_bits;
};
inline HopSortShape hop_sort_shape(uint32_t capacity, unsigned key_bits) {
  HopSortShape sh;
  sh.blocks = capacity ? static_cast<uint32_t>((static_cast<uint64_t>(capacity) + kHopSortChunk - 1) / kHopSortChunk) : 1u;
  if (key_bits == 0) key_bits = 1;
  sh.passes = (key_bits + kHopSortMaxDigitBits - 1) / kHopSortMaxDigitBits;
  sh.digit_bits = (key_bits + sh.passes - 1) / sh.passes;
  return sh;
}

__global__ __launch_bounds__(kHopSortThreads) void hop_sort_count_kernel(uint32_t *__restrict__ table,
                                                                         const uint32_t *__restrict__ keys,
                                                                         DevCount edges, unsigned shift,
                                                                         unsigned digit_bits) {
  __shared__ uint32_t hist[kHopSortMaxBins];
  const uint32_t E = edges.get();
  const uint64_t first = static_cast<uint64_t>(blockIdx.x) * kHopSortChunk;
  if (first >= E) return;
  const uint32_t bins = 1u << digit_bits, mask = bins - 1u;
  for (uint32_t d = threadIdx.x; d < bins; d += kHopSortThreads) hist[d] = 0;
  __syncthreads();
  const uint64_t last = first + kHopSortChunk < E ? first + kHopSortChunk : E;
  for (uint64_t e = first + threadIdx.x; e < last; e += kHopSortThreads) atomicAdd(&hist[(keys[e] >> shift) & mask], 1u);
  __syncthreads();
  for (uint32_t d = threadIdx.x; d < bins; d += kHopSortThreads) table[static_cast<size_t>(d) * gridDim.x + blockIdx.x] = hist[d];
}

// One block per digit; table rows are `blocks` long, totals follow the table.
__global__ __launch_bounds__(kHopSortThreads) void hop_sort_rows_kernel(uint32_t *__restrict__ table,
                                                                        uint32_t *__restrict__ totals, uint32_t blocks,
                                                                        DevCount edges) {
  __shared__ uint32_t wave_sums[kHopSortThreads / kWave];
  const uint32_t E = edges.get();
  const uint32_t live = static_cast<uint32_t>((static_cast<uint64_t>(E) + kHopSortChunk - 1) / kHopSortChunk);
  uint32_t *row = table + static_cast<size_t>(blockIdx.x) * blocks;
  const uint32_t per = (live + kHopSortThreads - 1) / kHopSortThreads;
  const uint32_t b = threadIdx.x * per, e = b + per < live ? b + per : live;
  uint32_t sum = 0;
  for (uint32_t i = b; i < e; ++i) sum += row[i];
  uint32_t total;
  uint32_t run = block_prefix<kHopSortThreads>(sum, wave_sums, &total);
  for (uint32_t i = b; i < e; ++i) {
    const uint32_t v = row[i];
    row[i] = run;
    run += v;
  }
  if (threadIdx.x == 0) totals[blockIdx.x] = total;
}

// vals_in == nullptr: the value of edge e is e.  THREADS x ITEMS = 2,048 edges per block.  Wavefront w
// takes the edges [512 w, 512 (w + 1)) of the chunk, 64 consecutive ones per round: the lanes that hold
// the same digit find each other with one ballot per digit bit, an edge's rank is the number of equal
// digits the wavefront has seen in earlier rounds (a histogram of its own in LDS) plus the equal digits
// on lower lanes, and the wavefronts' histograms, added up in wavefront order, give the rest -- the
// stable rank of every edge without sorting the chunk.
template <int THREADS, int ITEMS>
__global__ __launch_bounds__(THREADS) void hop_sort_scatter_kernel(uint32_t *__restrict__ keys_out,
                                                                           uint32_t *__restrict__ vals_out,
                                                                           const uint32_t *__restrict__ keys_in,
                                                                           const uint32_t *__restrict__ vals_in,
                                                                           const uint32_t *__restrict__ table,
                                                                           const uint32_t *__restrict__ totals,
                                                                           DevCount edges, unsigned shift,
                                                                           unsigned digit_bits) {
  constexpr int kWaves = THREADS / kWave;
  __shared__ uint32_t start[kHopSortMaxBins];  // output position of the first edge of each digit from this block
  __shared__ uint32_t wave_hist[kWaves][kHopSortMaxBins];
  __shared__ uint32_t wave_sums[kWaves];
  static_assert(THREADS * ITEMS == static_cast<int>(kHopSortChunk), "one chunk per block");
  const uint32_t E = edges.get();
  const uint64_t c0 = static_cast<uint64_t>(blockIdx.x) * kHopSortChunk;
  if (c0 >= E) return;
  const uint32_t n = static_cast<uint32_t>(E - c0 < kHopSortChunk ? E - c0 : kHopSortChunk);
  const uint32_t bins = 1u << digit_bits, mask = bins - 1u;
  const uint32_t lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  uint32_t key[ITEMS], val[ITEMS], rank[ITEMS];
#pragma unroll
  for (int j = 0; j < ITEMS; ++j) {  // coalesced: round j of this wavefront
    const uint32_t p = wave * (kWave * ITEMS) + j * kWave + lane;
    key[j] = 0;
    val[j] = 0;
    if (p < n) {
      key[j] = keys_in[c0 + p];
      val[j] = vals_in ? vals_in[c0 + p] : static_cast<uint32_t>(c0 + p);
    }
  }
#pragma unroll
  for (int w = 0; w < kWaves; ++w)
    for (uint32_t d = threadIdx.x; d < bins; d += THREADS) wave_hist[w][d] = 0;
  {  // first position of every digit: exclusive scan of the totals, plus this block's entry of the table
    const uint32_t per = (bins + THREADS - 1) / THREADS;
    const uint32_t b = threadIdx.x * per, e = b + per < bins ? b + per : bins;
    uint32_t sum = 0;
    for (uint32_t d = b; d < e; ++d) sum += totals[d];
    uint32_t total;
    uint32_t run = block_prefix<THREADS>(sum, wave_sums, &total);
    for (uint32_t d = b; d < e; ++d) {
      start[d] = run + table[static_cast<size_t>(d) * gridDim.x + blockIdx.x];
      run += totals[d];
    }
  }
  __syncthreads();
  uint32_t *hist = wave_hist[wave];
  const uint64_t below = (1ull << lane) - 1ull;
#pragma unroll
  for (int j = 0; j < ITEMS; ++j) {
    const uint32_t p = wave * (kWave * ITEMS) + j * kWave + lane;
    const bool active = p < n;
    const uint32_t d = (key[j] >> shift) & mask;
    uint64_t peers = __ballot(active);  // for an active lane: the active lanes with the same digit
    for (unsigned b = 0; b < digit_bits; ++b) {
      const bool one = (d >> b) & 1u;
      const uint64_t votes = __ballot(one);
      peers &= one ? votes : ~votes;
    }
    const uint32_t seen = active ? hist[d] : 0u;
    rank[j] = seen + __popcll(peers & below);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();  // every lane has read its count before a leader raises it
    if (active && (peers & below) == 0) hist[d] = seen + __popcll(peers);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  }
  __syncthreads();
  for (uint32_t d = threadIdx.x; d < bins; d += THREADS) {  // counts -> edges of the digit in earlier wavefronts
    uint32_t run = 0;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
      const uint32_t v = wave_hist[w][d];
      wave_hist[w][d] = run;
      run += v;
    }
  }
  __syncthreads();
#pragma unroll
  for (int j = 0; j < ITEMS; ++j) {
    const uint32_t p = wave * (kWave * ITEMS) + j * kWave + lane;
    if (p < n) {
      const uint32_t d = (key[j] >> shift) & mask;
      const uint32_t pos = start[d] + hist[d] + rank[j];
      keys_out[pos] = key[j];
      vals_out[pos] = val[j];
    }
  }
}

// Splits the (src, dst) pairs of an edge list into two key arrays.
__global__ __launch_bounds__(256) void split_pairs_kernel(uint32_t *__restrict__ src, uint32_t *__restrict__ dst,
                                                          const uint2 *__restrict__ pairs, uint32_t E) {
  const uint32_t e = blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= E) return;
  const uint2 p = pairs[e];
  src[e] = p.x;
  dst[e] = p.y;
}

hipError_t sort_pairs_temp_bytes(uint32_t E, size_t *bytes) {
  size_t tmp = 0;
  uint32_t *nul = nullptr;
  hipError_t err = rocprim::radix_sort_pairs(nullptr, tmp, nul, nul, nul, nul, E ? E : 1u, 0u, 32u,
                                             static_cast<hipStream_t>(nullptr), false);
  *bytes = tmp;
  return err;
}

}  // namespace

// Scratch layout: [sorted keys: n][keys between passes: n][values between passes: n]
//                 [digit table: 1,024 x ceil(n / 2048)][digit totals: 1,024], all u32.
size_t csr_from_csc_bytes(uint32_t sort_n) {
  const size_t arr = align_up(static_cast<size_t>(sort_n ? sort_n : 1) * sizeof(uint32_t), 256);
  const HopSortShape sh = hop_sort_shape(sort_n, 32);
  const size_t table = align_up((static_cast<size_t>(sh.blocks) + 1) * kHopSortMaxBins * sizeof(uint32_t), 256);
  return 3 * arr + table + 256;
}

int csr_from_csc(uint32_t *ro, uint32_t *ci, uint32_t *perm, const uint32_t *co, const uint32_t *ri, DevCount Vd,
                 DevCount Vs, DevCount E, uint32_t sort_n, unsigned key_bits, void *work, const uint32_t *owner,
                 hipStream_t stream) {
  unsigned char *w = static_cast<unsigned char *>(work);
  const size_t arr = align_up(static_cast<size_t>(sort_n ? sort_n : 1) * sizeof(uint32_t), 256);
  uint32_t *keys_sorted = reinterpret_cast<uint32_t *>(w);
  uint32_t *keys_mid[2] = {reinterpret_cast<uint32_t *>(w + arr), keys_sorted};
  uint32_t *vals_mid = reinterpret_cast<uint32_t *>(w + 2 * arr);
  uint32_t *table = reinterpret_cast<uint32_t *>(w + 3 * arr);
  // Without a caller buffer for perm, ci doubles as the sorted edge-id array and is rewritten in
  // place by a second pass (each thread reads its own element before writing it).
  uint32_t *perm_out = perm ? perm : ci;
  // Stable sort of (local source, CSC edge id): edge ids stay ascending within a source, which is
  // exactly the order the host counting sort produces.  Keys and values alternate between two
  // buffers so that the last pass lands in keys_sorted / perm_out.
  const HopSortShape sh = hop_sort_shape(sort_n, key_bits);
  uint32_t *totals = table + static_cast<size_t>(sh.blocks) * kHopSortMaxBins;
  uint32_t *vals_buf[2] = {vals_mid, perm_out};
  const uint32_t *kin = ri, *vin = nullptr;
  for (unsigned pass = 0; pass < sh.passes; ++pass) {
    const unsigned to = (sh.passes - 1 - pass) & 1u ? 0u : 1u;  // the last pass writes buffer 1
    uint32_t *kout = keys_mid[to], *vout = vals_buf[to];
    const unsigned shift = pass * sh.digit_bits;
    hipLaunchKernelGGL(hop_sort_count_kernel, dim3(sh.blocks), dim3(kHopSortThreads), 0, stream, table, kin, E, shift,
                       sh.digit_bits);
    hipLaunchKernelGGL(hop_sort_rows_kernel, dim3(1u << sh.digit_bits), dim3(kHopSortThreads), 0, stream, table, totals,
                       sh.blocks, E);
    hipLaunchKernelGGL((hop_sort_scatter_kernel<kHopSortThreads, kHopSortItems>), dim3(sh.blocks), dim3(kHopSortThreads), 0,
                       stream, kout, vout, kin, vin, table, totals, E, shift, sh.digit_bits);
    NTS_LAUNCH_CHECK("hop_sort kernels");
    kin = kout;
    vin = vout;
  }
  const uint64_t span = static_cast<uint64_t>(Vs.cap) + 1 > E.cap ? static_cast<uint64_t>(Vs.cap) + 1 : E.cap;
  hipLaunchKernelGGL(csr_finish_kernel, dim3(ceil_div(span, 256)), dim3(256), 0, stream, ro, ci, keys_sorted, perm_out,
                     co, Vd, Vs, E, owner);
  NTS_LAUNCH_CHECK("csr_finish_kernel");
  return NTS_OK;
}

int relabel_sources(uint32_t *source, uint32_t *n_source, uint32_t *n_source_copy, uint32_t *local,
                    const uint32_t *global_ids, DevCount E, uint32_t fill_to, uint32_t fill_value, uint32_t *e_out,
                    uint32_t V, void *work, bool marked, hipStream_t stream) {
  const uint32_t words = (V + 31) / 32;
  const size_t arr = align_up(static_cast<size_t>(words) * sizeof(uint32_t), 256);
  unsigned char *w = static_cast<unsigned char *>(work);
  uint32_t *bits = reinterpret_cast<uint32_t *>(w);
  uint32_t *prefix = reinterpret_cast<uint32_t *>(w + arr);
  size_t tmp = 0;
  NTS_HIP_TRY(scan_temp_bytes(words, &tmp));
  if (!marked) {
    if (int rc = nts_memset_zero(bits, static_cast<size_t>(words) * sizeof(uint32_t), stream)) return rc;
    hipLaunchKernelGGL(mark_bits_kernel, dim3(ceil_div(E.cap, 256)), dim3(256), 0, stream, bits, global_ids, E);
    NTS_LAUNCH_CHECK("mark_bits_kernel");
  }
  PopcountIterator counts(rocprim::counting_iterator<uint32_t>(0u), WordPopcount{bits});
  NTS_HIP_TRY(rocprim::exclusive_scan(w + 2 * arr, tmp, counts, prefix, 0u, words, rocprim::plus<uint32_t>(), stream,
                                      false));
  const uint64_t span = static_cast<uint64_t>(words) + (fill_to > E.cap ? fill_to : E.cap);
  hipLaunchKernelGGL(expand_relabel_kernel, dim3(ceil_div(span, 256)), dim3(256), 0, stream, source, n_source,
                     n_source_copy, local, global_ids, bits, prefix, words, E, fill_to, fill_value, e_out);
  NTS_LAUNCH_CHECK("expand_relabel_kernel");
  return NTS_OK;
}

int gcn_edge_weights(float *ewf, float *ewb, const uint32_t *co, const uint32_t *ri, const uint32_t *ro,
                     const uint32_t *ci, DevCount Vd, DevCount Vs, uint32_t *clear, uint32_t clear_words,
                     const uint32_t *csc_owner, const uint32_t *csr_owner, hipStream_t stream) {
  // The edge count lives on the device: the grid is sized from the vertex counts and the kernel
  // strides over co[Vd] edges, so the call neither needs the count nor synchronises.  Forward and
  // backward weights share one launch (grid.y).
  uint64_t blocks = (static_cast<uint64_t>(Vd.cap > Vs.cap ? Vd.cap : Vs.cap) * 32 + 255) / 256;
  if (blocks < 64) blocks = 64;
  if (blocks > 8192) blocks = 8192;
  if (!ewf && !ewb && !clear) return NTS_OK;
  const int first = ewf ? 0 : 1;
  const unsigned passes = (ewf && ewb) ? 2u : 1u;
  hipLaunchKernelGGL(edge_weights_kernel, dim3(static_cast<unsigned>(blocks), passes), dim3(256), 0, stream, ewf, ewb, co,
                     ri, ro, ci, Vd, Vs, first, clear, clear_words, csc_owner, csr_owner);
  NTS_LAUNCH_CHECK("edge_weights_kernel");
  return NTS_OK;
}

}  // namespace nts

using namespace nts;

extern "C" {

size_t nts_csr_from_csc_work_bytes(uint32_t Vd, uint32_t Vs, uint32_t E) {
  (void)Vd;
  (void)Vs;
  return csr_from_csc_bytes(E);
}

int nts_csr_from_csc(uint32_t *ro, uint32_t *ci, uint32_t *perm, const uint32_t *co, const uint32_t *ri, uint32_t Vd,
                     uint32_t Vs, uint32_t E, void *work, nts_stream_t stream) {
  NTS_TRACE_RANGE("nts_csr_from_csc");
  if (!ro) return fail(NTS_ERR_INVALID, "nts_csr_from_csc: null ro");
  if (E == 0) {
    return nts_memset_zero(ro, (static_cast<size_t>(Vs) + 1) * sizeof(uint32_t), stream);
  }
  if (!ci || !co || !ri || !work) return fail(NTS_ERR_INVALID, "nts_csr_from_csc: null pointer");
  if (!aligned_to(work, 256)) return fail(NTS_ERR_INVALID, "nts_csr_from_csc: work must be 256-byte aligned");
  return csr_from_csc(ro, ci, perm, co, ri, host_count(Vd), host_count(Vs), host_count(E), E, bits_for(Vs), work, nullptr,
                      stream);
}

size_t nts_chunk_from_edges_work_bytes(uint32_t V, uint32_t E) {
  (void)V;
  size_t tmp = 0;
  if (sort_pairs_temp_bytes(E, &tmp) != hipSuccess) return 0;
  return 3 * align_up(static_cast<size_t>(E) * sizeof(uint32_t), 256) + align_up(tmp, 256) + 256;
}

int nts_chunk_from_edges(uint32_t *co, uint32_t *ri, float *ewf, uint32_t *ro, uint32_t *ci, float *ewb,
                         const uint32_t *pairs, uint32_t E, uint32_t V, void *work, nts_stream_t stream) {
  NTS_TRACE_RANGE("nts_chunk_from_edges");
  if (!co || !ro) return fail(NTS_ERR_INVALID, "nts_chunk_from_edges: null offsets");
  if (E == 0) {
    if (int rc = nts_memset_zero(co, (static_cast<size_t>(V) + 1) * sizeof(uint32_t), stream)) return rc;
    return nts_memset_zero(ro, (static_cast<size_t>(V) + 1) * sizeof(uint32_t), stream);
  }
  if (V == 0) return fail(NTS_ERR_INVALID, "nts_chunk_from_edges: edges without vertices");
  if (!ri || !ci || !pairs || !work) return fail(NTS_ERR_INVALID, "nts_chunk_from_edges: null pointer");
  if (!aligned_to(work, 256) || !aligned_to(pairs, 8))
    return fail(NTS_ERR_INVALID, "nts_chunk_from_edges: work must be 256-byte and pairs 8-byte aligned");
  const size_t arr = align_up(static_cast<size_t>(E) * sizeof(uint32_t), 256);
  unsigned char *w = static_cast<unsigned char *>(work);
  uint32_t *a = reinterpret_cast<uint32_t *>(w);            // file-order sources, later destination-sorted keys
  uint32_t *b = reinterpret_cast<uint32_t *>(w + arr);      // file-order destinations
  uint32_t *c = reinterpret_cast<uint32_t *>(w + 2 * arr);  // sources in (source, file) order
  void *tmp_ptr = w + 3 * arr;
  size_t tmp = 0;
  NTS_HIP_TRY(sort_pairs_temp_bytes(E, &tmp));
  const unsigned bits = bits_for(V);
  hipLaunchKernelGGL(split_pairs_kernel, dim3(ceil_div(E, 256)), dim3(256), 0, stream, a, b,
                     reinterpret_cast<const uint2 *>(pairs), E);
  NTS_LAUNCH_CHECK("split_pairs_kernel");
  // The edge list ordered by source, file order kept inside a source (stable sort): the CSR rows.
  NTS_HIP_TRY(rocprim::radix_sort_pairs(tmp_ptr, tmp, a, c, b, ci, E, 0u, bits, stream, false));
  hipLaunchKernelGGL(offsets_from_sorted_kernel, dim3(ceil_div(static_cast<uint64_t>(V) + 1, 256)), dim3(256), 0,
                     stream, ro, c, host_count(V), host_count(E));
  NTS_LAUNCH_CHECK("offsets_from_sorted_kernel(ro)");
  // That list re-ordered by destination, again stable: the CSC rows (sources ascending inside a row).
  NTS_HIP_TRY(rocprim::radix_sort_pairs(tmp_ptr, tmp, ci, a, c, ri, E, 0u, bits, stream, false));
  hipLaunchKernelGGL(offsets_from_sorted_kernel, dim3(ceil_div(static_cast<uint64_t>(V) + 1, 256)), dim3(256), 0,
                     stream, co, a, host_count(V), host_count(E));
  NTS_LAUNCH_CHECK("offsets_from_sorted_kernel(co)");
  if (ewf || ewb) return nts_gcn_edge_weights(ewf, ewb, co, ri, ro, ci, V, V, stream);
  return NTS_OK;
}

size_t nts_relabel_sources_work_bytes(uint32_t V) {
  const size_t words = (static_cast<size_t>(V) + 31) / 32;
  size_t tmp = 0;
  if (scan_temp_bytes(static_cast<uint32_t>(words), &tmp) != hipSuccess) return 0;
  return 3 * align_up(words * sizeof(uint32_t), 256) + align_up(tmp, 256) + 256;
}

int nts_relabel_sources(uint32_t *source, uint32_t *n_source, uint32_t *local, const uint32_t *global_ids, uint32_t E,
                        uint32_t V, void *work, nts_stream_t stream) {
  NTS_TRACE_RANGE("nts_relabel_sources");
  if (!n_source) return fail(NTS_ERR_INVALID, "nts_relabel_sources: null n_source");
  if (E == 0 || V == 0) return nts_memset_zero(n_source, sizeof(uint32_t), stream);
  if (!source || !local || !global_ids || !work) return fail(NTS_ERR_INVALID, "nts_relabel_sources: null pointer");
  if (!aligned_to(work, 256)) return fail(NTS_ERR_INVALID, "nts_relabel_sources: work must be 256-byte aligned");
  return relabel_sources(source, n_source, nullptr, local, global_ids, host_count(E), 0, 0, nullptr, V, work, false,
                         stream);
}

int nts_gather_edge_to_src_unsorted(float *out, const float *msg, const uint32_t *ri, const uint32_t *co,
                                    const uint32_t *mirror, uint32_t Vd, uint32_t F, nts_stream_t stream) {
  NTS_TRACE_RANGE("nts_gather_edge_to_src_unsorted");
  if (F == 0) return fail(NTS_ERR_INVALID, "nts_gather_edge_to_src_unsorted: F is 0");
  if (Vd == 0) return NTS_OK;
  if (!out || !msg || !ri || !co) return fail(NTS_ERR_INVALID, "nts_gather_edge_to_src_unsorted: null pointer");
  uint32_t E = 0;
  NTS_HIP_TRY(hipMemcpyAsync(&E, co + Vd, sizeof(uint32_t), hipMemcpyDeviceToHost, stream));
  NTS_HIP_TRY(hipStreamSynchronize(stream));
  if (E == 0) return NTS_OK;
  size_t tmp = 0;
  NTS_HIP_TRY(rocprim::radix_sort_pairs(nullptr, tmp, static_cast<uint32_t *>(nullptr), static_cast<uint32_t *>(nullptr),
                                        rocprim::counting_iterator<uint32_t>(0u), static_cast<uint32_t *>(nullptr), E, 0u,
                                        32u, stream, false));
  const size_t arr = align_up(static_cast<size_t>(E) * sizeof(uint32_t), 256);
  unsigned char *work = nullptr;
  NTS_HIP_TRY(scratch_alloc(reinterpret_cast<void **>(&work), 3 * arr + align_up(tmp, 256), stream));
  uint32_t *keys = reinterpret_cast<uint32_t *>(work);
  uint32_t *keys_sorted = reinterpret_cast<uint32_t *>(work + arr);
  uint32_t *perm = reinterpret_cast<uint32_t *>(work + 2 * arr);
  hipLaunchKernelGGL(target_keys_kernel, dim3(ceil_div(E, 256)), dim3(256), 0, stream, keys, ri, mirror, E);
  hipError_t err = hipGetLastError();
  if (err == hipSuccess)
    err = rocprim::radix_sort_pairs(work + 3 * arr, tmp, keys, keys_sorted,
                                                     rocprim::counting_iterator<uint32_t>(0u), perm, E, 0u, 32u, stream,
                                                     false);
  if (err == hipSuccess) {
    hipLaunchKernelGGL(add_runs_kernel, dim3(ceil_div(E, 4)), dim3(256), 0, stream, out, msg, keys_sorted, perm, E, F);
    err = hipGetLastError();
  }
  hipError_t ferr = scratch_free(work, stream);
  if (err != hipSuccess) return fail_hip(err, "nts_gather_edge_to_src_unsorted");
  if (ferr != hipSuccess) return fail_hip(ferr, "nts_gather_edge_to_src_unsorted: hipFreeAsync");
  return NTS_OK;
}

int nts_gcn_edge_weights(float *ewf, float *ewb, const uint32_t *co, const uint32_t *ri, const uint32_t *ro,
                         const uint32_t *ci, uint32_t Vd, uint32_t Vs, nts_stream_t stream) {
  NTS_TRACE_RANGE("nts_gcn_edge_weights");
  if (!co || !ro) return fail(NTS_ERR_INVALID, "nts_gcn_edge_weights: null offsets");
  if (Vd == 0 || Vs == 0) return NTS_OK;
  if (ewf && !ri) return fail(NTS_ERR_INVALID, "nts_gcn_edge_weights: null ri");
  if (ewb && !ci) return fail(NTS_ERR_INVALID, "nts_gcn_edge_weights: null ci");
  return gcn_edge_weights(ewf, ewb, co, ri, ro, ci, host_count(Vd), host_count(Vs), nullptr, 0, nullptr, nullptr, stream);
}

}  // extern "C"
