// Edge <-> vertex movement, edge softmax and fused GAT attention kernels (replaces
// cuda/ntsCUDADistKernel.cuh:23-95, 166-260, cuda/ntsCUDAFuseKernel.cuh:492-506 and their
// launchers cuda/ntsCUDAGraphOP.cu:294-377, 449-474).
//
// Copies and per-edge products are edge-parallel (work per wavefront independent of any vertex's
// degree); per-destination reductions give one wavefront to one destination (or source) row, lanes
// spanning the feature / head dimension.  Sums run in edge order or through fixed-shape cross-lane
// butterflies, and nothing uses float atomics, so every result is bit-reproducible.
#include "common.hpp"

namespace nts {
namespace {

constexpr int kWavesPerBlock = 4;

__device__ __forceinline__ uint32_t wave_item() {
  return blockIdx.x * (blockDim.x / kWave) + (threadIdx.x / kWave);
}
__device__ __forceinline__ uint32_t lane_id() { return threadIdx.x & (kWave - 1); }

inline dim3 wave_grid(uint32_t items) { return dim3(ceil_div(items ? items : 1, kWavesPerBlock)); }
inline dim3 wave_block() { return dim3(kWavesPerBlock * kWave); }

// ---- vertex -> edge copies ------------------------------------------------------------------
//
// Edge-parallel: the edge count is read on the device (co[Vd]); a wavefront takes 64 consecutive
// edges per step, every lane looks up the feature row its edge copies from (the source id, or the
// destination that owns the edge, followed along the wavefront's contiguous span of edges), and
// sub-wavefront groups of G lanes then move 64/G rows at a time.  Work per wave does not depend on
// any vertex's degree.

enum CopyMode { kFromSrc = 0, kFromDst = 1, kAddFromDst = 2 };

// owner_of by the whole wavefront (all 64 lanes call it, the result is the same on every lane): the lanes
// probe 64 evenly spaced offsets of the remaining range at once, so a search over 10^5 rows is three
// rounds of one load instead of seventeen dependent ones -- what a wavefront that walks only a step or
// two of a small edge list otherwise spends most of its time on.
__device__ __forceinline__ uint32_t owner_of_wave(const uint32_t *__restrict__ off, uint32_t n, uint32_t pos) {
  const uint32_t lane = threadIdx.x & (kWave - 1);
  uint32_t lo = 0, hi = n;  // answer in [lo, hi)
  while (hi - lo > 1) {
    const uint32_t step = (hi - lo + kWave - 1) / kWave;
    const uint64_t idx = static_cast<uint64_t>(lo) + static_cast<uint64_t>(lane + 1) * step;  // ascending probes
    const bool behind = idx < hi && off[idx] <= pos;
    const uint32_t k = __popcll(__ballot(behind));  // probes are ascending: the first k are not beyond pos
    lo += k * step;
    hi = lo + step < hi ? lo + step : hi;
  }
  return lo;
}

template <typename V, int G>
__global__ __launch_bounds__(256) void edge_copy_kernel(V *__restrict__ msg, const V *__restrict__ feat,
                                                        const uint32_t *__restrict__ ri,
                                                        const uint32_t *__restrict__ co,
                                                        const uint32_t *__restrict__ mirror, uint32_t Vd, uint32_t Fv,
                                                        int mode) {
  const uint32_t E = co[Vd];
  const uint32_t lane = lane_id();
  const uint32_t gl = lane & (G - 1), grp = lane / G;
  constexpr uint32_t kEdgesPerStep = kWave / G;
  const uint64_t wave = (static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x) / kWave;
  const uint64_t n_waves = static_cast<uint64_t>(gridDim.x) * blockDim.x / kWave;
  // A wavefront walks a contiguous span of wave steps: the destination that owns each step's edges
  // follows from the previous step's (owners_of_step) instead of a search per lane.
  const uint64_t total_steps = (static_cast<uint64_t>(E) + kWave - 1) / kWave;
  const uint64_t per_wave = (total_steps + n_waves - 1) / n_waves;
  const uint64_t first_step = wave * per_wave;
  const uint64_t end_step = first_step + per_wave < total_steps ? first_step + per_wave : total_steps;
  if (first_step >= end_step) return;
  uint32_t d0 = mode == kFromSrc ? 0u : owner_of_wave(co, Vd, static_cast<uint32_t>(first_step * kWave));
  for (uint64_t step = first_step; step < end_step; ++step) {
    const uint64_t base = step * kWave;
    const uint64_t e = base + lane;
    uint32_t row = 0;
    if (mode == kFromSrc) {
      if (e < E) {
        row = ri[e];
        if (mirror) row = mirror[row];
      }
    } else {
      row = owners_of_step(co, Vd, static_cast<uint32_t>(base), d0);
    }
    for (uint32_t j = 0; j < G; ++j) {
      const uint32_t holder = j * kEdgesPerStep + grp;  // lane that looked up this group's edge
      const uint32_t r = __shfl(row, holder, kWave);
      const uint64_t ee = base + holder;
      if (ee < E) {
        const V *src = feat + static_cast<size_t>(r) * Fv;
        V *dst = msg + ee * Fv;
        for (uint32_t c = gl; c < Fv; c += G) {
          V v = src[c];
          if (mode == kAddFromDst) {
            const V o = dst[c];
            float *vf = reinterpret_cast<float *>(&v);
            const float *of = reinterpret_cast<const float *>(&o);
#pragma unroll
            for (int t = 0; t < static_cast<int>(sizeof(V) / 4); ++t) vf[t] = of[t] + vf[t];
          }
          dst[c] = v;
        }
      }
    }
  }
}

// ---- edge -> vertex sums ----------------------------------------------------------------------
//
// Rows with at most `long_limit` edges: a group of G lanes per row (64/G rows per wavefront) adds
// the row's edge rows in order; where the edge rows of consecutive vertices follow each other in
// memory (no permutation), a wavefront streams the edges of a run of rows through LDS instead (same
// sums).  Longer rows (power-law hubs) are listed first and summed by whole
// blocks -- the first blocks of the same launch where the row launch is the balanced kernel, the
// block kernels below otherwise -- which spread a row's edges over the slices of the block and add
// the slices' partial sums in a fixed order.

constexpr uint32_t kNoLimit = 0xFFFFFFFFu;
constexpr uint32_t kLongRowEdges = 1024;    // edges of a row above which the block kernel takes over
constexpr uint64_t kGiantValues = 131072;   // softmax segments above this many values are cut into pieces
constexpr uint64_t kGiantRowEdges = 16384;  // edges of a row above which it is cut into pieces for several blocks
constexpr uint32_t kLongRowValues = 32768;  // the same for softmax segments, in values (edges * heads)
constexpr uint32_t kLongMinVertices = 16384;  // vertex count below which the extra launches are not worth it
constexpr int kLongBlock = 1024;

// out[r,:] (+)= sum_{k in [off[r], off[r+1])} msg[perm ? perm[k] : k, :], added in k order.
template <typename V, int G>
__global__ __launch_bounds__(256) void gather_edge_to_row_kernel(V *__restrict__ out, const V *__restrict__ msg,
                                                                 const uint32_t *__restrict__ off,
                                                                 const uint32_t *__restrict__ perm, uint32_t rows,
                                                                 uint32_t Fv, int accumulate, uint32_t long_limit) {
  const uint32_t r = (blockIdx.x * blockDim.x + threadIdx.x) / G;
  if (r >= rows) return;
  const uint32_t gl = threadIdx.x & (G - 1);
  const uint32_t e0 = off[r], e1 = off[r + 1];
  if (e1 - e0 > long_limit) return;
  constexpr int NF = sizeof(V) / 4;
  for (uint32_t c = gl; c < Fv; c += G) {
    float a[NF];
#pragma unroll
    for (int t = 0; t < NF; ++t) a[t] = 0.f;
    // Eight edge rows are loaded before they are added, in order: the loads overlap, the order of
    // the additions stays the edge order.
    uint32_t k = e0;
    for (; k + 8 <= e1; k += 8) {
      V v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const uint32_t e = perm ? perm[k + u] : k + u;
        v[u] = msg[static_cast<size_t>(e) * Fv + c];
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const float *vf = reinterpret_cast<const float *>(&v[u]);
#pragma unroll
        for (int t = 0; t < NF; ++t) a[t] += vf[t];
      }
    }
    for (; k < e1; ++k) {
      const uint32_t e = perm ? perm[k] : k;
      const V v = msg[static_cast<size_t>(e) * Fv + c];
      const float *vf = reinterpret_cast<const float *>(&v);
#pragma unroll
      for (int t = 0; t < NF; ++t) a[t] += vf[t];
    }
    V *p = out + static_cast<size_t>(r) * Fv + c;
    if (accumulate) {
      const V o = *p;
      const float *of = reinterpret_cast<const float *>(&o);
#pragma unroll
      for (int t = 0; t < NF; ++t) a[t] += of[t];
    }
    V res;
    float *rf = reinterpret_cast<float *>(&res);
#pragma unroll
    for (int t = 0; t < NF; ++t) rf[t] = a[t];
    *p = res;
  }
}

// What the first blocks of a row launch do beside it when the rows above `long_limit` edges are summed
// in the same launch: the list of those rows, the piece table of the giant ones, where the pieces' sums
// go, the column tile of a 256-thread block and how many blocks are set aside (0: none).
template <typename V>
struct LongRowWork {
  const uint32_t *list, *count, *hdr;
  const uint4 *pieces;
  V *partial;
  uint32_t tile, blocks;
};

__device__ __forceinline__ void vadd(float &a, const float &b) { a += b; }
__device__ __forceinline__ void vadd(float4 &a, const float4 &b) {
  a.x += b.x;
  a.y += b.y;
  a.z += b.z;
  a.w += b.w;
}
template <typename V>
__device__ __forceinline__ V vnull();
template <>
__device__ __forceinline__ float vnull<float>() {
  return 0.f;
}
template <>
__device__ __forceinline__ float4 vnull<float4>() {
  return make_float4(0.f, 0.f, 0.f, 0.f);
}

// Sum of the edge rows [e0, e1) by one block of BLOCK threads, added into dst[0 .. Fv) (V = float, or
// float4 when rows are 16-byte aligned: a quarter of the load instructions and of the rounds a row
// takes).  Columns are taken in tiles of `tile` vectors (a power of two <= BLOCK); thread t owns
// column t % tile of slice t / tile, a slice adds every (BLOCK/tile)-th edge of the range in ascending
// order (eight loads in flight), and the slices' sums are then added pairwise in a fixed tree.
template <typename V, int BLOCK>
__device__ __forceinline__ void block_sum_edge_rows(V *__restrict__ dst, const V *__restrict__ msg,
                                                    const uint32_t *__restrict__ perm, uint32_t e0, uint32_t e1,
                                                    uint32_t Fv, uint32_t tile, int accumulate, V *part) {
  const uint32_t c = threadIdx.x & (tile - 1);
  const uint32_t slice = threadIdx.x / tile;
  const uint32_t n_slices = BLOCK / tile;
  for (uint32_t cb = 0; cb < Fv; cb += tile) {
    const uint32_t col = cb + c;
    V a = vnull<V>();
    if (col < Fv) {
      uint32_t k = e0 + slice;
      for (; static_cast<uint64_t>(k) + 7ull * n_slices < e1; k += 8 * n_slices) {
        V v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const uint32_t kk = k + u * n_slices;
          const uint32_t e = perm ? perm[kk] : kk;
          v[u] = msg[static_cast<size_t>(e) * Fv + col];
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) vadd(a, v[u]);
      }
      for (; k < e1; k += n_slices) {
        const uint32_t e = perm ? perm[k] : k;
        vadd(a, msg[static_cast<size_t>(e) * Fv + col]);
      }
    }
    part[threadIdx.x] = a;
    __syncthreads();
    for (uint32_t stride = n_slices / 2; stride >= 1; stride >>= 1) {
      if (slice < stride) {
        V lo = part[threadIdx.x];
        vadd(lo, part[threadIdx.x + stride * tile]);
        part[threadIdx.x] = lo;
      }
      __syncthreads();
    }
    if (slice == 0 && col < Fv) {
      V total = part[c];
      if (accumulate) vadd(total, dst[col]);
      dst[col] = total;
    }
    __syncthreads();
  }
}

// The first blocks of a row launch take the listed long rows, one 256-thread block per row, and the
// pieces of the giant ones (their partial sums are combined by a launch of its own afterwards); the
// rows of the launch proper fill the chip meanwhile.
template <typename V>
__device__ __forceinline__ void sum_long_rows_in_this_block(V *__restrict__ out, const V *__restrict__ msg,
                                                            const uint32_t *__restrict__ off,
                                                            const uint32_t *__restrict__ perm, uint32_t Fv,
                                                            int accumulate, const LongRowWork<V> &lw) {
  __shared__ V long_part[256];
  const uint32_t n_rows = *lw.count;
  for (uint32_t i = blockIdx.x; i < n_rows; i += lw.blocks) {
    const uint32_t r = lw.list[i];
    block_sum_edge_rows<V, 256>(out + static_cast<size_t>(r) * Fv, msg, perm, off[r], off[r + 1], Fv, lw.tile,
                                accumulate, long_part);
  }
  const uint32_t n_pieces = lw.hdr[1];
  for (uint32_t p = blockIdx.x; p < n_pieces; p += lw.blocks) {
    const uint4 pc = lw.pieces[p];
    block_sum_edge_rows<V, 256>(lw.partial + static_cast<size_t>(p) * Fv, msg, perm, pc.z, pc.w, Fv, lw.tile, 0,
                                long_part);
  }
}

// Smallest row r in [0, rows] whose weight before it, (off[r] - off0) + r, is at least x (x at most the
// weight before `rows`, the total), searched by the whole wavefront like owner_of_wave.
__device__ __forceinline__ uint32_t first_row_of_weight(const uint32_t *__restrict__ off, uint32_t rows, uint32_t off0,
                                                        uint64_t x) {
  if (x == 0) return 0;
  const uint32_t lane = threadIdx.x & (kWave - 1);
  const uint64_t pos = x - 1;
  uint32_t lo = 0, hi = rows + 1;  // the largest row whose weight is at most pos lies in [lo, hi)
  while (hi - lo > 1) {
    const uint32_t step = (hi - lo + kWave - 1) / kWave;
    const uint64_t idx = static_cast<uint64_t>(lo) + static_cast<uint64_t>(lane + 1) * step;
    const bool behind = idx < hi && static_cast<uint64_t>(off[idx] - off0) + idx <= pos;
    const uint32_t k = __popcll(__ballot(behind));
    lo += k * step;
    hi = lo + step < hi ? lo + step : hi;
  }
  return lo + 1 < rows ? lo + 1 : rows;  // at most `rows` for ascending offsets; never beyond them for any input
}

// Edge rows that lie one after the other in memory (no permutation: the sums over a destination's
// edges) and are at most one wavefront wide: a wavefront takes 64 consecutive rows, whose edges are one
// contiguous range, and streams that range through a tile of LDS private to it -- all 64 lanes load
// consecutive 4- or 16-byte vectors, the next round is requested before this one is added up -- while
// the lanes that each own one float of an output row (up to four from 32 lanes of 16 bytes on) walk the
// tile edge by edge and write a row out
// where it ends: the running fp32 sum in edge order, as in the kernel below, without a loop per lane
// group and its hand-out of rows.  Rows above `long_limit` edges are skipped (the first blocks of the
// launch sum them); empty rows are written as zeros (or left, when accumulating).
template <typename V, int G>
__global__ __launch_bounds__(256) void gather_edge_to_row_stream_kernel(V *__restrict__ out, const V *__restrict__ msg,
                                                                        const uint32_t *__restrict__ off,
                                                                        uint32_t rows, uint32_t Fv, int accumulate,
                                                                        uint32_t long_limit, LongRowWork<V> lw) {
  if (blockIdx.x < lw.blocks) {
    sum_long_rows_in_this_block(out, msg, off, static_cast<const uint32_t *>(nullptr), Fv, accumulate, lw);
    return;
  }
  constexpr int NF = sizeof(V) / 4;
  constexpr int U = 8;                            // loads per lane and round
  constexpr uint32_t kSlots = kWave / G;          // edge rows per load of the wavefront
  constexpr uint32_t kRound = kSlots * U;         // edge rows per round
  constexpr uint32_t kPitch = G * NF;             // floats of an edge row in the tile
  __shared__ float tiles[4][kWave * U * NF];
  float *tile = tiles[threadIdx.x / kWave];
  const uint32_t lane = lane_id();
  const uint32_t col = lane & (G - 1), slot = lane / G;
  const bool col_live = col < Fv;
  const uint32_t comps = Fv * NF;  // floats of an output row: lane c owns the floats c + 64 k below comps
  constexpr int OWN = (G * NF + kWave - 1) / kWave;  // floats a lane owns at most (1 up to 16 lanes of 16 bytes)
  const uint64_t wave = (static_cast<uint64_t>(blockIdx.x - lw.blocks) * blockDim.x + threadIdx.x) / kWave;
  const uint64_t n_waves = static_cast<uint64_t>(gridDim.x - lw.blocks) * blockDim.x / kWave;
  // The wavefronts share the rows by weight, a row counting one plus its edges: wavefront w takes the
  // rows r with w C <= (off[r] - off[0]) + r < (w + 1) C.
  const uint32_t off0 = off[0];
  const uint64_t total = static_cast<uint64_t>(off[rows] - off0) + rows;
  const uint64_t share = (total + n_waves - 1) / n_waves;
  const uint64_t x0 = wave * share < total ? wave * share : total;
  const uint64_t x1 = x0 + share < total ? x0 + share : total;
  if (x0 == x1) return;
  const uint32_t r_begin = first_row_of_weight(off, rows, off0, x0);
  const uint32_t r_end = first_row_of_weight(off, rows, off0, x1);
  for (uint64_t base = r_begin; base < r_end; base += kWave) {
    const uint32_t n_set = r_end - base < kWave ? static_cast<uint32_t>(r_end - base) : kWave;
    uint32_t my_e1 = 0;
    if (lane < n_set) my_e1 = off[base + lane + 1];
    uint32_t pos = off[base];                       // next edge to add (wave-uniform)
    const uint32_t range_end = wave_read(my_e1, n_set - 1);
    uint32_t j = 0;                                 // current row of the set
    float acc[OWN];
#pragma unroll
    for (int o = 0; o < OWN; ++o) acc[o] = 0.f;
    V cur[U];
    auto load_round = [&](uint32_t k) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        cur[u] = V{};
        const uint32_t idx = k + u * kSlots + slot;
        if (idx < range_end && col_live) cur[u] = msg[static_cast<size_t>(idx) * Fv + col];
      }
    };
    // Rows that end at `pos` are complete: written out (a skipped long row is not), next row.
    auto finish_rows = [&](bool skip_first) {
      bool skip = skip_first;
      while (j < n_set && wave_read(my_e1, j) == pos) {
        if (!skip) {
#pragma unroll
          for (int o = 0; o < OWN; ++o) {
            const uint32_t c = lane + o * kWave;
            if (c < comps) {
              float *p = reinterpret_cast<float *>(out) + (base + j) * comps + c;
              float v = acc[o];
              if (accumulate) v += *p;
              *p = v;
            }
          }
        }
        skip = false;
#pragma unroll
        for (int o = 0; o < OWN; ++o) acc[o] = 0.f;
        ++j;
      }
    };
    finish_rows(false);  // empty rows at the head of the set
    uint32_t loaded = 0xFFFFFFFFu;  // first edge of the round held in `cur`
    while (j < n_set) {
      const uint32_t row_end = wave_read(my_e1, j);
      if (row_end - pos > long_limit) {  // pos is this row's first edge: nothing of it has been added
        pos = row_end;
        finish_rows(true);
        continue;
      }
      const uint32_t ts = pos;  // this round covers [ts, ts + kRound)
      if (loaded != ts) load_round(ts);
      __builtin_amdgcn_wave_barrier();  // the previous round's reads of the tile are done
#pragma unroll
      for (int u = 0; u < U; ++u) reinterpret_cast<V *>(tile)[u * kWave + lane] = cur[u];
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      loaded = ts + kRound;
      if (loaded < range_end) load_round(loaded);  // in flight while this round is added up
      const uint32_t tile_end = range_end - ts < kRound ? range_end : ts + kRound;
      while (pos < tile_end && j < n_set) {
        const uint32_t e1 = wave_read(my_e1, j);
        if (e1 - pos > long_limit) break;  // a long row starts here (a shorter one never has that much left)
        const uint32_t end = e1 < tile_end ? e1 : tile_end;
#pragma unroll
        for (int o = 0; o < OWN; ++o) {
          if (lane + o * kWave < comps) {
            const float *t = tile + (pos - ts) * kPitch + lane + o * kWave;
            float a = acc[o];
            uint32_t i = pos;
            for (; i + 4 <= end; i += 4, t += 4 * kPitch) {
              a += t[0];
              a += t[kPitch];
              a += t[2 * kPitch];
              a += t[3 * kPitch];
            }
            for (; i < end; ++i, t += kPitch) a += t[0];
            acc[o] = a;
          }
        }
        pos = end;
        if (pos == e1) finish_rows(false);
      }
    }
  }
}

// The same sums for rows that fit one group (Fv <= G), with the rows of a wavefront handed out
// dynamically: a wavefront takes 64 consecutive rows, reads their offsets with one coalesced load,
// and its 64/G groups then pull rows from that set one after the other -- a group that finishes a
// short row takes the next pending one instead of idling until the longest row of a fixed
// assignment is done.  Every group adds its row's edge rows in order (eight loads in flight), so
// the result does not depend on which group happened to take which row.
//
// Narrow rows (G * sizeof(V) of 16 to 64 bytes) leave a lone lane or two with the whole row: a
// 1,000-edge row is then 125 dependent rounds of eight loads.  There S slices of G lanes share a
// row: together they load 8 S consecutive edge rows at once, and every lane of the group then adds
// those values in edge order, fetching each from the lane that loaded it.  The sum is the same
// running fp32 sum, bit for bit; only the loads are spread.
//
// Rows of more than `coop_limit` edges (G <= 8 only) are taken by the whole wavefront after the
// set's other rows: all 64 lanes load consecutive edge rows (256 values of type V per round), stage
// them in a tile of LDS private to the wavefront, and request the next round's rows before the
// lanes that each own one float of the output row add the staged values in edge order -- again the
// same running fp32 sum (the tile is padded with zeros, and a sum that starts at +0 is never -0, so
// the padding changes no bit).  A 1,000-edge row of 16-byte values is four such rounds instead of
// sixteen dependent ones.
template <typename V, int G, int S>
__global__ __launch_bounds__(256) void gather_edge_to_row_balanced_kernel(V *__restrict__ out,
                                                                          const V *__restrict__ msg,
                                                                          const uint32_t *__restrict__ off,
                                                                          const uint32_t *__restrict__ perm,
                                                                          uint32_t rows, uint32_t Fv, int accumulate,
                                                                          uint32_t long_limit, uint32_t coop_limit,
                                                                          LongRowWork<V> lw) {
  if (blockIdx.x < lw.blocks) {
    sum_long_rows_in_this_block(out, msg, off, perm, Fv, accumulate, lw);
    return;
  }
  constexpr bool kCoop = G <= 8;
  constexpr int kCoopU = sizeof(V) == 16 ? 4 : 8;           // loads per lane and round on the cooperative path
  constexpr uint32_t kCoopFloats = kWave * kCoopU * (sizeof(V) / 4);  // floats of a wavefront's tile
  __shared__ float coop_tile[kCoop ? 4 : 1][kCoop ? kCoopFloats : 1];
  // Rows a wavefront takes at a time: eight per lane group, so that a wavefront with two groups
  // (128-byte-wide vectors) is not left with 32 rows per group while others have finished.
  constexpr uint32_t kSet = (kWave / (G * S)) * 8 < kWave ? (kWave / (G * S)) * 8 : kWave;
  constexpr int NF = sizeof(V) / 4;
  const uint32_t lane = lane_id();
  constexpr int GG = G * S;  // lanes that share a row
  const uint32_t gl = lane & (GG - 1), grp = lane / GG;
  const uint32_t col = gl & (G - 1), slice = gl / G;
  const uint64_t wave = (static_cast<uint64_t>(blockIdx.x - lw.blocks) * blockDim.x + threadIdx.x) / kWave;
  const uint64_t n_waves = static_cast<uint64_t>(gridDim.x - lw.blocks) * blockDim.x / kWave;
  const bool col_live = col < Fv;
  for (uint64_t base = wave * kSet; base < rows; base += n_waves * kSet) {
    uint32_t my_e0 = 0, my_e1 = 0;
    bool mine = false;
    if (lane < kSet && base + lane < rows) {
      my_e0 = off[base + lane];
      my_e1 = off[base + lane + 1];
      mine = my_e1 - my_e0 <= long_limit;  // longer rows belong to the block kernels
    }
    uint64_t coop = 0;
    if (kCoop) {
      const bool shared = mine && my_e1 - my_e0 > coop_limit;
      coop = __ballot(shared);
      if (shared) mine = false;
    }
    if (G == 1) {
      // Rows one vector wide (the per-head values of an attention layer): a lane sums its own row when
      // the row has at most eight edges -- most rows of a sampled layer's transposed structure -- with
      // the eight loads in flight at once, added in edge order like everywhere else; only the longer
      // rows go through the sharing scheme below.
      const uint32_t deg = my_e1 - my_e0;
      if (mine && deg <= 8u) {
        V v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          v[u] = V{};
          if (static_cast<uint32_t>(u) < deg) {
            const uint32_t e = perm ? perm[my_e0 + u] : my_e0 + u;
            v[u] = msg[e];
          }
        }
        float s1[NF];
#pragma unroll
        for (int t = 0; t < NF; ++t) s1[t] = 0.f;
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          if (static_cast<uint32_t>(u) < deg) {
            const float *vf = reinterpret_cast<const float *>(&v[u]);
#pragma unroll
            for (int t = 0; t < NF; ++t) s1[t] += vf[t];
          }
        }
        V *p = out + (base + lane);
        if (accumulate) {
          const V o = *p;
          const float *of = reinterpret_cast<const float *>(&o);
#pragma unroll
          for (int t = 0; t < NF; ++t) s1[t] += of[t];
        }
        V res;
        float *rf = reinterpret_cast<float *>(&res);
#pragma unroll
        for (int t = 0; t < NF; ++t) rf[t] = s1[t];
        *p = res;
        mine = false;
      }
    }
    uint64_t pending = __ballot(mine);  // rows of this set not handed out yet (wave-uniform)
    bool have = false;
    uint32_t row = 0, k = 0, e1 = 0;
    float a[NF];
    while (true) {
      // Groups without a row take the lowest pending rows, in group order.
      const uint64_t need_mask = __ballot(!have && gl == 0);
      bool took = false;
      if (!have) {
        const uint32_t rank = __popcll(need_mask & ((1ull << (grp * GG)) - 1ull));
        uint64_t m = pending;
        for (uint32_t t = 0; t < rank && m; ++t) m &= m - 1;
        if (m) {
          row = static_cast<uint32_t>(__builtin_ctzll(m));
          took = true;
        }
      }
      const uint32_t from = took ? row : lane;
      const uint32_t new_e0 = __shfl(my_e0, from, kWave), new_e1 = __shfl(my_e1, from, kWave);
      if (took) {
        have = true;
        k = new_e0;
        e1 = new_e1;
#pragma unroll
        for (int t = 0; t < NF; ++t) a[t] = 0.f;
      }
      for (uint32_t t = __popcll(need_mask); t > 0 && pending; --t) pending &= pending - 1;  // handed out
      if (!__ballot(have)) break;
      if (have) {
        // up to 8 S edge rows of this group's row, loaded together (slice s takes the edges s, s + S,
        // ...), added in order
        V v[8];
        const uint32_t n = e1 - k < 8u * S ? e1 - k : 8u * S;
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          v[u] = V{};
          const uint32_t idx = u * S + slice;
          if (idx < n && col_live) {
            const uint32_t e = perm ? perm[k + idx] : k + idx;
            v[u] = msg[static_cast<size_t>(e) * Fv + col];
          }
        }
        if (S == 1) {
#pragma unroll
          for (int u = 0; u < 8; ++u) {
            if (static_cast<uint32_t>(u) < n && col_live) {
              const float *vf = reinterpret_cast<const float *>(&v[u]);
#pragma unroll
              for (int t = 0; t < NF; ++t) a[t] += vf[t];
            }
          }
        } else {
          const uint32_t first = lane - gl + col;  // the lane of slice 0 that holds this lane's column
#pragma unroll
          for (int u = 0; u < 8; ++u) {
            if (!__ballot(static_cast<uint32_t>(u * S) < n)) break;  // no group of the wavefront has edges left
            const float *vf = reinterpret_cast<const float *>(&v[u]);
#pragma unroll
            for (int sl = 0; sl < S; ++sl) {
              float val[NF];
#pragma unroll
              for (int t = 0; t < NF; ++t) val[t] = __shfl(vf[t], first + sl * G, kWave);
              if (static_cast<uint32_t>(u * S + sl) < n) {
#pragma unroll
                for (int t = 0; t < NF; ++t) a[t] += val[t];
              }
            }
          }
        }
        k += n;
        if (k >= e1) {
          if (col_live && slice == 0) {
            V *p = out + (base + row) * Fv + col;
            if (accumulate) {
              const V o = *p;
              const float *of = reinterpret_cast<const float *>(&o);
#pragma unroll
              for (int t = 0; t < NF; ++t) a[t] += of[t];
            }
            V res;
            float *rf = reinterpret_cast<float *>(&res);
#pragma unroll
            for (int t = 0; t < NF; ++t) rf[t] = a[t];
            *p = res;
          }
          have = false;
        }
      }
    }
    if (kCoop) {
      // The long rows of this set, one after the other, by the whole wavefront.
      constexpr uint32_t kSlots = kWave / G;           // edge rows per load of the wavefront
      constexpr uint32_t kRound = kSlots * kCoopU;     // edge rows per round
      constexpr uint32_t kPitch = G * NF;              // floats of an edge row in the tile
      float *tile = coop_tile[threadIdx.x / kWave];
      const uint32_t slot = lane / G;
      const uint32_t comps = Fv * NF;                  // floats of an output row: lane c < comps owns float c
      while (coop) {
        const uint32_t j = static_cast<uint32_t>(__builtin_ctzll(coop));
        coop &= coop - 1;
        const uint32_t r0 = wave_read(my_e0, j), r1 = wave_read(my_e1, j);
        V cur[kCoopU];
        auto load_round = [&](uint32_t k) {
#pragma unroll
          for (int u = 0; u < kCoopU; ++u) {
            cur[u] = V{};
            const uint32_t idx = k + u * kSlots + slot;
            if (idx < r1 && col_live) {
              const uint32_t e = perm ? perm[idx] : idx;
              cur[u] = msg[static_cast<size_t>(e) * Fv + col];
            }
          }
        };
        load_round(r0);
        float acc = 0.f;
        for (uint32_t k = r0; k < r1; k += kRound) {
          __builtin_amdgcn_wave_barrier();  // the previous round's reads of the tile are done
#pragma unroll
          for (int u = 0; u < kCoopU; ++u) reinterpret_cast<V *>(tile)[u * kWave + lane] = cur[u];
          __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
          __builtin_amdgcn_wave_barrier();
          __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
          if (k + kRound < r1) load_round(k + kRound);  // in flight while this round is added up
          const uint32_t n = r1 - k < kRound ? r1 - k : kRound;
          if (lane < comps) {
            for (uint32_t i = 0; i < n; i += 8) {  // whole groups of eight: the tile's tail holds zeros
#pragma unroll
              for (uint32_t t = 0; t < 8; ++t) acc += tile[(i + t) * kPitch + lane];
            }
          }
        }
        if (lane < comps) {
          float *p = reinterpret_cast<float *>(out) + static_cast<size_t>(base + j) * comps + lane;
          if (accumulate) acc += *p;
          *p = acc;
        }
      }
    }
  }
}

// Giant rows: a row so long that one block working through it alone would outlast the rest of the
// launch (a 300,000-edge hub next to 10^4 rows of a few thousand edges) is cut into pieces that
// separate blocks reduce, and a last kernel combines the pieces in order.  The caller's argument
// lists carry no edge count, so everything is sized by fixed capacities and decided on the device:
// up to kGiantCap rows are listed (further ones simply stay with the one-block-per-row kernel), and
// the piece length is chosen so that the listed rows need at most kPieceCap pieces.
constexpr uint32_t kGiantCap = 1024;
constexpr uint32_t kPieceCap = 8192;
constexpr uint32_t kGiantMinPiece = 4096;  // edges

// hdr: [0] giant rows seen (may exceed kGiantCap until the plan kernel clamps it), [1] pieces,
//      [2] edges per piece, [4..5] edges of the listed giant rows (64-bit), [6] the long-row counter
//      (`count` points here, so that one fill clears all of them).
// list[0 .. *count) = rows r with (off[r+1] - off[r]) * width > limit that are not listed as giant
// (any order); giant_rows[0 .. min(hdr[0], kGiantCap)) = rows above giant_limit values.
__global__ __launch_bounds__(256) void collect_long_rows_kernel(uint32_t *__restrict__ list,
                                                                uint32_t *__restrict__ count,
                                                                uint32_t *__restrict__ giant_rows,
                                                                uint32_t *__restrict__ hdr,
                                                                const uint32_t *__restrict__ off, uint32_t rows,
                                                                uint32_t width, uint32_t limit,
                                                                uint64_t giant_limit) {
  const uint32_t r = blockIdx.x * blockDim.x + threadIdx.x;
  if (r >= rows) return;
  const uint32_t deg = off[r + 1] - off[r];
  const uint64_t n = static_cast<uint64_t>(deg) * width;
  if (n > giant_limit) {
    const uint32_t gi = atomicAdd(&hdr[0], 1u);
    if (gi < kGiantCap) {
      giant_rows[gi] = r;
      atomicAdd(reinterpret_cast<unsigned long long *>(hdr + 4), static_cast<unsigned long long>(deg));
      return;
    }
  }
  if (n > limit) list[atomicAdd(count, 1u)] = r;
}

// One block: fixes the piece length, gives every listed giant row its first piece (a serial prefix
// over at most kGiantCap rows) and writes the piece table (list position, row, first edge, end).
__global__ __launch_bounds__(256) void giant_plan_kernel(uint32_t *__restrict__ hdr,
                                                         const uint32_t *__restrict__ giant_rows,
                                                         uint32_t *__restrict__ first, uint4 *__restrict__ pieces,
                                                         const uint32_t *__restrict__ off) {
  __shared__ uint32_t n_sh, len_sh;
  if (threadIdx.x == 0) {
    const uint32_t n = hdr[0] < kGiantCap ? hdr[0] : kGiantCap;
    const unsigned long long edges = *reinterpret_cast<const unsigned long long *>(hdr + 4);
    unsigned long long len = (edges + (kPieceCap - kGiantCap) - 1) / (kPieceCap - kGiantCap);
    if (len < kGiantMinPiece) len = kGiantMinPiece;
    uint32_t p = 0;
    for (uint32_t i = 0; i < n; ++i) {
      first[i] = p;
      const uint32_t r = giant_rows[i];
      p += static_cast<uint32_t>((off[r + 1] - off[r] + len - 1) / len);
    }
    first[n] = p;
    hdr[0] = n;
    hdr[1] = p;
    hdr[2] = static_cast<uint32_t>(len);
    n_sh = n;
    len_sh = static_cast<uint32_t>(len);
  }
  __syncthreads();
  for (uint32_t i = threadIdx.x; i < n_sh; i += blockDim.x) {
    const uint32_t r = giant_rows[i];
    const uint32_t e1 = off[r + 1];
    uint32_t p = first[i];
    for (uint64_t k = off[r]; k < e1; k += len_sh, ++p)
      pieces[p] = make_uint4(i, r, static_cast<uint32_t>(k), static_cast<uint32_t>(k + len_sh < e1 ? k + len_sh : e1));
  }
}

// One 1024-thread block per listed long row.
template <typename V>
__global__ __launch_bounds__(kLongBlock) void gather_edge_to_row_long_kernel(
    V *__restrict__ out, const V *__restrict__ msg, const uint32_t *__restrict__ off,
    const uint32_t *__restrict__ perm, const uint32_t *__restrict__ list, const uint32_t *__restrict__ count,
    uint32_t Fv, uint32_t tile, int accumulate) {
  __shared__ V part[kLongBlock];
  const uint32_t n_rows = *count;
  for (uint32_t i = blockIdx.x; i < n_rows; i += gridDim.x) {
    const uint32_t r = list[i];
    block_sum_edge_rows<V, kLongBlock>(out + static_cast<size_t>(r) * Fv, msg, perm, off[r], off[r + 1], Fv, tile,
                                       accumulate, part);
  }
}

// One block per piece of a giant row: partial[piece, :] = sum of the piece's edge rows.
template <typename V>
__global__ __launch_bounds__(kLongBlock) void giant_sum_pieces_kernel(V *__restrict__ partial,
                                                                      const V *__restrict__ msg,
                                                                      const uint32_t *__restrict__ perm,
                                                                      const uint32_t *__restrict__ hdr,
                                                                      const uint4 *__restrict__ pieces, uint32_t Fv,
                                                                      uint32_t tile) {
  __shared__ V part[kLongBlock];
  const uint32_t n_pieces = hdr[1];
  for (uint32_t p = blockIdx.x; p < n_pieces; p += gridDim.x) {
    const uint4 pc = pieces[p];
    block_sum_edge_rows<V, kLongBlock>(partial + static_cast<size_t>(p) * Fv, msg, perm, pc.z, pc.w, Fv, tile, 0, part);
  }
}

// out[row, :] (+)= the row's piece sums, added in piece order.
__global__ __launch_bounds__(256) void giant_sum_combine_kernel(float *__restrict__ out,
                                                                const float *__restrict__ partial,
                                                                const uint32_t *__restrict__ hdr,
                                                                const uint32_t *__restrict__ giant_rows,
                                                                const uint32_t *__restrict__ first, uint32_t F,
                                                                int accumulate) {
  const uint32_t n = hdr[0];
  for (uint32_t i = blockIdx.x; i < n; i += gridDim.x) {
    const uint32_t r = giant_rows[i];
    const uint32_t p0 = first[i], p1 = first[i + 1];
    for (uint32_t c = threadIdx.x; c < F; c += blockDim.x) {
      float a = 0.f;
      for (uint32_t p = p0; p < p1; ++p) a += partial[static_cast<size_t>(p) * F + c];
      float *dst = out + static_cast<size_t>(r) * F + c;
      *dst = accumulate ? *dst + a : a;
    }
  }
}

// ---- segment softmax --------------------------------------------------------------------------
//
// A destination's scores x[e0*H .. e1*H) are contiguous.  Lane l walks flat positions l, l+64, ...
// When H is a power of two <= 64 a lane always meets the same head (l mod H), so the per-head
// maximum and sum are a lane-local reduction followed by a butterfly over the lanes that share a
// head (xor masks 32 .. H).  Other head counts take one strided pass per head.

template <int MODE>  // 0 = max, 1 = sum
__device__ __forceinline__ float head_reduce(float v, uint32_t H) {
  for (uint32_t m = kWave / 2; m >= H; m >>= 1) {
    const float o = __shfl_xor(v, m, kWave);
    v = MODE == 0 ? fmaxf(v, o) : v + o;
  }
  return v;
}

__device__ __forceinline__ float leaky(float s, float slope) { return s > 0.f ? s : s * slope; }

// exp for the softmax kernels: the hardware's 2^x of x * log2(e), two instructions instead of the
// fourteen of the correctly rounded library routine -- these kernels are bound by their vector
// instructions for short segments.  Arguments are <= 0 (a value minus its segment's maximum); the
// product's rounding puts the relative error at |x| * 6e-8 (1e-6 at x = -20, where the result is
// 2e-9 of the segment's largest term), well inside the 1e-4 these operators are held to.
__device__ __forceinline__ float softmax_exp(float x) { return __expf(x); }

// Multi-pass softmax forward of one segment with 16-byte lanes (H a multiple of 4, 16-byte aligned
// arrays): lane l of a group of WIDTH threads takes the vectors l, l + WIDTH, ... of the segment, i.e.
// four consecutive values = heads (4 l mod H) .. +3 of one edge, so a pass needs a quarter of the load
// rounds of the 4-byte version.  `load4(i)` fetches vector i (for the fused form: the four scores of
// its edge), `keep4(i, v)` may store it.  Leaves per-component running (max, sum) pairs in mx / sum.
template <int U, typename Load4, typename Keep4>
__device__ __forceinline__ void strided_max_sum_pass4(uint64_t first, uint64_t nv, uint64_t stride, Load4 load4,
                                                      Keep4 keep4, float (&mx)[4], float (&sum)[4]) {
  auto fold = [&](const float4 *v, int count) {
    float m[4] = {mx[0], mx[1], mx[2], mx[3]};
    for (int u = 0; u < count; ++u) {
      m[0] = fmaxf(m[0], v[u].x);
      m[1] = fmaxf(m[1], v[u].y);
      m[2] = fmaxf(m[2], v[u].z);
      m[3] = fmaxf(m[3], v[u].w);
    }
    float add[4] = {0.f, 0.f, 0.f, 0.f};
    for (int u = 0; u < count; ++u) {
      add[0] += softmax_exp(v[u].x - m[0]);
      add[1] += softmax_exp(v[u].y - m[1]);
      add[2] += softmax_exp(v[u].z - m[2]);
      add[3] += softmax_exp(v[u].w - m[3]);
    }
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      sum[c] = sum[c] * softmax_exp(mx[c] - m[c]) + add[c];  // mx = -inf at the start: the old sum is 0 and stays 0
      mx[c] = m[c];
    }
  };
  uint64_t i = first;
  for (; i + (U - 1) * stride < nv; i += U * stride) {
    float4 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) v[u] = load4(i + u * stride);
#pragma unroll
    for (int u = 0; u < U; ++u) keep4(i + u * stride, v[u]);
    fold(v, U);
  }
  for (; i < nv; i += stride) {
    const float4 v = load4(i);
    keep4(i, v);
    fold(&v, 1);
  }
}

// Three kernels share a launch, by segment size n = degree * H (values):
//   short   n <= 128, power-of-two H <= 16: a group of 16 lanes per destination, the segment held
//           in registers -- one pass over memory, four destinations per wavefront in flight;
//   wave    up to kLongRowValues (or any size when the block kernel is not used): one wavefront per
//           destination; segments of at most 512 values are register-resident too, larger ones take
//           the three passes (max, sum, write) / two passes (dot, write) over memory;
//   block   longer segments (hub destinations), listed by collect_long_rows.
// The short and the wave kernel stride over the destinations (a wavefront of the wave kernel looks
// at 64 destinations at a time and visits only those that fall in its size class), so their launch
// size does not grow with the vertex count.

constexpr int kShortG = 16;        // lanes per destination in the short kernel
constexpr int kShortK = 8;         // values per lane held in registers there
constexpr uint32_t kShortValues = kShortG * kShortK;
constexpr int kWaveK = 8;          // values per lane the wave kernel can hold in registers
constexpr uint32_t kWaveRegValues = kWave * kWaveK;
constexpr uint32_t kWaveMidValues = kWave * 32;  // the fused forward's launch for the class above that: 32 per lane

// One strided pass over a segment with U loads in flight: positions first, first + stride, ...
// below n; `load(i)` fetches, `use(i, v)` consumes, in ascending position order.
template <int U, typename Load, typename Use>
__device__ __forceinline__ void strided_pass(uint64_t first, uint64_t n, uint64_t stride, Load load, Use use) {
  uint64_t i = first;
  for (; i + (U - 1) * stride < n; i += U * stride) {
    decltype(load(i)) v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) v[u] = load(i + u * stride);
#pragma unroll
    for (int u = 0; u < U; ++u) use(i + u * stride, v[u]);
  }
  for (; i < n; i += stride) use(i, load(i));
}

// One strided pass that leaves a running (maximum, sum of exp(v - maximum)) pair, so that the maximum
// and the sum of a segment come out of a single read.  The U values in flight are folded in together:
// their maximum first, then one rescale of the old sum and U independent exponentials.
template <int U, typename Load, typename Seen>
__device__ __forceinline__ void strided_max_sum_pass(uint64_t first, uint64_t n, uint64_t stride, Load load,
                                                     Seen seen, float &mx, float &sum) {
  uint64_t i = first;
  for (; i + (U - 1) * stride < n; i += U * stride) {
    float v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) v[u] = load(i + u * stride);
    float m = mx;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      seen(i + u * stride, v[u]);
      m = fmaxf(m, v[u]);
    }
    float add = 0.f;
#pragma unroll
    for (int u = 0; u < U; ++u) add += softmax_exp(v[u] - m);
    sum = sum * softmax_exp(mx - m) + add;  // mx = -inf at the start: the old sum is 0 and stays 0
    mx = m;
  }
  for (; i < n; i += stride) {
    const float v = load(i);
    seen(i, v);
    const float m = fmaxf(mx, v);
    sum = sum * softmax_exp(mx - m) + softmax_exp(v - m);
    mx = m;
  }
}

// Reduction over the lanes of an aligned group of WIDTH lanes that share a head (lane mod H).
template <int MODE, int WIDTH>  // 0 = max, 1 = sum
__device__ __forceinline__ float head_reduce_w(float v, uint32_t H) {
  for (uint32_t m = WIDTH / 2; m >= H; m >>= 1) {
    const float o = __shfl_xor(v, m, WIDTH);
    v = MODE == 0 ? fmaxf(v, o) : v + o;
  }
  return v;
}

// Register-resident forward of one segment by WIDTH lanes (lane index gl), K values per lane;
// n <= WIDTH*K values, H a power of two <= WIDTH.
template <bool FUSED, int WIDTH, int K>
__device__ __forceinline__ void softmax_fwd_regs(float *__restrict__ ys, const float *__restrict__ xs,
                                                 const float *__restrict__ el, const float *__restrict__ er,
                                                 const uint32_t *__restrict__ ri, uint32_t d, uint32_t e0, uint32_t n,
                                                 uint32_t H, float slope, uint32_t gl) {
  const uint32_t h = gl & (H - 1);
  float erv = 0.f;
  if (FUSED) erv = er[static_cast<size_t>(d) * H + h];
  float v[K];
  float mx = -INFINITY;
#pragma unroll
  for (int k = 0; k < K; ++k) {
    const uint32_t i = gl + WIDTH * k;
    v[k] = -INFINITY;
    if (i < n) {
      if (FUSED) {
        const uint32_t src = ri[e0 + i / H];
        v[k] = leaky(el[static_cast<size_t>(src) * H + h] + erv, slope);
      } else {
        v[k] = xs[i];
      }
    }
    mx = fmaxf(mx, v[k]);
  }
  mx = head_reduce_w<0, WIDTH>(mx, H);
  float sum = 0.f;
#pragma unroll
  for (int k = 0; k < K; ++k) {
    v[k] = (gl + WIDTH * k < n) ? softmax_exp(v[k] - mx) : 0.f;
    sum += v[k];
  }
  sum = head_reduce_w<1, WIDTH>(sum, H);
  const float inv = 1.f / sum;  // one division per lane instead of one per value
#pragma unroll
  for (int k = 0; k < K; ++k) {
    const uint32_t i = gl + WIDTH * k;
    if (i < n) ys[i] = v[k] * inv;
  }
}

// Register-resident backward, same shape.  Writes ger[d, :] when FUSED (zeros for an empty segment).
template <bool FUSED, int WIDTH, int K>
__device__ __forceinline__ void softmax_bwd_regs(float *__restrict__ gxs, float *__restrict__ ger,
                                                 const float *__restrict__ gys, const float *__restrict__ ys,
                                                 const float *__restrict__ el, const float *__restrict__ er,
                                                 const uint32_t *__restrict__ ri, uint32_t d, uint32_t e0, uint32_t n,
                                                 uint32_t H, float slope, uint32_t gl) {
  const uint32_t h = gl & (H - 1);
  float yv[K], gv[K];
  float dot = 0.f;
#pragma unroll
  for (int k = 0; k < K; ++k) {
    const uint32_t i = gl + WIDTH * k;
    yv[k] = 0.f;
    gv[k] = 0.f;
    if (i < n) {
      yv[k] = ys[i];
      gv[k] = gys[i];
    }
    dot += gv[k] * yv[k];
  }
  dot = head_reduce_w<1, WIDTH>(dot, H);
  float erv = 0.f, gsum = 0.f;
  if (FUSED) erv = er[static_cast<size_t>(d) * H + h];
#pragma unroll
  for (int k = 0; k < K; ++k) {
    const uint32_t i = gl + WIDTH * k;
    if (i < n) {
      float g = yv[k] * (gv[k] - dot);
      if (FUSED) {
        const uint32_t src = ri[e0 + i / H];
        const float pre = el[static_cast<size_t>(src) * H + h] + erv;
        g *= pre > 0.f ? 1.f : slope;
        gsum += g;
      }
      gxs[i] = g;
    }
  }
  if (FUSED) {
    gsum = head_reduce_w<1, WIDTH>(gsum, H);
    if (gl < H) ger[static_cast<size_t>(d) * H + gl] = gsum;
  }
}

// These kernels are bound by their vector instructions, not by memory (253 per 256-value segment
// were counted, a wave64 instruction holding its SIMD for four cycles: 80 % of the launch time), and
// most of them served register slots beyond the segment's end.  The register paths are therefore
// instantiated for 1, 2, 4 and 8 slots per lane and called with the smallest count that covers
// every segment the wavefront is working on (`n`, the caller's segment size, must be in scope).
#define NTS_BY_SLOTS(WIDTH, FN, ...)                                        \
  do {                                                                      \
    if (!any_lane(n > 4u * (WIDTH))) {                                      \
      if (!any_lane(n > 2u * (WIDTH))) {                                    \
        if (!any_lane(n > 1u * (WIDTH))) FN<FUSED, WIDTH, 1>(__VA_ARGS__);  \
        else FN<FUSED, WIDTH, 2>(__VA_ARGS__);                              \
      } else {                                                              \
        FN<FUSED, WIDTH, 4>(__VA_ARGS__);                                   \
      }                                                                     \
    } else {                                                                \
      FN<FUSED, WIDTH, 8>(__VA_ARGS__);                                     \
    }                                                                       \
  } while (0)

// True if `pred` holds on any active lane of the wavefront.
__device__ __forceinline__ bool any_lane(bool pred) { return __ballot(pred) != 0; }

// Short segments (n <= kShortValues; power-of-two H <= kShortG): a group of kShortG lanes per
// destination, striding over the destinations.  BWD selects the backward formula.
// A segment of any length by one group of kShortG lanes, with plain strided passes (the safety net of a
// launch that was told no segment exceeds the short class: correct, not fast).
template <bool FUSED, bool BWD>
__device__ void softmax_group_any(float *__restrict__ outs, float *__restrict__ ger, const float *__restrict__ xs,
                                  const float *__restrict__ ys, const float *__restrict__ el,
                                  const float *__restrict__ er, const uint32_t *__restrict__ ri, uint32_t d,
                                  uint32_t e0, uint64_t n, uint32_t H, float slope, uint32_t gl) {
  const uint32_t h = gl & (H - 1);
  const float erv = FUSED ? er[static_cast<size_t>(d) * H + h] : 0.f;
  auto score = [&](uint64_t i) {
    if (!FUSED) return xs[i];
    return leaky(el[static_cast<size_t>(ri[e0 + i / H]) * H + h] + erv, slope);
  };
  if (!BWD) {
    float mx = -INFINITY;
    for (uint64_t i = gl; i < n; i += kShortG) mx = fmaxf(mx, score(i));
    mx = head_reduce_w<0, kShortG>(mx, H);
    float sum = 0.f;
    for (uint64_t i = gl; i < n; i += kShortG) sum += softmax_exp(score(i) - mx);
    sum = head_reduce_w<1, kShortG>(sum, H);
    const float inv = 1.f / sum;
    for (uint64_t i = gl; i < n; i += kShortG) outs[i] = softmax_exp(score(i) - mx) * inv;
  } else {
    float dot = 0.f;
    for (uint64_t i = gl; i < n; i += kShortG) dot += xs[i] * ys[i];
    dot = head_reduce_w<1, kShortG>(dot, H);
    float gsum = 0.f;
    for (uint64_t i = gl; i < n; i += kShortG) {
      float g = ys[i] * (xs[i] - dot);
      if (FUSED) {
        const float pre = el[static_cast<size_t>(ri[e0 + i / H]) * H + h] + erv;
        g *= pre > 0.f ? 1.f : slope;
        gsum += g;
      }
      outs[i] = g;
    }
    if (FUSED) {
      gsum = head_reduce_w<1, kShortG>(gsum, H);
      if (gl < H) ger[static_cast<size_t>(d) * H + gl] = gsum;
    }
  }
}

// ALL: the launch is the only one of its call (the caller bounded every segment by the short class), so
// a segment beyond the class is not skipped but computed by the group with plain strided passes.
template <bool FUSED, bool BWD, bool ALL = false>
__global__ __launch_bounds__(256) void edge_softmax_short_kernel(float *__restrict__ out, float *__restrict__ ger,
                                                                 const float *__restrict__ x_or_gy,
                                                                 const float *__restrict__ y,
                                                                 const float *__restrict__ el,
                                                                 const float *__restrict__ er,
                                                                 const uint32_t *__restrict__ co,
                                                                 const uint32_t *__restrict__ ri, uint32_t Vd,
                                                                 uint32_t H, float slope) {
  const uint32_t gl = threadIdx.x & (kShortG - 1);
  const uint64_t n_groups = static_cast<uint64_t>(gridDim.x) * (256 / kShortG);
  for (uint64_t d64 = (static_cast<uint64_t>(blockIdx.x) * 256 + threadIdx.x) / kShortG; d64 < Vd; d64 += n_groups) {
    const uint32_t d = static_cast<uint32_t>(d64);
    const uint32_t e0 = co[d], e1 = co[d + 1];
    const uint64_t n64 = static_cast<uint64_t>(e1 - e0) * H;
    const size_t base = static_cast<size_t>(e0) * H;
    if (n64 > kShortValues) {  // the whole group takes the same way
      if (ALL)
        softmax_group_any<FUSED, BWD>(out + base, ger, x_or_gy ? x_or_gy + base : nullptr, y ? y + base : nullptr, el, er,
                                      ri, d, e0, n64, H, slope, gl);
      continue;
    }
    const uint32_t n = static_cast<uint32_t>(n64);
    if (BWD) {
      if (FUSED) {  // the four instances together would cost this kernel a wavefront per SIMD
        softmax_bwd_regs<FUSED, kShortG, kShortK>(out + base, ger, x_or_gy + base, y + base, el, er, ri, d, e0, n, H,
                                                  slope, gl);
      } else {
        NTS_BY_SLOTS(kShortG, softmax_bwd_regs, out + base, ger, x_or_gy + base, y + base, el, er, ri, d, e0, n, H,
                     slope, gl);
      }
    } else {
      if (n == 0) continue;
      NTS_BY_SLOTS(kShortG, softmax_fwd_regs, out + base, FUSED ? nullptr : x_or_gy + base, el, er, ri, d, e0, n, H,
                   slope, gl);
    }
  }
}

// The destinations of [base, base + 64) whose segment size lies in [min_values, max_values], as a
// wave-uniform bit mask; every lane keeps the offsets of its own destination for the visit.
__device__ __forceinline__ uint64_t wave_rows_in_class(const uint32_t *__restrict__ co, uint32_t Vd, uint64_t base,
                                                       uint32_t H, uint32_t min_values, uint32_t max_values,
                                                       uint32_t &my_e0, uint32_t &my_e1) {
  const uint64_t d = base + lane_id();
  my_e0 = 0;
  my_e1 = 0;
  bool mine = false;
  if (d < Vd) {
    my_e0 = co[d];
    my_e1 = co[d + 1];
    const uint64_t n = static_cast<uint64_t>(my_e1 - my_e0) * H;
    mine = n >= min_values && n <= max_values;
  }
  return __ballot(mine);
}

// FUSED = false: y = softmax_seg(x).   FUSED = true: x is ignored and the score is
// leaky_relu(el[ri[e],h] + er[d,h], slope); in the three-pass path y first holds the raw score, then
// alpha.  Visits the destinations with min_values <= n <= max_values.
// PART: 0 = every segment size in one launch; 1 = the register-resident segments only, 2 = the
// longer ones only, 3 = segments of 513 .. 2,048 values held 16 or 32 per lane in registers -- launches
// of their own, each instance allotted the registers of its own path.  The fused form is launched in
// parts: its longer segments read el[src] with 16-byte lanes, which costs registers that the short
// ones should not pay for (Products-shaped graph: 3.05 -> 2.82 ms), and the class between them is
// still one pass over memory instead of writing raw scores and reading them back (2.76 -> 2.65 ms); for
// the plain softmax one launch is as fast as two or three (every variant runs at the rate of a copy).
template <bool FUSED, bool POW2, int PART>
__global__ __launch_bounds__(256) void edge_softmax_fwd_kernel(float *__restrict__ y, const float *__restrict__ x,
                                                               const float *__restrict__ el,
                                                               const float *__restrict__ er,
                                                               const uint32_t *__restrict__ co,
                                                               const uint32_t *__restrict__ ri, uint32_t Vd,
                                                               uint32_t H, float slope, uint32_t min_values,
                                                               uint32_t max_values, uint32_t vec4) {
  const uint32_t lane = lane_id();
  const uint64_t wave = (static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x) / kWave;
  const uint64_t n_waves = static_cast<uint64_t>(gridDim.x) * blockDim.x / kWave;
  for (uint64_t first = wave * kWave; first < Vd; first += n_waves * kWave) {
    uint32_t my_e0, my_e1;
    uint64_t todo = wave_rows_in_class(co, Vd, first, H, min_values < 1 ? 1 : min_values, max_values, my_e0, my_e1);
    while (todo) {
      const uint32_t j = static_cast<uint32_t>(__builtin_ctzll(todo));
      todo &= todo - 1;
      const uint32_t d = static_cast<uint32_t>(first) + j;
      const uint32_t e0 = wave_read(my_e0, j), e1 = wave_read(my_e1, j);
      const size_t base = static_cast<size_t>(e0) * H;
      const uint32_t n = (e1 - e0) * H;
      float *ys = y + base;
      const float *xs = FUSED ? nullptr : x + base;

      if (POW2) {
        if (PART <= 1 && n <= kWaveRegValues) {
          NTS_BY_SLOTS(kWave, softmax_fwd_regs, ys, xs, el, er, ri, d, e0, n, H, slope, lane);
          continue;
        }
        if (PART == 1) continue;
        if (PART == 3) {  // 513 .. 2,048 values: still one pass, 16 or 32 values per lane in registers
          if (n <= 16u * kWave) softmax_fwd_regs<FUSED, kWave, 16>(ys, xs, el, er, ri, d, e0, n, H, slope, lane);
          else softmax_fwd_regs<FUSED, kWave, 32>(ys, xs, el, er, ri, d, e0, n, H, slope, lane);
          continue;
        }
        if (PART == 2 && vec4 && n >= 2048u) {  // at least two full rounds of four vectors per lane
          const uint32_t h0 = (lane * 4u) & (H - 1);  // head of this lane's first value; 256 k = 0 mod H
          const uint32_t hq = H / 4;                  // lanes hq apart hold the same heads
          float4 erv = make_float4(0.f, 0.f, 0.f, 0.f);
          if (FUSED) erv = *reinterpret_cast<const float4 *>(er + static_cast<size_t>(d) * H + h0);
          const float4 *xs4 = reinterpret_cast<const float4 *>(xs);
          float4 *ys4 = reinterpret_cast<float4 *>(ys);
          float mx4[4] = {-INFINITY, -INFINITY, -INFINITY, -INFINITY}, sum4[4] = {0.f, 0.f, 0.f, 0.f};
          strided_max_sum_pass4<4>(
              lane, n / 4, kWave,
              [&](uint64_t i) -> float4 {
                if (!FUSED) return xs4[i];
                const uint32_t src = ri[e0 + static_cast<uint32_t>(i * 4 / H)];
                const float4 e = *reinterpret_cast<const float4 *>(el + static_cast<size_t>(src) * H + h0);
                return make_float4(leaky(e.x + erv.x, slope), leaky(e.y + erv.y, slope), leaky(e.z + erv.z, slope),
                                   leaky(e.w + erv.w, slope));
              },
              [&](uint64_t i, float4 sc) {
                if (FUSED) ys4[i] = sc;
              },
              mx4, sum4);
          float inv4[4];
#pragma unroll
          for (int c = 0; c < 4; ++c) {
            const float lane_mx = mx4[c];
            mx4[c] = head_reduce<0>(mx4[c], hq);
            sum4[c] = head_reduce<1>(sum4[c] * softmax_exp(lane_mx - mx4[c]), hq);
            inv4[c] = 1.f / sum4[c];
          }
          strided_pass<4>(lane, n / 4, kWave, [&](uint64_t i) -> float4 { return FUSED ? ys4[i] : xs4[i]; },
                          [&](uint64_t i, float4 sc) {
                            ys4[i] = make_float4(softmax_exp(sc.x - mx4[0]) * inv4[0], softmax_exp(sc.y - mx4[1]) * inv4[1],
                                                 softmax_exp(sc.z - mx4[2]) * inv4[2], softmax_exp(sc.w - mx4[3]) * inv4[3]);
                          });
          continue;
        }
        const uint32_t h = lane & (H - 1);
        float erv = 0.f;
        if (FUSED) erv = er[static_cast<size_t>(d) * H + h];
        float mx = -INFINITY, sum = 0.f;
        strided_max_sum_pass<8>(
            lane, n, kWave,
            [&](uint64_t i) -> float {
              if (!FUSED) return xs[i];
              const uint32_t src = ri[e0 + i / H];
              return leaky(el[static_cast<size_t>(src) * H + h] + erv, slope);
            },
            [&](uint64_t i, float sc) {
              if (FUSED) ys[i] = sc;
            },
            mx, sum);
        // every lane's pair is brought to the head's maximum before the sums are added
        const float lane_mx = mx;
        mx = head_reduce<0>(mx, H);
        sum = head_reduce<1>(sum * softmax_exp(lane_mx - mx), H);
        const float inv = 1.f / sum;
        strided_pass<8>(lane, n, kWave, [&](uint64_t i) -> float { return FUSED ? ys[i] : xs[i]; },
                        [&](uint64_t i, float sc) { ys[i] = softmax_exp(sc - mx) * inv; });
      } else {
        const uint32_t deg = e1 - e0;
        for (uint32_t h = 0; h < H; ++h) {
          float erv = 0.f;
          if (FUSED) erv = er[static_cast<size_t>(d) * H + h];
          float mx = -INFINITY;
          for (uint32_t k = lane; k < deg; k += kWave) {
            float sc;
            if (FUSED) {
              const uint32_t src = ri[e0 + k];
              sc = leaky(el[static_cast<size_t>(src) * H + h] + erv, slope);
              ys[static_cast<size_t>(k) * H + h] = sc;
            } else {
              sc = xs[static_cast<size_t>(k) * H + h];
            }
            mx = fmaxf(mx, sc);
          }
          mx = group_max<kWave>(mx);
          float sum = 0.f;
          for (uint32_t k = lane; k < deg; k += kWave) {
            const float sc = FUSED ? ys[static_cast<size_t>(k) * H + h] : xs[static_cast<size_t>(k) * H + h];
            sum += softmax_exp(sc - mx);
          }
          sum = group_sum<kWave>(sum);
          const float inv = 1.f / sum;
          for (uint32_t k = lane; k < deg; k += kWave) {
            const float sc = FUSED ? ys[static_cast<size_t>(k) * H + h] : xs[static_cast<size_t>(k) * H + h];
            ys[static_cast<size_t>(k) * H + h] = softmax_exp(sc - mx) * inv;
          }
        }
      }
    }
  }
}

// FUSED = false: gx = y * (gy - sum_seg gy*y).
// FUSED = true : additionally multiplies by leaky_relu'(el[src]+er[d]) and writes
//                ger[d,h] = sum_seg gx[e,h].
// Visits the destinations with min_values <= n <= max_values (empty segments included when
// min_values is 0, so that ger is written for every destination).
// PART as in the forward kernel: the fused form is launched in two parts.
template <bool FUSED, bool POW2, int PART>
__global__ __launch_bounds__(256) void edge_softmax_bwd_kernel(float *__restrict__ gx, float *__restrict__ ger,
                                                               const float *__restrict__ gy,
                                                               const float *__restrict__ y,
                                                               const float *__restrict__ el,
                                                               const float *__restrict__ er,
                                                               const uint32_t *__restrict__ co,
                                                               const uint32_t *__restrict__ ri, uint32_t Vd,
                                                               uint32_t H, float slope, uint32_t min_values,
                                                               uint32_t max_values, uint32_t vec4) {
  const uint32_t lane = lane_id();
  const uint64_t wave = (static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x) / kWave;
  const uint64_t n_waves = static_cast<uint64_t>(gridDim.x) * blockDim.x / kWave;
  for (uint64_t first = wave * kWave; first < Vd; first += n_waves * kWave) {
    uint32_t my_e0, my_e1;
    uint64_t todo = wave_rows_in_class(co, Vd, first, H, min_values, max_values, my_e0, my_e1);
    while (todo) {
      const uint32_t j = static_cast<uint32_t>(__builtin_ctzll(todo));
      todo &= todo - 1;
      const uint32_t d = static_cast<uint32_t>(first) + j;
      const uint32_t e0 = wave_read(my_e0, j), e1 = wave_read(my_e1, j);
      const size_t base = static_cast<size_t>(e0) * H;
      const uint32_t n = (e1 - e0) * H;
      const float *gys = gy + base;
      const float *ys = y + base;
      float *gxs = gx + base;

      if (POW2) {
        if (PART <= 1 && n <= kWaveRegValues) {
          NTS_BY_SLOTS(kWave, softmax_bwd_regs, gxs, ger, gys, ys, el, er, ri, d, e0, n, H, slope, lane);
          continue;
        }
        if (PART == 1) continue;

        if (PART == 2 && FUSED && vec4 && n >= 2048u) {
          // 16-byte lanes: four consecutive values = heads (4 lane mod H) .. +3 of one edge
          const uint32_t h0 = (lane * 4u) & (H - 1);
          const uint32_t hq = H / 4;
          const float4 *gys4 = reinterpret_cast<const float4 *>(gys);
          const float4 *ys4 = reinterpret_cast<const float4 *>(ys);
          float4 *gxs4 = reinterpret_cast<float4 *>(gxs);
          float dot4[4] = {0.f, 0.f, 0.f, 0.f};
          strided_pass<4>(lane, n / 4, kWave, [&](uint64_t i) -> float4 { return gys4[i]; },
                          [&](uint64_t i, float4 g) {
                            const float4 a = ys4[i];
                            dot4[0] += g.x * a.x;
                            dot4[1] += g.y * a.y;
                            dot4[2] += g.z * a.z;
                            dot4[3] += g.w * a.w;
                          });
#pragma unroll
          for (int c = 0; c < 4; ++c) dot4[c] = head_reduce<1>(dot4[c], hq);
          const float4 erv = *reinterpret_cast<const float4 *>(er + static_cast<size_t>(d) * H + h0);
          float gsum4[4] = {0.f, 0.f, 0.f, 0.f};
          strided_pass<4>(lane, n / 4, kWave,
                          [&](uint64_t i) -> float4 {
                            const uint32_t src = ri[e0 + static_cast<uint32_t>(i * 4 / H)];
                            return *reinterpret_cast<const float4 *>(el + static_cast<size_t>(src) * H + h0);
                          },
                          [&](uint64_t i, float4 e) {
                            const float4 g = gys4[i], a = ys4[i];
                            float4 r;
                            r.x = a.x * (g.x - dot4[0]) * (e.x + erv.x > 0.f ? 1.f : slope);
                            r.y = a.y * (g.y - dot4[1]) * (e.y + erv.y > 0.f ? 1.f : slope);
                            r.z = a.z * (g.z - dot4[2]) * (e.z + erv.z > 0.f ? 1.f : slope);
                            r.w = a.w * (g.w - dot4[3]) * (e.w + erv.w > 0.f ? 1.f : slope);
                            gsum4[0] += r.x;
                            gsum4[1] += r.y;
                            gsum4[2] += r.z;
                            gsum4[3] += r.w;
                            gxs4[i] = r;
                          });
#pragma unroll
          for (int c = 0; c < 4; ++c) gsum4[c] = head_reduce<1>(gsum4[c], hq);
          if (lane < hq) {
            *reinterpret_cast<float4 *>(ger + static_cast<size_t>(d) * H + h0) =
                make_float4(gsum4[0], gsum4[1], gsum4[2], gsum4[3]);
          }
          continue;
        }
        const uint32_t h = lane & (H - 1);
        float dot = 0.f;
        strided_pass<8>(lane, n, kWave, [&](uint64_t i) -> float2 { return make_float2(gys[i], ys[i]); },
                        [&](uint64_t, float2 v) { dot += v.x * v.y; });
        dot = head_reduce<1>(dot, H);
        float erv = 0.f, gsum = 0.f;
        if (FUSED) erv = er[static_cast<size_t>(d) * H + h];
        strided_pass<8>(lane, n, kWave,
                        [&](uint64_t i) -> float4 {
                          float pre = 1.f;
                          if (FUSED) pre = el[static_cast<size_t>(ri[e0 + i / H]) * H + h] + erv;
                          return make_float4(gys[i], ys[i], pre, 0.f);
                        },
                        [&](uint64_t i, float4 v) {
                          float g = v.y * (v.x - dot);
                          if (FUSED) {
                            g *= v.z > 0.f ? 1.f : slope;
                            gsum += g;
                          }
                          gxs[i] = g;
                        });
        if (FUSED) {
          gsum = head_reduce<1>(gsum, H);
          if (lane < H) ger[static_cast<size_t>(d) * H + lane] = gsum;
        }
      } else {
        const uint32_t deg = e1 - e0;
        for (uint32_t h = 0; h < H; ++h) {
          float dot = 0.f;
          for (uint32_t k = lane; k < deg; k += kWave) {
            const size_t i = static_cast<size_t>(k) * H + h;
            dot += gys[i] * ys[i];
          }
          dot = group_sum<kWave>(dot);
          float erv = 0.f, gsum = 0.f;
          if (FUSED) erv = er[static_cast<size_t>(d) * H + h];
          for (uint32_t k = lane; k < deg; k += kWave) {
            const size_t i = static_cast<size_t>(k) * H + h;
            float g = ys[i] * (gys[i] - dot);
            if (FUSED) {
              const uint32_t src = ri[e0 + k];
              const float pre = el[static_cast<size_t>(src) * H + h] + erv;
              g *= pre > 0.f ? 1.f : slope;
              gsum += g;
            }
            gxs[i] = g;
          }
          if (FUSED) {
            gsum = group_sum<kWave>(gsum);
            if (lane == 0) ger[static_cast<size_t>(d) * H + h] = gsum;
          }
        }
      }
    }
  }
}

// Block kernels for long segments (power-of-two H <= 64 only; other head counts stay on the wave
// kernels).  1024 threads walk the segment's values; thread t always meets head t mod H.  Per-head
// maxima / sums are reduced inside each wave with the head butterfly, then across the 16 waves
// through LDS in wave order.
template <int MODE>  // 0 = max, 1 = sum
__device__ __forceinline__ float block_head_reduce(float v, uint32_t H, float (*red)[kWave]) {
  const uint32_t lane = lane_id(), wave = threadIdx.x / kWave;
  v = head_reduce<MODE>(v, H);
  if (lane < H) red[wave][lane] = v;
  __syncthreads();
  const uint32_t h = lane & (H - 1);
  float r = red[0][h];
  for (uint32_t wv = 1; wv < kLongBlock / kWave; ++wv) r = MODE == 0 ? fmaxf(r, red[wv][h]) : r + red[wv][h];
  __syncthreads();
  return r;
}

template <bool FUSED>
__global__ __launch_bounds__(kLongBlock) void edge_softmax_fwd_long_kernel(
    float *__restrict__ y, const float *__restrict__ x, const float *__restrict__ el, const float *__restrict__ er,
    const uint32_t *__restrict__ co, const uint32_t *__restrict__ ri, const uint32_t *__restrict__ list,
    const uint32_t *__restrict__ count, uint32_t H, float slope) {
  __shared__ float red[kLongBlock / kWave][kWave];
  const uint32_t n_rows = *count;
  const uint32_t h = threadIdx.x & (H - 1);
  for (uint32_t i = blockIdx.x; i < n_rows; i += gridDim.x) {
    const uint32_t d = list[i];
    const uint32_t e0 = co[d], e1 = co[d + 1];
    const size_t base = static_cast<size_t>(e0) * H;
    const size_t n = static_cast<size_t>(e1 - e0) * H;
    float *ys = y + base;
    const float *xs = FUSED ? nullptr : x + base;
    float erv = 0.f;
    if (FUSED) erv = er[static_cast<size_t>(d) * H + h];
    float mx = -INFINITY, sum = 0.f;
    strided_max_sum_pass<8>(
        threadIdx.x, n, kLongBlock,
        [&](uint64_t j) -> float {
          if (!FUSED) return xs[j];
          const uint32_t src = ri[e0 + j / H];
          return leaky(el[static_cast<size_t>(src) * H + h] + erv, slope);
        },
        [&](uint64_t j, float sc) {
          if (FUSED) ys[j] = sc;
        },
        mx, sum);
    const float thread_mx = mx;
    mx = block_head_reduce<0>(mx, H, red);
    sum = block_head_reduce<1>(sum * softmax_exp(thread_mx - mx), H, red);
    const float inv = 1.f / sum;
    strided_pass<8>(threadIdx.x, n, kLongBlock, [&](uint64_t j) -> float { return FUSED ? ys[j] : xs[j]; },
                    [&](uint64_t j, float sc) { ys[j] = softmax_exp(sc - mx) * inv; });
  }
}

template <bool FUSED>
__global__ __launch_bounds__(kLongBlock) void edge_softmax_bwd_long_kernel(
    float *__restrict__ gx, float *__restrict__ ger, const float *__restrict__ gy, const float *__restrict__ y,
    const float *__restrict__ el, const float *__restrict__ er, const uint32_t *__restrict__ co,
    const uint32_t *__restrict__ ri, const uint32_t *__restrict__ list, const uint32_t *__restrict__ count, uint32_t H,
    float slope) {
  __shared__ float red[kLongBlock / kWave][kWave];
  const uint32_t n_rows = *count;
  const uint32_t h = threadIdx.x & (H - 1);
  for (uint32_t i = blockIdx.x; i < n_rows; i += gridDim.x) {
    const uint32_t d = list[i];
    const uint32_t e0 = co[d], e1 = co[d + 1];
    const size_t base = static_cast<size_t>(e0) * H;
    const size_t n = static_cast<size_t>(e1 - e0) * H;
    const float *gys = gy + base;
    const float *ys = y + base;
    float *gxs = gx + base;
    float dot = 0.f;
    strided_pass<8>(threadIdx.x, n, kLongBlock, [&](uint64_t j) -> float2 { return make_float2(gys[j], ys[j]); },
                    [&](uint64_t, float2 v) { dot += v.x * v.y; });
    dot = block_head_reduce<1>(dot, H, red);
    float erv = 0.f, gsum = 0.f;
    if (FUSED) erv = er[static_cast<size_t>(d) * H + h];
    strided_pass<8>(threadIdx.x, n, kLongBlock,
                    [&](uint64_t j) -> float4 {
                      float pre = 1.f;
                      if (FUSED) pre = el[static_cast<size_t>(ri[e0 + j / H]) * H + h] + erv;
                      return make_float4(gys[j], ys[j], pre, 0.f);
                    },
                    [&](uint64_t j, float4 v) {
                      float g = v.y * (v.x - dot);
                      if (FUSED) {
                        g *= v.z > 0.f ? 1.f : slope;
                        gsum += g;
                      }
                      gxs[j] = g;
                    });
    if (FUSED) {
      gsum = block_head_reduce<1>(gsum, H, red);
      if (threadIdx.x < H) ger[static_cast<size_t>(d) * H + threadIdx.x] = gsum;
    }
  }
}

// ---- giant segments of the softmax operators ----------------------------------------------------
//
// A piece of a giant destination is reduced by one block; per-head results of the pieces are
// combined in piece order.  Forward uses the online form: a piece keeps (m_p, s_p = sum exp(x - m_p));
// the destination's maximum is max_p m_p and its sum is sum_p s_p * exp(m_p - m).
// stats[piece, 0..H) / [H..2H) and rowstat[giant row, 0..H) / [H..2H) hold the two values per head.

template <bool FUSED>
__global__ __launch_bounds__(kLongBlock) void giant_softmax_stats_kernel(
    float *__restrict__ stats, float *__restrict__ y, const float *__restrict__ x, const float *__restrict__ el,
    const float *__restrict__ er, const uint32_t *__restrict__ ri, const uint32_t *__restrict__ hdr,
    const uint4 *__restrict__ pieces, uint32_t H, float slope) {
  __shared__ float red[kLongBlock / kWave][kWave];
  const uint32_t n_pieces = hdr[1];
  const uint32_t h = threadIdx.x & (H - 1);
  for (uint32_t p = blockIdx.x; p < n_pieces; p += gridDim.x) {
    const uint4 pc = pieces[p];
    const uint32_t d = pc.y, e0 = pc.z;
    const size_t base = static_cast<size_t>(e0) * H;
    const uint64_t n = static_cast<uint64_t>(pc.w - e0) * H;
    float *ys = y + base;
    const float *xs = FUSED ? nullptr : x + base;
    float erv = 0.f;
    if (FUSED) erv = er[static_cast<size_t>(d) * H + h];
    float mx = -INFINITY;
    strided_pass<8>(threadIdx.x, n, kLongBlock,
                    [&](uint64_t j) -> float {
                      if (!FUSED) return xs[j];
                      const uint32_t src = ri[e0 + j / H];
                      return leaky(el[static_cast<size_t>(src) * H + h] + erv, slope);
                    },
                    [&](uint64_t j, float sc) {
                      if (FUSED) ys[j] = sc;
                      mx = fmaxf(mx, sc);
                    });
    mx = block_head_reduce<0>(mx, H, red);
    float sum = 0.f;
    strided_pass<8>(threadIdx.x, n, kLongBlock, [&](uint64_t j) -> float { return FUSED ? ys[j] : xs[j]; },
                    [&](uint64_t, float sc) { sum += softmax_exp(sc - mx); });
    sum = block_head_reduce<1>(sum, H, red);
    if (threadIdx.x < H) {
      stats[static_cast<size_t>(p) * 2 * H + threadIdx.x] = mx;
      stats[static_cast<size_t>(p) * 2 * H + H + threadIdx.x] = sum;
    }
  }
}

// MODE 0: online-softmax combine of (m_p, s_p).  MODE 1: plain sum of stats[piece, 0..H) in piece
// order; the result goes to rowstat[giant row, 0..H) or, when `to_rows` is set, to to_rows[row, 0..H)
// (the per-destination gradient sum of the fused backward).
template <int MODE>
__global__ __launch_bounds__(64) void giant_softmax_combine_kernel(float *__restrict__ rowstat,
                                                                   float *__restrict__ to_rows,
                                                                   const float *__restrict__ stats,
                                                                   const uint32_t *__restrict__ hdr,
                                                                   const uint32_t *__restrict__ giant_rows,
                                                                   const uint32_t *__restrict__ first, uint32_t H) {
  const uint32_t n = hdr[0];
  const uint32_t h = threadIdx.x;
  if (h >= H) return;
  const uint32_t width = MODE == 0 ? 2 * H : H;
  for (uint32_t i = blockIdx.x; i < n; i += gridDim.x) {
    const uint32_t p0 = first[i], p1 = first[i + 1];
    if (MODE == 0) {
      float m = -INFINITY;
      for (uint32_t p = p0; p < p1; ++p) m = fmaxf(m, stats[static_cast<size_t>(p) * width + h]);
      float sum = 0.f;
      for (uint32_t p = p0; p < p1; ++p)
        sum += stats[static_cast<size_t>(p) * width + H + h] * softmax_exp(stats[static_cast<size_t>(p) * width + h] - m);
      rowstat[static_cast<size_t>(i) * 2 * H + h] = m;
      rowstat[static_cast<size_t>(i) * 2 * H + H + h] = sum;
    } else {
      float sum = 0.f;
      for (uint32_t p = p0; p < p1; ++p) sum += stats[static_cast<size_t>(p) * width + h];
      if (to_rows) to_rows[static_cast<size_t>(giant_rows[i]) * H + h] = sum;
      else rowstat[static_cast<size_t>(i) * 2 * H + h] = sum;
    }
  }
}

template <bool FUSED>
__global__ __launch_bounds__(kLongBlock) void giant_softmax_apply_kernel(float *__restrict__ y,
                                                                         const float *__restrict__ x,
                                                                         const float *__restrict__ rowstat,
                                                                         const uint32_t *__restrict__ hdr,
                                                                         const uint4 *__restrict__ pieces,
                                                                         uint32_t H) {
  const uint32_t n_pieces = hdr[1];
  const uint32_t h = threadIdx.x & (H - 1);
  for (uint32_t p = blockIdx.x; p < n_pieces; p += gridDim.x) {
    const uint4 pc = pieces[p];
    const size_t base = static_cast<size_t>(pc.z) * H;
    const uint64_t n = static_cast<uint64_t>(pc.w - pc.z) * H;
    const float mx = rowstat[static_cast<size_t>(pc.x) * 2 * H + h];
    const float sum = rowstat[static_cast<size_t>(pc.x) * 2 * H + H + h];
    float *ys = y + base;
    const float *xs = FUSED ? ys : x + base;  // the fused forward left the raw score in y
    const float inv = 1.f / sum;
    strided_pass<8>(threadIdx.x, n, kLongBlock, [&](uint64_t j) -> float { return xs[j]; },
                    [&](uint64_t j, float sc) { ys[j] = softmax_exp(sc - mx) * inv; });
  }
}

// Backward, first stage: stats[piece, h] = sum over the piece of gy * y.
__global__ __launch_bounds__(kLongBlock) void giant_softmax_dot_kernel(float *__restrict__ stats,
                                                                       const float *__restrict__ gy,
                                                                       const float *__restrict__ y,
                                                                       const uint32_t *__restrict__ hdr,
                                                                       const uint4 *__restrict__ pieces, uint32_t H) {
  __shared__ float red[kLongBlock / kWave][kWave];
  const uint32_t n_pieces = hdr[1];
  for (uint32_t p = blockIdx.x; p < n_pieces; p += gridDim.x) {
    const uint4 pc = pieces[p];
    const size_t base = static_cast<size_t>(pc.z) * H;
    const uint64_t n = static_cast<uint64_t>(pc.w - pc.z) * H;
    const float *gys = gy + base;
    const float *ys = y + base;
    float dot = 0.f;
    strided_pass<8>(threadIdx.x, n, kLongBlock, [&](uint64_t j) -> float2 { return make_float2(gys[j], ys[j]); },
                    [&](uint64_t, float2 v) { dot += v.x * v.y; });
    dot = block_head_reduce<1>(dot, H, red);
    if (threadIdx.x < H) stats[static_cast<size_t>(p) * H + threadIdx.x] = dot;
  }
}

// Backward, last stage: gx over the piece; with FUSED also stats[piece, h] = sum of the piece's gx.
template <bool FUSED>
__global__ __launch_bounds__(kLongBlock) void giant_softmax_bwd_apply_kernel(
    float *__restrict__ gx, float *__restrict__ stats, const float *__restrict__ gy, const float *__restrict__ y,
    const float *__restrict__ el, const float *__restrict__ er, const uint32_t *__restrict__ ri,
    const float *__restrict__ rowstat, const uint32_t *__restrict__ hdr, const uint4 *__restrict__ pieces, uint32_t H,
    float slope) {
  __shared__ float red[kLongBlock / kWave][kWave];
  const uint32_t n_pieces = hdr[1];
  const uint32_t h = threadIdx.x & (H - 1);
  for (uint32_t p = blockIdx.x; p < n_pieces; p += gridDim.x) {
    const uint4 pc = pieces[p];
    const uint32_t d = pc.y, e0 = pc.z;
    const size_t base = static_cast<size_t>(e0) * H;
    const uint64_t n = static_cast<uint64_t>(pc.w - e0) * H;
    const float *gys = gy + base;
    const float *ys = y + base;
    float *gxs = gx + base;
    const float dot = rowstat[static_cast<size_t>(pc.x) * 2 * H + h];
    float erv = 0.f, gsum = 0.f;
    if (FUSED) erv = er[static_cast<size_t>(d) * H + h];
    strided_pass<8>(threadIdx.x, n, kLongBlock,
                    [&](uint64_t j) -> float4 {
                      float pre = 1.f;
                      if (FUSED) pre = el[static_cast<size_t>(ri[e0 + j / H]) * H + h] + erv;
                      return make_float4(gys[j], ys[j], pre, 0.f);
                    },
                    [&](uint64_t j, float4 v) {
                      float g = v.y * (v.x - dot);
                      if (FUSED) {
                        g *= v.z > 0.f ? 1.f : slope;
                        gsum += g;
                      }
                      gxs[j] = g;
                    });
    if (FUSED) {
      gsum = block_head_reduce<1>(gsum, H, red);
      if (threadIdx.x < H) stats[static_cast<size_t>(p) * H + threadIdx.x] = gsum;
    }
  }
}

// ---- gradient of the attention-weighted aggregation with respect to alpha ----------------------
//
// galpha[e,h] = < in[ri[e], h-th slice], gout[d, h-th slice] > for e in CSC(d).  Edge-parallel like
// the copies: 64 consecutive edges per wave step, (source, owner) looked up per lane.

// Fast path: G = (H*Fh)/VEC lanes cover one edge's row (G a power of two <= 64), the Fh/VEC lanes of
// a head add their products with an xor butterfly.  A wave step takes 64 consecutive edges and each
// of the 64/G lane groups G consecutive ones of them, so a group's destination changes rarely and
// its gout row stays in registers until it does: one gathered row per edge instead of two.
template <int VEC>
__global__ __launch_bounds__(256) void sddmm_edge_kernel(float *__restrict__ galpha, const float *__restrict__ in,
                                                         const float *__restrict__ gout,
                                                         const uint32_t *__restrict__ co,
                                                         const uint32_t *__restrict__ ri, uint32_t Vd, uint32_t H,
                                                         uint32_t Fh, uint32_t G, uint32_t lanes_per_head) {
  const uint32_t E = co[Vd];
  const uint32_t F = H * Fh;
  const uint32_t lane = lane_id();
  const uint32_t gl = lane & (G - 1), grp = lane / G;
  const uint64_t wave = (static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x) / kWave;
  const uint64_t n_waves = static_cast<uint64_t>(gridDim.x) * blockDim.x / kWave;
  uint32_t d_held = 0xFFFFFFFFu;
  float4 y4 = make_float4(0.f, 0.f, 0.f, 0.f);
  float y1 = 0.f;
  // A wavefront walks a contiguous span of wave steps, so that the owner of each step's edges is
  // found from the previous step's instead of by a search per lane.
  const uint64_t total_steps = (static_cast<uint64_t>(E) + kWave - 1) / kWave;
  const uint64_t per_wave = (total_steps + n_waves - 1) / n_waves;
  const uint64_t first_step = wave * per_wave;
  const uint64_t end_step = first_step + per_wave < total_steps ? first_step + per_wave : total_steps;
  if (first_step >= end_step) return;
  uint32_t d0 = owner_of_wave(co, Vd, static_cast<uint32_t>(first_step * kWave));
  for (uint64_t step = first_step; step < end_step; ++step) {
    const uint64_t base = step * kWave;
    const uint64_t e = base + lane;
    const uint32_t own = owners_of_step(co, Vd, static_cast<uint32_t>(base), d0);
    const uint32_t src = e < E ? ri[e] : 0u;
    // Eight edges at a time: their gathered rows -- and the destination rows of the edges at which the
    // destination changes -- are requested before the first is used (four measure the same on a whole
    // graph; on a sampled layer of 410 k edges, where the launch is a few dependent rounds long, eight
    // take the mini-batch epoch's backward stage from 8.2 to 8.0 ms).
    constexpr uint32_t U = 8;
    for (uint32_t j0 = 0; j0 < G; j0 += U) {
      uint32_t d[U];
      bool valid[U], fresh[U];
      float4 x4[U], w4[U];
      float x1[U], w1[U];
#pragma unroll
      for (uint32_t u = 0; u < U; ++u) {
        const uint32_t holder = grp * G + j0 + u;
        const uint32_t s = __shfl(src, holder & (kWave - 1), kWave);
        d[u] = __shfl(own, holder & (kWave - 1), kWave);
        valid[u] = j0 + u < G && base + holder < E;
        fresh[u] = valid[u] && d[u] != (u ? d[u - 1] : d_held);  // an edge is valid only if the one before it is
        x4[u] = w4[u] = make_float4(0.f, 0.f, 0.f, 0.f);
        x1[u] = w1[u] = 0.f;
        if (valid[u]) {
          const float *a = in + static_cast<size_t>(s) * F + gl * VEC;
          if (VEC == 4) x4[u] = *reinterpret_cast<const float4 *>(a); else x1[u] = a[0];
        }
        if (fresh[u]) {
          const float *b = gout + static_cast<size_t>(d[u]) * F + gl * VEC;
          if (VEC == 4) w4[u] = *reinterpret_cast<const float4 *>(b); else w1[u] = b[0];
        }
      }
#pragma unroll
      for (uint32_t u = 0; u < U; ++u) {
        float p = 0.f;
        if (valid[u]) {
          if (fresh[u]) {
            if (VEC == 4) y4 = w4[u]; else y1 = w1[u];
            d_held = d[u];
          }
          p = VEC == 4 ? fmaf(x4[u].w, y4.w, fmaf(x4[u].z, y4.z, fmaf(x4[u].y, y4.y, x4[u].x * y4.x))) : x1[u] * y1;
        }
        for (uint32_t m = lanes_per_head / 2; m >= 1; m >>= 1) p += __shfl_xor(p, m, kWave);
        if (valid[u] && (gl & (lanes_per_head - 1)) == 0)
          galpha[(base + grp * G + j0 + u) * H + gl / lanes_per_head] = p;
      }
    }
  }
}

// General shapes: the 64 edges of a step are taken one after the other; for each edge and head the
// lanes stride over the head's slice and a full-wave butterfly adds the partial products.
__global__ __launch_bounds__(256) void sddmm_edge_generic_kernel(float *__restrict__ galpha,
                                                                 const float *__restrict__ in,
                                                                 const float *__restrict__ gout,
                                                                 const uint32_t *__restrict__ co,
                                                                 const uint32_t *__restrict__ ri, uint32_t Vd,
                                                                 uint32_t H, uint32_t Fh) {
  const uint32_t E = co[Vd];
  const uint32_t F = H * Fh;
  const uint32_t lane = lane_id();
  const uint64_t wave = (static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x) / kWave;
  const uint64_t n_waves = static_cast<uint64_t>(gridDim.x) * blockDim.x / kWave;
  for (uint64_t base = wave * kWave; base < E; base += n_waves * kWave) {
    const uint64_t e = base + lane;
    uint32_t src = 0, own = 0;
    if (e < E) {
      src = ri[e];
      own = owner_of(co, Vd, static_cast<uint32_t>(e));
    }
    const uint32_t n = static_cast<uint32_t>(min(static_cast<uint64_t>(kWave), E - base));
    for (uint32_t j = 0; j < n; ++j) {
      const float *a = in + static_cast<size_t>(wave_read(src, j)) * F;
      const float *b = gout + static_cast<size_t>(wave_read(own, j)) * F;
      for (uint32_t h = 0; h < H; ++h) {
        float p = 0.f;
        for (uint32_t f = lane; f < Fh; f += kWave) p = fmaf(a[h * Fh + f], b[h * Fh + f], p);
        p = group_sum<kWave>(p);
        if (lane == 0) galpha[(base + j) * H + h] = p;
      }
    }
  }
}

inline bool is_pow2(uint32_t v) { return v && !(v & (v - 1)); }

}  // namespace
}  // namespace nts

using namespace nts;

namespace {
// Grid for the edge-parallel kernels: the edge count lives on the device, so the grid is sized from
// the vertex count (assuming a few dozen edges per vertex) and the kernels stride over the edges.
inline dim3 edge_grid(uint32_t Vd) {
  uint64_t blocks = (static_cast<uint64_t>(Vd) * 32 + 255) / 256;
  if (blocks < 64) blocks = 64;
  if (blocks > 8192) blocks = 8192;
  return dim3(static_cast<unsigned>(blocks));
}

// Lanes per row for a row of Fv vector elements: the smallest power of two >= Fv, at most 64.
inline int lanes_for(uint32_t Fv) {
  int g = 1;
  while (g < 64 && static_cast<uint32_t>(g) < Fv) g <<= 1;
  return g;
}

template <typename V>
void launch_edge_copy(V *msg, const V *feat, const uint32_t *ri, const uint32_t *co, const uint32_t *mirror,
                      uint32_t Vd, uint32_t Fv, int mode, hipStream_t stream) {
  const dim3 grid = edge_grid(Vd), block(256);
#define NTS_COPY(GG)                                                                                              \
  hipLaunchKernelGGL((edge_copy_kernel<V, GG>), grid, block, 0, stream, msg, feat, ri, co, mirror, Vd, Fv, mode)
  switch (lanes_for(Fv)) {
    case 1: NTS_COPY(1); break;
    case 2: NTS_COPY(2); break;
    case 4: NTS_COPY(4); break;
    case 8: NTS_COPY(8); break;
    case 16: NTS_COPY(16); break;
    case 32: NTS_COPY(32); break;
    default: NTS_COPY(64); break;
  }
#undef NTS_COPY
}

int edge_copy_impl(float *msg, const float *feat, const uint32_t *ri, const uint32_t *co, const uint32_t *mirror,
                   uint32_t Vd, uint32_t F, int mode, hipStream_t stream, const char *who) {
  if (F == 0) return fail(NTS_ERR_INVALID, who);
  if (Vd == 0) return NTS_OK;
  if (!msg || !feat || !co || (mode == kFromSrc && !ri)) return fail(NTS_ERR_INVALID, who);
  if (F % 4 == 0 && aligned_to(msg, 16) && aligned_to(feat, 16))
    launch_edge_copy(reinterpret_cast<float4 *>(msg), reinterpret_cast<const float4 *>(feat), ri, co, mirror, Vd,
                     F / 4, mode, stream);
  else
    launch_edge_copy(msg, feat, ri, co, mirror, Vd, F, mode, stream);
  NTS_LAUNCH_CHECK(who);
  return NTS_OK;
}

// Scratch of the long-row path in one stream-ordered allocation: list[rows], its counter, and the
// tables of the giant rows (header, row list, first-piece prefix, piece table).
struct LongRows {
  ScratchBlock block;  // owns the allocation: returned to the pool on every way out of the caller
  uint32_t *list = nullptr;
  uint32_t *count = nullptr;
  uint32_t *hdr = nullptr;
  uint32_t *giant_rows = nullptr;
  uint32_t *first = nullptr;
  uint4 *pieces = nullptr;
};

// Collects the rows whose segment holds more than `limit` values (edges * width) when the vertex
// count makes hubs likely, the ones above `giant_limit` values separately (with their piece table);
// returns with lr.list == nullptr when the long path is not used.
int collect_long_rows(LongRows &lr, const uint32_t *off, uint32_t rows, uint32_t width, uint32_t limit,
                      uint64_t giant_limit, hipStream_t stream) {
  if (rows < kLongMinVertices) return NTS_OK;
  const size_t list_bytes = (static_cast<size_t>(rows) + 7) / 8 * 8 * sizeof(uint32_t);  // list, 32-byte multiple
  const size_t small_bytes = (8 + kGiantCap + kGiantCap + 8) * sizeof(uint32_t);         // hdr (with the counter), rows, first
  NTS_HIP_TRY(lr.block.alloc(list_bytes + small_bytes + kPieceCap * sizeof(uint4), stream));
  unsigned char *buf = static_cast<unsigned char *>(lr.block.ptr);
  lr.list = reinterpret_cast<uint32_t *>(buf);
  lr.hdr = reinterpret_cast<uint32_t *>(buf + list_bytes);
  lr.count = lr.hdr + 6;
  lr.giant_rows = lr.hdr + 8;
  lr.first = lr.giant_rows + kGiantCap;
  lr.pieces = reinterpret_cast<uint4 *>(buf + list_bytes + small_bytes);
  if (int rc = nts_memset_zero(lr.hdr, 8 * sizeof(uint32_t), stream)) return rc;  // counters and the ticket
  hipLaunchKernelGGL(collect_long_rows_kernel, dim3(ceil_div(rows, 256)), dim3(256), 0, stream, lr.list, lr.count,
                     lr.giant_rows, lr.hdr, off, rows, width, limit, giant_limit);
  NTS_LAUNCH_CHECK("collect_long_rows_kernel");
  hipLaunchKernelGGL(giant_plan_kernel, dim3(1), dim3(256), 0, stream, lr.hdr, lr.giant_rows, lr.first, lr.pieces, off);
  NTS_LAUNCH_CHECK("giant_plan_kernel");
  return NTS_OK;
}

int release_long_rows(LongRows &lr) {
  lr.list = nullptr;
  NTS_HIP_TRY(lr.block.release());
  return NTS_OK;
}

constexpr unsigned kLongGrid = 512;  // blocks of the long-row kernels; they stride over the list

// Edges of a row above which the whole wavefront takes it (rows up to eight lanes wide); NTS_EDGE_SUM_COOP
// in the environment overrides it (0 = never).
uint32_t coop_limit() {
  static const uint32_t value = [] {
    const char *env = getenv("NTS_EDGE_SUM_COOP");
    if (!env) return 64u;
    const long v = atol(env);
    return v <= 0 ? kNoLimit : static_cast<uint32_t>(v);
  }();
  return value;
}

// Blocks of a row launch set aside for the long rows when they are summed in the same launch: as many
// threads as the long-row kernels of their own bring (512 blocks of 1,024).
constexpr uint32_t kMergedLongBlocks = 2048;
// NTS_EDGE_SUM_MERGE in the environment: 0 = long rows always in launches of their own; n > 0 = that many
// blocks of the row launch for them.
uint32_t merged_long_blocks() {
  static const uint32_t value = [] {
    const char *env = getenv("NTS_EDGE_SUM_MERGE");
    if (!env) return kMergedLongBlocks;
    const long v = atol(env);
    return v <= 0 ? 0u : static_cast<uint32_t>(v);
  }();
  return value;
}

// The row launch whose first blocks also sum the long rows: one-group rows of a vertex set large enough.
bool rows_launch_takes_long_rows(uint32_t rows, uint32_t Fv) { return Fv <= 64 && rows >= 4096; }

// NTS_EDGE_SUM_STREAM=0 in the environment: contiguous edge rows take the lane-group kernel like permuted ones.
bool stream_contiguous_rows() {
  static const bool value = [] {
    const char *env = getenv("NTS_EDGE_SUM_STREAM");
    return !(env && atol(env) == 0);
  }();
  return value;
}

template <typename V>
void launch_gather_rows(V *out, const V *msg, const uint32_t *off, const uint32_t *perm, uint32_t rows, uint32_t Fv,
                        int accumulate, uint32_t limit, const LongRowWork<V> &lw, hipStream_t stream) {
  if (rows_launch_takes_long_rows(rows, Fv) && !perm && stream_contiguous_rows()) {
    // a wavefront streams the contiguous edges of 64 rows at a time
    const uint32_t blocks = ceil_div(rows, 4 * kWave);
    const dim3 grid((blocks < 16384u ? blocks : 16384u) + lw.blocks);
#define NTS_STREAM(GG)                                                                                          \
  hipLaunchKernelGGL((gather_edge_to_row_stream_kernel<V, GG>), grid, dim3(256), 0, stream, out, msg, off, rows, Fv, \
                     accumulate, limit, lw)
    switch (lanes_for(Fv)) {
      case 1: NTS_STREAM(1); break;
      case 2: NTS_STREAM(2); break;
      case 4: NTS_STREAM(4); break;
      case 8: NTS_STREAM(8); break;
      case 16: NTS_STREAM(16); break;
      case 32: NTS_STREAM(32); break;
      default: NTS_STREAM(64); break;
    }
#undef NTS_STREAM
    return;
  }
  if (rows_launch_takes_long_rows(rows, Fv)) {
    // One group covers a row: wavefronts hand their 64 rows out dynamically (strided launch).
#define NTS_BALANCED(GG, SS)                                                                                    \
  do {                                                                                                          \
    const uint32_t set = (kWave / ((GG) * (SS))) * 8 < kWave ? (kWave / ((GG) * (SS))) * 8 : kWave;            \
    const uint32_t blocks = ceil_div(rows, 4 * set); /* at most `set` rows per wavefront at a time */          \
    hipLaunchKernelGGL((gather_edge_to_row_balanced_kernel<V, GG, SS>),                                         \
                       dim3((blocks < 16384u ? blocks : 16384u) + lw.blocks), dim3(256), 0, stream, out, msg, off, \
                       perm, rows, Fv, accumulate, limit, coop_limit(), lw);                                    \
  } while (0)
    switch (lanes_for(Fv)) {  // rows narrower than eight lanes are shared by eight lanes all the same
      case 1: NTS_BALANCED(1, 8); break;
      case 2: NTS_BALANCED(2, 4); break;
      case 4: NTS_BALANCED(4, 2); break;
      case 8: NTS_BALANCED(8, 1); break;
      case 16: NTS_BALANCED(16, 1); break;
      case 32: NTS_BALANCED(32, 1); break;
      default: NTS_BALANCED(64, 1); break;
    }
#undef NTS_BALANCED
    return;
  }
#define NTS_GATHER(GG)                                                                                          \
  hipLaunchKernelGGL((gather_edge_to_row_kernel<V, GG>), dim3(ceil_div(static_cast<uint64_t>(rows) * GG, 256)),  \
                     dim3(256), 0, stream, out, msg, off, perm, rows, Fv, accumulate, limit)
  switch (lanes_for(Fv)) {
    case 1: NTS_GATHER(1); break;
    case 2: NTS_GATHER(2); break;
    case 4: NTS_GATHER(4); break;
    case 8: NTS_GATHER(8); break;
    case 16: NTS_GATHER(16); break;
    case 32: NTS_GATHER(32); break;
    default: NTS_GATHER(64); break;
  }
#undef NTS_GATHER
}

int gather_edge_impl(float *out, const float *msg, const uint32_t *off, const uint32_t *perm, uint32_t rows,
                     uint32_t F, int accumulate, hipStream_t stream, const char *who) {
  if (F == 0) return fail(NTS_ERR_INVALID, who);
  if (rows == 0) return NTS_OK;
  if (!out || !msg || !off) return fail(NTS_ERR_INVALID, who);
  LongRows lr;
  if (int rc = collect_long_rows(lr, off, rows, 1u, kLongRowEdges, kGiantRowEdges, stream)) return rc;
  const uint32_t limit = lr.list ? kLongRowEdges : kNoLimit;
  // 16-byte vectors for the row kernels and the block kernels alike
  const bool v4 = F % 4 == 0 && aligned_to(out, 16) && aligned_to(msg, 16);
  const uint32_t Fv = v4 ? F / 4 : F;
  // Long rows: in the first blocks of the row launch where that launch has them (256-thread blocks),
  // else in launches of their own after it (1,024-thread blocks).  Giant rows: pieces by separate
  // blocks into stream-ordered scratch, then the ordered combine.
  const bool merged = lr.list && rows_launch_takes_long_rows(rows, Fv) && merged_long_blocks() > 0;
  const uint32_t block_threads = merged ? 256u : static_cast<uint32_t>(kLongBlock);
  uint32_t tile = 1;
  while (tile < Fv && tile < block_threads) tile <<= 1;
  ScratchBlock partial_block;
  float *partial = nullptr;
  if (lr.list) {
    NTS_HIP_TRY(partial_block.alloc(static_cast<size_t>(kPieceCap) * F * sizeof(float), stream));
    partial = static_cast<float *>(partial_block.ptr);
  }
  if (v4) {
    LongRowWork<float4> lw{lr.list, lr.count, lr.hdr, lr.pieces, reinterpret_cast<float4 *>(partial), tile,
                           merged ? merged_long_blocks() : 0u};
    launch_gather_rows(reinterpret_cast<float4 *>(out), reinterpret_cast<const float4 *>(msg), off, perm, rows, Fv,
                       accumulate, limit, lw, stream);
  } else {
    LongRowWork<float> lw{lr.list, lr.count, lr.hdr, lr.pieces, partial, tile, merged ? merged_long_blocks() : 0u};
    launch_gather_rows(out, msg, off, perm, rows, Fv, accumulate, limit, lw, stream);
  }
  hipError_t launch_err = hipGetLastError();
  if (lr.list && launch_err == hipSuccess) {
    if (!merged) {
      if (v4) {
        hipLaunchKernelGGL(gather_edge_to_row_long_kernel<float4>, dim3(kLongGrid), dim3(kLongBlock), 0, stream,
                           reinterpret_cast<float4 *>(out), reinterpret_cast<const float4 *>(msg), off, perm, lr.list,
                           lr.count, Fv, tile, accumulate);
        hipLaunchKernelGGL(giant_sum_pieces_kernel<float4>, dim3(kLongGrid), dim3(kLongBlock), 0, stream,
                           reinterpret_cast<float4 *>(partial), reinterpret_cast<const float4 *>(msg), perm, lr.hdr,
                           lr.pieces, Fv, tile);
      } else {
        hipLaunchKernelGGL(gather_edge_to_row_long_kernel<float>, dim3(kLongGrid), dim3(kLongBlock), 0, stream, out, msg,
                           off, perm, lr.list, lr.count, Fv, tile, accumulate);
        hipLaunchKernelGGL(giant_sum_pieces_kernel<float>, dim3(kLongGrid), dim3(kLongBlock), 0, stream, partial, msg,
                           perm, lr.hdr, lr.pieces, Fv, tile);
      }
    }
    hipLaunchKernelGGL(giant_sum_combine_kernel, dim3(kGiantCap / 4), dim3(256), 0, stream, out, partial, lr.hdr,
                       lr.giant_rows, lr.first, F, accumulate);
    launch_err = hipGetLastError();
  }
  if (lr.list) NTS_HIP_TRY(partial_block.release());
  if (launch_err != hipSuccess) {
    (void)release_long_rows(lr);
    return fail_hip(launch_err, who);
  }
  return release_long_rows(lr);
}

// A second stream per host thread and device, for launches that a call runs beside those on the
// caller's stream (the block kernels of the few hub rows, which leave most of the chip idle, beside the
// kernels of all other rows).  Created at first use and kept until the process ends; a thread that
// ends leaves its stream and events behind (destroying them from a thread-exit hook could run after the
// runtime has shut down).  NTS_SOFTMAX_SIDE_STREAM=0 in the environment: everything on the caller's stream.
struct SideLane {
  hipStream_t stream = nullptr;
  hipEvent_t fork = nullptr, join = nullptr;
};
SideLane *side_lane() {
  static const bool enabled = [] {
    const char *env = getenv("NTS_SOFTMAX_SIDE_STREAM");
    return !(env && atol(env) == 0);
  }();
  if (!enabled) return nullptr;
  constexpr int kDevices = 16;
  thread_local SideLane lanes[kDevices];
  thread_local bool tried[kDevices] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kDevices) return nullptr;
  SideLane &l = lanes[dev];
  if (!tried[dev]) {
    tried[dev] = true;
    hipStream_t st = nullptr;
    hipEvent_t a = nullptr, b = nullptr;
    if (hipStreamCreateWithFlags(&st, hipStreamNonBlocking) == hipSuccess &&
        hipEventCreateWithFlags(&a, hipEventDisableTiming) == hipSuccess &&
        hipEventCreateWithFlags(&b, hipEventDisableTiming) == hipSuccess) {
      l.stream = st;
      l.fork = a;
      l.join = b;
    } else {
      if (a) (void)hipEventDestroy(a);
      if (st) (void)hipStreamDestroy(st);
      (void)hipGetLastError();
    }
  }
  return l.stream ? &l : nullptr;
}

// The side lane between a fork (it waits for everything enqueued on `main` so far) and the join (`main`
// waits for it), which also happens on every way out of the scope.
class SideWork {
 public:
  SideWork(hipStream_t main, bool wanted) : main_(main), lane_(wanted ? side_lane() : nullptr) {
    // a stream that is recording a graph keeps all of the call's launches: the side stream is shared by
    // the thread's calls and must not become part of a recording
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (lane_ && (hipStreamIsCapturing(main_, &capturing) != hipSuccess || capturing != hipStreamCaptureStatusNone)) {
      (void)hipGetLastError();
      lane_ = nullptr;
    }
    if (lane_ && (hipEventRecord(lane_->fork, main_) != hipSuccess ||
                  hipStreamWaitEvent(lane_->stream, lane_->fork, 0) != hipSuccess)) {
      (void)hipGetLastError();
      lane_ = nullptr;  // nothing has been enqueued on the side stream: the caller's stream takes the work
    }
  }
  SideWork(const SideWork &) = delete;
  SideWork &operator=(const SideWork &) = delete;
  hipStream_t stream() const { return lane_ ? lane_->stream : main_; }
  hipError_t join() {
    if (!lane_) return hipSuccess;
    SideLane *l = lane_;
    lane_ = nullptr;
    const hipError_t e = hipEventRecord(l->join, l->stream);
    return e != hipSuccess ? e : hipStreamWaitEvent(main_, l->join, 0);
  }
  ~SideWork() { (void)join(); }

 private:
  hipStream_t main_;
  SideLane *lane_;
};

// Edge softmax / fused attention, forward (gy == nullptr) or backward; x / el / er / ri / ger are
// null where the variant does not use them.
int softmax_impl(bool backward, bool fused, float *out, float *ger, const float *x_or_gy, const float *y,
                 const float *el, const float *er, const uint32_t *co, const uint32_t *ri, uint32_t Vd, uint32_t H,
                 float slope, hipStream_t stream, const char *who, uint32_t max_degree = 0) {
  const bool pow2 = is_pow2(H) && H <= kWave;
  LongRows lr;
  // A caller that bounds every segment below the block kernels' class (a sampled layer: at most `fanout`
  // edges per destination) needs none of the launches that look for hub rows; a longer segment than
  // stated is still computed, by one wavefront.
  const bool no_hubs = max_degree != 0 && static_cast<uint64_t>(max_degree) * H <= kLongRowValues;
  if (pow2 && !no_hubs)
    if (int rc = collect_long_rows(lr, co, Vd, H, kLongRowValues, kGiantValues, stream)) return rc;
  const uint32_t max_values = lr.list ? kLongRowValues : kNoLimit;
  // The block kernels of the hub rows and the kernels of the giant ones' pieces run on the side lane,
  // beside the launches for all other rows below (they write other rows); their scratch is taken
  // before the fork, so that whatever the pool ordered for it on `stream` lies before it too.
  const size_t stats_floats = static_cast<size_t>(kPieceCap) * 2 * H, row_floats = static_cast<size_t>(kGiantCap) * 2 * H;
  ScratchBlock stats_block;
  if (lr.list) NTS_HIP_TRY(stats_block.alloc((stats_floats + row_floats) * sizeof(float), stream));
  SideWork side(stream, lr.list != nullptr);
  const hipStream_t hub_stream = side.stream();
  // 16-byte lanes for the segments that do not fit the register paths: whole heads per lane and
  // every array 16-byte aligned (a segment starts at e0 * H floats).
  const uint32_t vec4 = pow2 && H % 4 == 0 && aligned_to(out, 16) && aligned_to(x_or_gy, 16) && aligned_to(y, 16) &&
                        aligned_to(el, 16) && aligned_to(er, 16) && aligned_to(ger, 16);
  const bool use_short = pow2 && H <= static_cast<uint32_t>(kShortG);
  const uint32_t min_values = use_short ? kShortValues + 1 : 0u;
  // Both strided kernels: enough wavefronts to fill the chip several times, never more than the work.
  const dim3 block(256);
  const uint32_t short_blocks = ceil_div(static_cast<uint64_t>(Vd) * kShortG, 256);
  const dim3 short_grid(short_blocks < 16384u ? short_blocks : 16384u);
  const uint32_t wave_blocks = ceil_div(Vd, 4);  // at most one destination per wavefront
  const dim3 grid(wave_blocks < 8192u ? wave_blocks : 8192u);
  if (lr.list) {
    // The hub rows first: their few large blocks take their places on the chip before the launches for
    // all other rows fill it.
    if (!backward) {
      if (fused)
        hipLaunchKernelGGL(edge_softmax_fwd_long_kernel<true>, dim3(kLongGrid), dim3(kLongBlock), 0, hub_stream, out,
                           x_or_gy, el, er, co, ri, lr.list, lr.count, H, slope);
      else
        hipLaunchKernelGGL(edge_softmax_fwd_long_kernel<false>, dim3(kLongGrid), dim3(kLongBlock), 0, hub_stream, out,
                           x_or_gy, el, er, co, ri, lr.list, lr.count, H, slope);
    } else {
      if (fused)
        hipLaunchKernelGGL(edge_softmax_bwd_long_kernel<true>, dim3(kLongGrid), dim3(kLongBlock), 0, hub_stream, out, ger,
                           x_or_gy, y, el, er, co, ri, lr.list, lr.count, H, slope);
      else
        hipLaunchKernelGGL(edge_softmax_bwd_long_kernel<false>, dim3(kLongGrid), dim3(kLongBlock), 0, hub_stream, out, ger,
                           x_or_gy, y, el, er, co, ri, lr.list, lr.count, H, slope);
    }
    NTS_LAUNCH_CHECK(who);
    // Giant segments: per-piece statistics, ordered combine, apply (see the kernels above).
    float *stats = static_cast<float *>(stats_block.ptr);
    float *rowstat = stats + stats_floats;
    const dim3 pgrid(kLongGrid), pblock(kLongBlock), cgrid(kGiantCap / 4), cblock(64);
    if (!backward) {
      if (fused)
        hipLaunchKernelGGL(giant_softmax_stats_kernel<true>, pgrid, pblock, 0, hub_stream, stats, out, x_or_gy, el, er, ri,
                           lr.hdr, lr.pieces, H, slope);
      else
        hipLaunchKernelGGL(giant_softmax_stats_kernel<false>, pgrid, pblock, 0, hub_stream, stats, out, x_or_gy, el, er, ri,
                           lr.hdr, lr.pieces, H, slope);
      hipLaunchKernelGGL(giant_softmax_combine_kernel<0>, cgrid, cblock, 0, hub_stream, rowstat,
                         static_cast<float *>(nullptr), stats, lr.hdr, lr.giant_rows, lr.first, H);
      if (fused)
        hipLaunchKernelGGL(giant_softmax_apply_kernel<true>, pgrid, pblock, 0, hub_stream, out, x_or_gy, rowstat, lr.hdr,
                           lr.pieces, H);
      else
        hipLaunchKernelGGL(giant_softmax_apply_kernel<false>, pgrid, pblock, 0, hub_stream, out, x_or_gy, rowstat, lr.hdr,
                           lr.pieces, H);
    } else {
      hipLaunchKernelGGL(giant_softmax_dot_kernel, pgrid, pblock, 0, hub_stream, stats, x_or_gy, y, lr.hdr, lr.pieces, H);
      hipLaunchKernelGGL(giant_softmax_combine_kernel<1>, cgrid, cblock, 0, hub_stream, rowstat,
                         static_cast<float *>(nullptr), stats, lr.hdr, lr.giant_rows, lr.first, H);
      if (fused) {
        hipLaunchKernelGGL(giant_softmax_bwd_apply_kernel<true>, pgrid, pblock, 0, hub_stream, out, stats, x_or_gy, y, el, er,
                           ri, rowstat, lr.hdr, lr.pieces, H, slope);
        hipLaunchKernelGGL(giant_softmax_combine_kernel<1>, cgrid, cblock, 0, hub_stream, rowstat, ger, stats, lr.hdr,
                           lr.giant_rows, lr.first, H);
      } else {
        hipLaunchKernelGGL(giant_softmax_bwd_apply_kernel<false>, pgrid, pblock, 0, hub_stream, out, stats, x_or_gy, y, el, er,
                           ri, rowstat, lr.hdr, lr.pieces, H, slope);
      }
    }
    NTS_LAUNCH_CHECK(who);
  }
  if (use_short && fused && max_degree != 0 && static_cast<uint64_t>(max_degree) * H <= kShortValues) {
    // Every segment fits the short class by the caller's word: one launch (which still computes a
    // longer segment, slowly, should there be one).
    if (backward)
      hipLaunchKernelGGL((edge_softmax_short_kernel<true, true, true>), short_grid, block, 0, stream, out, ger, x_or_gy,
                         y, el, er, co, ri, Vd, H, slope);
    else
      hipLaunchKernelGGL((edge_softmax_short_kernel<true, false, true>), short_grid, block, 0, stream, out, ger, x_or_gy,
                         y, el, er, co, ri, Vd, H, slope);
    NTS_LAUNCH_CHECK(who);
    return NTS_OK;
  }
  if (use_short) {
#define NTS_SHORT(FU, BW)                                                                                          \
  hipLaunchKernelGGL((edge_softmax_short_kernel<FU, BW>), short_grid, block, 0, stream, out, ger, x_or_gy, y, el, er, \
                     co, ri, Vd, H, slope)
    if (fused) { if (backward) NTS_SHORT(true, true); else NTS_SHORT(true, false); }
    else       { if (backward) NTS_SHORT(false, true); else NTS_SHORT(false, false); }
#undef NTS_SHORT
    NTS_LAUNCH_CHECK(who);
  }
  if (!backward) {
#define NTS_FWD(FU, P2, PART, LO, HI)                                                                             \
  hipLaunchKernelGGL((edge_softmax_fwd_kernel<FU, P2, PART>), grid, block, 0, stream, out, x_or_gy, el, er, co, ri, \
                     Vd, H, slope, LO, HI, vec4)
    if (pow2 && fused) {
      // the register-resident segments, then the longer ones
      const uint32_t regs_hi = max_values < kWaveRegValues ? max_values : kWaveRegValues;
      NTS_FWD(true, true, 1, min_values, regs_hi);
      // 513 .. 2,048 values in a launch of their own: 16 or 32 values per lane in registers, one pass over
      // memory, and the registers that costs are not the other classes' (64 per lane measured slower)
      if (max_values > kWaveRegValues) {
        const uint32_t mid_hi = max_values < kWaveMidValues ? max_values : kWaveMidValues;
        NTS_FWD(true, true, 3, kWaveRegValues + 1, mid_hi);
        if (max_values > kWaveMidValues) NTS_FWD(true, true, 2, kWaveMidValues + 1, max_values);
      }
    } else if (pow2) {
      NTS_FWD(false, true, 0, min_values, max_values);
    } else {
      if (fused) NTS_FWD(true, false, 0, min_values, max_values); else NTS_FWD(false, false, 0, min_values, max_values);
    }
#undef NTS_FWD
    NTS_LAUNCH_CHECK(who);
  } else {
#define NTS_BWD(FU, P2, PART, LO, HI)                                                                            \
  hipLaunchKernelGGL((edge_softmax_bwd_kernel<FU, P2, PART>), grid, block, 0, stream, out, ger, x_or_gy, y, el, er, co, \
                     ri, Vd, H, slope, LO, HI, vec4)
    if (pow2 && fused) {
      const uint32_t regs_hi = max_values < kWaveRegValues ? max_values : kWaveRegValues;
      NTS_BWD(true, true, 1, min_values, regs_hi);
      // (a launch of its own for the class above that, held in registers as in the forward pass, measured no
      // gain up to 1,024 values and 3.36 -> 3.57 ms up to 2,048: the backward holds two arrays per lane)
      if (max_values > kWaveRegValues) NTS_BWD(true, true, 2, kWaveRegValues + 1, max_values);
    } else if (pow2) {
      NTS_BWD(false, true, 0, min_values, max_values);
    } else {
      if (fused) NTS_BWD(true, false, 0, min_values, max_values); else NTS_BWD(false, false, 0, min_values, max_values);
    }
#undef NTS_BWD
    NTS_LAUNCH_CHECK(who);
  }
  if (lr.list) {
    const hipError_t join_err = side.join();  // `stream` waits for the hub rows before their scratch goes back
    NTS_HIP_TRY(stats_block.release());
    if (join_err != hipSuccess) return fail_hip(join_err, who);
  }
  return release_long_rows(lr);
}
}  // namespace

extern "C" {

int nts_scatter_src_to_edge(float *msg, const float *feat, const uint32_t *ri, const uint32_t *co,
                            const uint32_t *mirror, uint32_t Vd, uint32_t F, nts_stream_t stream) {
  NTS_TRACE_RANGE("nts_scatter_src_to_edge");
  return edge_copy_impl(msg, feat, ri, co, mirror, Vd, F, kFromSrc, stream, "nts_scatter_src_to_edge: bad argument");
}

int nts_scatter_dst_to_edge(float *msg, const float *feat, const uint32_t *co, uint32_t Vd, uint32_t F,
                            nts_stream_t stream) {
  NTS_TRACE_RANGE("nts_scatter_dst_to_edge");
  return edge_copy_impl(msg, feat, nullptr, co, nullptr, Vd, F, kFromDst, stream,
                        "nts_scatter_dst_to_edge: bad argument");
}

int nts_scatter_grad_to_edge(float *msg_grad, const float *gout, const uint32_t *co, uint32_t Vd, uint32_t F,
                             nts_stream_t stream) {
  NTS_TRACE_RANGE("nts_scatter_grad_to_edge");
  return edge_copy_impl(msg_grad, gout, nullptr, co, nullptr, Vd, F, kAddFromDst, stream,
                        "nts_scatter_grad_to_edge: bad argument");
}

int nts_gather_edge_to_dst(float *out, const float *msg, const uint32_t *co, uint32_t Vd, uint32_t F, int accumulate,
                           nts_stream_t stream) {
  NTS_TRACE_RANGE("nts_gather_edge_to_dst");
  return gather_edge_impl(out, msg, co, nullptr, Vd, F, accumulate, stream, "nts_gather_edge_to_dst: bad argument");
}

int nts_gather_edge_to_src(float *out, const float *msg, const uint32_t *ro, const uint32_t *perm, uint32_t Vs,
                           uint32_t F, int accumulate, nts_stream_t stream) {
  NTS_TRACE_RANGE("nts_gather_edge_to_src");
  if (Vs != 0 && !perm) return fail(NTS_ERR_INVALID, "nts_gather_edge_to_src: null perm");
  return gather_edge_impl(out, msg, ro, perm, Vs, F, accumulate, stream, "nts_gather_edge_to_src: bad argument");
}

int nts_edge_softmax_fwd(float *y, const float *x, const uint32_t *co, uint32_t Vd, uint32_t H,
                         nts_stream_t stream) {
  NTS_TRACE_RANGE("nts_edge_softmax_fwd");
  if (H == 0) return fail(NTS_ERR_INVALID, "nts_edge_softmax_fwd: H is 0");
  if (Vd == 0) return NTS_OK;
  if (!y || !x || !co) return fail(NTS_ERR_INVALID, "nts_edge_softmax_fwd: null pointer");
  return softmax_impl(false, false, y, nullptr, x, nullptr, nullptr, nullptr, co, nullptr, Vd, H, 0.f, stream,
                      "nts_edge_softmax_fwd");
}

int nts_edge_softmax_bwd(float *gx, const float *gy, const float *y, const uint32_t *co, uint32_t Vd, uint32_t H,
                         nts_stream_t stream) {
  NTS_TRACE_RANGE("nts_edge_softmax_bwd");
  if (H == 0) return fail(NTS_ERR_INVALID, "nts_edge_softmax_bwd: H is 0");
  if (Vd == 0) return NTS_OK;
  if (!gx || !gy || !y || !co) return fail(NTS_ERR_INVALID, "nts_edge_softmax_bwd: null pointer");
  return softmax_impl(true, false, gx, nullptr, gy, y, nullptr, nullptr, co, nullptr, Vd, H, 0.f, stream,
                      "nts_edge_softmax_bwd");
}

int nts_gat_attention_fwd(float *alpha, const float *el, const float *er, const uint32_t *co, const uint32_t *ri,
                          uint32_t Vd, uint32_t H, float slope, nts_stream_t stream) {
  NTS_TRACE_RANGE("nts_gat_attention_fwd");
  if (H == 0) return fail(NTS_ERR_INVALID, "nts_gat_attention_fwd: H is 0");
  if (Vd == 0) return NTS_OK;
  if (!alpha || !el || !er || !co || !ri) return fail(NTS_ERR_INVALID, "nts_gat_attention_fwd: null pointer");
  return softmax_impl(false, true, alpha, nullptr, nullptr, nullptr, el, er, co, ri, Vd, H, slope, stream,
                      "nts_gat_attention_fwd");
}

int nts_gat_attention_fwd_bounded(float *alpha, const float *el, const float *er, const uint32_t *co,
                                  const uint32_t *ri, uint32_t Vd, uint32_t H, float slope, uint32_t max_degree,
                                  nts_stream_t stream) {
  NTS_TRACE_RANGE("nts_gat_attention_fwd_bounded");
  if (H == 0) return fail(NTS_ERR_INVALID, "nts_gat_attention_fwd_bounded: H is 0");
  if (Vd == 0) return NTS_OK;
  if (!alpha || !el || !er || !co || !ri) return fail(NTS_ERR_INVALID, "nts_gat_attention_fwd_bounded: null pointer");
  return softmax_impl(false, true, alpha, nullptr, nullptr, nullptr, el, er, co, ri, Vd, H, slope, stream,
                      "nts_gat_attention_fwd_bounded", max_degree);
}

int nts_gat_attention_bwd_bounded(float *gs, float *ger, const float *galpha, const float *alpha, const float *el,
                                  const float *er, const uint32_t *co, const uint32_t *ri, uint32_t Vd, uint32_t H,
                                  float slope, uint32_t max_degree, nts_stream_t stream) {
  NTS_TRACE_RANGE("nts_gat_attention_bwd_bounded");
  if (H == 0) return fail(NTS_ERR_INVALID, "nts_gat_attention_bwd_bounded: H is 0");
  if (Vd == 0) return NTS_OK;
  if (!gs || !ger || !galpha || !alpha || !el || !er || !co || !ri)
    return fail(NTS_ERR_INVALID, "nts_gat_attention_bwd_bounded: null pointer");
  return softmax_impl(true, true, gs, ger, galpha, alpha, el, er, co, ri, Vd, H, slope, stream,
                      "nts_gat_attention_bwd_bounded", max_degree);
}

int nts_gat_attention_bwd(float *gs, float *ger, const float *galpha, const float *alpha, const float *el,
                          const float *er, const uint32_t *co, const uint32_t *ri, uint32_t Vd, uint32_t H,
                          float slope, nts_stream_t stream) {
  NTS_TRACE_RANGE("nts_gat_attention_bwd");
  if (H == 0) return fail(NTS_ERR_INVALID, "nts_gat_attention_bwd: H is 0");
  if (Vd == 0) return NTS_OK;
  if (!gs || !ger || !galpha || !alpha || !el || !er || !co || !ri)
    return fail(NTS_ERR_INVALID, "nts_gat_attention_bwd: null pointer");
  return softmax_impl(true, true, gs, ger, galpha, alpha, el, er, co, ri, Vd, H, slope, stream,
                      "nts_gat_attention_bwd");
}

int nts_sddmm_heads(float *galpha, const float *in, const float *gout, const uint32_t *co, const uint32_t *ri,
                    uint32_t Vd, uint32_t H, uint32_t Fh, nts_stream_t stream) {
  NTS_TRACE_RANGE("nts_sddmm_heads");
  if (H == 0 || Fh == 0) return fail(NTS_ERR_INVALID, "nts_sddmm_heads: H or Fh is 0");
  if (static_cast<uint64_t>(H) * Fh > 0xFFFFFFFFull) return fail(NTS_ERR_INVALID, "nts_sddmm_heads: H*Fh overflows");
  if (Vd == 0) return NTS_OK;
  if (!galpha || !in || !gout || !co || !ri) return fail(NTS_ERR_INVALID, "nts_sddmm_heads: null pointer");
  const uint32_t F = H * Fh;
  const dim3 grid = edge_grid(Vd), block(256);
  const bool v4 = Fh % 4 == 0 && aligned_to(in, 16) && aligned_to(gout, 16);
  const uint32_t vec = v4 ? 4 : 1;
  const uint32_t lanes = F / vec, lanes_per_head = Fh / vec;
  if (lanes <= kWave && is_pow2(lanes) && is_pow2(lanes_per_head)) {
    if (v4)
      hipLaunchKernelGGL(sddmm_edge_kernel<4>, grid, block, 0, stream, galpha, in, gout, co, ri, Vd, H, Fh, lanes,
                         lanes_per_head);
    else
      hipLaunchKernelGGL(sddmm_edge_kernel<1>, grid, block, 0, stream, galpha, in, gout, co, ri, Vd, H, Fh, lanes,
                         lanes_per_head);
  } else {
    hipLaunchKernelGGL(sddmm_edge_generic_kernel, grid, block, 0, stream, galpha, in, gout, co, ri, Vd, H, Fh);
  }
  NTS_LAUNCH_CHECK("nts_sddmm_heads");
  return NTS_OK;
}

}  // extern "C"
