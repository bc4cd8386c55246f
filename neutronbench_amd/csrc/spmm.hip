// Aggregation kernels: weighted / unweighted SpMM executed as a row gather, forward over CSC and
// backward over CSR (replaces cuda/ntsCUDAFuseKernel.cuh:147-290, 327-487 and their launchers
// cuda/ntsCUDAGraphOP.cu:186-292).
//
// Mapping.  One wavefront (64 lanes) owns one work item = one output row, or one chunk of a long
// row.  The 64 lanes span the feature dimension: lane l holds NACC register accumulators of VEC
// consecutive floats at columns (l + 64*k)*VEC (VEC = 4 when rows are 16-byte aligned, else 1), so
// every row read is a fully coalesced 64*VEC*4-byte wave load and each output element is written
// exactly once, without atomics.
// Neighbour (index, weight) pairs are fetched 64 at a time with one coalesced load per wave, staged
// in a wave-private LDS tile and read back one pair at a time by all lanes at once (a broadcast
// read), then moved to scalar registers, so the source-row base address is scalar and every
// index/weight is read from memory once per row instead of once per lane.
// Narrow rows (F <= 32*VEC) use sub-wavefront groups of G lanes per row (spmm_group_kernel).
//
// Accumulation order within a row is the edge order of the offsets array, one fused multiply-add
// per edge and element -- the order of the CPU operators (core/ntsMiniBatchGraphOp.hpp:154-240),
// so unsplit rows reproduce an FMA-contracted CPU build bit for bit.
#include <stdlib.h>
#include <string.h>

#include <rocprim/device/device_radix_sort.hpp>
#include <rocprim/device/device_scan.hpp>
#include <rocprim/iterator/counting_iterator.hpp>
#include <rocprim/iterator/transform_iterator.hpp>

#include <algorithm>
#include <atomic>
#include <mutex>
#include <new>
#include <thread>
#include <vector>

#include "common.hpp"

// Fixed scratch of nts_spmm_gather_static_scratch, the entry point for callers that must not allocate:
// each device that loads this library holds one copy of the array until the process ends.  Host code
// never passes the array's name to a kernel (on the host the name is only a stand-in for the symbol):
// its device address is looked up once per device and kept in g_static_scratch_ptr.
constexpr size_t kStaticScratchBytes = NTS_SPMM_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace nts {
namespace {

constexpr int kMaxScratchDevices = 64;
std::mutex g_static_scratch_mutex;
unsigned char *g_static_scratch_ptr[kMaxScratchDevices] = {};

// Device address of `scratch` on the current device (looked up on the first call per device).
int static_scratch_address(unsigned char **out) {
  int dev = -1;
  NTS_HIP_TRY(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxScratchDevices) return fail(NTS_ERR_INVALID, "static scratch: device ordinal out of range");
  std::lock_guard<std::mutex> lock(g_static_scratch_mutex);
  if (!g_static_scratch_ptr[dev]) {
    unsigned char *p = nullptr;
    NTS_HIP_TRY(hipGetSymbolAddress(reinterpret_cast<void **>(&p), HIP_SYMBOL(scratch)));
    if (!p) return fail(NTS_ERR_HIP, "static scratch: hipGetSymbolAddress returned a null address");
    g_static_scratch_ptr[dev] = p;
  }
  *out = g_static_scratch_ptr[dev];
  return NTS_OK;
}

template <int VEC>
struct Vec;
template <>
struct Vec<1> {
  using type = float;
};
template <>
struct Vec<2> {
  using type = float2;
};
template <>
struct Vec<4> {
  using type = float4;
};

template <int VEC>
__device__ __forceinline__ typename Vec<VEC>::type vzero();
template <>
__device__ __forceinline__ float vzero<1>() {
  return 0.f;
}
template <>
__device__ __forceinline__ float2 vzero<2>() {
  return make_float2(0.f, 0.f);
}
template <>
__device__ __forceinline__ float4 vzero<4>() {
  return make_float4(0.f, 0.f, 0.f, 0.f);
}

__device__ __forceinline__ void vfma(float &a, float x, float w) { a = fmaf(x, w, a); }
__device__ __forceinline__ void vfma(float2 &a, float2 x, float w) {
  a.x = fmaf(x.x, w, a.x);
  a.y = fmaf(x.y, w, a.y);
}
__device__ __forceinline__ void vfma(float4 &a, float4 x, float w) {
  a.x = fmaf(x.x, w, a.x);
  a.y = fmaf(x.y, w, a.y);
  a.z = fmaf(x.z, w, a.z);
  a.w = fmaf(x.w, w, a.w);
}
__device__ __forceinline__ void vadd(float &a, float x) { a += x; }
__device__ __forceinline__ void vadd(float2 &a, float2 x) {
  a.x += x.x;
  a.y += x.y;
}
__device__ __forceinline__ void vadd(float4 &a, float4 x) {
  a.x += x.x;
  a.y += x.y;
  a.z += x.z;
  a.w += x.w;
}

// Edges processed per inner step: keeps 8..16 independent row loads in flight per lane.
// With 4-byte lanes and six to ten accumulators (F = 602: ten) four edges per step were measured
// against one, two and three: 11.04 ms against 11.54 / 11.13 / 11.13 for the Reddit-shaped F=602 pass --
// a step's loads are all requested before the first is used, so a wavefront then has 40 row loads in
// flight instead of 10.  With 16-byte lanes the same count would cost 160 registers.
__host__ __device__ constexpr int unroll_for(int nacc, int vec) {
  return nacc >= 6 ? (vec == 1 ? 4 : 1) : nacc >= 4 ? 2 : nacc >= 2 ? 4 : 8;
}

// Work item of a planned launch: row, first edge, one-past-last edge, partial slot (kNoSlot = the
// item is a whole row and writes `out` directly).
using Item = uint4;

// Per-head edge weights (attention-weighted aggregation): w is alpha [E_csc, H], a column belongs
// to head column / Fh, and the weight of edge position e is alpha[(perm ? perm[e] : e) * H + head].
struct HeadArgs {
  const uint32_t *perm;
  uint32_t H;
  uint32_t Fh;
};

template <int VEC, int NACC, bool LDS_TILE, bool HEADS, bool REMAP, bool RUNS>
__global__ __launch_bounds__(256) void spmm_wave_kernel(const float *__restrict__ in, float *__restrict__ out,
                                                        const float *__restrict__ w,
                                                        const uint32_t *__restrict__ offsets,
                                                        const uint32_t *__restrict__ indices, uint32_t index_base,
                                                        uint32_t n_items, uint32_t n_list, uint32_t F,
                                                        uint32_t col_base, const Item *__restrict__ items,
                                                        float *__restrict__ partial,
                                                        int accumulate, HeadArgs heads, uint32_t row_edge_limit,
                                                        const uint32_t *__restrict__ edge_ids, uint32_t in_ld,
                                                        uint32_t partial_ld, int out_scalar) {
  using V = typename Vec<VEC>::type;
  constexpr int U = unroll_for(NACC, VEC);
  const uint32_t lane = threadIdx.x & (kWave - 1);
  const uint32_t item = blockIdx.x * (blockDim.x / kWave) + (threadIdx.x / kWave);
  if (item >= n_items) return;

  // Work items [0, n_list) come from the list, the ones after it are the rows 0, 1, ... themselves
  // (a launch may hold both: the pieces of long rows first, then every row that fits one wavefront).
  uint32_t row, e0, e1, slot;
  if (item < n_list) {
    const Item it = items[item];
    row = wave_first(it.x);
    e0 = wave_first(it.y);
    e1 = wave_first(it.z);
    slot = wave_first(it.w);
  } else {
    row = item - n_list;
    e0 = wave_first(offsets[row]);
    e1 = wave_first(offsets[row + 1]);
    slot = kNoSlot;
    if (e1 - e0 > row_edge_limit) return;  // a long row: its pieces are separate work items
  }

  // Lanes past the end of the row (only possible in the last accumulator) read the row's last
  // VEC columns instead, so that loads need no predication; their sums are never stored.
  uint32_t col[NACC];
  uint32_t lcol[NACC];
  uint32_t head[NACC];
  bool live[NACC];
  V acc[NACC];
#pragma unroll
  for (int k = 0; k < NACC; ++k) {
    col[k] = col_base + (lane + kWave * k) * VEC;
    live[k] = col[k] < F;
    lcol[k] = live[k] ? col[k] : in_ld - VEC;
    head[k] = HEADS ? lcol[k] / heads.Fh : 0u;
    acc[k] = vzero<VEC>();
  }

  // Tile of up to 64 neighbour (index, weight) pairs, fetched with one coalesced load per wave; the
  // next tile is fetched while the current one is consumed.  The pairs are then handed to the whole
  // wave one at a time as scalars: either straight from the registers that hold them (readlane), or
  // (LDS_TILE) through a wave-private LDS tile that every lane reads at the same address.  The LDS
  // region belongs to one wave and LDS operations of a wave complete in order, so no block barrier
  // is needed -- which matters because waves of a block run different trip counts.
  __shared__ uint2 lds_tile[LDS_TILE ? 4 : 1][LDS_TILE ? kWave : 1];
  uint2 *tile = lds_tile[LDS_TILE ? (threadIdx.x / kWave) : 0];
  // Second component of a pair: the edge weight (as bits), or with per-head weights the id of the
  // edge in alpha's (CSC) order.
  // edge_ids (a schedule that gathers through its own, re-ordered copy of the indices): position of
  // edge e in the caller's weight / alpha order.
  auto second_of = [&](uint32_t e) -> uint32_t {
    const uint32_t id = REMAP ? edge_ids[e] : e;
    if (HEADS) return heads.perm ? heads.perm[id] : id;
    return w ? __float_as_uint(w[id]) : __float_as_uint(1.f);
  };
  uint32_t nxt_i = 0;
  uint32_t nxt_s = HEADS ? 0u : __float_as_uint(1.f);
  if (e0 + lane < e1) {
    nxt_i = indices[e0 + lane] - index_base;
    nxt_s = second_of(e0 + lane);
  }
  for (uint32_t eb = e0; eb < e1; eb += kWave) {
    const uint32_t n = min(static_cast<uint32_t>(kWave), e1 - eb);
    const uint32_t my_i = nxt_i;
    const uint32_t my_s = nxt_s;
    if (LDS_TILE) {
      __builtin_amdgcn_wave_barrier();  // earlier reads of the tile are done before it is overwritten
      tile[lane] = make_uint2(my_i, my_s);
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
    const uint32_t en = eb + kWave + lane;
    if (en < e1) {
      nxt_i = indices[en] - index_base;
      nxt_s = second_of(en);
    }
    auto pair_at = [&](uint32_t j, uint32_t &idx, uint32_t &second) {
      if (LDS_TILE) {
        const uint2 p = tile[j];
        idx = wave_first(p.x);
        second = wave_first(p.y);
      } else {
        idx = wave_read(my_i, j);
        second = wave_read(my_s, j);
      }
    };
    if (RUNS && LDS_TILE && !HEADS) {
      // Runs of consecutive edges with the same neighbour (a multigraph's parallel edges, adjacent in
      // sorted rows): the row is loaded once and added once per edge of the run, in edge order with
      // each edge's own weight, so the result is the same bit for bit.  Up to U runs per step.
      const uint32_t prev = tile[lane ? lane - 1 : 0].x;
      uint64_t starts = __ballot(lane < n && (lane == 0 || my_i != prev));
      while (starts) {
        uint32_t rs[U + 1];
        int nr = 0;
#pragma unroll
        for (int u = 0; u < U; ++u) {
          rs[u] = n;
          if (starts) {
            rs[u] = static_cast<uint32_t>(__builtin_ctzll(starts));
            starts &= starts - 1;
            nr = u + 1;
          }
        }
        rs[U] = starts ? static_cast<uint32_t>(__builtin_ctzll(starts)) : n;
        V v[U][NACC];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          if (u < nr) {
            const float *src = in + static_cast<size_t>(wave_first(tile[rs[u]].x)) * in_ld;
#pragma unroll
            for (int k = 0; k < NACC; ++k) v[u][k] = *reinterpret_cast<const V *>(src + lcol[k]);
          }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
          if (u < nr) {
            const uint32_t end = (u + 1 < U) ? rs[u + 1] : rs[U];
            for (uint32_t q = rs[u]; q < end; ++q) {
              const float wgt = __uint_as_float(wave_first(tile[q].y));
#pragma unroll
              for (int k = 0; k < NACC; ++k) vfma(acc[k], v[u][k], wgt);
            }
          }
        }
      }
      continue;
    }
    uint32_t j = 0;
    for (; j + U <= n; j += U) {
      const float *src[U];
      uint32_t ss[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        uint32_t si;
        pair_at(j + u, si, ss[u]);
        src[u] = in + static_cast<size_t>(si) * in_ld;
      }
      V v[U][NACC];
      float wv[U][HEADS ? NACC : 1];
#pragma unroll
      for (int u = 0; u < U; ++u) {
#pragma unroll
        for (int k = 0; k < NACC; ++k) {
          v[u][k] = *reinterpret_cast<const V *>(src[u] + lcol[k]);
          if (HEADS) wv[u][k] = w[static_cast<size_t>(ss[u]) * heads.H + head[k]];
        }
        if (!HEADS) wv[u][0] = __uint_as_float(ss[u]);
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
#pragma unroll
        for (int k = 0; k < NACC; ++k) {
          vfma(acc[k], v[u][k], wv[u][HEADS ? k : 0]);
        }
      }
    }
    for (; j < n; ++j) {
      uint32_t si, ss;
      pair_at(j, si, ss);
      const float *src = in + static_cast<size_t>(si) * in_ld;
#pragma unroll
      for (int k = 0; k < NACC; ++k) {
        const float wgt = HEADS ? w[static_cast<size_t>(ss) * heads.H + head[k]] : __uint_as_float(ss);
        vfma(acc[k], *reinterpret_cast<const V *>(src + lcol[k]), wgt);
      }
    }
  }

  if (VEC > 1 && out_scalar && slot == kNoSlot) {
    // Output rows that do not start on a 16-byte boundary (F not a multiple of four while the gather
    // runs over a padded copy of the input): the row is stored one float at a time.
    float *dst = out + static_cast<size_t>(row) * F;
#pragma unroll
    for (int k = 0; k < NACC; ++k) {
      const float *r = reinterpret_cast<const float *>(&acc[k]);
#pragma unroll
      for (int c = 0; c < VEC; ++c) {
        const uint32_t cc = col[k] + c;
        if (cc < F) dst[cc] = accumulate ? r[c] + dst[cc] : r[c];
      }
    }
    return;
  }
  float *dst =
      (slot == kNoSlot) ? out + static_cast<size_t>(row) * F : partial + static_cast<size_t>(slot) * partial_ld;
  const bool add = accumulate && slot == kNoSlot;
#pragma unroll
  for (int k = 0; k < NACC; ++k) {
    if (live[k]) {
      V *p = reinterpret_cast<V *>(dst + col[k]);
      V r = acc[k];
      if (add) vadd(r, *p);
      *p = r;
    }
  }
}

// Sub-wavefront variant for narrow rows: G lanes per row (G = 4, 8, 16 or 32), 64/G rows per
// wavefront, one VEC-wide accumulator per lane (F <= G*VEC).  Neighbour pairs are fetched G at a
// time per group and broadcast inside the group with cross-lane shuffles.
template <int G, int VEC, bool HEADS, bool REMAP, bool RUNS>
__global__ __launch_bounds__(256) void spmm_group_kernel(const float *__restrict__ in, float *__restrict__ out,
                                                         const float *__restrict__ w,
                                                         const uint32_t *__restrict__ offsets,
                                                         const uint32_t *__restrict__ indices, uint32_t index_base,
                                                         uint32_t n_items, uint32_t n_list, uint32_t F,
                                                         const Item *__restrict__ items, float *__restrict__ partial,
                                                         int accumulate, HeadArgs heads,
                                                         uint32_t row_edge_limit,
                                                         const uint32_t *__restrict__ edge_ids) {
  using V = typename Vec<VEC>::type;
  constexpr int U = G >= 8 ? 8 : 4;  // edges per step: their rows are requested together
  const uint32_t gl = threadIdx.x & (G - 1);
  const uint32_t item = (blockIdx.x * blockDim.x + threadIdx.x) / G;
  if (item >= n_items) return;  // whole groups leave together; shuffles stay inside a group

  uint32_t row, e0, e1, slot;
  if (item < n_list) {  // listed work items first, then the rows themselves
    const Item it = items[item];
    row = it.x;
    e0 = it.y;
    e1 = it.z;
    slot = it.w;
  } else {
    row = item - n_list;
    e0 = offsets[row];
    e1 = offsets[row + 1];
    slot = kNoSlot;
    if (e1 - e0 > row_edge_limit) return;  // a long row: its pieces are separate work items
  }
  const uint32_t col = gl * VEC;
  const bool live = col < F;
  const uint32_t lcol = live ? col : F - VEC;  // idle lanes re-read the last columns, never store
  const uint32_t head = HEADS ? lcol / heads.Fh : 0u;
  V acc = vzero<VEC>();

  // The (index, weight) pairs of the next G edges are requested while the current ones are used, so
  // that a group does not wait for them at the start of every tile.
  auto fetch_pair = [&](uint32_t e, uint32_t &pi, uint32_t &ps) {
    pi = 0;
    ps = HEADS ? 0u : __float_as_uint(1.f);  // weight bits, or the edge's id in alpha's order
    if (e < e1) {
      pi = indices[e] - index_base;
      const uint32_t id = REMAP ? edge_ids[e] : e;
      if (HEADS)
        ps = heads.perm ? heads.perm[id] : id;
      else if (w)
        ps = __float_as_uint(w[id]);
    }
  };
  uint32_t nxt_i, nxt_s;
  fetch_pair(e0 + gl, nxt_i, nxt_s);
  V held = vzero<VEC>();            // RUNS: the row loaded last and its index
  uint32_t held_i = 0xFFFFFFFFu;
  for (uint32_t eb = e0; eb < e1; eb += G) {
    const uint32_t n = min(static_cast<uint32_t>(G), e1 - eb);
    const uint32_t my_i = nxt_i, my_s = nxt_s;
    fetch_pair(eb + G + gl, nxt_i, nxt_s);
    uint32_t j = 0;
    for (; j + U <= n; j += U) {
      uint32_t si[U];
      uint32_t ss[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        si[u] = __shfl(my_i, j + u, G);
        ss[u] = __shfl(my_s, j + u, G);
      }
      V v[U];
      float wv[U];
      if (RUNS) {
        // An edge that repeats its predecessor's index (a parallel edge) does not load the row again:
        // the group keeps the last row it loaded in `held` and adds it with the edge's own weight.
        bool fresh[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          fresh[u] = si[u] != (u ? si[u - 1] : held_i);
          v[u] = vzero<VEC>();
          if (fresh[u]) v[u] = *reinterpret_cast<const V *>(in + static_cast<size_t>(si[u]) * F + lcol);
          wv[u] = HEADS ? w[static_cast<size_t>(ss[u]) * heads.H + head] : __uint_as_float(ss[u]);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
          if (fresh[u]) held = v[u];
          vfma(acc, held, wv[u]);
        }
        held_i = si[U - 1];
        continue;
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        v[u] = *reinterpret_cast<const V *>(in + static_cast<size_t>(si[u]) * F + lcol);
        wv[u] = HEADS ? w[static_cast<size_t>(ss[u]) * heads.H + head] : __uint_as_float(ss[u]);
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        vfma(acc, v[u], wv[u]);
      }
    }
    if (!RUNS && j < n) {
      // The last, partial step: its rows are requested together like a full step's (a sampled layer's
      // rows are a step or two long; one edge after the other, each waited for, doubled their time),
      // and added in the same order.
      const uint32_t left = n - j;
      V v[U];
      float wv[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const uint32_t si = __shfl(my_i, (j + u) & (G - 1), G);
        const uint32_t ss = __shfl(my_s, (j + u) & (G - 1), G);
        v[u] = vzero<VEC>();
        wv[u] = 0.f;
        if (static_cast<uint32_t>(u) < left) {
          v[u] = *reinterpret_cast<const V *>(in + static_cast<size_t>(si) * F + lcol);
          wv[u] = HEADS ? w[static_cast<size_t>(ss) * heads.H + head] : __uint_as_float(ss);
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (static_cast<uint32_t>(u) < left) vfma(acc, v[u], wv[u]);
      }
      j = n;
    }
    for (; j < n; ++j) {
      const uint32_t si = __shfl(my_i, j, G);
      const uint32_t ss = __shfl(my_s, j, G);
      const float wgt = HEADS ? w[static_cast<size_t>(ss) * heads.H + head] : __uint_as_float(ss);
      if (RUNS) {
        if (si != held_i) held = *reinterpret_cast<const V *>(in + static_cast<size_t>(si) * F + lcol);
        held_i = si;
        vfma(acc, held, wgt);
        continue;
      }
      vfma(acc, *reinterpret_cast<const V *>(in + static_cast<size_t>(si) * F + lcol), wgt);
    }
  }

  if (live) {
    float *dst = (slot == kNoSlot) ? out + static_cast<size_t>(row) * F : partial + static_cast<size_t>(slot) * F;
    V *p = reinterpret_cast<V *>(dst + col);
    V r = acc;
    if (accumulate && slot == kNoSlot) vadd(r, *p);
    *p = r;
  }
}

// Second stage for split rows: out[row,:] (+)= partial[first,:] + partial[first+1,:] + ... in slot
// order.  Block (x, y) owns 256 columns (tile y) of split row x; `splits[i]` = (row, first slot,
// slot count, unused).  Eight slots are loaded at a time and then added one after the other, so the
// loads overlap while the order of the additions stays fixed.
__global__ __launch_bounds__(256) void spmm_reduce_partials_kernel(float *__restrict__ out,
                                                                   const float *__restrict__ partial,
                                                                   const uint4 *__restrict__ splits, uint32_t F,
                                                                   int accumulate, uint32_t ld) {
  const uint4 s = splits[blockIdx.x];
  const uint32_t c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= F) return;
  const float *src = partial + static_cast<size_t>(s.y) * ld + c;
  float a = src[0];
  uint32_t k = 1;
  for (; k + 8 <= s.z; k += 8) {
    float v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = src[static_cast<size_t>(k + u) * ld];
#pragma unroll
    for (int u = 0; u < 8; ++u) a += v[u];
  }
  for (; k < s.z; ++k) a += src[static_cast<size_t>(k) * ld];
  float *dst = out + static_cast<size_t>(s.x) * F + c;
  if (accumulate) a += *dst;
  *dst = a;
}

// The same for rows of up to 1,024 columns: one block per split row covers all columns (thread t
// adds columns t, t + 256, ...), so that a block reads whole, contiguous partial rows.
template <int J>
__global__ __launch_bounds__(256) void spmm_reduce_partials_wide_kernel(float *__restrict__ out,
                                                                        const float *__restrict__ partial,
                                                                        const uint4 *__restrict__ splits, uint32_t F,
                                                                        int accumulate, uint32_t ld) {
  const uint4 s = splits[blockIdx.x];
  const float *src = partial + static_cast<size_t>(s.y) * ld;
  uint32_t c[J];
  bool live[J];
  float a[J];
#pragma unroll
  for (int j = 0; j < J; ++j) {
    c[j] = threadIdx.x + 256u * j;
    live[j] = c[j] < F;
    if (!live[j]) c[j] = F - 1;  // re-read the last column, never stored
    a[j] = src[c[j]];
  }
  uint32_t k = 1;
  for (; k + 8 <= s.z; k += 8) {
    float v[8][J];
#pragma unroll
    for (int u = 0; u < 8; ++u)
#pragma unroll
      for (int j = 0; j < J; ++j) v[u][j] = src[static_cast<size_t>(k + u) * ld + c[j]];
#pragma unroll
    for (int u = 0; u < 8; ++u)
#pragma unroll
      for (int j = 0; j < J; ++j) a[j] += v[u][j];
  }
  for (; k + 2 <= s.z; k += 2) {
    float v[2][J];
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int j = 0; j < J; ++j) v[u][j] = src[static_cast<size_t>(k + u) * ld + c[j]];
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int j = 0; j < J; ++j) a[j] += v[u][j];
  }
  for (; k < s.z; ++k)
#pragma unroll
    for (int j = 0; j < J; ++j) a[j] += src[static_cast<size_t>(k) * ld + c[j]];
  float *dst = out + static_cast<size_t>(s.x) * F;
#pragma unroll
  for (int j = 0; j < J; ++j)
    if (live[j]) dst[c[j]] = accumulate ? a[j] + dst[c[j]] : a[j];
}

// Launches the second stage for a plan's split rows.
inline void launch_reduce_partials(float *out, const float *partial, const uint4 *splits, uint32_t n_splits, uint32_t F,
                                   int accumulate, hipStream_t stream, uint32_t ld = 0) {
  if (!ld) ld = F;  // row stride of the partial sums
  // Up to 1,024 columns one block adds whole rows (contiguous reads: 29.6 -> 29.2 ms per step on the
  // Reddit-shaped F=602 workload); wider rows are tiled 256 columns per block.
#define NTS_REDUCE_WIDE(J)                                                                                          \
  hipLaunchKernelGGL(spmm_reduce_partials_wide_kernel<J>, dim3(n_splits), dim3(256), 0, stream, out, partial, splits, \
                     F, accumulate, ld)
  if (F > 256 && F <= 512)
    NTS_REDUCE_WIDE(2);
  else if (F > 512 && F <= 768)
    NTS_REDUCE_WIDE(3);
  else if (F > 768 && F <= 1024)
    NTS_REDUCE_WIDE(4);
  else
    hipLaunchKernelGGL(spmm_reduce_partials_kernel, dim3(n_splits, ceil_div(F, 256)), dim3(256), 0, stream, out, partial,
                       splits, F, accumulate, ld);
#undef NTS_REDUCE_WIDE
}

// Copy of a [rows, F] matrix with the row stride padded to `ld` floats (a multiple of four; the pad
// columns are zero), so that every row starts on a 16-byte boundary and the gather can use 16-byte
// lanes.  One thread per 16 bytes written.
__global__ __launch_bounds__(256) void pad_rows_kernel(float4 *__restrict__ dst, const float *__restrict__ src,
                                                       uint32_t rows, uint32_t F, uint32_t ld) {
  const uint32_t per_row = ld / 4;
  const uint64_t total = static_cast<uint64_t>(rows) * per_row;
  for (uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < total;
       i += static_cast<uint64_t>(gridDim.x) * blockDim.x) {
    const uint32_t r = static_cast<uint32_t>(i / per_row);
    const uint32_t c = static_cast<uint32_t>(i % per_row) * 4;
    const float *p = src + static_cast<size_t>(r) * F + c;
    float4 v;
    v.x = c + 0 < F ? p[0] : 0.f;
    v.y = c + 1 < F ? p[1] : 0.f;
    v.z = c + 2 < F ? p[2] : 0.f;
    v.w = c + 3 < F ? p[3] : 0.f;
    dst[i] = v;
  }
}

struct LaunchArgs {
  const float *in;
  float *out;
  const float *w;
  const uint32_t *offsets;
  const uint32_t *indices;
  uint32_t index_base;
  uint32_t n_items;
  uint32_t F;
  const Item *items;
  float *partial;
  int accumulate;
  hipStream_t stream;
  HeadArgs heads = HeadArgs{nullptr, 0u, 0u};  // H == 0: one weight per edge
  uint32_t row_edge_limit = 0xFFFFFFFFu;       // whole-row launches skip rows with more edges than this
  const uint32_t *edge_ids = nullptr;          // schedules with their own index copy: edge -> caller's edge position
  uint32_t in_ld = 0;                          // row stride of `in` in floats (0 = F)
  uint32_t partial_ld = 0;                     // row stride of `partial` in floats (0 = F)
  bool dup_runs = false;                       // rows hold runs of equal indices worth loading once per run
  uint32_t rows_after_items = 0;               // with items: this many whole rows follow the listed items in the launch
};

template <int VEC, int NACC>
void launch_wave(const LaunchArgs &a, uint32_t col_base) {
  constexpr int kWavesPerBlock = 4;
  const uint32_t n_list = a.items ? a.n_items : 0u, n_total = a.n_items + (a.items ? a.rows_after_items : 0u);
  const uint32_t blocks = ceil_div(n_total, kWavesPerBlock);
  const dim3 grid(blocks), block(kWavesPerBlock * kWave);
  // Neighbour pairs always go through the wave-private LDS tile (a register-broadcast variant measured
  // the same: 12.44 ms against 12.40 ms for the 114.8 M-edge F=602 gather).
#define NTS_LAUNCH_WAVE(HD, RM, RUNS)                                                                                  \
  hipLaunchKernelGGL((spmm_wave_kernel<VEC, NACC, true, HD, RM, RUNS>), grid, block, 0, a.stream, a.in, a.out, a.w,    \
                     a.offsets, a.indices, a.index_base, n_total, n_list, a.F, col_base, a.items, a.partial,         \
                     a.accumulate,                                                                                     \
                     a.heads, a.row_edge_limit, a.edge_ids, a.in_ld ? a.in_ld : a.F,                                  \
                     a.partial_ld ? a.partial_ld : a.F,                                                                \
                     (VEC > 1 && (a.F % VEC != 0 || !aligned_to(a.out, 4 * VEC))) ? 1 : 0)
  if (a.edge_ids) {
    if (a.heads.H) NTS_LAUNCH_WAVE(true, true, false);
    else if (a.dup_runs) NTS_LAUNCH_WAVE(false, true, true);
    else NTS_LAUNCH_WAVE(false, true, false);
  } else {
    if (a.heads.H) NTS_LAUNCH_WAVE(true, false, false);
    else if (a.dup_runs) NTS_LAUNCH_WAVE(false, false, true);
    else NTS_LAUNCH_WAVE(false, false, false);
  }
#undef NTS_LAUNCH_WAVE
}

template <int G, int VEC>
void launch_group(const LaunchArgs &a) {
  const uint32_t per_block = 256 / G;
  const uint32_t n_list = a.items ? a.n_items : 0u, n_total = a.n_items + (a.items ? a.rows_after_items : 0u);
  const uint32_t blocks = ceil_div(n_total, per_block);
#define NTS_LAUNCH_GROUP(HD, RM, RUNS)                                                                                  \
  hipLaunchKernelGGL((spmm_group_kernel<G, VEC, HD, RM, RUNS>), dim3(blocks), dim3(256), 0, a.stream, a.in, a.out, a.w, \
                     a.offsets, a.indices, a.index_base, n_total, n_list, a.F, a.items, a.partial, a.accumulate,        \
                     a.heads,                                                                                          \
                     a.row_edge_limit, a.edge_ids)
  if (a.edge_ids) {
    if (a.heads.H) NTS_LAUNCH_GROUP(true, true, false);
    else if (a.dup_runs) NTS_LAUNCH_GROUP(false, true, true);
    else NTS_LAUNCH_GROUP(false, true, false);
  } else {
    if (a.heads.H) NTS_LAUNCH_GROUP(true, false, false);
    else if (a.dup_runs) NTS_LAUNCH_GROUP(false, false, true);
    else NTS_LAUNCH_GROUP(false, false, false);
  }
#undef NTS_LAUNCH_GROUP
}

template <int VEC>
void launch_wave_vec(const LaunchArgs &a) {
  // Column panels of at most 10 accumulators per lane, balanced; wider rows are covered by several
  // launches over disjoint column ranges (each panel re-walks the edge list; outputs are disjoint).
  constexpr uint32_t kMaxAcc = 10;
  const uint32_t per_acc = kWave * VEC;
  const uint32_t total_acc = ceil_div(a.F, per_acc);
  const uint32_t panels = ceil_div(total_acc, kMaxAcc);
  const uint32_t acc_per_panel = ceil_div(total_acc, panels);
  uint32_t col_base = 0;
  while (col_base < a.F) {
    const uint32_t remaining = a.F - col_base;
    uint32_t nacc = ceil_div(remaining, per_acc);
    if (nacc > acc_per_panel) nacc = acc_per_panel;
    switch (nacc) {
      case 1: launch_wave<VEC, 1>(a, col_base); break;
      case 2: launch_wave<VEC, 2>(a, col_base); break;
      case 3: launch_wave<VEC, 3>(a, col_base); break;
      case 4: launch_wave<VEC, 4>(a, col_base); break;
      case 5: launch_wave<VEC, 5>(a, col_base); break;
      case 6: launch_wave<VEC, 6>(a, col_base); break;
      case 7: launch_wave<VEC, 7>(a, col_base); break;
      case 8: launch_wave<VEC, 8>(a, col_base); break;
      case 9: launch_wave<VEC, 9>(a, col_base); break;
      default: launch_wave<VEC, 10>(a, col_base); break;
    }
    col_base += nacc * per_acc;
  }
}

// Vector width of the row loads: 16-byte lanes when every row starts 16-byte aligned (rows start
// at multiples of F floats from the base pointers), otherwise 4-byte lanes.  8-byte lanes are not
// used: measured on MI355X, dwordx2 gathers run ~20 % slower than either dword or dwordx4 gathers of
// the same bytes (F=512: 15.4 ms vs 12.8 / 11.7 ms; F=602: 18.8 ms vs 15.3 ms with dword lanes).
int pick_vec(const LaunchArgs &a) {
  const bool heads_ok = a.heads.H == 0 || a.heads.Fh % 4 == 0;  // a 16-byte lane must stay inside one head
  if (a.in_ld) {
    // Gather over a padded copy of the input (row stride a multiple of four floats): 16-byte lanes
    // whatever F is; output rows off a 16-byte boundary are stored float by float.
    const uint32_t pld = a.partial_ld ? a.partial_ld : a.F;
    if (a.in_ld % 4 == 0 && aligned_to(a.in, 16) && (!a.partial || (pld % 4 == 0 && aligned_to(a.partial, 16))) &&
        a.heads.H == 0)
      return 4;
    return 1;
  }
  const bool a16 = aligned_to(a.in, 16) && aligned_to(a.out, 16) && (!a.partial || aligned_to(a.partial, 16));
  if (a.F % 4 == 0 && a16 && heads_ok) return 4;
  return 1;
}

void launch_spmm(const LaunchArgs &a) {
  if (a.n_items == 0) return;
  const int vec = pick_vec(a);
  const uint32_t F = a.F;
  // Narrow rows: sub-wavefront groups so that lanes are not left idle.
  if (vec == 4 && F <= 16) return launch_group<4, 4>(a);
  if (vec == 4 && F <= 32) return launch_group<8, 4>(a);
  if (vec == 4 && F <= 64) return launch_group<16, 4>(a);
  if (vec == 4 && F <= 128) return launch_group<32, 4>(a);
  if (vec == 1 && F <= 4) return launch_group<4, 1>(a);
  if (vec == 1 && F <= 8) return launch_group<8, 1>(a);
  if (vec == 1 && F <= 16) return launch_group<16, 1>(a);
  if (vec == 1 && F <= 32) return launch_group<32, 1>(a);
  // Wave per row.
  if (vec == 4) return launch_wave_vec<4>(a);
  return launch_wave_vec<1>(a);
}

// ---- launches without a plan: hub rows are cut into pieces on the device ---------------------------
//
// A call that brings no plan still must not let one wavefront walk a 10^5-edge row alone.  For edge
// counts where that can matter, the pieces are derived on the device in the same stream, without
// any copy to the host: pieces[r] = ceil(deg/chunk) for rows longer than `chunk` = 256 edges (else 0), an
// exclusive scan gives each long row its first partial slot, one thread per possible piece writes
// the work item (binary search of the scan), whole-row wavefronts skip the long rows, the piece
// wavefronts write partial sums and a last kernel adds each long row's partials in slot order.
// The number of pieces is not known on the host, so grids and buffers are sized for its upper bound
// E/chunk + min(rows, E/chunk); surplus work items are empty.  Scratch is stream-ordered
// (hipMallocAsync / hipFreeAsync).  Calls below kAutoLargeEdges take the pieces' slots from a counter
// instead of a scan (launch_spmm_cut_small).

constexpr uint32_t kAutoMinEdges = 1u << 16;  // below this a serial hub row costs less than the set-up
// Piece length.  Shorter pieces mean more partial rows but also narrower index spans per piece
// (rows ascend), hence better locality once the pieces are ordered by source, and more parallelism
// for calls with few long rows: on the 114.8 M-edge graph at F=602 1,024-edge pieces take 18.9 ms,
// 256-edge pieces 16.3 ms; a 2.3 M-edge sampled layer has only 2,300 pieces of 1,024 edges.
constexpr uint32_t kAutoChunk = 256;
// Calls below this many edges (sampled layers) skip the ordering of the pieces by source: their
// source rows fit the caches anyway and every launch saved counts at this size.
constexpr uint32_t kAutoLargeEdges = 1u << 22;

// Pieces of row r: 0 for a row that fits one wavefront, else ceil(degree / chunk); 0 for r == rows,
// so that the exclusive scan's last entry is the total.  Evaluated inside the scan (no launch and no
// array of its own).
struct PieceCount {
  const uint32_t *off;
  uint32_t rows, chunk;
  __host__ __device__ uint32_t operator()(uint32_t r) const {
    if (r >= rows) return 0u;
    const uint32_t deg = off[r + 1] - off[r];
    return deg > chunk ? (deg + chunk - 1) / chunk : 0u;
  }
};
using PieceCountIterator = rocprim::transform_iterator<rocprim::counting_iterator<uint32_t>, PieceCount, uint32_t>;

// Also writes keys[i] = the gather index of the piece's first edge (0xFFFFFFFF for an empty item):
// the pieces are then issued in ascending key order, so that wavefronts resident at the same time
// gather from nearby source rows (with sorted adjacency a piece covers a narrow index range).
__global__ __launch_bounds__(256) void auto_items_kernel(Item *__restrict__ items, uint32_t *__restrict__ keys,
                                                         const uint32_t *__restrict__ base,
                                                         const uint32_t *__restrict__ off,
                                                         const uint32_t *__restrict__ indices, uint32_t index_base,
                                                         uint32_t rows, uint32_t chunk, uint32_t p_max) {
  const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= p_max) return;
  if (i >= base[rows]) {
    items[i] = make_uint4(0u, 0u, 0u, i);  // empty item: writes zeros to its own unused slot
    keys[i] = 0xFFFFFFFFu;
    return;
  }
  const uint32_t r = owner_of(base, rows, i);  // the last row whose first slot is <= i is the long row itself
  const uint32_t e0 = off[r] + (i - base[r]) * chunk;
  items[i] = make_uint4(r, e0, min(off[r + 1], e0 + chunk), i);
  keys[i] = indices[e0] - index_base;
}

__global__ __launch_bounds__(256) void auto_order_items_kernel(Item *__restrict__ ordered,
                                                               const Item *__restrict__ items,
                                                               const uint32_t *__restrict__ order, uint32_t p_max) {
  const uint32_t j = blockIdx.x * blockDim.x + threadIdx.x;
  if (j < p_max) ordered[j] = items[order[j]];
}

// Block (x, y): if work item x is the first piece of its row, adds that row's partials in slot order
// into out (256 columns per block, tile y).
__global__ __launch_bounds__(256) void auto_reduce_kernel(float *__restrict__ out, const float *__restrict__ partial,
                                                          const Item *__restrict__ items,
                                                          const uint32_t *__restrict__ base, uint32_t F,
                                                          int accumulate, uint32_t p_max) {
  const uint32_t i = blockIdx.x;
  const uint32_t r = items[i].x;
  if (base[r] != i) return;
  // Slots at or beyond p_max were never written (only possible when the caller's edge count is
  // smaller than offsets[rows]): they are not read.
  const uint32_t n = min(base[r + 1], p_max) - i;
  if (n == 0) return;
  const uint32_t c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= F) return;
  const float *src = partial + static_cast<size_t>(i) * F + c;
  float a = src[0];
  uint32_t k = 1;
  for (; k + 8 <= n; k += 8) {
    float v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = src[static_cast<size_t>(k + u) * F];
#pragma unroll
    for (int u = 0; u < 8; ++u) a += v[u];
  }
  for (; k < n; ++k) a += src[static_cast<size_t>(k) * F];
  float *dst = out + static_cast<size_t>(r) * F + c;
  if (accumulate) a += *dst;
  *dst = a;
}

// The same with one block per work item covering all columns (rows of up to 1,024 columns): whole,
// contiguous partial rows are read, and a third or a quarter as many blocks are launched.
template <int J>
__global__ __launch_bounds__(256) void auto_reduce_wide_kernel(float *__restrict__ out,
                                                               const float *__restrict__ partial,
                                                               const Item *__restrict__ items,
                                                               const uint32_t *__restrict__ base, uint32_t F,
                                                               int accumulate, uint32_t p_max) {
  const uint32_t i = blockIdx.x;
  const uint32_t r = items[i].x;
  if (base[r] != i) return;
  const uint32_t n = min(base[r + 1], p_max) - i;  // as in auto_reduce_kernel
  if (n == 0) return;
  const float *src = partial + static_cast<size_t>(i) * F;
  uint32_t c[J];
  bool live[J];
  float a[J];
#pragma unroll
  for (int j = 0; j < J; ++j) {
    c[j] = threadIdx.x + 256u * j;
    live[j] = c[j] < F;
    if (!live[j]) c[j] = F - 1;  // re-read the last column, never stored
    a[j] = src[c[j]];
  }
  uint32_t k = 1;
  for (; k + 8 <= n; k += 8) {
    float v[8][J];
#pragma unroll
    for (int u = 0; u < 8; ++u)
#pragma unroll
      for (int j = 0; j < J; ++j) v[u][j] = src[static_cast<size_t>(k + u) * F + c[j]];
#pragma unroll
    for (int u = 0; u < 8; ++u)
#pragma unroll
      for (int j = 0; j < J; ++j) a[j] += v[u][j];
  }
  for (; k < n; ++k)
#pragma unroll
    for (int j = 0; j < J; ++j) a[j] += src[static_cast<size_t>(k) * F + c[j]];
  float *dst = out + static_cast<size_t>(r) * F;
#pragma unroll
  for (int j = 0; j < J; ++j)
    if (live[j]) dst[c[j]] = accumulate ? a[j] + dst[c[j]] : a[j];
}

inline size_t up256(size_t v) { return (v + 255) / 256 * 256; }

// Calls below kAutoLargeEdges (sampled layers) need no order among the pieces, so they need no scan
// either: a long row takes its consecutive partial slots from a counter (integer atomic: which slots a
// row gets varies from call to call, the order of its pieces inside them and therefore every sum does
// not), and lists itself for the second stage.
//   ctr[0] = slots handed out, ctr[1] = rows listed.  Items are pre-filled as empty, so the slots beyond
//   the live count cost a wavefront that writes zeros to a slot nobody reads.
__global__ __launch_bounds__(256) void auto_fill_kernel(Item *__restrict__ items, uint32_t *__restrict__ ctr,
                                                        uint32_t p_max) {
  const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < 2) ctr[i] = 0;
  if (i < p_max) items[i] = make_uint4(0u, 0u, 0u, i);
}

__global__ __launch_bounds__(256) void auto_cut_kernel(Item *__restrict__ items, uint4 *__restrict__ splits,
                                                       uint32_t *__restrict__ ctr, const uint32_t *__restrict__ off,
                                                       uint32_t rows, uint32_t chunk, uint32_t p_max, uint32_t s_max) {
  const uint32_t r = blockIdx.x * blockDim.x + threadIdx.x;
  if (r >= rows) return;
  const uint32_t b = off[r], e = off[r + 1], deg = e - b;
  if (deg <= chunk) return;
  uint32_t n = (deg + chunk - 1) / chunk;
  const uint32_t first = atomicAdd(&ctr[0], n);
  // Slots at or beyond p_max do not exist (only possible when the caller's edge count is smaller than
  // offsets[rows]): such pieces are not created and not read.
  if (first >= p_max) return;
  if (first + n > p_max) n = p_max - first;
  for (uint32_t j = 0; j < n; ++j) {
    const uint32_t e0 = b + j * chunk;
    items[first + j] = make_uint4(r, e0, min(e, e0 + chunk), first + j);
  }
  const uint32_t s = atomicAdd(&ctr[1], 1u);
  if (s < s_max) splits[s] = make_uint4(r, first, n, 0u);
}

// Block (x, y): adds the partials of listed row x in slot order into out (256 columns per block, tile y).
__global__ __launch_bounds__(256) void auto_reduce_listed_kernel(float *__restrict__ out,
                                                                 const float *__restrict__ partial,
                                                                 const uint4 *__restrict__ splits,
                                                                 const uint32_t *__restrict__ ctr, uint32_t F,
                                                                 int accumulate, uint32_t s_max) {
  const uint32_t live = ctr[1] < s_max ? ctr[1] : s_max;
  if (blockIdx.x >= live) return;
  const uint4 sp = splits[blockIdx.x];
  const uint32_t c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= F || sp.z == 0) return;
  const float *src = partial + static_cast<size_t>(sp.y) * F + c;
  float a = src[0];
  uint32_t k = 1;
  for (; k + 8 <= sp.z; k += 8) {
    float v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = src[static_cast<size_t>(k + u) * F];
#pragma unroll
    for (int u = 0; u < 8; ++u) a += v[u];
  }
  for (; k < sp.z; ++k) a += src[static_cast<size_t>(k) * F];
  float *dst = out + static_cast<size_t>(sp.x) * F + c;
  if (accumulate) a += *dst;
  *dst = a;
}

int launch_spmm_cut_small(const LaunchArgs &a, uint32_t edges, unsigned char *fixed, size_t fixed_cap) {
  const uint32_t rows = a.n_items;
  const uint32_t chunk = kAutoChunk;
  const uint32_t by_edges = edges / chunk;
  const uint32_t s_max = (rows < by_edges ? rows : by_edges) + 1;  // rows of more than `chunk` edges
  const uint32_t p_max = by_edges + s_max;
  const size_t n_items_b = up256(static_cast<size_t>(p_max) * sizeof(Item));
  const size_t n_splits_b = up256(static_cast<size_t>(s_max) * sizeof(uint4));
  const size_t n_partial = up256(static_cast<size_t>(p_max) * a.F * sizeof(float));
  const size_t need = 256 + n_items_b + n_splits_b + n_partial;
  unsigned char *buf = fixed;
  if (fixed) {
    if (need > fixed_cap) {
      char msg[200];
      snprintf(msg, sizeof msg, "spmm: the call needs %zu bytes of scratch, the fixed scratch holds %zu", need,
               fixed_cap);
      return fail(NTS_ERR_INVALID, msg);
    }
  } else {
    NTS_HIP_TRY(scratch_alloc(reinterpret_cast<void **>(&buf), need, a.stream));
  }
  uint32_t *ctr = reinterpret_cast<uint32_t *>(buf);
  Item *items = reinterpret_cast<Item *>(buf + 256);
  uint4 *splits = reinterpret_cast<uint4 *>(buf + 256 + n_items_b);
  float *partial = reinterpret_cast<float *>(buf + 256 + n_items_b + n_splits_b);
  hipLaunchKernelGGL(auto_fill_kernel, dim3(ceil_div(p_max, 256)), dim3(256), 0, a.stream, items, ctr, p_max);
  hipLaunchKernelGGL(auto_cut_kernel, dim3(ceil_div(rows, 256)), dim3(256), 0, a.stream, items, splits, ctr, a.offsets,
                     rows, chunk, p_max, s_max);
  LaunchArgs pc = a;
  pc.n_items = p_max;
  pc.items = items;
  pc.partial = partial;
  pc.rows_after_items = rows;
  pc.row_edge_limit = chunk;
  launch_spmm(pc);
  hipLaunchKernelGGL(auto_reduce_listed_kernel, dim3(s_max, ceil_div(a.F, 256)), dim3(256), 0, a.stream, a.out, partial,
                     splits, ctr, a.F, a.accumulate, s_max);
  const hipError_t err = hipGetLastError();
  if (!fixed) {
    const hipError_t freed = scratch_free(buf, a.stream);
    if (err == hipSuccess && freed != hipSuccess) return fail_hip(freed, "spmm: scratch");
  }
  if (err != hipSuccess) return fail_hip(err, "spmm: balanced launch");
  return NTS_OK;
}

// `a` describes the whole-row launch (a.n_items = rows, no items).  Scratch comes from the library's
// stream-ordered pool, or, when `fixed` is set, from that caller-held region of `fixed_cap` bytes
// (nothing is allocated or freed then; a call that needs more is refused).
int launch_spmm_balanced(LaunchArgs a, uint32_t edges, unsigned char *fixed = nullptr, size_t fixed_cap = 0) {
  const uint32_t rows = a.n_items;
  if (edges < kAutoMinEdges) {
    launch_spmm(a);
    return NTS_OK;
  }
  const bool large = edges >= kAutoLargeEdges;
  if (!large) return launch_spmm_cut_small(a, edges, fixed, fixed_cap);
  const uint32_t chunk = kAutoChunk;
  const uint32_t by_edges = edges / chunk;
  const uint32_t p_max = by_edges + (rows < by_edges ? rows : by_edges) + 1;
  size_t scan_bytes = 0, sort_bytes = 0;
  {
    uint32_t *nul = nullptr;
    PieceCountIterator none(rocprim::counting_iterator<uint32_t>(0u), PieceCount{nullptr, 0u, chunk});
    NTS_HIP_TRY(rocprim::exclusive_scan(nullptr, scan_bytes, none, nul, 0u, static_cast<size_t>(rows) + 1,
                                        rocprim::plus<uint32_t>(), a.stream, false));
    NTS_HIP_TRY(rocprim::radix_sort_pairs(nullptr, sort_bytes, nul, nul, rocprim::counting_iterator<uint32_t>(0u), nul,
                                          p_max, 0u, 32u, a.stream, false));
  }
  const size_t tmp_bytes = up256(scan_bytes > sort_bytes ? scan_bytes : sort_bytes);
  const size_t n_off = up256((static_cast<size_t>(rows) + 1) * sizeof(uint32_t));
  const size_t n_items_b = up256(static_cast<size_t>(p_max) * sizeof(Item));
  const size_t n_keys_b = up256(static_cast<size_t>(p_max) * sizeof(uint32_t));
  const size_t n_partial = up256(static_cast<size_t>(p_max) * a.F * sizeof(float));
  const size_t need = n_off + 2 * n_items_b + 3 * n_keys_b + tmp_bytes + n_partial;
  unsigned char *buf = fixed;
  if (fixed) {
    if (need > fixed_cap) {
      char msg[200];
      snprintf(msg, sizeof msg, "spmm: the call needs %zu bytes of scratch, the fixed scratch holds %zu", need,
               fixed_cap);
      return fail(NTS_ERR_INVALID, msg);
    }
  } else {
    NTS_HIP_TRY(scratch_alloc(reinterpret_cast<void **>(&buf), need, a.stream));
  }
  unsigned char *cursor = buf;
  auto take = [&cursor](size_t bytes) {
    unsigned char *p = cursor;
    cursor += bytes;
    return p;
  };
  uint32_t *base = reinterpret_cast<uint32_t *>(take(n_off));
  Item *items = reinterpret_cast<Item *>(take(n_items_b));
  Item *ordered = reinterpret_cast<Item *>(take(n_items_b));
  uint32_t *keys = reinterpret_cast<uint32_t *>(take(n_keys_b));
  uint32_t *keys_sorted = reinterpret_cast<uint32_t *>(take(n_keys_b));
  uint32_t *order = reinterpret_cast<uint32_t *>(take(n_keys_b));
  void *tmp = take(tmp_bytes);
  float *partial = reinterpret_cast<float *>(take(n_partial));
  auto bail = [&](hipError_t err, const char *what) {
    if (!fixed) (void)scratch_free(buf, a.stream);
    return fail_hip(err, what);
  };
  PieceCountIterator counts(rocprim::counting_iterator<uint32_t>(0u), PieceCount{a.offsets, rows, chunk});
  hipError_t err = rocprim::exclusive_scan(tmp, scan_bytes, counts, base, 0u, static_cast<size_t>(rows) + 1,
                                           rocprim::plus<uint32_t>(), a.stream, false);
  if (err != hipSuccess) return bail(err, "spmm: scan of piece counts");
  hipLaunchKernelGGL(auto_items_kernel, dim3(ceil_div(p_max, 256)), dim3(256), 0, a.stream, items, keys, base, a.offsets,
                     a.indices, a.index_base, rows, chunk, p_max);
  err = hipGetLastError();
  if (err != hipSuccess) return bail(err, "auto_items_kernel");
  if (large) {
    err = rocprim::radix_sort_pairs(tmp, sort_bytes, keys, keys_sorted, rocprim::counting_iterator<uint32_t>(0u), order,
                                    p_max, 0u, 32u, a.stream, false);
    if (err != hipSuccess) return bail(err, "spmm: ordering of the pieces");
    hipLaunchKernelGGL(auto_order_items_kernel, dim3(ceil_div(p_max, 256)), dim3(256), 0, a.stream, ordered, items,
                       order, p_max);
    err = hipGetLastError();
    if (err != hipSuccess) return bail(err, "auto_order_items_kernel");
  }
  // One launch: the pieces first (the heavy, uniform work), then the rows that fit one wavefront,
  // so that the rows fill the chip while the last pieces, each a serial chain, finish.
  LaunchArgs pc = a;
  pc.n_items = p_max;
  pc.items = large ? ordered : items;
  pc.partial = partial;
  pc.rows_after_items = rows;
  pc.row_edge_limit = chunk;
  launch_spmm(pc);
#define NTS_AUTO_REDUCE_WIDE(J)                                                                                     \
  hipLaunchKernelGGL(auto_reduce_wide_kernel<J>, dim3(p_max), dim3(256), 0, a.stream, a.out, partial, items, base, a.F, \
                     a.accumulate, p_max)
  if (a.F > 256 && a.F <= 512)
    NTS_AUTO_REDUCE_WIDE(2);
  else if (a.F > 512 && a.F <= 768)
    NTS_AUTO_REDUCE_WIDE(3);
  else if (a.F > 768 && a.F <= 1024)
    NTS_AUTO_REDUCE_WIDE(4);
  else
    hipLaunchKernelGGL(auto_reduce_kernel, dim3(p_max, ceil_div(a.F, 256)), dim3(256), 0, a.stream, a.out, partial, items,
                       base, a.F, a.accumulate, p_max);
#undef NTS_AUTO_REDUCE_WIDE
  err = hipGetLastError();
  if (err != hipSuccess) return bail(err, "spmm: balanced launch");
  if (!fixed) NTS_HIP_TRY(scratch_free(buf, a.stream));
  return NTS_OK;
}

// ---- the same schedule built on the device -----------------------------------------------------------
//
// nts_spmm_plan_create_slabs needs the index array to cut rows at source-range boundaries; copying it
// to the host and scheduling there costs seconds per 10^8 edges.  The kernels below build the item
// list of make_schedule -- the same pieces, slots, order of pieces, order of whole rows and order of
// split rows, entry for entry -- from the arrays where they lie:
//   plan_cut_rows_kernel      one thread per row: the row's range count by its length, a lower_bound per
//                             range boundary, pieces per (row, range) into a [rows, n_slabs] table
//   exclusive scan of the table = first partial slot of every (row, range); its total = slots
//   plan_emit_pieces_kernel   one thread per non-empty (row, range): its pieces and their sort keys
//                             (range id, then longer pieces first); slot order is creation order, so a
//                             stable radix sort by key reproduces the host's stable_sort
//   plan_row_keys_kernel      per row: key of the whole rows (descending length, stable by row) and of
//                             the split rows (descending slot count, stable by row)
//   plan_finish_kernel        whole rows behind the pieces; the split-row table
// Rows long enough to be cut must ascend; plan_scan_edges_kernel lists every descent idx[k-1] > idx[k]
// (in a sorted graph these sit at row starts only) and plan_check_descents_kernel flags one inside such
// a row -- then the host path, which sorts those rows in a copy of its own, takes over.

struct PlanShape {
  uint32_t chunk, n_slabs, wide_ranges;
  uint64_t fine_width;
  // Ranges a row of `deg` edges is cut at (0 = the row stays whole): see make_schedule.
  __host__ __device__ uint32_t ranges_for(uint32_t deg) const {
    if (deg <= chunk) return (wide_ranges && deg > chunk / 4) ? wide_ranges : 0u;
    return (wide_ranges && deg <= 4ull * chunk) ? n_slabs / 2 : n_slabs;
  }
};

struct PlanCounters {  // device words read back once
  unsigned long long repeated_raw;  // k in [1, E) with idx[k] == idx[k-1], row starts included
  uint32_t boundary_equal;          // of those, the ones at a row start
  uint32_t n_descents;
  uint32_t descent_overflow;
  uint32_t unsorted_long_row;
  uint32_t n_splits;
  uint32_t pad;
};

__device__ __forceinline__ uint32_t lower_bound_index(const uint32_t *__restrict__ idx, uint32_t lo, uint32_t hi,
                                                      uint64_t lim, uint32_t base) {
  while (lo < hi) {
    const uint32_t mid = lo + (hi - lo) / 2;
    if (static_cast<uint64_t>(idx[mid] - base) < lim) lo = mid + 1; else hi = mid;
  }
  return lo;
}

__global__ __launch_bounds__(256) void plan_cut_rows_kernel(uint32_t *__restrict__ counts, uint32_t *__restrict__ stops,
                                                            const uint32_t *__restrict__ off,
                                                            const uint32_t *__restrict__ idx, uint32_t index_base,
                                                            uint32_t rows, PlanShape sh) {
  const uint32_t r = blockIdx.x * blockDim.x + threadIdx.x;
  if (r >= rows) return;
  const uint32_t b = off[r], e = off[r + 1], deg = e - b;
  const uint32_t R = sh.ranges_for(deg);
  if (R == 0) return;  // the table was cleared: a whole row has no pieces
  uint32_t *cnt = counts + static_cast<size_t>(r) * sh.n_slabs;
  uint32_t *stp = stops + static_cast<size_t>(r) * sh.n_slabs;
  const uint32_t per = sh.n_slabs / R;
  uint32_t cut = b, nonempty = 0;
  for (uint32_t c = 0; c < R; ++c) {
    const uint64_t hi = static_cast<uint64_t>(c + 1) * per * sh.fine_width;  // first index of the next range
    const uint32_t stop = (c + 1 == R || cut >= e) ? e : lower_bound_index(idx, cut, e, hi, index_base);
    const uint32_t n = stop - cut;
    cnt[c] = deg > sh.chunk ? (n + sh.chunk - 1) / sh.chunk : (n ? 1u : 0u);
    stp[c] = stop;
    nonempty += n ? 1u : 0u;
    cut = stop;
  }
  if (deg <= sh.chunk && nonempty <= 1)  // all edges in one wide range: the row stays whole
    for (uint32_t c = 0; c < R; ++c) cnt[c] = 0;
}

__global__ __launch_bounds__(256) void plan_emit_pieces_kernel(Item *__restrict__ pieces, uint32_t *__restrict__ keys,
                                                               const uint32_t *__restrict__ counts,
                                                               const uint32_t *__restrict__ stops,
                                                               const uint32_t *__restrict__ slot_base,
                                                               const uint32_t *__restrict__ off, uint32_t rows,
                                                               PlanShape sh) {
  const uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= static_cast<uint64_t>(rows) * sh.n_slabs) return;
  const uint32_t n = counts[i];
  if (!n) return;
  const uint32_t r = static_cast<uint32_t>(i / sh.n_slabs), c = static_cast<uint32_t>(i % sh.n_slabs);
  const uint32_t b = off[r], deg = off[r + 1] - b;
  const uint32_t per = sh.n_slabs / sh.ranges_for(deg);
  const uint32_t lo = c ? stops[i - 1] : b, hi = stops[i];
  const uint32_t first = slot_base[i];
  for (uint32_t j = 0; j < n; ++j) {
    const uint32_t e0 = lo + j * sh.chunk, e1 = min(hi, e0 + sh.chunk);
    pieces[first + j] = make_uint4(r, e0, e1, first + j);
    keys[first + j] = c * per * (sh.chunk + 1) + (sh.chunk - (e1 - e0));
  }
}

__global__ __launch_bounds__(256) void plan_row_keys_kernel(uint32_t *__restrict__ whole_key,
                                                            uint32_t *__restrict__ split_key,
                                                            const uint32_t *__restrict__ slot_base,
                                                            const uint32_t *__restrict__ off, uint32_t rows,
                                                            PlanShape sh, PlanCounters *__restrict__ counters) {
  const uint32_t r = blockIdx.x * blockDim.x + threadIdx.x;
  uint32_t split = 0;
  if (r < rows) {
    const uint32_t P = slot_base[static_cast<size_t>(r + 1) * sh.n_slabs] - slot_base[static_cast<size_t>(r) * sh.n_slabs];
    const uint32_t deg = off[r + 1] - off[r];
    whole_key[r] = P == 0 ? sh.chunk - deg : sh.chunk + 1;  // whole rows by descending length, cut rows last
    split_key[r] = ~P;                                      // split rows by descending slot count, whole rows last
    split = P ? 1u : 0u;
  }
  const uint32_t n = __popcll(__ballot(split));
  if ((threadIdx.x & (kWave - 1)) == 0 && n) atomicAdd(&counters->n_splits, n);
}

__global__ __launch_bounds__(256) void plan_finish_kernel(Item *__restrict__ items, uint4 *__restrict__ splits,
                                                          const uint32_t *__restrict__ whole_order,
                                                          const uint32_t *__restrict__ split_order,
                                                          const uint32_t *__restrict__ slot_base,
                                                          const uint32_t *__restrict__ off, uint32_t n_pieces,
                                                          uint32_t n_whole, uint32_t n_splits, uint32_t n_slabs) {
  const uint32_t j = blockIdx.x * blockDim.x + threadIdx.x;
  if (j < n_whole) {
    const uint32_t r = whole_order[j];
    items[n_pieces + j] = make_uint4(r, off[r], off[r + 1], kNoSlot);
  }
  if (j < n_splits) {
    const uint32_t r = split_order[j];
    const uint32_t first = slot_base[static_cast<size_t>(r) * n_slabs];
    splits[j] = make_uint4(r, first, slot_base[static_cast<size_t>(r + 1) * n_slabs] - first, 0u);
  }
}

__global__ __launch_bounds__(256) void plan_scan_edges_kernel(const uint32_t *__restrict__ idx, uint32_t edges,
                                                              uint32_t *__restrict__ descents, uint32_t descent_cap,
                                                              PlanCounters *__restrict__ counters) {
  unsigned long long equal = 0;
  for (uint64_t k = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x + 1; k < edges;
       k += static_cast<uint64_t>(gridDim.x) * blockDim.x) {
    const uint32_t a = idx[k - 1], b = idx[k];
    equal += a == b ? 1u : 0u;
    if (a > b) {
      const uint32_t at = atomicAdd(&counters->n_descents, 1u);  // list order does not matter
      if (at < descent_cap) descents[at] = static_cast<uint32_t>(k); else counters->descent_overflow = 1u;
    }
  }
#pragma unroll
  for (int m = kWave / 2; m >= 1; m >>= 1) equal += __shfl_xor(equal, m, kWave);
  if ((threadIdx.x & (kWave - 1)) == 0 && equal) atomicAdd(&counters->repeated_raw, equal);
}

__global__ __launch_bounds__(256) void plan_row_starts_kernel(const uint32_t *__restrict__ off,
                                                              const uint32_t *__restrict__ idx, uint32_t rows,
                                                              uint32_t edges, PlanCounters *__restrict__ counters) {
  const uint32_t r = blockIdx.x * blockDim.x + threadIdx.x + 1;
  uint32_t hit = 0;
  if (r < rows) {
    const uint32_t p = off[r];
    // every edge position that starts a row is met once: at the first row that starts there
    hit = (off[r - 1] < p && p < edges && idx[p] == idx[p - 1]) ? 1u : 0u;
  }
  const uint32_t n = __popcll(__ballot(hit));
  if ((threadIdx.x & (kWave - 1)) == 0 && n) atomicAdd(&counters->boundary_equal, n);
}

__global__ __launch_bounds__(256) void plan_check_descents_kernel(const uint32_t *__restrict__ descents,
                                                                  const uint32_t *__restrict__ off, uint32_t rows,
                                                                  uint32_t cut_above, uint32_t descent_cap,
                                                                  PlanCounters *__restrict__ counters) {
  const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
  const uint32_t n = min(counters->n_descents, descent_cap);
  if (i >= n) return;
  const uint32_t k = descents[i];
  const uint32_t r = owner_of(off, rows, k);
  if (k != off[r] && off[r + 1] - off[r] > cut_above) counters->unsorted_long_row = 1u;
}

int check_common(const float *in, float *out, const uint32_t *offsets, const uint32_t *indices, uint32_t rows,
                 uint32_t edges, uint32_t F, const char *who) {
  if (F == 0) return fail(NTS_ERR_INVALID, "spmm: feature width F is 0");
  if (rows == 0) return NTS_OK;
  if (!out || !offsets) return fail(NTS_ERR_INVALID, who);
  if (edges != 0 && (!in || !indices)) return fail(NTS_ERR_INVALID, who);
  return NTS_OK;
}

}  // namespace
}  // namespace nts

namespace {
// fn(first, last) over [0, n) on up to 16 host threads, in contiguous blocks.
template <typename Fn>
void parallel_blocks(uint32_t n, Fn fn) {
  unsigned t = std::thread::hardware_concurrency();
  if (t > 16) t = 16;
  if (t < 2 || n < 4096) {
    fn(0u, n);
    return;
  }
  std::vector<std::thread> pool;
  const uint32_t per = (n + t - 1) / t;
  for (uint32_t b = 0; b < n; b += per) pool.emplace_back(fn, b, std::min(n, b + per));
  for (std::thread &th : pool) th.join();
}

}  // namespace

struct nts_spmm_plan {
  uint32_t rows = 0;
  uint32_t edges = 0;
  uint32_t chunk = 0;
  uint32_t n_items = 0;
  uint32_t n_splits = 0;
  uint32_t n_partials = 0;
  const uint32_t *offsets = nullptr;  // identity check only
  uint4 *items = nullptr;             // device
  uint4 *splits = nullptr;            // device
  // Scratch shared by every call on this plan: the partial sums of split rows and, for widths whose
  // rows do not start on 16-byte boundaries, a padded copy of the input.  `mu` serialises the host
  // side of the calls (growing the scratch, enqueueing); `done` is recorded after the last kernel of
  // each call, and a call on another stream waits for it before it touches the scratch.
  float *partial = nullptr;           // device
  size_t partial_floats = 0;          // its capacity
  float *in_padded = nullptr;         // device
  size_t in_padded_floats = 0;
  uint32_t n_index = 0;               // rows of the gathered matrix (0 = not known: no padded copy)
  // At least 1 in 20 edges repeats the gather index of the edge before it: the wave kernel then loads
  // a row once per run of equal indices (and widths off 16-byte boundaries get the padded copy).
  bool dup_runs = false;
  uint64_t repeated_edges = 0;
  std::mutex mu;
  hipEvent_t done = nullptr;
  hipStream_t last_stream = nullptr;
  bool in_flight = false;
  // Only when rows had to be re-ordered for the source ranges: the schedule's own copy of the gather
  // indices (base already subtracted), and for each of its edges the position in the caller's order.
  uint32_t *sorted_idx = nullptr;     // device, [edges]
  uint32_t *edge_ids = nullptr;       // device, [edges]
  hipEvent_t ev_start = nullptr;      // optional profiling events around the main kernel
  hipEvent_t ev_stop = nullptr;
};

extern "C" {

int nts_spmm_gather(const float *in, float *out, const float *w, const uint32_t *offsets, const uint32_t *indices,
                    uint32_t index_base, uint32_t rows, uint32_t edges, uint32_t F, int accumulate,
                    nts_stream_t stream) {
  NTS_TRACE_RANGE("nts_spmm_gather");
  if (int rc = nts::check_common(in, out, offsets, indices, rows, edges, F, "nts_spmm_gather: null pointer")) return rc;
  if (rows == 0) return NTS_OK;
  nts::LaunchArgs a{in, out, w, offsets, indices, index_base, rows, F, nullptr, nullptr, accumulate, stream};
  if (int rc = nts::launch_spmm_balanced(a, edges)) return rc;
  NTS_LAUNCH_CHECK("nts_spmm_gather");
  return NTS_OK;
}

int nts_spmm_gather_bounded(const float *in, float *out, const float *w, const uint32_t *offsets,
                            const uint32_t *indices, uint32_t index_base, uint32_t rows, uint32_t edges, uint32_t F,
                            int accumulate, uint32_t max_row_edges, nts_stream_t stream) {
  NTS_TRACE_RANGE("nts_spmm_gather_bounded");
  if (int rc = nts::check_common(in, out, offsets, indices, rows, edges, F, "nts_spmm_gather_bounded: null pointer"))
    return rc;
  if (rows == 0) return NTS_OK;
  nts::LaunchArgs a{in, out, w, offsets, indices, index_base, rows, F, nullptr, nullptr, accumulate, stream};
  if (max_row_edges != 0 && max_row_edges <= nts::kAutoChunk) {
    // No row can need cutting: one launch, a wavefront (or lane group) per row, no scratch.
    nts::launch_spmm(a);
  } else if (int rc = nts::launch_spmm_balanced(a, edges)) {
    return rc;
  }
  NTS_LAUNCH_CHECK("nts_spmm_gather_bounded");
  return NTS_OK;
}

int nts_spmm_gather_static_scratch(const float *in, float *out, const float *w, const uint32_t *offsets,
                                   const uint32_t *indices, uint32_t index_base, uint32_t rows, uint32_t edges,
                                   uint32_t F, int accumulate, nts_stream_t stream) {
  NTS_TRACE_RANGE("nts_spmm_gather_static_scratch");
  if (int rc = nts::check_common(in, out, offsets, indices, rows, edges, F,
                                 "nts_spmm_gather_static_scratch: null pointer"))
    return rc;
  if (rows == 0) return NTS_OK;
  unsigned char *fixed = nullptr;
  if (int rc = nts::static_scratch_address(&fixed)) return rc;
  nts::LaunchArgs a{in, out, w, offsets, indices, index_base, rows, F, nullptr, nullptr, accumulate, stream};
  if (int rc = nts::launch_spmm_balanced(a, edges, fixed, kStaticScratchBytes)) return rc;
  NTS_LAUNCH_CHECK("nts_spmm_gather_static_scratch");
  return NTS_OK;
}

namespace {

struct Piece {
  uint32_t slab, row, e0, e1, slot;
};

// Builds the work-item list.  Rows with more than `chunk` edges are split into pieces that write
// partial sums (slots numbered in ascending edge order inside a row, so the second-stage sum has
// a fixed order).  With n_slabs > 1 and a host copy of the gather indices, pieces of rows whose
// indices ascend are additionally cut at the boundaries of n_slabs equal ranges of the gather
// index space and the pieces are ordered slab by slab: wavefronts that run at the same time then
// gather from the same 1/n_slabs of the source rows, which is what lets each 4 MB L2 keep that
// range's hot rows resident.  Items: all pieces (slab-major, longest first inside a slab), then
// the unsplit rows by descending degree.
struct Schedule {
  std::vector<uint4> items;   // (row, first edge, end edge, partial slot or kNoSlot)
  std::vector<uint4> splits;  // (row, first slot, slot count, 0)
  uint32_t n_partials = 0;
  // Empty unless some row that is cut by source range did not have ascending indices: then a copy
  // of the index array in which those rows are sorted (stable), and the original position of each
  // of its edges.  Rows that are never cut keep their order.
  std::vector<uint32_t> sorted_idx;
  std::vector<uint32_t> edge_ids;
  // Edges whose gather index equals that of the edge before them in the same row (parallel edges of
  // a multigraph, adjacent when rows are sorted); counted in the index array the schedule gathers through.
  uint64_t repeated_edges = 0;
};

// Host-only: needs nothing but the two index arrays.
void make_schedule(Schedule &out, const uint32_t *off, const uint32_t *idx_in, uint32_t rows, uint32_t chunk,
                   uint32_t n_slabs, uint32_t n_index) {
  const uint32_t *idx = idx_in;
  std::vector<Piece> pieces;
  std::vector<uint4> &splits = out.splits;
  uint32_t n_partials = 0;
  std::vector<uint32_t> bucket(static_cast<size_t>(chunk) + 2, 0u);
  const bool slabbed = n_slabs > 1 && idx != nullptr && n_index > 0;
  // Source ranges come in three widths and a row is cut at the width that suits its length: every
  // piece costs one partial row (written, then read by the second stage), so shorter rows get
  // fewer, wider ranges.
  //   more than 4 * chunk edges    n_slabs ranges
  //   more than chunk edges        n_slabs / 2 ranges (2,048-edge rows at 32 ranges would be cut into 19-edge
  //                                pieces on average; 24.7 -> 24.2 ms per four-pass step on the 114.8 M-edge graph)
  //   more than chunk / 4 edges    n_slabs / 4 ranges; a row whose edges all fall into one of them stays whole
  // A piece is issued with the first narrow range it covers, so that wavefronts resident at the
  // same time gather from the same part of the source rows whatever the width of their ranges.
  // (Twice or four times as many, narrower ranges for rows above 2,048 .. 16,384 edges were
  // measured as well: no gain on the 114.8 M-edge power-law graph.)
  const uint32_t fine = slabbed ? n_slabs : 1;
  const uint64_t fine_width = slabbed ? (static_cast<uint64_t>(n_index) + fine - 1) / fine : 0;
  const uint32_t wide_ranges = slabbed && n_slabs >= 8 ? n_slabs / 4 : 0;
  std::vector<uint8_t> was_cut(wide_ranges ? rows : 0, 0);
  if (slabbed) {
    // Rows long enough to be cut by source range must ascend.  Edge files are not always sorted
    // (the reference's loader leaves a CSR row in thread-arrival order), so such rows are sorted in
    // a copy of the index array that the schedule then gathers through; a stable sort, so equal
    // indices keep their edge order.  Sums of those rows are associated in source order.
    const uint32_t cut_above = wide_ranges ? chunk / 4 : chunk;
    std::vector<uint8_t> unsorted(rows, 0);
    std::atomic<bool> any(false);
    parallel_blocks(rows, [&](uint32_t r0, uint32_t r1) {
      for (uint32_t r = r0; r < r1; ++r) {
        const uint32_t b = off[r], e = off[r + 1];
        if (e - b <= cut_above) continue;
        for (uint32_t k = b + 1; k < e; ++k)
          if (idx_in[k - 1] > idx_in[k]) {
            unsorted[r] = 1;
            any.store(true, std::memory_order_relaxed);
            break;
          }
      }
    });
    if (any.load()) {
      const uint32_t edges = off[rows];
      out.sorted_idx.assign(idx_in, idx_in + edges);
      out.edge_ids.resize(edges);
      parallel_blocks(edges, [&](uint32_t e0, uint32_t e1) {
        for (uint32_t e = e0; e < e1; ++e) out.edge_ids[e] = e;
      });
      parallel_blocks(rows, [&](uint32_t r0, uint32_t r1) {
        for (uint32_t r = r0; r < r1; ++r) {
          if (!unsorted[r]) continue;
          uint32_t *ids = out.edge_ids.data() + off[r], *ids_end = out.edge_ids.data() + off[r + 1];
          std::stable_sort(ids, ids_end, [&](uint32_t a, uint32_t b) { return idx_in[a] < idx_in[b]; });
          for (uint32_t k = off[r]; k < off[r + 1]; ++k) out.sorted_idx[k] = idx_in[out.edge_ids[k]];
        }
      });
      idx = out.sorted_idx.data();
    }
  }
  std::vector<uint32_t> stops;  // (narrow range id, end edge) of the non-empty ranges of one row
  // Cuts edges [b, e) of a row with ascending indices at `ranges` equal ranges; ranges divides fine.
  auto range_stops = [&](uint32_t b, uint32_t e, uint32_t ranges) {
    stops.clear();
    const uint32_t per = fine / ranges;
    uint32_t cut = b;
    for (uint32_t c = 0; c < ranges && cut < e; ++c) {
      const uint64_t hi = static_cast<uint64_t>(c + 1) * per * fine_width;  // first index of the next range
      const uint32_t stop =
          c + 1 == ranges ? e
                          : static_cast<uint32_t>(std::lower_bound(idx + cut, idx + e, hi,
                                                                   [](uint32_t v, uint64_t lim) { return v < lim; }) -
                                                  idx);
      if (stop > cut) {
        stops.push_back(c * per);
        stops.push_back(stop);
      }
      cut = stop;
    }
  };
  for (uint32_t r = 0; r < rows; ++r) {
    const uint32_t b = off[r], e = off[r + 1], deg = e - b;
    if (deg <= chunk) {
      if (wide_ranges && deg > chunk / 4) {
        range_stops(b, e, wide_ranges);
        if (stops.size() > 2) {
          const uint32_t first = n_partials;
          uint32_t from = b;
          for (size_t q = 0; q < stops.size(); q += 2) {
            pieces.push_back(Piece{stops[q], r, from, stops[q + 1], n_partials++});
            from = stops[q + 1];
          }
          splits.push_back(make_uint4(r, first, n_partials - first, 0u));
          was_cut[r] = 1;
          continue;
        }
      }
      ++bucket[chunk - deg + 1];  // descending degree
      continue;
    }
    const uint32_t first = n_partials;
    if (slabbed) {
      range_stops(b, e, (wide_ranges && deg <= 4 * static_cast<uint64_t>(chunk)) ? n_slabs / 2 : n_slabs);
      uint32_t from = b;
      for (size_t q = 0; q < stops.size(); q += 2) {
        for (uint32_t k = from; k < stops[q + 1]; k += chunk)
          pieces.push_back(Piece{stops[q], r, k, std::min(stops[q + 1], k + chunk), n_partials++});
        from = stops[q + 1];
      }
    } else {
      for (uint32_t k = b; k < e; k += chunk) pieces.push_back(Piece{0u, r, k, std::min(e, k + chunk), n_partials++});
    }
    splits.push_back(make_uint4(r, first, n_partials - first, 0u));
  }
  if (idx) {
    std::atomic<uint64_t> repeated(0);
    parallel_blocks(rows, [&](uint32_t r0, uint32_t r1) {
      uint64_t n = 0;
      for (uint32_t r = r0; r < r1; ++r)
        for (uint32_t k = off[r] + 1; k < off[r + 1]; ++k) n += idx[k] == idx[k - 1];
      repeated.fetch_add(n, std::memory_order_relaxed);
    });
    out.repeated_edges = repeated.load();
  }
  std::stable_sort(splits.begin(), splits.end(), [](const uint4 &a, const uint4 &b) { return a.z > b.z; });
  std::stable_sort(pieces.begin(), pieces.end(), [](const Piece &a, const Piece &b) {
    if (a.slab != b.slab) return a.slab < b.slab;
    return (a.e1 - a.e0) > (b.e1 - b.e0);
  });
  std::vector<uint4> &items = out.items;
  items.reserve(pieces.size() + rows);
  for (const Piece &pc : pieces) items.push_back(make_uint4(pc.row, pc.e0, pc.e1, pc.slot));
  for (size_t i = 1; i < bucket.size(); ++i) bucket[i] += bucket[i - 1];
  const size_t base = items.size();
  items.resize(base + bucket.back());
  for (uint32_t r = 0; r < rows; ++r) {
    const uint32_t deg = off[r + 1] - off[r];
    if (deg <= chunk && !(wide_ranges && was_cut[r]))
      items[base + bucket[chunk - deg]++] = make_uint4(r, off[r], off[r + 1], nts::kNoSlot);
  }
  out.n_partials = n_partials;
}

int build_plan(nts_spmm_plan_t **plan_out, const uint32_t *offsets_dev, const std::vector<uint32_t> &off,
               const uint32_t *idx, uint32_t rows, uint32_t edges, uint32_t chunk, uint32_t n_slabs,
               uint32_t n_index) {
  Schedule sched;
  make_schedule(sched, off.data(), idx, rows, chunk, n_slabs, n_index);
  const std::vector<uint4> &items = sched.items;
  const std::vector<uint4> &splits = sched.splits;
  const uint32_t n_partials = sched.n_partials;

  nts_spmm_plan *p = new (std::nothrow) nts_spmm_plan();
  if (!p) return nts::fail(NTS_ERR_NOMEM, "nts_spmm_plan_create: host allocation failed");
  p->rows = rows;
  p->edges = edges;
  p->chunk = chunk;
  p->offsets = offsets_dev;
  p->n_items = static_cast<uint32_t>(items.size());
  p->n_splits = static_cast<uint32_t>(splits.size());
  p->n_partials = n_partials;
  p->n_index = n_index;
  p->repeated_edges = sched.repeated_edges;
  p->dup_runs = edges > 0 && sched.repeated_edges * 20 >= edges;
  hipError_t err = hipEventCreateWithFlags(&p->done, hipEventDisableTiming);
  if (err == hipSuccess && !items.empty()) {
    err = hipMalloc(reinterpret_cast<void **>(&p->items), items.size() * sizeof(uint4));
    if (err == hipSuccess)
      err = hipMemcpy(p->items, items.data(), items.size() * sizeof(uint4), hipMemcpyHostToDevice);
  }
  if (err == hipSuccess && !splits.empty()) {
    err = hipMalloc(reinterpret_cast<void **>(&p->splits), splits.size() * sizeof(uint4));
    if (err == hipSuccess)
      err = hipMemcpy(p->splits, splits.data(), splits.size() * sizeof(uint4), hipMemcpyHostToDevice);
  }
  if (err == hipSuccess && !sched.sorted_idx.empty()) {
    const size_t bytes = sched.sorted_idx.size() * sizeof(uint32_t);
    err = hipMalloc(reinterpret_cast<void **>(&p->sorted_idx), bytes);
    if (err == hipSuccess) err = hipMemcpy(p->sorted_idx, sched.sorted_idx.data(), bytes, hipMemcpyHostToDevice);
    if (err == hipSuccess) err = hipMalloc(reinterpret_cast<void **>(&p->edge_ids), bytes);
    if (err == hipSuccess) err = hipMemcpy(p->edge_ids, sched.edge_ids.data(), bytes, hipMemcpyHostToDevice);
  }
  if (err != hipSuccess) {
    nts_spmm_plan_destroy(p);
    return nts::fail_hip(err, "nts_spmm_plan_create: device upload");
  }
  *plan_out = p;
  return NTS_OK;
}

// Builds the schedule of make_schedule on the device (kernels above).  *fell_back is set, and nothing
// built, when a row that would be cut does not ascend (the host path sorts such rows in a copy).
int build_plan_device(nts_spmm_plan_t **plan_out, const uint32_t *offsets, const uint32_t *indices,
                      uint32_t index_base, uint32_t n_index, uint32_t rows, uint32_t edges, uint32_t chunk,
                      uint32_t n_slabs, hipStream_t stream, bool *fell_back) {
  using nts::Item;
  *fell_back = false;
  nts::PlanShape sh;
  sh.chunk = chunk;
  sh.n_slabs = n_slabs;
  sh.wide_ranges = n_slabs >= 8 ? n_slabs / 4 : 0;
  sh.fine_width = (static_cast<uint64_t>(n_index) + n_slabs - 1) / n_slabs;
  const size_t cells = static_cast<size_t>(rows) * n_slabs;
  const uint32_t descent_cap = rows + 1;
  unsigned key_bits = 1;
  while ((1ull << key_bits) < static_cast<uint64_t>(n_slabs) * (chunk + 1)) ++key_bits;
  unsigned whole_bits = 1;
  while ((1ull << whole_bits) < static_cast<uint64_t>(chunk) + 2) ++whole_bits;

  size_t scan_bytes = 0, sort_rows_bytes = 0;
  uint32_t *nul = nullptr;
  NTS_HIP_TRY(rocprim::exclusive_scan(nullptr, scan_bytes, nul, nul, 0u, cells + 1, rocprim::plus<uint32_t>(), stream,
                                      false));
  NTS_HIP_TRY(rocprim::radix_sort_pairs(nullptr, sort_rows_bytes, nul, nul, rocprim::counting_iterator<uint32_t>(0u), nul,
                                        rows, 0u, 32u, stream, false));
  const size_t tmp1_bytes = nts::up256(std::max(scan_bytes, sort_rows_bytes));
  const size_t cell_words = nts::up256((cells + 1) * sizeof(uint32_t));
  const size_t row_words = nts::up256((static_cast<size_t>(rows) + 1) * sizeof(uint32_t));
  struct Block {  // freed on every path out
    unsigned char *p = nullptr;
    ~Block() {
      if (p) (void)hipFree(p);
    }
  } work, work2;
  NTS_HIP_TRY(hipMalloc(reinterpret_cast<void **>(&work.p), 3 * cell_words + 7 * row_words + 256 + tmp1_bytes));
  unsigned char *cursor = work.p;
  auto take = [&cursor](size_t bytes) {
    unsigned char *q = cursor;
    cursor += bytes;
    return q;
  };
  uint32_t *counts = reinterpret_cast<uint32_t *>(take(cell_words));
  uint32_t *stops = reinterpret_cast<uint32_t *>(take(cell_words));
  uint32_t *slot_base = reinterpret_cast<uint32_t *>(take(cell_words));
  uint32_t *whole_key = reinterpret_cast<uint32_t *>(take(row_words));
  uint32_t *split_key = reinterpret_cast<uint32_t *>(take(row_words));
  uint32_t *key_sorted = reinterpret_cast<uint32_t *>(take(row_words));
  uint32_t *whole_order = reinterpret_cast<uint32_t *>(take(row_words));
  uint32_t *split_order = reinterpret_cast<uint32_t *>(take(row_words));
  uint32_t *descents = reinterpret_cast<uint32_t *>(take(2 * row_words));
  nts::PlanCounters *counters = reinterpret_cast<nts::PlanCounters *>(take(256));
  void *tmp1 = take(tmp1_bytes);

  NTS_HIP_TRY(hipMemsetAsync(counts, 0, (cells + 1) * sizeof(uint32_t), stream));
  NTS_HIP_TRY(hipMemsetAsync(counters, 0, sizeof(nts::PlanCounters), stream));
  const uint32_t row_blocks = nts::ceil_div(static_cast<uint64_t>(rows) + 1, 256);
  if (edges > 1) {
    const uint32_t edge_blocks = static_cast<uint32_t>(std::min<uint64_t>((static_cast<uint64_t>(edges) + 255) / 256, 1u << 14));
    hipLaunchKernelGGL(nts::plan_scan_edges_kernel, dim3(edge_blocks), dim3(256), 0, stream, indices, edges, descents,
                       descent_cap, counters);
    hipLaunchKernelGGL(nts::plan_row_starts_kernel, dim3(row_blocks), dim3(256), 0, stream, offsets, indices, rows, edges,
                       counters);
    hipLaunchKernelGGL(nts::plan_check_descents_kernel, dim3(row_blocks), dim3(256), 0, stream, descents, offsets, rows,
                       sh.wide_ranges ? chunk / 4 : chunk, descent_cap, counters);
  }
  hipLaunchKernelGGL(nts::plan_cut_rows_kernel, dim3(row_blocks), dim3(256), 0, stream, counts, stops, offsets, indices,
                     index_base, rows, sh);
  NTS_LAUNCH_CHECK("plan_cut_rows_kernel");
  NTS_HIP_TRY(rocprim::exclusive_scan(tmp1, scan_bytes, counts, slot_base, 0u, cells + 1, rocprim::plus<uint32_t>(),
                                      stream, false));
  hipLaunchKernelGGL(nts::plan_row_keys_kernel, dim3(row_blocks), dim3(256), 0, stream, whole_key, split_key, slot_base,
                     offsets, rows, sh, counters);
  NTS_LAUNCH_CHECK("plan_row_keys_kernel");
  nts::PlanCounters host_counters;
  uint32_t n_pieces = 0;
  NTS_HIP_TRY(hipMemcpyAsync(&host_counters, counters, sizeof(host_counters), hipMemcpyDeviceToHost, stream));
  NTS_HIP_TRY(hipMemcpyAsync(&n_pieces, slot_base + cells, sizeof(n_pieces), hipMemcpyDeviceToHost, stream));
  NTS_HIP_TRY(hipStreamSynchronize(stream));
  if (host_counters.unsorted_long_row || host_counters.descent_overflow) {
    *fell_back = true;
    return NTS_OK;
  }
  const uint32_t n_splits = host_counters.n_splits, n_whole = rows - n_splits;
  const uint64_t n_items64 = static_cast<uint64_t>(n_pieces) + n_whole;
  if (n_items64 > 0xFFFFFFF0ull) return nts::fail(NTS_ERR_INVALID, "nts_spmm_plan_create_slabs: too many work items");

  nts_spmm_plan *p = new (std::nothrow) nts_spmm_plan();
  if (!p) return nts::fail(NTS_ERR_NOMEM, "nts_spmm_plan_create_slabs: host allocation failed");
  p->rows = rows;
  p->edges = edges;
  p->chunk = chunk;
  p->offsets = offsets;
  p->n_items = static_cast<uint32_t>(n_items64);
  p->n_splits = n_splits;
  p->n_partials = n_pieces;
  p->n_index = n_index;
  p->repeated_edges = host_counters.repeated_raw - host_counters.boundary_equal;
  p->dup_runs = edges > 0 && p->repeated_edges * 20 >= edges;
  auto bail = [&](hipError_t err, const char *what) {
    nts_spmm_plan_destroy(p);
    return nts::fail_hip(err, what);
  };
  hipError_t err = hipEventCreateWithFlags(&p->done, hipEventDisableTiming);
  if (err == hipSuccess && p->n_items) err = hipMalloc(reinterpret_cast<void **>(&p->items), p->n_items * sizeof(uint4));
  if (err == hipSuccess && n_splits) err = hipMalloc(reinterpret_cast<void **>(&p->splits), n_splits * sizeof(uint4));
  if (err != hipSuccess) return bail(err, "nts_spmm_plan_create_slabs: device allocation");

  if (n_pieces) {
    size_t sort_pieces_bytes = 0;
    err = rocprim::radix_sort_pairs(nullptr, sort_pieces_bytes, nul, nul, rocprim::counting_iterator<uint32_t>(0u), nul,
                                    n_pieces, 0u, key_bits, stream, false);
    if (err != hipSuccess) return bail(err, "nts_spmm_plan_create_slabs: sort size");
    const size_t piece_items = nts::up256(static_cast<size_t>(n_pieces) * sizeof(Item));
    const size_t piece_words = nts::up256(static_cast<size_t>(n_pieces) * sizeof(uint32_t));
    err = hipMalloc(reinterpret_cast<void **>(&work2.p), piece_items + 3 * piece_words + nts::up256(sort_pieces_bytes));
    if (err != hipSuccess) return bail(err, "nts_spmm_plan_create_slabs: device allocation");
    Item *pieces = reinterpret_cast<Item *>(work2.p);
    uint32_t *keys = reinterpret_cast<uint32_t *>(work2.p + piece_items);
    uint32_t *keys_sorted = reinterpret_cast<uint32_t *>(work2.p + piece_items + piece_words);
    uint32_t *order = reinterpret_cast<uint32_t *>(work2.p + piece_items + 2 * piece_words);
    void *tmp2 = work2.p + piece_items + 3 * piece_words;
    hipLaunchKernelGGL(nts::plan_emit_pieces_kernel, dim3(nts::ceil_div(cells, 256)), dim3(256), 0, stream, pieces, keys,
                       counts, stops, slot_base, offsets, rows, sh);
    err = hipGetLastError();
    if (err == hipSuccess)
      err = rocprim::radix_sort_pairs(tmp2, sort_pieces_bytes, keys, keys_sorted, rocprim::counting_iterator<uint32_t>(0u),
                                      order, n_pieces, 0u, key_bits, stream, false);
    if (err != hipSuccess) return bail(err, "nts_spmm_plan_create_slabs: ordering of the pieces");
    hipLaunchKernelGGL(nts::auto_order_items_kernel, dim3(nts::ceil_div(n_pieces, 256)), dim3(256), 0, stream, p->items,
                       pieces, order, n_pieces);
  }
  err = rocprim::radix_sort_pairs(tmp1, sort_rows_bytes, whole_key, key_sorted, rocprim::counting_iterator<uint32_t>(0u),
                                  whole_order, rows, 0u, whole_bits, stream, false);
  if (err == hipSuccess)
    err = rocprim::radix_sort_pairs(tmp1, sort_rows_bytes, split_key, key_sorted, rocprim::counting_iterator<uint32_t>(0u),
                                    split_order, rows, 0u, 32u, stream, false);
  if (err != hipSuccess) return bail(err, "nts_spmm_plan_create_slabs: ordering of the rows");
  if (n_whole || n_splits)
    hipLaunchKernelGGL(nts::plan_finish_kernel, dim3(nts::ceil_div(std::max(n_whole, n_splits), 256)), dim3(256), 0, stream,
                       p->items, p->splits, whole_order, split_order, slot_base, offsets, n_pieces, n_whole, n_splits,
                       n_slabs);
  err = hipGetLastError();
  if (err == hipSuccess) err = hipStreamSynchronize(stream);
  if (err != hipSuccess) return bail(err, "nts_spmm_plan_create_slabs: device schedule");
  *plan_out = p;
  return NTS_OK;
}

int read_offsets(std::vector<uint32_t> &off, const uint32_t *offsets, uint32_t rows, uint32_t edges,
                 hipStream_t stream) {
  off.assign(static_cast<size_t>(rows) + 1, 0u);
  if (!rows) return NTS_OK;
  NTS_HIP_TRY(hipMemcpyAsync(off.data(), offsets, off.size() * sizeof(uint32_t), hipMemcpyDeviceToHost, stream));
  NTS_HIP_TRY(hipStreamSynchronize(stream));
  if (off[rows] != edges) return nts::fail(NTS_ERR_INVALID, "nts_spmm_plan_create: offsets[rows] != edges");
  for (uint32_t r = 0; r < rows; ++r)
    if (off[r + 1] < off[r]) return nts::fail(NTS_ERR_INVALID, "nts_spmm_plan_create: offsets not ascending");
  return NTS_OK;
}

}  // namespace

int nts_spmm_plan_create(nts_spmm_plan_t **plan_out, const uint32_t *offsets, uint32_t rows, uint32_t edges,
                         uint32_t chunk_edges, nts_stream_t stream) {
  NTS_TRACE_RANGE("nts_spmm_plan_create");
  if (!plan_out) return nts::fail(NTS_ERR_INVALID, "nts_spmm_plan_create: null out-pointer");
  *plan_out = nullptr;
  if (rows != 0 && !offsets) return nts::fail(NTS_ERR_INVALID, "nts_spmm_plan_create: null offsets");
  std::vector<uint32_t> off;
  if (int rc = read_offsets(off, offsets, rows, edges, stream)) return rc;
  return build_plan(plan_out, offsets, off, nullptr, rows, edges, chunk_edges ? chunk_edges : 4096u, 1u, 0u);
}

int nts_spmm_plan_create_slabs(nts_spmm_plan_t **plan_out, const uint32_t *offsets, const uint32_t *indices,
                               uint32_t index_base, uint32_t n_index, uint32_t rows, uint32_t edges,
                               uint32_t chunk_edges, uint32_t n_slabs, nts_stream_t stream) {
  NTS_TRACE_RANGE("nts_spmm_plan_create_slabs");
  if (!plan_out) return nts::fail(NTS_ERR_INVALID, "nts_spmm_plan_create_slabs: null out-pointer");
  *plan_out = nullptr;
  if (rows != 0 && !offsets) return nts::fail(NTS_ERR_INVALID, "nts_spmm_plan_create_slabs: null offsets");
  if (edges != 0 && !indices) return nts::fail(NTS_ERR_INVALID, "nts_spmm_plan_create_slabs: null indices");
  std::vector<uint32_t> off;
  if (int rc = read_offsets(off, offsets, rows, edges, stream)) return rc;
  const uint32_t chunk = chunk_edges ? chunk_edges : 512u, slabs = n_slabs ? n_slabs : 32u;
  // The schedule is built on the device where that reproduces the host's (source ranges in use, sizes
  // within the 32-bit sort keys and the range table); NTS_SPMM_PLAN_HOST=1 forces the host path.
  static const bool force_host = [] {
    const char *e = getenv("NTS_SPMM_PLAN_HOST");
    return e && e[0] != '0';
  }();
  if (!force_host && slabs > 1 && n_index > 0 && rows > 0 && edges > 0 &&
      static_cast<uint64_t>(slabs) * (static_cast<uint64_t>(chunk) + 1) < (1ull << 32) && slabs <= 4096 &&
      static_cast<uint64_t>(rows) * slabs < (1ull << 31)) {
    bool fell_back = false;
    if (int rc = build_plan_device(plan_out, offsets, indices, index_base, n_index, rows, edges, chunk, slabs, stream,
                                   &fell_back))
      return rc;
    if (!fell_back) return NTS_OK;
  }
  std::vector<uint32_t> idx(edges);
  if (edges) {
    NTS_HIP_TRY(hipMemcpyAsync(idx.data(), indices, idx.size() * sizeof(uint32_t), hipMemcpyDeviceToHost, stream));
    NTS_HIP_TRY(hipStreamSynchronize(stream));
    if (index_base)
      for (uint32_t &v : idx) v -= index_base;
  }
  return build_plan(plan_out, offsets, off, idx.data(), rows, edges, chunk, slabs, n_index);
}

int nts_spmm_plan_schedule_host(const uint32_t *offsets_host, const uint32_t *indices_host, uint32_t n_index,
                                uint32_t rows, uint32_t chunk_edges, uint32_t n_slabs, uint32_t *items_out,
                                uint64_t items_cap, uint32_t *n_items, uint32_t *n_split_rows, uint32_t *n_partials) {
  if (rows != 0 && !offsets_host) return nts::fail(NTS_ERR_INVALID, "nts_spmm_plan_schedule_host: null offsets");
  for (uint32_t r = 0; r < rows; ++r)
    if (offsets_host[r + 1] < offsets_host[r])
      return nts::fail(NTS_ERR_INVALID, "nts_spmm_plan_schedule_host: offsets not ascending");
  if (rows && offsets_host[rows] != 0 && n_slabs > 1 && !indices_host)
    return nts::fail(NTS_ERR_INVALID, "nts_spmm_plan_schedule_host: null indices");
  Schedule sched;
  const bool with_ranges = indices_host != nullptr;
  make_schedule(sched, offsets_host, indices_host, rows, chunk_edges ? chunk_edges : (with_ranges ? 512u : 4096u),
                with_ranges ? (n_slabs ? n_slabs : 32u) : 1u, n_index);
  if (n_items) *n_items = static_cast<uint32_t>(sched.items.size());
  if (n_split_rows) *n_split_rows = static_cast<uint32_t>(sched.splits.size());
  if (n_partials) *n_partials = sched.n_partials;
  if (items_out) {
    if (items_cap < sched.items.size())
      return nts::fail(NTS_ERR_INVALID, "nts_spmm_plan_schedule_host: items_out too small");
    memcpy(items_out, sched.items.data(), sched.items.size() * sizeof(uint4));
  }
  return NTS_OK;
}

int nts_spmm_plan_destroy(nts_spmm_plan_t *plan) {
  NTS_TRACE_RANGE("nts_spmm_plan_destroy");
  if (!plan) return NTS_OK;
  { std::lock_guard<std::mutex> lock(plan->mu); }  // a call that is still enqueueing finishes first
  hipError_t e1 = plan->items ? hipFree(plan->items) : hipSuccess;
  hipError_t e2 = plan->splits ? hipFree(plan->splits) : hipSuccess;
  hipError_t e3 = plan->partial ? hipFree(plan->partial) : hipSuccess;
  if (plan->in_padded && hipFree(plan->in_padded) != hipSuccess) e3 = hipErrorUnknown;
  if (plan->done && hipEventDestroy(plan->done) != hipSuccess) e3 = hipErrorUnknown;
  if (plan->sorted_idx && hipFree(plan->sorted_idx) != hipSuccess) e3 = hipErrorUnknown;
  if (plan->edge_ids && hipFree(plan->edge_ids) != hipSuccess) e3 = hipErrorUnknown;
  delete plan;
  if (e1 != hipSuccess) return nts::fail_hip(e1, "nts_spmm_plan_destroy");
  if (e2 != hipSuccess) return nts::fail_hip(e2, "nts_spmm_plan_destroy");
  if (e3 != hipSuccess) return nts::fail_hip(e3, "nts_spmm_plan_destroy");
  return NTS_OK;
}

int nts_spmm_plan_copy_schedule(const nts_spmm_plan_t *plan, uint32_t *items_out, uint64_t items_cap,
                                uint32_t *splits_out, uint64_t splits_cap) {
  NTS_TRACE_RANGE("nts_spmm_plan_copy_schedule");
  if (!plan) return nts::fail(NTS_ERR_INVALID, "nts_spmm_plan_copy_schedule: null plan");
  if (items_out) {
    if (items_cap < plan->n_items) return nts::fail(NTS_ERR_INVALID, "nts_spmm_plan_copy_schedule: items_out too small");
    if (plan->n_items)
      NTS_HIP_TRY(hipMemcpy(items_out, plan->items, plan->n_items * sizeof(uint4), hipMemcpyDeviceToHost));
  }
  if (splits_out) {
    if (splits_cap < plan->n_splits)
      return nts::fail(NTS_ERR_INVALID, "nts_spmm_plan_copy_schedule: splits_out too small");
    if (plan->n_splits)
      NTS_HIP_TRY(hipMemcpy(splits_out, plan->splits, plan->n_splits * sizeof(uint4), hipMemcpyDeviceToHost));
  }
  return NTS_OK;
}

int nts_spmm_plan_info(const nts_spmm_plan_t *plan, uint32_t *items, uint32_t *split_rows, uint32_t *partials) {
  NTS_TRACE_RANGE("nts_spmm_plan_info");
  if (!plan) return nts::fail(NTS_ERR_INVALID, "nts_spmm_plan_info: null plan");
  if (items) *items = plan->n_items;
  if (split_rows) *split_rows = plan->n_splits;
  if (partials) *partials = plan->n_partials;
  return NTS_OK;
}

namespace {

// Row stride, in floats, of the padded input copy and of the partial sums for width F: rows of more
// than 128 floats that do not start on 16-byte boundaries can be gathered from a copy whose rows are
// padded to a multiple of 32 floats (whole 128-byte lines), so that the gather runs with 16-byte
// lanes -- three loads per neighbour row at F = 602 instead of ten.  0 = no copy (F itself is the
// stride).  Measured on the 114.8 M-edge R-MAT graph at F = 602: with one load per run of equal
// indices the copy pays (9.75 -> 9.21 ms per pass, the 0.25 ms copy not included; 25.7 -> 25.0 ms per
// four-pass step with it); without runs it does not (11.05 -> 11.7 ms, and 8.79 -> 8.93 ms on the same
// graph with its parallel edges removed), so only schedules with runs use it.  NTS_SPMM_PAD=0 / 1 in
// the environment forces it off / on.
uint32_t padded_stride(const nts_spmm_plan *plan, uint32_t F, bool heads) {
  static const int forced = [] {
    const char *e = getenv("NTS_SPMM_PAD");
    return e ? (e[0] != '0' ? 1 : 0) : -1;
  }();
  if (heads || plan->n_index == 0 || F <= 128 || F % 4 == 0) return 0;
  if (forced == 0 || (forced < 0 && !plan->dup_runs)) return 0;
  return (F + 31) / 32 * 32;
}

// NTS_SPMM_RUNS=0 / 1 forces the one-load-per-run kernel off / on whatever the schedule found.
bool use_runs(const nts_spmm_plan *plan) {
  static const int forced = [] {
    const char *e = getenv("NTS_SPMM_RUNS");
    return e ? (e[0] != '0' ? 1 : 0) : -1;
  }();
  return forced < 0 ? plan->dup_runs : forced == 1;
}

// Grows the plan's scratch for width F.  Caller holds plan->mu.
int reserve_locked(nts_spmm_plan *plan, uint32_t F, bool heads) {
  const uint32_t ld = padded_stride(plan, F, heads);
  const size_t want_partial = static_cast<size_t>(plan->n_partials) * (ld ? ld : F);
  const size_t want_padded = ld ? static_cast<size_t>(plan->n_index) * ld : 0;
  if (want_partial > plan->partial_floats) {
    // The old buffer may still be read by work queued earlier: hipFree waits for the device.
    if (plan->partial) {
      NTS_HIP_TRY(hipFree(plan->partial));
      plan->partial = nullptr;
      plan->partial_floats = 0;
    }
    NTS_HIP_TRY(hipMalloc(reinterpret_cast<void **>(&plan->partial), want_partial * sizeof(float)));
    plan->partial_floats = want_partial;
  }
  if (want_padded > plan->in_padded_floats) {
    if (plan->in_padded) {
      NTS_HIP_TRY(hipFree(plan->in_padded));
      plan->in_padded = nullptr;
      plan->in_padded_floats = 0;
    }
    NTS_HIP_TRY(hipMalloc(reinterpret_cast<void **>(&plan->in_padded), want_padded * sizeof(float)));
    plan->in_padded_floats = want_padded;
  }
  return NTS_OK;
}

// A call on `stream` is about to use the plan's scratch: if the previous call ran on another stream,
// `stream` first waits for it (in stream order, the host does not block).  Caller holds plan->mu.
// A stream that is being captured records its launches instead of running them: a call under capture
// neither waits for the plan's event (that would pull the other stream's work into the capture, or
// fail) nor records it, and leaves the plan's bookkeeping alone -- replays of the captured call are
// ordered against other uses of the plan by the caller.
bool stream_is_capturing(hipStream_t stream) {
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &status) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  return status != hipStreamCaptureStatusNone;
}
int enter_stream(nts_spmm_plan *plan, hipStream_t stream) {
  if (stream_is_capturing(stream)) return NTS_OK;
  if (plan->in_flight && plan->last_stream != stream) NTS_HIP_TRY(hipStreamWaitEvent(stream, plan->done, 0));
  return NTS_OK;
}
int leave_stream(nts_spmm_plan *plan, hipStream_t stream) {
  if (stream_is_capturing(stream)) return NTS_OK;
  NTS_HIP_TRY(hipEventRecord(plan->done, stream));
  plan->last_stream = stream;
  plan->in_flight = true;
  return NTS_OK;
}

}  // namespace

int nts_spmm_plan_scratch_info(nts_spmm_plan_t *plan, uint32_t F, size_t *partial_bytes, size_t *padded_input_bytes,
                               uint64_t *repeated_edges, int *loads_once_per_run) {
  NTS_TRACE_RANGE("nts_spmm_plan_scratch_info");
  if (!plan) return nts::fail(NTS_ERR_INVALID, "nts_spmm_plan_scratch_info: null plan");
  if (F == 0) return nts::fail(NTS_ERR_INVALID, "nts_spmm_plan_scratch_info: F is 0");
  const uint32_t ld = padded_stride(plan, F, false);
  if (partial_bytes) *partial_bytes = static_cast<size_t>(plan->n_partials) * (ld ? ld : F) * sizeof(float);
  if (padded_input_bytes) *padded_input_bytes = ld ? static_cast<size_t>(plan->n_index) * ld * sizeof(float) : 0;
  if (repeated_edges) *repeated_edges = plan->repeated_edges;
  if (loads_once_per_run) *loads_once_per_run = use_runs(plan) ? 1 : 0;
  return NTS_OK;
}

int nts_spmm_plan_reserve(nts_spmm_plan_t *plan, uint32_t F) {
  NTS_TRACE_RANGE("nts_spmm_plan_reserve");
  if (!plan) return nts::fail(NTS_ERR_INVALID, "nts_spmm_plan_reserve: null plan");
  if (F == 0) return nts::fail(NTS_ERR_INVALID, "nts_spmm_plan_reserve: F is 0");
  std::lock_guard<std::mutex> lock(plan->mu);
  return reserve_locked(plan, F, false);
}

namespace {
int check_heads(const float *alpha, uint32_t H, uint32_t Fh, const char *who) {
  if (H == 0 || Fh == 0) return nts::fail(NTS_ERR_INVALID, who);
  if (static_cast<uint64_t>(H) * Fh > 0xFFFFFFFFull) return nts::fail(NTS_ERR_INVALID, who);
  if (!alpha) return nts::fail(NTS_ERR_INVALID, who);
  return NTS_OK;
}
}  // namespace

int nts_spmm_gather_heads(const float *in, float *out, const float *alpha, const uint32_t *perm,
                          const uint32_t *offsets, const uint32_t *indices, uint32_t rows, uint32_t edges, uint32_t H,
                          uint32_t Fh, int accumulate, nts_stream_t stream) {
  NTS_TRACE_RANGE("nts_spmm_gather_heads");
  if (int rc = check_heads(alpha, H, Fh, "nts_spmm_gather_heads: bad H / Fh / alpha")) return rc;
  if (rows == 0) return NTS_OK;
  if (!in || !out || !offsets || !indices) return nts::fail(NTS_ERR_INVALID, "nts_spmm_gather_heads: null pointer");
  nts::LaunchArgs a{in, out, alpha, offsets, indices, 0u, rows, H * Fh, nullptr, nullptr, accumulate, stream};
  a.heads = nts::HeadArgs{perm, H, Fh};
  if (int rc = nts::launch_spmm_balanced(a, edges)) return rc;
  NTS_LAUNCH_CHECK("nts_spmm_gather_heads");
  return NTS_OK;
}

int nts_spmm_gather_heads_bounded(const float *in, float *out, const float *alpha, const uint32_t *perm,
                                  const uint32_t *offsets, const uint32_t *indices, uint32_t rows, uint32_t edges,
                                  uint32_t H, uint32_t Fh, int accumulate, uint32_t max_row_edges, nts_stream_t stream) {
  NTS_TRACE_RANGE("nts_spmm_gather_heads_bounded");
  if (int rc = check_heads(alpha, H, Fh, "nts_spmm_gather_heads_bounded: bad H / Fh / alpha")) return rc;
  if (rows == 0) return NTS_OK;
  if (!in || !out || !offsets || !indices)
    return nts::fail(NTS_ERR_INVALID, "nts_spmm_gather_heads_bounded: null pointer");
  nts::LaunchArgs a{in, out, alpha, offsets, indices, 0u, rows, H * Fh, nullptr, nullptr, accumulate, stream};
  a.heads = nts::HeadArgs{perm, H, Fh};
  if (max_row_edges != 0 && max_row_edges <= nts::kAutoChunk) {
    nts::launch_spmm(a);
  } else if (int rc = nts::launch_spmm_balanced(a, edges)) {
    return rc;
  }
  NTS_LAUNCH_CHECK("nts_spmm_gather_heads_bounded");
  return NTS_OK;
}

int nts_spmm_gather_heads_planned(nts_spmm_plan_t *plan, const float *in, float *out, const float *alpha,
                                  const uint32_t *perm, const uint32_t *offsets, const uint32_t *indices, uint32_t H,
                                  uint32_t Fh, int accumulate, nts_stream_t stream) {
  NTS_TRACE_RANGE("nts_spmm_gather_heads_planned");
  if (!plan) return nts::fail(NTS_ERR_INVALID, "nts_spmm_gather_heads_planned: null plan");
  if (offsets != plan->offsets)
    return nts::fail(NTS_ERR_INVALID,
                     "nts_spmm_gather_heads_planned: offsets differ from the array the plan was built from");
  if (int rc = check_heads(alpha, H, Fh, "nts_spmm_gather_heads_planned: bad H / Fh / alpha")) return rc;
  const uint32_t F = H * Fh;
  if (int rc = nts::check_common(in, out, offsets, indices, plan->rows, plan->edges, F,
                                 "nts_spmm_gather_heads_planned: null pointer"))
    return rc;
  if (plan->rows == 0) return NTS_OK;
  std::lock_guard<std::mutex> lock(plan->mu);
  if (int rc = reserve_locked(plan, F, true)) return rc;
  if (int rc = enter_stream(plan, stream)) return rc;
  nts::LaunchArgs a{in,  out,         alpha,         offsets,    indices, 0u, plan->n_items,
                    F,   plan->items, plan->partial, accumulate, stream};
  a.heads = nts::HeadArgs{perm, H, Fh};
  if (plan->sorted_idx) {
    a.indices = plan->sorted_idx;
    a.edge_ids = plan->edge_ids;
  }
  nts::launch_spmm(a);
  NTS_LAUNCH_CHECK("nts_spmm_gather_heads_planned");
  if (plan->n_splits) {
    nts::launch_reduce_partials(out, plan->partial, plan->splits, plan->n_splits, F, accumulate, stream);
    NTS_LAUNCH_CHECK("spmm_reduce_partials_kernel");
  }
  return leave_stream(plan, stream);
}

int nts_spmm_plan_set_events(nts_spmm_plan_t *plan, nts_event_t start, nts_event_t stop) {
  NTS_TRACE_RANGE("nts_spmm_plan_set_events");
  if (!plan) return nts::fail(NTS_ERR_INVALID, "nts_spmm_plan_set_events: null plan");
  if ((start == nullptr) != (stop == nullptr))
    return nts::fail(NTS_ERR_INVALID, "nts_spmm_plan_set_events: pass both events or neither");
  plan->ev_start = start;
  plan->ev_stop = stop;
  return NTS_OK;
}

int nts_spmm_gather_planned(nts_spmm_plan_t *plan, const float *in, float *out, const float *w,
                            const uint32_t *offsets, const uint32_t *indices, uint32_t index_base, uint32_t F,
                            int accumulate, nts_stream_t stream) {
  NTS_TRACE_RANGE("nts_spmm_gather_planned");
  if (!plan) return nts::fail(NTS_ERR_INVALID, "nts_spmm_gather_planned: null plan");
  if (offsets != plan->offsets)
    return nts::fail(NTS_ERR_INVALID, "nts_spmm_gather_planned: offsets differ from the array the plan was built from");
  if (int rc = nts::check_common(in, out, offsets, indices, plan->rows, plan->edges, F,
                                 "nts_spmm_gather_planned: null pointer"))
    return rc;
  if (plan->rows == 0) return NTS_OK;
  std::lock_guard<std::mutex> lock(plan->mu);
  if (int rc = reserve_locked(plan, F, false)) return rc;
  if (int rc = enter_stream(plan, stream)) return rc;
  nts::LaunchArgs a{in,  out,         w,           offsets,       indices,   index_base, plan->n_items,
                    F,   plan->items, plan->partial, accumulate, stream};
  if (plan->sorted_idx) {  // the schedule's own copy of the indices, base already subtracted
    a.indices = plan->sorted_idx;
    a.index_base = 0;
    a.edge_ids = plan->edge_ids;
  }
  a.dup_runs = use_runs(plan);
  if (const uint32_t ld = padded_stride(plan, F, false)) {
    // Rows off 16-byte boundaries: gather from a padded copy with 16-byte lanes.
    const uint64_t vecs = static_cast<uint64_t>(plan->n_index) * (ld / 4);
    const uint32_t blocks = static_cast<uint32_t>(std::min<uint64_t>((vecs + 255) / 256, 1u << 16));
    hipLaunchKernelGGL(nts::pad_rows_kernel, dim3(blocks), dim3(256), 0, stream,
                       reinterpret_cast<float4 *>(plan->in_padded), in, plan->n_index, F, ld);
    NTS_LAUNCH_CHECK("pad_rows_kernel");
    a.in = plan->in_padded;
    a.in_ld = ld;
    a.partial_ld = ld;
  }
  if (plan->ev_start && plan->ev_stop) NTS_HIP_TRY(hipEventRecord(plan->ev_start, stream));
  nts::launch_spmm(a);
  NTS_LAUNCH_CHECK("nts_spmm_gather_planned");
  if (plan->ev_start && plan->ev_stop) NTS_HIP_TRY(hipEventRecord(plan->ev_stop, stream));
  if (plan->n_splits) {
    nts::launch_reduce_partials(out, plan->partial, plan->splits, plan->n_splits, F, accumulate, stream, a.partial_ld);
    NTS_LAUNCH_CHECK("spmm_reduce_partials_kernel");
  }
  return leave_stream(plan, stream);
}

}  // extern "C"
