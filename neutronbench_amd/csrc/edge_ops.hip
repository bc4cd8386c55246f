// Edge <-> vertex movement, edge softmax and fused GAT attention kernels (replaces
// cuda/ntsCUDADistKernel.cuh:23-95, 166-260, cuda/ntsCUDAFuseKernel.cuh:492-506 and their
// launchers cuda/ntsCUDAGraphOP.cu:294-377, 449-474).
//
// All kernels give one wavefront to one destination (or source) row; lanes span the feature /
// head dimension, sums over a segment run in edge order or through fixed-shape cross-lane
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

// msg[e,:] = feat[mirror ? mirror[ri[e]] : ri[e], :] for e in CSC(d); one wave per destination.
template <typename V>
__global__ __launch_bounds__(256) void scatter_src_to_edge_kernel(V *__restrict__ msg, const V *__restrict__ feat,
                                                                  const uint32_t *__restrict__ ri,
                                                                  const uint32_t *__restrict__ co,
                                                                  const uint32_t *__restrict__ mirror, uint32_t Vd,
                                                                  uint32_t Fv) {
  const uint32_t d = wave_item();
  if (d >= Vd) return;
  const uint32_t lane = lane_id();
  const uint32_t e0 = wave_first(co[d]), e1 = wave_first(co[d + 1]);
  for (uint32_t e = e0; e < e1; ++e) {
    uint32_t s = ri[e];
    if (mirror) s = mirror[s];
    const V *src = feat + static_cast<size_t>(s) * Fv;
    V *dst = msg + static_cast<size_t>(e) * Fv;
    for (uint32_t c = lane; c < Fv; c += kWave) dst[c] = src[c];
  }
}

// msg[e,:] (+)= feat[d,:] for e in CSC(d); the destination row is read once per column.
template <typename V, bool ADD>
__global__ __launch_bounds__(256) void scatter_dst_to_edge_kernel(V *__restrict__ msg, const V *__restrict__ feat,
                                                                  const uint32_t *__restrict__ co, uint32_t Vd,
                                                                  uint32_t Fv) {
  const uint32_t d = wave_item();
  if (d >= Vd) return;
  const uint32_t lane = lane_id();
  const uint32_t e0 = wave_first(co[d]), e1 = wave_first(co[d + 1]);
  for (uint32_t c = lane; c < Fv; c += kWave) {
    const V v = feat[static_cast<size_t>(d) * Fv + c];
    for (uint32_t e = e0; e < e1; ++e) {
      V *p = msg + static_cast<size_t>(e) * Fv + c;
      if (ADD) {
        V o = *p;
        float *of = reinterpret_cast<float *>(&o);
        const float *vf = reinterpret_cast<const float *>(&v);
#pragma unroll
        for (int t = 0; t < static_cast<int>(sizeof(V) / 4); ++t) of[t] += vf[t];
        *p = o;
      } else {
        *p = v;
      }
    }
  }
}

// ---- edge -> vertex sums ----------------------------------------------------------------------

// out[r,:] (+)= sum_{k in [off[r], off[r+1])} msg[perm ? perm[k] : k, :], added in k order.
template <typename V>
__global__ __launch_bounds__(256) void gather_edge_to_row_kernel(V *__restrict__ out, const V *__restrict__ msg,
                                                                 const uint32_t *__restrict__ off,
                                                                 const uint32_t *__restrict__ perm, uint32_t rows,
                                                                 uint32_t Fv, int accumulate) {
  const uint32_t r = wave_item();
  if (r >= rows) return;
  const uint32_t lane = lane_id();
  const uint32_t e0 = wave_first(off[r]), e1 = wave_first(off[r + 1]);
  constexpr int NF = sizeof(V) / 4;
  for (uint32_t c = lane; c < Fv; c += kWave) {
    float a[NF];
#pragma unroll
    for (int t = 0; t < NF; ++t) a[t] = 0.f;
    for (uint32_t k = e0; k < e1; ++k) {
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

// FUSED = false: y = softmax_seg(x).   FUSED = true: x is ignored and the score is
// leaky_relu(el[ri[e],h] + er[d,h], slope); y first holds the raw score, then alpha.
template <bool FUSED, bool POW2>
__global__ __launch_bounds__(256) void edge_softmax_fwd_kernel(float *__restrict__ y, const float *__restrict__ x,
                                                               const float *__restrict__ el,
                                                               const float *__restrict__ er,
                                                               const uint32_t *__restrict__ co,
                                                               const uint32_t *__restrict__ ri, uint32_t Vd,
                                                               uint32_t H, float slope) {
  const uint32_t d = wave_item();
  if (d >= Vd) return;
  const uint32_t lane = lane_id();
  const uint32_t e0 = wave_first(co[d]), e1 = wave_first(co[d + 1]);
  if (e0 == e1) return;
  const size_t base = static_cast<size_t>(e0) * H;
  const uint32_t n = (e1 - e0) * H;
  float *ys = y + base;
  const float *xs = FUSED ? nullptr : x + base;

  if (POW2) {
    const uint32_t h = lane & (H - 1);
    float erv = 0.f;
    if (FUSED) erv = er[static_cast<size_t>(d) * H + h];
    float mx = -INFINITY;
    for (uint32_t i = lane; i < n; i += kWave) {
      float s;
      if (FUSED) {
        const uint32_t src = ri[e0 + i / H];
        s = leaky(el[static_cast<size_t>(src) * H + h] + erv, slope);
        ys[i] = s;
      } else {
        s = xs[i];
      }
      mx = fmaxf(mx, s);
    }
    mx = head_reduce<0>(mx, H);
    float sum = 0.f;
    for (uint32_t i = lane; i < n; i += kWave) {
      const float s = FUSED ? ys[i] : xs[i];
      sum += expf(s - mx);
    }
    sum = head_reduce<1>(sum, H);
    for (uint32_t i = lane; i < n; i += kWave) {
      const float s = FUSED ? ys[i] : xs[i];
      ys[i] = expf(s - mx) / sum;
    }
  } else {
    const uint32_t deg = e1 - e0;
    for (uint32_t h = 0; h < H; ++h) {
      float erv = 0.f;
      if (FUSED) erv = er[static_cast<size_t>(d) * H + h];
      float mx = -INFINITY;
      for (uint32_t k = lane; k < deg; k += kWave) {
        float s;
        if (FUSED) {
          const uint32_t src = ri[e0 + k];
          s = leaky(el[static_cast<size_t>(src) * H + h] + erv, slope);
          ys[static_cast<size_t>(k) * H + h] = s;
        } else {
          s = xs[static_cast<size_t>(k) * H + h];
        }
        mx = fmaxf(mx, s);
      }
      mx = group_max<kWave>(mx);
      float sum = 0.f;
      for (uint32_t k = lane; k < deg; k += kWave) {
        const float s = FUSED ? ys[static_cast<size_t>(k) * H + h] : xs[static_cast<size_t>(k) * H + h];
        sum += expf(s - mx);
      }
      sum = group_sum<kWave>(sum);
      for (uint32_t k = lane; k < deg; k += kWave) {
        const float s = FUSED ? ys[static_cast<size_t>(k) * H + h] : xs[static_cast<size_t>(k) * H + h];
        ys[static_cast<size_t>(k) * H + h] = expf(s - mx) / sum;
      }
    }
  }
}

// FUSED = false: gx = y * (gy - sum_seg gy*y).
// FUSED = true : additionally multiplies by leaky_relu'(el[src]+er[d]) and writes
//                ger[d,h] = sum_seg gx[e,h].
template <bool FUSED, bool POW2>
__global__ __launch_bounds__(256) void edge_softmax_bwd_kernel(float *__restrict__ gx, float *__restrict__ ger,
                                                               const float *__restrict__ gy,
                                                               const float *__restrict__ y,
                                                               const float *__restrict__ el,
                                                               const float *__restrict__ er,
                                                               const uint32_t *__restrict__ co,
                                                               const uint32_t *__restrict__ ri, uint32_t Vd,
                                                               uint32_t H, float slope) {
  const uint32_t d = wave_item();
  if (d >= Vd) return;
  const uint32_t lane = lane_id();
  const uint32_t e0 = wave_first(co[d]), e1 = wave_first(co[d + 1]);
  const size_t base = static_cast<size_t>(e0) * H;
  const uint32_t n = (e1 - e0) * H;
  const float *gys = gy + base;
  const float *ys = y + base;
  float *gxs = gx + base;

  if (POW2) {
    const uint32_t h = lane & (H - 1);
    float dot = 0.f;
    for (uint32_t i = lane; i < n; i += kWave) dot += gys[i] * ys[i];
    dot = head_reduce<1>(dot, H);
    float erv = 0.f, gsum = 0.f;
    if (FUSED) erv = er[static_cast<size_t>(d) * H + h];
    for (uint32_t i = lane; i < n; i += kWave) {
      float g = ys[i] * (gys[i] - dot);
      if (FUSED) {
        const uint32_t src = ri[e0 + i / H];
        const float pre = el[static_cast<size_t>(src) * H + h] + erv;
        g *= pre > 0.f ? 1.f : slope;
        gsum += g;
      }
      gxs[i] = g;
    }
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

// ---- gradient of the attention-weighted aggregation with respect to alpha ----------------------

// galpha[e,h] = < in[ri[e], h-th slice], gout[d, h-th slice] > for e in CSC(d).  One wave per
// destination; for each edge and head the lanes stride over the slice and a full-wave butterfly
// adds the partial products.
__global__ __launch_bounds__(256) void sddmm_heads_kernel(float *__restrict__ galpha, const float *__restrict__ in,
                                                          const float *__restrict__ gout,
                                                          const uint32_t *__restrict__ co,
                                                          const uint32_t *__restrict__ ri, uint32_t Vd, uint32_t H,
                                                          uint32_t Fh) {
  const uint32_t d = wave_item();
  if (d >= Vd) return;
  const uint32_t lane = lane_id();
  const uint32_t F = H * Fh;
  const uint32_t e0 = wave_first(co[d]), e1 = wave_first(co[d + 1]);
  const float *g = gout + static_cast<size_t>(d) * F;
  for (uint32_t e = e0; e < e1; ++e) {
    const float *src = in + static_cast<size_t>(wave_first(ri[e])) * F;
    for (uint32_t h = 0; h < H; ++h) {
      float p = 0.f;
      for (uint32_t f = lane; f < Fh; f += kWave) p = fmaf(src[h * Fh + f], g[h * Fh + f], p);
      p = group_sum<kWave>(p);
      if (lane == 0) galpha[static_cast<size_t>(e) * H + h] = p;
    }
  }
}

// Fast path of the above when every head is a power-of-two number L = Fh <= 64 of lanes wide and
// the whole row fits one wave pass (H*Fh <= 64): lane l owns column l, the per-head sum is a
// butterfly over L lanes.
__global__ __launch_bounds__(256) void sddmm_heads_pow2_kernel(float *__restrict__ galpha,
                                                               const float *__restrict__ in,
                                                               const float *__restrict__ gout,
                                                               const uint32_t *__restrict__ co,
                                                               const uint32_t *__restrict__ ri, uint32_t Vd,
                                                               uint32_t H, uint32_t Fh) {
  const uint32_t d = wave_item();
  if (d >= Vd) return;
  const uint32_t lane = lane_id();
  const uint32_t F = H * Fh;
  const uint32_t e0 = wave_first(co[d]), e1 = wave_first(co[d + 1]);
  const bool live = lane < F;
  const float g = live ? gout[static_cast<size_t>(d) * F + lane] : 0.f;
  for (uint32_t e = e0; e < e1; ++e) {
    const float *src = in + static_cast<size_t>(wave_first(ri[e])) * F;
    float p = live ? src[lane] * g : 0.f;
    for (uint32_t m = Fh / 2; m >= 1; m >>= 1) p += __shfl_xor(p, m, kWave);
    if (live && (lane & (Fh - 1)) == 0) galpha[static_cast<size_t>(e) * H + lane / Fh] = p;
  }
}

inline bool is_pow2(uint32_t v) { return v && !(v & (v - 1)); }

// Vector width (in floats) usable for [*, F] row-major operands at the given base pointers.
inline int row_vec(uint32_t F, const void *a, const void *b) {
  if (F % 4 == 0 && aligned_to(a, 16) && aligned_to(b, 16)) return 4;
  if (F % 2 == 0 && aligned_to(a, 8) && aligned_to(b, 8)) return 2;
  return 1;
}

}  // namespace
}  // namespace nts

using namespace nts;

namespace {
template <bool ADD>
int scatter_dst_impl(float *msg, const float *feat, const uint32_t *co, uint32_t Vd, uint32_t F, hipStream_t stream,
                     const char *who) {
  if (F == 0) return fail(NTS_ERR_INVALID, who);
  if (Vd == 0) return NTS_OK;
  if (!msg || !feat || !co) return fail(NTS_ERR_INVALID, who);
  switch (row_vec(F, msg, feat)) {
    case 4:
      hipLaunchKernelGGL((scatter_dst_to_edge_kernel<float4, ADD>), wave_grid(Vd), wave_block(), 0, stream,
                         reinterpret_cast<float4 *>(msg), reinterpret_cast<const float4 *>(feat), co, Vd, F / 4);
      break;
    case 2:
      hipLaunchKernelGGL((scatter_dst_to_edge_kernel<float2, ADD>), wave_grid(Vd), wave_block(), 0, stream,
                         reinterpret_cast<float2 *>(msg), reinterpret_cast<const float2 *>(feat), co, Vd, F / 2);
      break;
    default:
      hipLaunchKernelGGL((scatter_dst_to_edge_kernel<float, ADD>), wave_grid(Vd), wave_block(), 0, stream, msg, feat,
                         co, Vd, F);
  }
  NTS_LAUNCH_CHECK(who);
  return NTS_OK;
}

int gather_edge_impl(float *out, const float *msg, const uint32_t *off, const uint32_t *perm, uint32_t rows,
                     uint32_t F, int accumulate, hipStream_t stream, const char *who) {
  if (F == 0) return fail(NTS_ERR_INVALID, who);
  if (rows == 0) return NTS_OK;
  if (!out || !msg || !off) return fail(NTS_ERR_INVALID, who);
  switch (row_vec(F, out, msg)) {
    case 4:
      hipLaunchKernelGGL(gather_edge_to_row_kernel<float4>, wave_grid(rows), wave_block(), 0, stream,
                         reinterpret_cast<float4 *>(out), reinterpret_cast<const float4 *>(msg), off, perm, rows,
                         F / 4, accumulate);
      break;
    case 2:
      hipLaunchKernelGGL(gather_edge_to_row_kernel<float2>, wave_grid(rows), wave_block(), 0, stream,
                         reinterpret_cast<float2 *>(out), reinterpret_cast<const float2 *>(msg), off, perm, rows,
                         F / 2, accumulate);
      break;
    default:
      hipLaunchKernelGGL(gather_edge_to_row_kernel<float>, wave_grid(rows), wave_block(), 0, stream, out, msg, off,
                         perm, rows, F, accumulate);
  }
  NTS_LAUNCH_CHECK(who);
  return NTS_OK;
}
}  // namespace

extern "C" {

int nts_scatter_src_to_edge(float *msg, const float *feat, const uint32_t *ri, const uint32_t *co,
                            const uint32_t *mirror, uint32_t Vd, uint32_t F, nts_stream_t stream) {
  if (F == 0) return fail(NTS_ERR_INVALID, "nts_scatter_src_to_edge: F is 0");
  if (Vd == 0) return NTS_OK;
  if (!msg || !feat || !ri || !co) return fail(NTS_ERR_INVALID, "nts_scatter_src_to_edge: null pointer");
  switch (row_vec(F, msg, feat)) {
    case 4:
      hipLaunchKernelGGL(scatter_src_to_edge_kernel<float4>, wave_grid(Vd), wave_block(), 0, stream,
                         reinterpret_cast<float4 *>(msg), reinterpret_cast<const float4 *>(feat), ri, co, mirror, Vd,
                         F / 4);
      break;
    case 2:
      hipLaunchKernelGGL(scatter_src_to_edge_kernel<float2>, wave_grid(Vd), wave_block(), 0, stream,
                         reinterpret_cast<float2 *>(msg), reinterpret_cast<const float2 *>(feat), ri, co, mirror, Vd,
                         F / 2);
      break;
    default:
      hipLaunchKernelGGL(scatter_src_to_edge_kernel<float>, wave_grid(Vd), wave_block(), 0, stream, msg, feat, ri, co,
                         mirror, Vd, F);
  }
  NTS_LAUNCH_CHECK("nts_scatter_src_to_edge");
  return NTS_OK;
}

int nts_scatter_dst_to_edge(float *msg, const float *feat, const uint32_t *co, uint32_t Vd, uint32_t F,
                            nts_stream_t stream) {
  return scatter_dst_impl<false>(msg, feat, co, Vd, F, stream, "nts_scatter_dst_to_edge: bad argument");
}

int nts_scatter_grad_to_edge(float *msg_grad, const float *gout, const uint32_t *co, uint32_t Vd, uint32_t F,
                             nts_stream_t stream) {
  return scatter_dst_impl<true>(msg_grad, gout, co, Vd, F, stream, "nts_scatter_grad_to_edge: bad argument");
}

int nts_gather_edge_to_dst(float *out, const float *msg, const uint32_t *co, uint32_t Vd, uint32_t F, int accumulate,
                           nts_stream_t stream) {
  return gather_edge_impl(out, msg, co, nullptr, Vd, F, accumulate, stream, "nts_gather_edge_to_dst: bad argument");
}

int nts_gather_edge_to_src(float *out, const float *msg, const uint32_t *ro, const uint32_t *perm, uint32_t Vs,
                           uint32_t F, int accumulate, nts_stream_t stream) {
  if (Vs != 0 && !perm) return fail(NTS_ERR_INVALID, "nts_gather_edge_to_src: null perm");
  return gather_edge_impl(out, msg, ro, perm, Vs, F, accumulate, stream, "nts_gather_edge_to_src: bad argument");
}

int nts_edge_softmax_fwd(float *y, const float *x, const uint32_t *co, uint32_t Vd, uint32_t H,
                         nts_stream_t stream) {
  if (H == 0) return fail(NTS_ERR_INVALID, "nts_edge_softmax_fwd: H is 0");
  if (Vd == 0) return NTS_OK;
  if (!y || !x || !co) return fail(NTS_ERR_INVALID, "nts_edge_softmax_fwd: null pointer");
  if (is_pow2(H) && H <= kWave)
    hipLaunchKernelGGL((edge_softmax_fwd_kernel<false, true>), wave_grid(Vd), wave_block(), 0, stream, y, x, nullptr,
                       nullptr, co, nullptr, Vd, H, 0.f);
  else
    hipLaunchKernelGGL((edge_softmax_fwd_kernel<false, false>), wave_grid(Vd), wave_block(), 0, stream, y, x, nullptr,
                       nullptr, co, nullptr, Vd, H, 0.f);
  NTS_LAUNCH_CHECK("nts_edge_softmax_fwd");
  return NTS_OK;
}

int nts_edge_softmax_bwd(float *gx, const float *gy, const float *y, const uint32_t *co, uint32_t Vd, uint32_t H,
                         nts_stream_t stream) {
  if (H == 0) return fail(NTS_ERR_INVALID, "nts_edge_softmax_bwd: H is 0");
  if (Vd == 0) return NTS_OK;
  if (!gx || !gy || !y || !co) return fail(NTS_ERR_INVALID, "nts_edge_softmax_bwd: null pointer");
  if (is_pow2(H) && H <= kWave)
    hipLaunchKernelGGL((edge_softmax_bwd_kernel<false, true>), wave_grid(Vd), wave_block(), 0, stream, gx, nullptr, gy,
                       y, nullptr, nullptr, co, nullptr, Vd, H, 0.f);
  else
    hipLaunchKernelGGL((edge_softmax_bwd_kernel<false, false>), wave_grid(Vd), wave_block(), 0, stream, gx, nullptr,
                       gy, y, nullptr, nullptr, co, nullptr, Vd, H, 0.f);
  NTS_LAUNCH_CHECK("nts_edge_softmax_bwd");
  return NTS_OK;
}

int nts_gat_attention_fwd(float *alpha, const float *el, const float *er, const uint32_t *co, const uint32_t *ri,
                          uint32_t Vd, uint32_t H, float slope, nts_stream_t stream) {
  if (H == 0) return fail(NTS_ERR_INVALID, "nts_gat_attention_fwd: H is 0");
  if (Vd == 0) return NTS_OK;
  if (!alpha || !el || !er || !co || !ri) return fail(NTS_ERR_INVALID, "nts_gat_attention_fwd: null pointer");
  if (is_pow2(H) && H <= kWave)
    hipLaunchKernelGGL((edge_softmax_fwd_kernel<true, true>), wave_grid(Vd), wave_block(), 0, stream, alpha, nullptr,
                       el, er, co, ri, Vd, H, slope);
  else
    hipLaunchKernelGGL((edge_softmax_fwd_kernel<true, false>), wave_grid(Vd), wave_block(), 0, stream, alpha, nullptr,
                       el, er, co, ri, Vd, H, slope);
  NTS_LAUNCH_CHECK("nts_gat_attention_fwd");
  return NTS_OK;
}

int nts_gat_attention_bwd(float *gs, float *ger, const float *galpha, const float *alpha, const float *el,
                          const float *er, const uint32_t *co, const uint32_t *ri, uint32_t Vd, uint32_t H,
                          float slope, nts_stream_t stream) {
  if (H == 0) return fail(NTS_ERR_INVALID, "nts_gat_attention_bwd: H is 0");
  if (Vd == 0) return NTS_OK;
  if (!gs || !ger || !galpha || !alpha || !el || !er || !co || !ri)
    return fail(NTS_ERR_INVALID, "nts_gat_attention_bwd: null pointer");
  if (is_pow2(H) && H <= kWave)
    hipLaunchKernelGGL((edge_softmax_bwd_kernel<true, true>), wave_grid(Vd), wave_block(), 0, stream, gs, ger, galpha,
                       alpha, el, er, co, ri, Vd, H, slope);
  else
    hipLaunchKernelGGL((edge_softmax_bwd_kernel<true, false>), wave_grid(Vd), wave_block(), 0, stream, gs, ger, galpha,
                       alpha, el, er, co, ri, Vd, H, slope);
  NTS_LAUNCH_CHECK("nts_gat_attention_bwd");
  return NTS_OK;
}

int nts_sddmm_heads(float *galpha, const float *in, const float *gout, const uint32_t *co, const uint32_t *ri,
                    uint32_t Vd, uint32_t H, uint32_t Fh, nts_stream_t stream) {
  if (H == 0 || Fh == 0) return fail(NTS_ERR_INVALID, "nts_sddmm_heads: H or Fh is 0");
  if (Vd == 0) return NTS_OK;
  if (!galpha || !in || !gout || !co || !ri) return fail(NTS_ERR_INVALID, "nts_sddmm_heads: null pointer");
  if (is_pow2(Fh) && static_cast<uint64_t>(H) * Fh <= kWave)
    hipLaunchKernelGGL(sddmm_heads_pow2_kernel, wave_grid(Vd), wave_block(), 0, stream, galpha, in, gout, co, ri, Vd,
                       H, Fh);
  else
    hipLaunchKernelGGL(sddmm_heads_kernel, wave_grid(Vd), wave_block(), 0, stream, galpha, in, gout, co, ri, Vd, H,
                       Fh);
  NTS_LAUNCH_CHECK("nts_sddmm_heads");
  return NTS_OK;
}

}  // extern "C"
