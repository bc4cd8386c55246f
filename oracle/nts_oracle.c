/*
 * nts_oracle.c -- CPU restatement of NeutronBench's own CPU graph operators for the single-GPU
 * hot path.  TEST INFRASTRUCTURE ONLY: this file is the checker that the HIP kernels are compared
 * against (tests/, the smoke check and the cpu_baseline leg of the benchmark); nothing in the
 * product path may call it.
 *
 * Each function names the reference code it follows (file:line relative to the NeutronBench
 * tree).  Arithmetic is fp32 with the reference's operation order; the file is compiled with
 * -ffp-contract=off so that "mul then add" stays two roundings unless a function says otherwise.
 *
 * Pinning status (the independent evidence each function is checked against lives in
 * tests/test_oracle_pins.py, tests/test_golden.py, tests/test_oracle_vs_reference_build.py,
 * tests/test_reference_operators.py and tests/test_dataset_formats.py):
 *   norm_degree, comp, spmm (fwd/bwd), build_chunk, scatter / aggregate edge ops, edge_softmax fwd/bwd:
 *   pinned by closed forms, brute force and library routines, AND against the reference's own code
 *   compiled from its tree (oracle/build_ref.sh): nts_comp / nts_norm_degree bit for bit, and the
 *   operator classes ForwardCPUfuseOp (bit for bit, forward and backward), SingleCPUSrcDstScatterOp,
 *   SingleCPUDstAggregateOp (bit for bit) and SingleEdgeSoftMax (to rounding: it calls libtorch's
 *   softmax) run on graphs loaded by the reference's loader and partitioner.
 *   postprocess, csr_from_csc, layer weights: additionally against the reference's sampCSC itself
 *   (core/coocsc.hpp compiles against the HIP veneer; postprocessing, generate_csr_from_csc,
 *   update_degree, compute_weight_forward / backward run on sampled lists made by the tests), bit for bit.
 *   init_co, gathers, cache split: the reference code for these (core/ntsSampler.hpp,
 *   core/ntsMiniBatchGraphOp.hpp) needs METIS headers the tree does not carry and cannot be
 *   compiled; pinned by brute force and exact fixtures.
 *   dataset readers: pinned by exact rational rounding of every token and by the file definitions, and
 *   against the reference's GNNDatum::readFeature_Label_Mask itself (GPU test: its tables are pinned memory).
 */
#define _GNU_SOURCE /* getline */
#include <math.h>
#include <stdio.h>
#include <sys/types.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define NTS_EXPORT __attribute__((visibility("default")))

/* ---------------------------------------------------------------------------------------------
 * A.1  nts_norm_degree  (core/ntsBaseOp.hpp:183-186)
 *   1 / ((ValueType)std::sqrt(out_degree[src]) * (ValueType)std::sqrt(in_degree[dst]))
 * std::sqrt on an unsigned integer promotes to double; each root is narrowed to float, the
 * product and the reciprocal are float operations.
 * ------------------------------------------------------------------------------------------- */
NTS_EXPORT float nts_oracle_norm_degree(uint32_t out_deg_src, uint32_t in_deg_dst) {
  const float a = (float)sqrt((double)out_deg_src);
  const float b = (float)sqrt((double)in_deg_dst);
  const float prod = a * b;
  return 1 / prod;
}

/* nts_comp (core/ntsBaseOp.hpp:76-97): output[i] += input[i] * weight, written there as an AVX
 * multiply followed by an AVX add (8 lanes, scalar tail) -- element-wise the same two roundings. */
static inline void comp_mul_add(float *output, const float *input, float weight, uint32_t n) {
  for (uint32_t i = 0; i < n; ++i) {
    const float prod = input[i] * weight;
    output[i] = output[i] + prod;
  }
}

/* The same loop as a compiler emits it when it contracts the multiply and the add into one fused
 * multiply-add (GCC's default -ffp-contract=fast together with -march=native, CMakeLists.txt:128). */
static inline void comp_fma(float *output, const float *input, float weight, uint32_t n) {
  for (uint32_t i = 0; i < n; ++i) output[i] = fmaf(input[i], weight, output[i]);
}

NTS_EXPORT void nts_oracle_comp(float *output, const float *input, float weight, uint32_t n, int fused) {
  if (fused) comp_fma(output, input, weight, n); else comp_mul_add(output, input, weight, n);
}

/* ---------------------------------------------------------------------------------------------
 * A.3 / A.4  aggregation forward and backward (pull)
 *   MiniBatchFuseOp::forward  (core/ntsMiniBatchGraphOp.hpp:154-184): per destination, in CSC edge
 *     order, nts_comp(out[dst], in[row_indices[e]], edge_weight_forward[e]).
 *   MiniBatchFuseOp::backward, pull branch (:214-240): per source, in CSR edge order,
 *     nts_comp(gin[src], gout[column_indices[e]], edge_weight_backward[e]).
 *   ForwardCPUfuseOp::forward / backward (core/ntsCPUFusedGraphOp.hpp:41-141) run the same loops
 *     with global ids and nts_norm_degree evaluated per edge.
 * Both are the one loop below: rows = destinations with CSC arrays, or sources with CSR arrays.
 * Rows are independent and distributed over threads exactly like SampledSubgraph::compute_one_layer
 * (core/FullyRepGraph.hpp:366-395: omp parallel for over rows).
 *   w == NULL: unweighted sum (weight 1).  fused: see comp_fma.  threads <= 0: leave OpenMP default.
 * ------------------------------------------------------------------------------------------- */
NTS_EXPORT void nts_oracle_spmm(const float *in, float *out, const float *w, const uint32_t *offsets,
                                const uint32_t *indices, uint32_t index_base, uint32_t rows, uint32_t F,
                                int fused, int threads) {
#ifdef _OPENMP
  if (threads > 0) omp_set_num_threads(threads);
#else
  (void)threads;
#endif
#pragma omp parallel for schedule(dynamic, 64)
  for (int64_t r = 0; r < (int64_t)rows; ++r) {
    float *o = out + (size_t)r * F;
    memset(o, 0, sizeof(float) * F);
    for (uint32_t e = offsets[r]; e < offsets[r + 1]; ++e) {
      const float *src = in + (size_t)(indices[e] - index_base) * F;
      const float weight = w ? w[e] : 1.0f;
      if (fused) comp_fma(o, src, weight, F); else comp_mul_add(o, src, weight, F);
    }
  }
}

/* MiniBatchFuseOp::backward, push branch (core/ntsMiniBatchGraphOp.hpp:194-213, mini_pull == 0):
 * for each destination in order, for each CSC edge, gin[row_indices[e]] += gout[dst] * ewf[e].
 * Serial here (the reference's parallel version races on gin). */
NTS_EXPORT void nts_oracle_spmm_push(const float *gout, float *gin, const float *ewf, const uint32_t *co,
                                     const uint32_t *ri, uint32_t Vd, uint32_t Vs, uint32_t F) {
  memset(gin, 0, sizeof(float) * (size_t)Vs * F);
  for (uint32_t d = 0; d < Vd; ++d)
    for (uint32_t e = co[d]; e < co[d + 1]; ++e) comp_mul_add(gin + (size_t)ri[e] * F, gout + (size_t)d * F, ewf[e], F);
}

/* ---------------------------------------------------------------------------------------------
 * A.2  full-graph chunk layout  (PartitionedGraph::PartitionToChunks, core/PartitionedGraph.hpp:298-388,
 * one partition).  Input: the COO edge list in the order generatePartitionedSubgraph produces it
 * (:281-297), and the global degree arrays.  Output: CSC (column_offset, row_indices = global
 * source ids, edge_weight_forward) and CSR (row_offset, column_indices = global destination ids,
 * edge_weight_backward); edges keep COO order inside every row; weights = nts_norm_degree(src, dst).
 * ------------------------------------------------------------------------------------------- */
NTS_EXPORT void nts_oracle_build_chunk(const uint32_t *coo_src, const uint32_t *coo_dst, uint64_t E, uint32_t V,
                                       const uint32_t *out_degree, const uint32_t *in_degree,
                                       uint32_t *column_offset, uint32_t *row_indices, float *ewf,
                                       uint32_t *row_offset, uint32_t *column_indices, float *ewb) {
  uint32_t *tc = (uint32_t *)calloc((size_t)V + 1, sizeof(uint32_t));
  uint32_t *tr = (uint32_t *)calloc((size_t)V + 1, sizeof(uint32_t));
  for (uint64_t j = 0; j < E; ++j) {
    tc[coo_dst[j] + 1] += 1;
    tr[coo_src[j] + 1] += 1;
  }
  column_offset[0] = 0;
  row_offset[0] = 0;
  for (uint32_t j = 0; j < V; ++j) {
    tc[j + 1] += tc[j];
    column_offset[j + 1] = tc[j + 1];
    tr[j + 1] += tr[j];
    row_offset[j + 1] = tr[j + 1];
  }
  for (uint64_t j = 0; j < E; ++j) {
    const uint32_t s = coo_src[j], d = coo_dst[j];
    const float wgt = nts_oracle_norm_degree(out_degree[s], in_degree[d]);
    row_indices[tc[d]] = s;
    ewf[tc[d]++] = wgt;
    column_indices[tr[s]] = d;
    ewb[tr[s]++] = wgt;
  }
  free(tc);
  free(tr);
}

/* Degrees as Gemini counts them for the weight function: every edge of the file counts (duplicates
 * and self loops included) and zero degrees are raised to one (core/graph.hpp:3983-3986). */
NTS_EXPORT void nts_oracle_degrees(const uint32_t *coo_src, const uint32_t *coo_dst, uint64_t E, uint32_t V,
                                   uint32_t *out_degree, uint32_t *in_degree) {
  memset(out_degree, 0, sizeof(uint32_t) * V);
  memset(in_degree, 0, sizeof(uint32_t) * V);
  for (uint64_t j = 0; j < E; ++j) {
    out_degree[coo_src[j]] += 1;
    in_degree[coo_dst[j]] += 1;
  }
  for (uint32_t v = 0; v < V; ++v) {
    if (out_degree[v] == 0) out_degree[v] = 1;
    if (in_degree[v] == 0) in_degree[v] = 1;
  }
}

/* ---------------------------------------------------------------------------------------------
 * A.5  sampCSC::postprocessing  (core/coocsc.hpp:338-424)
 * The sampled global source ids of all edges are marked in a bitmap by the sampler; the scan below
 * walks the bitmap words in ascending order, appends every set bit to `source` and records its
 * position in node_idx; then every row index is replaced by node_idx[row index].
 *   row_indices: in = global ids, out = local ids.   source: capacity >= number of distinct ids.
 *   node_idx: scratch of V entries (only marked entries are written, as in the reference).
 * Returns src_size.
 * ------------------------------------------------------------------------------------------- */
NTS_EXPORT uint32_t nts_oracle_postprocess(uint32_t *row_indices, uint32_t E, uint32_t V, uint32_t *source,
                                           uint32_t *node_idx) {
  const size_t words = ((size_t)V >> 6) + 1;
  uint64_t *bits = (uint64_t *)calloc(words, sizeof(uint64_t));
  for (uint32_t e = 0; e < E; ++e) bits[row_indices[e] >> 6] |= (uint64_t)1 << (row_indices[e] & 63);
  uint32_t src_size = 0;
  for (uint32_t base = 0; base < V; base += 64) {
    uint64_t word = bits[base >> 6];
    uint32_t offset = 0;
    while (word != 0) {
      if (word & 1) {
        source[src_size] = base + offset;
        node_idx[base + offset] = src_size++;
      }
      offset++;
      word >>= 1;
    }
  }
  for (uint32_t e = 0; e < E; ++e) row_indices[e] = node_idx[row_indices[e]];
  free(bits);
  return src_size;
}

/* A.6  sampCSC::generate_csr_from_csc  (core/coocsc.hpp:243-309): histogram of local sources,
 * inclusive prefix sum, fill walking destinations in ascending order while post-incrementing the
 * running offsets, then shift the offsets back by one position. */
NTS_EXPORT void nts_oracle_csr_from_csc(const uint32_t *co, const uint32_t *ri, uint32_t Vd, uint32_t Vs, uint32_t E,
                                        uint32_t *ro, uint32_t *ci) {
  memset(ro, 0, sizeof(uint32_t) * ((size_t)Vs + 1));
  for (uint32_t i = 0; i < E; ++i) ro[ri[i] + 1]++;
  for (uint32_t i = 1; i <= Vs; ++i) ro[i] += ro[i - 1];
  for (uint32_t d = 0; d < Vd; ++d)
    for (uint32_t j = co[d]; j < co[d + 1]; ++j) ci[ro[ri[j]]++] = d;
  for (uint32_t i = Vs; i > 0; --i) ro[i] = ro[i - 1];
  ro[0] = 0;
}

/* A.7  sampCSC::update_degree (core/coocsc.hpp:166-216) followed by compute_weight_forward /
 * compute_weight_backward (:136-163), as driven per layer by SampledSubgraph::compute_weight
 * (core/FullyRepGraph.hpp:128-143).  The degree arrays are the GLOBAL ones (V entries) and keep
 * the values written here, like the reference's graph->in/out_degree_for_backward. */
NTS_EXPORT void nts_oracle_layer_weights(const uint32_t *co, const uint32_t *ri, const uint32_t *ro,
                                         const uint32_t *ci, const uint32_t *source, const uint32_t *destination,
                                         uint32_t Vd, uint32_t Vs, uint32_t *out_degree, uint32_t *in_degree,
                                         float *ewf, float *ewb) {
  for (uint32_t i = 0; i < Vd; ++i) in_degree[destination[i]] = 0;
  for (uint32_t i = 0; i < Vd; ++i) in_degree[destination[i]] += co[i + 1] - co[i];
  for (uint32_t i = 0; i < Vs; ++i) out_degree[source[i]] = 0;
  for (uint32_t i = 0; i < Vs; ++i) out_degree[source[i]] += ro[i + 1] - ro[i];
  for (uint32_t i = 0; i < Vd; ++i)
    for (uint32_t j = co[i]; j < co[i + 1]; ++j)
      ewf[j] = nts_oracle_norm_degree(out_degree[source[ri[j]]], in_degree[destination[i]]);
  for (uint32_t i = 0; i < Vs; ++i)
    for (uint32_t j = ro[i]; j < ro[i + 1]; ++j)
      ewb[j] = nts_oracle_norm_degree(out_degree[source[i]], in_degree[destination[ci[j]]]);
}

/* init_co (core/FullyRepGraph.hpp:199-209) with the neighbour count of Sampler::sample_one
 * (core/ntsSampler.hpp:843-1106): fanout < 0 takes every in-neighbour, otherwise min(deg, fanout). */
NTS_EXPORT void nts_oracle_init_co(const uint32_t *graph_co, const uint32_t *dst, uint32_t n_dst, int fanout,
                                   uint32_t *co) {
  uint32_t offset = 0;
  for (uint32_t i = 0; i < n_dst; ++i) {
    co[i] = offset;
    const uint32_t deg = graph_co[dst[i] + 1] - graph_co[dst[i]];
    offset += (fanout < 0 || deg < (uint32_t)fanout) ? deg : (uint32_t)fanout;
  }
  co[n_dst] = offset;
}

/* ---------------------------------------------------------------------------------------------
 * A.8  batch assembly
 * ------------------------------------------------------------------------------------------- */

/* get_feature (core/ntsMiniBatchGraphOp.hpp:77-91): memcpy of one feature row per sampled source. */
NTS_EXPORT void nts_oracle_get_feature(float *out, const float *whole, const uint32_t *src, uint32_t n, uint32_t F) {
#pragma omp parallel for
  for (int64_t i = 0; i < (int64_t)n; ++i)
    memcpy(out + (size_t)i * F, whole + (size_t)src[i] * F, sizeof(float) * F);
}

/* get_label (core/ntsMiniBatchGraphOp.hpp:36-54) at one partition (offset 0); `classes` values per
 * row for multi-label data, as Sampler::load_label_gpu lays them out (core/ntsSampler.hpp:471-529). */
NTS_EXPORT void nts_oracle_get_label(int64_t *out, const int64_t *whole, const uint32_t *dst, uint32_t n,
                                     uint32_t classes) {
  for (uint32_t i = 0; i < n; ++i)
    for (uint32_t c = 0; c < classes; ++c) out[(size_t)i * classes + c] = whole[(size_t)dst[i] * classes + c];
}

/* mark_cache_node (toolkits/GCN_GPU_NEIGHBOR.hpp:930-956): every entry -1 (0xFFFFFFFF), then the
 * first n_cache nodes of `order` receive slots 0, 1, 2, ...   `order` is the caller's ranking (the
 * reference's cache_high_degree sorts by out-degree with std::sort, whose order among equal
 * degrees is unspecified, so the ranking is an input here). */
NTS_EXPORT void nts_oracle_mark_cache(uint32_t *hashmap, uint32_t V, const uint32_t *order, uint32_t n_cache) {
  for (uint32_t i = 0; i < V; ++i) hashmap[i] = 0xFFFFFFFFu;
  for (uint32_t i = 0; i < n_cache; ++i) hashmap[order[i]] = i;
}

/* gater_cpu_cache_feature_and_trans_to_gpu (toolkits/GCN_GPU_NEIGHBOR.hpp:899-928): the cache
 * table holds feature[node] at row hashmap[node]. */
NTS_EXPORT void nts_oracle_fill_cache(float *cache, const float *feature, const uint32_t *order, uint32_t n_cache,
                                      const uint32_t *hashmap, uint32_t F) {
  for (uint32_t i = 0; i < n_cache; ++i)
    memcpy(cache + (size_t)hashmap[order[i]] * F, feature + (size_t)order[i] * F, sizeof(float) * F);
}

/* Sampler::load_feature_gpu_cache (core/ntsSampler.hpp:424-469): host split of the batch's source
 * positions into cache hits and misses (both ascending), then hit rows come from the cache table
 * and miss rows from the feature table.  Returns the number of hits. */
NTS_EXPORT uint32_t nts_oracle_load_feature_cached(float *out, const float *feature, const float *cache,
                                                   const uint32_t *source, uint32_t n, const uint32_t *hashmap,
                                                   uint32_t F, uint32_t *local_idx, uint32_t *local_idx_cache) {
  uint32_t n_miss = 0, n_hit = 0;
  for (uint32_t i = 0; i < n; ++i) {
    if (hashmap[source[i]] != 0xFFFFFFFFu) local_idx_cache[n_hit++] = i; else local_idx[n_miss++] = i;
  }
  for (uint32_t k = 0; k < n_miss; ++k) {
    const uint32_t i = local_idx[k];
    memcpy(out + (size_t)i * F, feature + (size_t)source[i] * F, sizeof(float) * F);
  }
  for (uint32_t k = 0; k < n_hit; ++k) {
    const uint32_t i = local_idx_cache[k];
    memcpy(out + (size_t)i * F, cache + (size_t)hashmap[source[i]] * F, sizeof(float) * F);
  }
  return n_hit;
}

/* ---------------------------------------------------------------------------------------------
 * A.9  GAT operators on one (bipartite) block: CSC over Vd destinations, sources indexed by ri.
 * The full-graph operators are the special case where sources and destinations share one id space.
 * ------------------------------------------------------------------------------------------- */

/* SingleCPUSrcDstScatterOp::forward (core/ntsSingleCPUGraphOp.hpp:43-59):
 * edge row e = [ x_src[ri[e]] | x_dst[d] ], width 2F. */
NTS_EXPORT void nts_oracle_scatter_src_dst(float *msg, const float *x_src, const float *x_dst, const uint32_t *co,
                                           const uint32_t *ri, uint32_t Vd, uint32_t F) {
  for (uint32_t d = 0; d < Vd; ++d)
    for (uint32_t e = co[d]; e < co[d + 1]; ++e) {
      memcpy(msg + (size_t)e * 2 * F, x_src + (size_t)ri[e] * F, sizeof(float) * F);
      memcpy(msg + (size_t)e * 2 * F + F, x_dst + (size_t)d * F, sizeof(float) * F);
    }
}

/* SingleCPUSrcDstScatterOp::backward (:61-83): the two halves of every edge gradient row are
 * added (nts_acc) to the source row and to the destination row, destinations ascending, edges in
 * CSC order.  g_src [Vs,F] and g_dst [Vd,F] are zeroed here. */
NTS_EXPORT void nts_oracle_scatter_src_dst_bwd(float *g_src, float *g_dst, const float *g_msg, const uint32_t *co,
                                               const uint32_t *ri, uint32_t Vd, uint32_t Vs, uint32_t F) {
  memset(g_src, 0, sizeof(float) * (size_t)Vs * F);
  memset(g_dst, 0, sizeof(float) * (size_t)Vd * F);
  for (uint32_t d = 0; d < Vd; ++d)
    for (uint32_t e = co[d]; e < co[d + 1]; ++e)
      for (uint32_t f = 0; f < F; ++f) {
        g_src[(size_t)ri[e] * F + f] += g_msg[(size_t)e * 2 * F + f];
        g_dst[(size_t)d * F + f] += g_msg[(size_t)e * 2 * F + F + f];
      }
}

/* SingleCPUSrcScatterOp::forward (:94-109) / scatter_src_mirror_to_msg: msg[e] = x[ri[e]]. */
NTS_EXPORT void nts_oracle_scatter_src(float *msg, const float *x_src, const uint32_t *co, const uint32_t *ri,
                                       const uint32_t *mirror, uint32_t Vd, uint32_t F) {
  for (uint32_t d = 0; d < Vd; ++d)
    for (uint32_t e = co[d]; e < co[d + 1]; ++e) {
      const uint32_t s = mirror ? mirror[ri[e]] : ri[e];
      memcpy(msg + (size_t)e * F, x_src + (size_t)s * F, sizeof(float) * F);
    }
}

/* Adjoint of the above (what SingleCPUSrcScatterOp::backward is meant to compute; the reference's
 * own body has its nts_acc operands swapped, core/ntsSingleCPUGraphOp.hpp:111-128, and is not
 * followed): g_src[ri[e]] += g_msg[e], destinations ascending. */
NTS_EXPORT void nts_oracle_gather_to_src(float *g_src, const float *g_msg, const uint32_t *co, const uint32_t *ri,
                                         uint32_t Vd, uint32_t Vs, uint32_t F) {
  memset(g_src, 0, sizeof(float) * (size_t)Vs * F);
  for (uint32_t d = 0; d < Vd; ++d)
    for (uint32_t e = co[d]; e < co[d + 1]; ++e)
      for (uint32_t f = 0; f < F; ++f) g_src[(size_t)ri[e] * F + f] += g_msg[(size_t)e * F + f];
}

/* scatter_dst_to_msg (cuda/ntsCUDADistKernel.cuh:65-79) == SingleCPUDstAggregateOp::backward
 * (core/ntsSingleCPUGraphOp.hpp:157-174): msg[e] = x_dst[d] for e in CSC(d). */
NTS_EXPORT void nts_oracle_scatter_dst(float *msg, const float *x_dst, const uint32_t *co, uint32_t Vd, uint32_t F) {
  for (uint32_t d = 0; d < Vd; ++d)
    for (uint32_t e = co[d]; e < co[d + 1]; ++e) memcpy(msg + (size_t)e * F, x_dst + (size_t)d * F, sizeof(float) * F);
}

/* SingleCPUDstAggregateOp::forward (:139-155): out[d] = sum of edge rows in CSC order (nts_acc). */
NTS_EXPORT void nts_oracle_aggregate_dst(float *out, const float *msg, const uint32_t *co, uint32_t Vd, uint32_t F) {
  memset(out, 0, sizeof(float) * (size_t)Vd * F);
  for (uint32_t d = 0; d < Vd; ++d)
    for (uint32_t e = co[d]; e < co[d + 1]; ++e)
      for (uint32_t f = 0; f < F; ++f) out[(size_t)d * F + f] += msg[(size_t)e * F + f];
}

/* SingleEdgeSoftMax::forward (:297-319): softmax over dim 0 of every destination's slice
 * x[co[d]:co[d+1], :], each of the H columns on its own.  libtorch's softmax is restated in its
 * textbook stable form exp(x - max) / sum(exp(x - max)). */
NTS_EXPORT void nts_oracle_edge_softmax(float *y, const float *x, const uint32_t *co, uint32_t Vd, uint32_t H) {
  for (uint32_t d = 0; d < Vd; ++d) {
    const uint32_t e0 = co[d], e1 = co[d + 1];
    for (uint32_t h = 0; h < H; ++h) {
      if (e0 == e1) continue;
      float mx = x[(size_t)e0 * H + h];
      for (uint32_t e = e0 + 1; e < e1; ++e) mx = fmaxf(mx, x[(size_t)e * H + h]);
      float sum = 0.f;
      for (uint32_t e = e0; e < e1; ++e) sum += expf(x[(size_t)e * H + h] - mx);
      for (uint32_t e = e0; e < e1; ++e) y[(size_t)e * H + h] = expf(x[(size_t)e * H + h] - mx) / sum;
    }
  }
}

/* SingleEdgeSoftMax::backward (:321-341): d_o = (imr * d) - imr * (d^T imr) per destination slice.
 * The reference expression is only shape-correct for one column; each column is treated on its
 * own here (H independent heads), which for H == 1 is the reference's formula. */
NTS_EXPORT void nts_oracle_edge_softmax_bwd(float *gx, const float *gy, const float *y, const uint32_t *co,
                                            uint32_t Vd, uint32_t H) {
  for (uint32_t d = 0; d < Vd; ++d) {
    const uint32_t e0 = co[d], e1 = co[d + 1];
    for (uint32_t h = 0; h < H; ++h) {
      float dot = 0.f;
      for (uint32_t e = e0; e < e1; ++e) dot += gy[(size_t)e * H + h] * y[(size_t)e * H + h];
      for (uint32_t e = e0; e < e1; ++e) {
        const size_t i = (size_t)e * H + h;
        gx[i] = y[i] * gy[i] - y[i] * dot;
      }
    }
  }
}

/* ---------------------------------------------------------------------------------------------
 * On-disk formats.  Sequential restatements of the reference's readers for one partition that
 * owns every vertex (p_v_s = 0, p_v_e = V).  `stream >> x` is restated with fscanf, which like the
 * stream extraction skips white space and converts with the C library's strtof / strtol.
 * ------------------------------------------------------------------------------------------- */

static int mask_word_code(const char *w) {
  if (strcmp(w, "train") == 0) return 0;
  if (strcmp(w, "eval") == 0 || strcmp(w, "val") == 0) return 1;
  if (strcmp(w, "test") == 0) return 2;
  return 3;
}

/* GNNDatum::readFeature_Label_Mask (core/ntsDataloador.hpp:264-395).  The three files are read in
 * step: the k-th record of the label and of the mask file belongs to the vertex named by the k-th
 * record of the feature file (local_*); afterwards label and mask files are read again on their
 * own ids (global_*).  Tables must come in zeroed, as the constructor leaves them (:78-88). */
NTS_EXPORT int nts_oracle_read_feature_label_mask(const char *path_f, const char *path_l, const char *path_m,
                                                  uint32_t V, uint32_t F, uint32_t classes, float *local_feature,
                                                  int64_t *local_label, int32_t *local_mask, int64_t *global_label,
                                                  int32_t *global_mask) {
  FILE *ff = fopen(path_f, "r"), *fl = fopen(path_l, "r"), *fm = fopen(path_m, "r");
  if (!ff || !fl || !fm) {
    if (ff) fclose(ff);
    if (fl) fclose(fl);
    if (fm) fclose(fm);
    return -1;
  }
  char la[256], msk[256];
  unsigned id = 0;
  float skip;
  while (fscanf(ff, "%u", &id) == 1) {
    if (id < V) {
      for (uint32_t i = 0; i < F; ++i)
        if (fscanf(ff, "%f", &local_feature[(size_t)F * id + i]) != 1) break;
      if (fscanf(fl, "%255s", la) != 1) la[0] = 0;
      if (classes > 1) {
        int sz = 0, idx = 0;
        if (fscanf(fl, "%d", &sz) != 1) sz = 0;
        while (sz--) {
          if (fscanf(fl, "%d", &idx) != 1) break;
          local_label[(size_t)id * classes + idx] = 1;
        }
      } else {
        long v = 0;
        if (fscanf(fl, "%ld", &v) == 1) local_label[id] = v;
      }
      if (fscanf(fm, "%255s", la) != 1) la[0] = 0;
      if (fscanf(fm, "%255s", msk) != 1) msk[0] = 0;
      local_mask[id] = mask_word_code(msk);
    } else {
      for (uint32_t i = 0; i < F; ++i)
        if (fscanf(ff, "%f", &skip) != 1) break;
      if (fscanf(fl, "%255s", la) != 1 || fscanf(fl, "%255s", la) != 1) la[0] = 0;
      if (fscanf(fm, "%255s", la) != 1 || fscanf(fm, "%255s", la) != 1) la[0] = 0;
    }
  }
  fclose(ff);
  rewind(fl);
  while (fscanf(fl, "%u", &id) == 1) {
    if (classes > 1) {
      int sz = 0, idx = 0;
      if (fscanf(fl, "%d", &sz) != 1) sz = 0;
      while (sz--) {
        if (fscanf(fl, "%d", &idx) != 1) break;
        if (id < V) global_label[(size_t)id * classes + idx] = 1;
      }
    } else {
      long v = 0;
      if (fscanf(fl, "%ld", &v) == 1 && id < V) global_label[id] = v;
    }
  }
  rewind(fm);
  while (fscanf(fm, "%u", &id) == 1) {
    if (fscanf(fm, "%255s", msk) != 1) msk[0] = 0;
    if (id < V) global_mask[id] = mask_word_code(msk);
  }
  fclose(fl);
  fclose(fm);
  return 0;
}

/* GNNDatum::readFeature_Label_Mask_OGB (core/ntsDataloador.hpp:397-471): line k of the feature file
 * holds vertex k's values separated by commas, converted with atof; the label file holds one
 * integer per vertex; <dir>/train.csv, valid.csv, test.csv list the vertex ids of the splits. */
NTS_EXPORT int nts_oracle_read_feature_label_mask_ogb(const char *path_f, const char *path_l, const char *dir_m,
                                                      uint32_t V, uint32_t F, float *local_feature,
                                                      int64_t *local_label, int32_t *local_mask) {
  FILE *ff = fopen(path_f, "r"), *fl = fopen(path_l, "r");
  if (!ff || !fl) {
    if (ff) fclose(ff);
    if (fl) fclose(fl);
    return -1;
  }
  char *line = NULL;
  size_t cap = 0;
  int rc = 0;
  for (uint32_t id = 0; id < V; ++id) {
    ssize_t len = getline(&line, &cap, ff);
    if (len < 0) {
      rc = -2;
      break;
    }
    if (len > 0 && line[len - 1] == '\n') line[--len] = 0;
    uint32_t i = 0;
    char *p = line;
    while (p < line + len) { /* getline(ss, field, ','): a field ends at a comma or at the end */
      char *q = p;
      while (*q && *q != ',') ++q;
      const char saved = *q;
      *q = 0;
      if (i < F) local_feature[(size_t)F * id + i] = (float)atof(p);
      ++i;
      if (!saved) break;
      p = q + 1;
    }
    if (i != F) { /* the reference asserts i == size_0 */
      rc = -3;
      break;
    }
    long v = 0;
    if (fscanf(fl, "%ld", &v) == 1) local_label[id] = v;
  }
  free(line);
  fclose(ff);
  fclose(fl);
  if (rc) return rc;
  static const char *names[3] = {"/train.csv", "/valid.csv", "/test.csv"};
  for (int k = 0; k < 3; ++k) {
    char path[4096];
    snprintf(path, sizeof(path), "%s%s", dir_m, names[k]);
    FILE *fm = fopen(path, "r");
    if (!fm) return -1;
    unsigned vtx = 0;
    while (fscanf(fm, "%u", &vtx) == 1)
      if (vtx < V) local_mask[vtx] = k;
    fclose(fm);
  }
  return 0;
}

/* Binary edge list (EdgeUnit<Empty>, dep/gemini/type.hpp:99-106): file bytes / 8 records of
 * {uint32 src, uint32 dst} (core/graph.hpp:1059-1060).  Returns the number of records read. */
NTS_EXPORT uint64_t nts_oracle_read_edges(const char *path, uint32_t *src, uint32_t *dst, uint64_t capacity) {
  FILE *f = fopen(path, "rb");
  if (!f) return 0;
  uint32_t rec[2];
  uint64_t n = 0;
  while (n < capacity && fread(rec, sizeof(uint32_t), 2, f) == 2) {
    src[n] = rec[0];
    dst[n] = rec[1];
    ++n;
  }
  fclose(f);
  return n;
}

NTS_EXPORT int nts_oracle_version(void) { return 1; }

NTS_EXPORT int nts_oracle_max_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}
