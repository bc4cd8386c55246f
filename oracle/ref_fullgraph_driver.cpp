// Driver around the REFERENCE's own full-graph operators, compiled from the reference tree where it
// lies (see build_ref.sh).  TEST INFRASTRUCTURE ONLY: it exists so that tests can compare the oracle
// and the HIP library with what the reference's code itself computes.
//
// It loads a binary edge file through the reference's loader (Graph::load_directed), builds the
// reference's chunks (PartitionedGraph::GenerateAll with nts_norm_degree) and runs, on inputs read
// from raw little-endian float32 files, the reference's operator classes unchanged:
//   CPU  ForwardCPUfuseOp                  (core/ntsCPUFusedGraphOp.hpp)
//        SingleCPUSrcDstScatterOp, SingleEdgeSoftMax, SingleCPUDstAggregateOp
//                                          (core/ntsSingleCPUGraphOp.hpp)
//   GPU  (only when built with CUDA_ENABLE=1 against the HIP veneer and libntship.so)
//        ForwardSingleGPUfuseOp            (core/ntsSingleGPUFusedGraphOp.hpp)
//        DistGPUScatterSrc, DistGPUScatterDst, DistGPUEdgeSoftMax, DistGPUAggregateDst
//                                          (core/ntsDistGPUGraphOp.hpp)
// and writes every result as a raw file <prefix>.<name>.
//
//   usage: ref_fullgraph <edge_file> <vertices> <F> <H> <prefix> <cpu|gpu|both|agg-cpu>
//   agg-cpu runs ForwardCPUfuseOp only; <F> may be a comma-separated list, and for every width the
//   input is <prefix>.x<F>.  NTS_REF_WARMUP (default 2) untimed and NTS_REF_REPS (default 5) timed
//   repetitions per width; the median and the best forward and backward times are printed: the CPU
//   baseline of the aggregation benchmark.
//   agg-gpu (GPU build only): ForwardSingleGPUfuseOp only, on the reference's GPU chunk
//   (GenerateAll(GPU_T) + CopyGraphToDevice), same width list, inputs and repetitions as agg-cpu; prints
//   the median and best wall time of forward and backward (each call ends with the operator's own stream synchronisation).
//   samp (GPU build only, but makes no device call): <H> is a number of sampled layers; for layer k
//   the files <prefix>.l<k>.dst [Vd], .co [Vd+1], .ri [E] (uint32; ri = GLOBAL source ids of the
//   sampled edges) are run through the reference's sampCSC (core/coocsc.hpp): postprocessing,
//   generate_csr_from_csc, update_degree, compute_weight_forward / backward, and the resulting
//   source, row_indices (local), row_offset, column_indices and both weight arrays are written as
//   <prefix>.l<k>.<name>.
//   mini (GPU build only): the sampled layers of `samp`, held one after the other in a single sampCSC
//   object as the reference's sampler re-uses it, are mirrored on the device by the reference's own
//   alloc_dev_array_async / copy_data_to_device_async / copy_ewf/ewb_to_device_async (grow-only
//   device arrays, core/coocsc.hpp:673-773) and aggregated forward and backward with the calls of
//   SingleGPUSampleGraphOp (core/ntsMiniBatchGraphOp.hpp:288-375) on <prefix>.l<k>.x [src_size, F] and
//   <prefix>.l<k>.g [v_size, F]; writes <prefix>.l<k>.fwd and .bwd next to the arrays of `samp`.
//   data (GPU build only; allocates the feature table in pinned memory, so it needs the device):
//   GNNDatum::readFeature_Label_Mask (core/ntsDataloador.hpp:264-395) on <prefix>.feat / .label /
//   .mask with F features and <H> classes; writes local_feature, local_label, local_mask,
//   global_label, global_mask as <prefix>.<name>.
//   inputs:  <prefix>.x  [V, F]   vertex features, also used as the vertex-side gradient
//            <prefix>.m  [E, H]   edge scores;  <prefix>.gm [E, H] their gradient
//            <prefix>.e  [E, F]   edge messages;  <prefix>.g2 [E, 2F] gradient of the (src | dst) scatter
#include "comm/logger.h"
#include "core/PartitionedGraph.hpp"
#include "core/graph.hpp"
#include "core/ntsBaseOp.hpp"
#include "core/ntsCPUFusedGraphOp.hpp"
#include "core/ntsSingleCPUGraphOp.hpp"
#if CUDA_ENABLE
#include "core/coocsc.hpp"
#include "core/ntsDataloador.hpp"
#include "core/ntsDistGPUGraphOp.hpp"
#include "core/ntsSingleGPUFusedGraphOp.hpp"
#endif

#include <algorithm>
#include <chrono>
#include <cstdio>
#include <sstream>
#include <string>
#include <vector>

static std::string g_prefix;
static int g_warmup = 2, g_reps = 5;  // NTS_REF_WARMUP / NTS_REF_REPS (timing modes)

static double median(std::vector<double> v) {
  std::sort(v.begin(), v.end());
  const size_t n = v.size();
  return n == 0 ? 0.0 : (n % 2 ? v[n / 2] : 0.5 * (v[n / 2 - 1] + v[n / 2]));
}

static NtsVar read_matrix(const std::string &name, long rows, long cols) {
  const std::string path = g_prefix + "." + name;
  NtsVar t = torch::zeros({rows, cols}, torch::kFloat);
  FILE *f = fopen(path.c_str(), "rb");
  const size_t n = static_cast<size_t>(rows) * cols;
  if (!f || fread(t.data_ptr<float>(), sizeof(float), n, f) != n) {
    fprintf(stderr, "cannot read %ld x %ld floats from %s\n", rows, cols, path.c_str());
    exit(2);
  }
  fclose(f);
  return t;
}

static void write_raw(const std::string &name, const void *p, size_t bytes) {
  const std::string path = g_prefix + "." + name;
  FILE *f = fopen(path.c_str(), "wb");
  if (!f || (bytes && fwrite(p, 1, bytes, f) != bytes)) {
    fprintf(stderr, "cannot write %s\n", path.c_str());
    exit(2);
  }
  fclose(f);
}

static void write_tensor(const std::string &name, const NtsVar &t_in) {
  NtsVar t = t_in.detach().cpu().contiguous();
  write_raw(name, t.data_ptr<float>(), static_cast<size_t>(t.numel()) * sizeof(float));
}

static std::vector<VertexId> read_ids(const std::string &name) {
  const std::string path = g_prefix + "." + name;
  FILE *f = fopen(path.c_str(), "rb");
  if (!f) {
    fprintf(stderr, "cannot open %s\n", path.c_str());
    exit(2);
  }
  fseek(f, 0, SEEK_END);
  const size_t n = static_cast<size_t>(ftell(f)) / sizeof(VertexId);
  fseek(f, 0, SEEK_SET);
  std::vector<VertexId> v(n);
  if (n && fread(v.data(), sizeof(VertexId), n, f) != n) exit(2);
  fclose(f);
  return v;
}

#if CUDA_ENABLE
// The reference's per-layer construction steps of Sampler::sample_one after the neighbour pick
// (core/ntsSampler.hpp:1006-1106), on sampled lists handed in by the caller.
static void run_sampled_layers(Graph<Empty> *graph, int layers, bool on_device, int F) {
  VertexId *node_idx = new VertexId[graph->vertices];
  // Never destroyed: ~sampCSC frees device pointers its constructors leave uninitialised.
  sampCSC *shared = new sampCSC();
  Cuda_Stream *cs = on_device ? new Cuda_Stream() : nullptr;
  for (int k = 0; k < layers; ++k) {
    const std::string tag = "l" + std::to_string(k) + ".";
    std::vector<VertexId> dst = read_ids(tag + "dst"), co = read_ids(tag + "co"), ri = read_ids(tag + "ri");
    sampCSC *sg = on_device ? shared : new sampCSC(static_cast<VertexId>(dst.size()), static_cast<VertexId>(ri.size()));
    sg->update_vertices(static_cast<VertexId>(dst.size()));
    sg->update_edges(static_cast<VertexId>(ri.size()));
    sg->dst() = dst;
    sg->c_o() = co;
    sg->r_i() = ri;
    Bitmap bits(graph->vertices);
    for (VertexId g : ri) bits.set_bit(g);
    sg->postprocessing(&bits, node_idx);
    sg->generate_csr_from_csc();
    sg->update_degree(graph);
    sg->compute_weight_forward(graph);
    sg->compute_weight_backward(graph);
    write_raw(tag + "source", sg->src().data(), sg->src().size() * sizeof(VertexId));
    write_raw(tag + "row_indices", sg->r_i().data(), sg->r_i().size() * sizeof(VertexId));
    write_raw(tag + "row_offset", sg->r_o().data(), sg->r_o().size() * sizeof(VertexId));
    write_raw(tag + "column_indices", sg->c_i().data(), sg->c_i().size() * sizeof(VertexId));
    write_raw(tag + "edge_weight_forward", sg->edge_weight_forward.data(), sg->edge_weight_forward.size() * sizeof(ValueType));
    write_raw(tag + "edge_weight_backward", sg->edge_weight_backward.data(), sg->edge_weight_backward.size() * sizeof(ValueType));
    if (on_device) {
      sg->alloc_dev_array_async(cs->stream);
      sg->copy_data_to_device_async(cs->stream);
      sg->copy_ewf_to_device_async(cs->stream);
      sg->copy_ewb_to_device_async(cs->stream);
      const long Vd = sg->v_size, Vs = sg->src_size;
      NtsVar x = read_matrix(tag + "x", Vs, F).cuda(), g = read_matrix(tag + "g", Vd, F).cuda();
      NtsVar y = torch::zeros({Vd, (long)F}, x.options()), gx = torch::zeros({Vs, (long)F}, x.options());
      torch::cuda::synchronize();
      cs->Gather_By_Dst_From_Src(x.data_ptr<float>(), y.data_ptr<float>(), sg->dev_ewf(), sg->dev_r_i(), sg->dev_c_o(), 0, 0,
                                 0, 0, sg->e_size, sg->v_size, F, true, false);
      cs->Gather_By_Src_From_Dst(g.data_ptr<float>(), gx.data_ptr<float>(), sg->dev_ewb(), sg->dev_r_o(), sg->dev_c_i(), 0,
                                 0, 0, 0, sg->e_size, sg->src_size, F, true, false);
      cs->CUDA_DEVICE_SYNCHRONIZE();
      write_tensor(tag + "fwd", y);
      write_tensor(tag + "bwd", gx);
    }
  }
  printf("reference sampCSC construction done for %d layers\n", layers);
}
#endif

static double now() {
  return std::chrono::duration<double>(std::chrono::steady_clock::now().time_since_epoch()).count();
}

int main(int argc, char **argv) {
  MPI_Instance mpi(&argc, &argv);
  if (argc < 7) {
    fprintf(stderr, "usage: %s edge_file vertices F H prefix cpu|gpu|both|agg-cpu\n", argv[0]);
    return 2;
  }
  const std::string edge_file = argv[1];
  const VertexId vertices = static_cast<VertexId>(std::stoul(argv[2]));
  std::vector<int> widths;
  {
    std::stringstream ss(argv[3]);
    std::string item;
    while (std::getline(ss, item, ',')) widths.push_back(std::stoi(item));
  }
  const int F = widths.at(0);
  const int H = std::stoi(argv[4]);
  g_prefix = argv[5];
  if (const char *e = getenv("NTS_REF_WARMUP")) g_warmup = std::max(0, atoi(e));
  if (const char *e = getenv("NTS_REF_REPS")) g_reps = std::max(1, atoi(e));
  const std::string mode = argv[6];
  const bool agg_only = mode == "agg-cpu";
  const bool run_cpu = mode == "cpu" || mode == "both";
  const bool run_gpu = mode == "gpu" || mode == "both";

  Graph<Empty> *graph = new Graph<Empty>();
  graph->config->vertices = vertices;
  graph->config->edge_file = edge_file;
  graph->config->layer_string = std::to_string(F) + "-" + std::to_string(F);
  graph->replication_threshold = 0;
  graph->load_directed(edge_file, vertices);
  graph->generate_backward_structure();

#if CUDA_ENABLE
  if (mode == "agg-gpu") {
    VertexSubset *all = graph->alloc_vertex_subset();
    all->fill();
    graph->init_gnnctx(graph->config->layer_string);
    graph->init_rtminfo();
    graph->rtminfo->with_weight = true;
    graph->rtminfo->with_cuda = true;
    graph->rtminfo->copy_data = false;
    graph->rtminfo->process_local = false;
    graph->rtminfo->reduce_comm = false;
    graph->rtminfo->process_overlap = false;
    graph->rtminfo->lock_free = false;
    PartitionedGraph *pgg = new PartitionedGraph(graph, all);
    pgg->GenerateAll([&](VertexId src, VertexId dst) { return nts::op::nts_norm_degree(graph, src, dst); }, GPU_T);
    graph->init_message_buffer();
    nts::op::ForwardSingleGPUfuseOp op(pgg, all);
    for (int width : widths) {
      NtsVar X = read_matrix("x" + std::to_string(width), vertices, width).cuda();
      std::vector<double> tf, tb;
      for (int rep = 0; rep < g_warmup + g_reps; ++rep) {
        double t0 = now();
        NtsVar Y = op.forward(X);
        double t1 = now();
        NtsVar G = op.backward(X);
        double t2 = now();
        if (rep >= g_warmup) {
          tf.push_back(t1 - t0);
          tb.push_back(t2 - t1);
        }
      }
      printf("reference ForwardSingleGPUfuseOp over libntship timing: V=%u E=%u F=%d forward_s=%.6f backward_s=%.6f "
             "best_forward_s=%.6f best_backward_s=%.6f reps=%d warmup=%d\n",
             vertices, pgg->owned_edges, width, median(tf), median(tb), *std::min_element(tf.begin(), tf.end()),
             *std::min_element(tb.begin(), tb.end()), g_reps, g_warmup);
    }
    return 0;
  }
  if (mode == "samp" || mode == "mini") {
    run_sampled_layers(graph, H, mode == "mini", F);
    return 0;
  }
  if (mode == "data") {
    graph->config->classes = H;
    graph->config->mode = "zerocopy";
    graph->init_gnnctx(graph->config->layer_string);
    GNNDatum *datum = new GNNDatum(graph->gnnctx, graph);
    datum->readFeature_Label_Mask(g_prefix + ".feat", g_prefix + ".label", g_prefix + ".mask");
    const size_t V = vertices, width = H > 1 ? H : 1;
    write_raw("local_feature", datum->local_feature, V * F * sizeof(ValueType));
    write_raw("local_label", datum->local_label, V * width * sizeof(long));
    write_raw("global_label", datum->global_label, V * width * sizeof(long));
    write_raw("local_mask", datum->local_mask, V * sizeof(int));
    write_raw("global_mask", datum->global_mask, V * sizeof(int));
    printf("reference GNNDatum::readFeature_Label_Mask done\n");
    return 0;
  }
#endif

  VertexSubset *active = graph->alloc_vertex_subset();
  active->fill();
  graph->init_gnnctx(graph->config->layer_string);
  graph->init_rtminfo();
  graph->rtminfo->process_local = false;
  graph->rtminfo->reduce_comm = false;
  graph->rtminfo->copy_data = false;
  graph->rtminfo->process_overlap = false;
  graph->rtminfo->with_weight = true;
  graph->rtminfo->lock_free = false;
  graph->rtminfo->with_cuda = false;

  // One CPU-side partitioned graph with the mirror index and whole-graph topology (dist = true), as
  // GAT_GPU_DIST sets it up (toolkits/GAT_GPU_DIST.hpp:67-70): the CPU operators read its chunks, the
  // DistGPU* operators upload its column_offset / row_indices / MirrorIndex themselves.
  PartitionedGraph *pg = new PartitionedGraph(graph, active);
  pg->GenerateAll([&](VertexId src, VertexId dst) { return nts::op::nts_norm_degree(graph, src, dst); }, CPU_T, true);
  graph->init_communicatior();
  const long V = vertices, E = pg->owned_edges;
  printf("reference graph: V=%ld E=%ld mirrors=%u\n", V, E, pg->owned_mirrors);

  if (agg_only) {
    nts::op::ForwardCPUfuseOp op(pg, active);
    for (int width : widths) {
      NtsVar X = read_matrix("x" + std::to_string(width), V, width);
      std::vector<double> tf, tb;
      for (int rep = 0; rep < g_warmup + g_reps; ++rep) {
        double t0 = now();
        NtsVar Y = op.forward(X);
        double t1 = now();
        NtsVar G = op.backward(X);
        double t2 = now();
        if (rep >= g_warmup) {
          tf.push_back(t1 - t0);
          tb.push_back(t2 - t1);
        }
      }
      printf("reference ForwardCPUfuseOp timing: V=%ld E=%ld F=%d forward_s=%.6f backward_s=%.6f threads=%d "
             "best_forward_s=%.6f best_backward_s=%.6f reps=%d warmup=%d\n",
             V, E, width, median(tf), median(tb), graph->threads, *std::min_element(tf.begin(), tf.end()),
             *std::min_element(tb.begin(), tb.end()), g_reps, g_warmup);
    }
    return 0;
  }

  CSC_segment_pinned *chunk = pg->graph_chunks[0];
  write_raw("column_offset", chunk->column_offset, (V + 1) * sizeof(VertexId));
  write_raw("row_indices", chunk->row_indices, E * sizeof(VertexId));
  write_raw("edge_weight_forward", chunk->edge_weight_forward, E * sizeof(ValueType));
  write_raw("row_offset", chunk->row_offset, (V + 1) * sizeof(VertexId));
  write_raw("column_indices", chunk->column_indices, E * sizeof(VertexId));
  write_raw("edge_weight_backward", chunk->edge_weight_backward, E * sizeof(ValueType));
  write_raw("mirror_index", pg->MirrorIndex, (V + 1) * sizeof(VertexId));

  NtsVar X = read_matrix("x", V, F);
  NtsVar M = read_matrix("m", E, H), GM = read_matrix("gm", E, H);
  NtsVar Emsg = read_matrix("e", E, F), G2 = read_matrix("g2", E, 2 * F);
  NtsVar M1 = M.slice(1, 0, 1).contiguous(), GM1 = GM.slice(1, 0, 1).contiguous();

  if (run_cpu) {
    {
      nts::op::ForwardCPUfuseOp op(pg, active);
      double t0 = now();
      NtsVar Y = op.forward(X);
      double t1 = now();
      NtsVar G = op.backward(X);
      double t2 = now();
      write_tensor("cpu_fwd", Y);
      write_tensor("cpu_bwd", G);
      printf("reference ForwardCPUfuseOp: forward %.6f s backward %.6f s threads %d\n", t1 - t0, t2 - t1,
             graph->threads);
    }
    {
      nts::op::SingleCPUSrcDstScatterOp op(pg, active);
      write_tensor("cpu_scatter", op.forward(X));
      write_tensor("cpu_scatter_bwd", op.backward(G2));
    }
    {
      nts::op::SingleEdgeSoftMax op(pg, active);
      write_tensor("cpu_softmax", op.forward(M));
      // The backward expression is only shape-correct for one column (d.t().mm(imr) is H x H).
      nts::op::SingleEdgeSoftMax op1(pg, active);
      NtsVar y1 = op1.forward(M1);
      write_tensor("cpu_softmax1", y1);
      write_tensor("cpu_softmax1_bwd", op1.backward(GM1));
    }
    {
      nts::op::SingleCPUDstAggregateOp op(pg, active);
      write_tensor("cpu_agg", op.forward(Emsg));
      write_tensor("cpu_agg_bwd", op.backward(X));
    }
    printf("reference CPU operators done\n");
  }
#if CUDA_ENABLE
  if (run_gpu) {
    {
      graph->rtminfo->with_cuda = true;
      PartitionedGraph *pgg = new PartitionedGraph(graph, active);
      pgg->GenerateAll([&](VertexId src, VertexId dst) { return nts::op::nts_norm_degree(graph, src, dst); }, GPU_T);
      graph->init_message_buffer();
      NtsVar Xg = X.cuda();
      nts::op::ForwardSingleGPUfuseOp op(pgg, active);
      write_tensor("gpu_fwd", op.forward(Xg));
      write_tensor("gpu_bwd", op.backward(Xg));
    }
    {
      // DistGPUScatterSrc reads rows of the mirror tensor: row MirrorIndex[v] holds vertex v, for
      // every vertex with an outgoing edge (what DistGPUGetDepNbrOp delivers at one partition).
      std::vector<long> mirror_vertices;
      for (long v = 0; v < V; ++v)
        if (pg->MirrorIndex[v + 1] != pg->MirrorIndex[v]) mirror_vertices.push_back(v);
      NtsVar sel = torch::from_blob(mirror_vertices.data(), {static_cast<long>(mirror_vertices.size())}, torch::kLong);
      NtsVar mirror = X.index_select(0, sel).cuda();
      NtsVar Xg = X.cuda(), G2g = G2.cuda();
      nts::op::DistGPUScatterSrc src_op(pg, active);
      nts::op::DistGPUScatterDst dst_op(pg, active);
      write_tensor("gpu_scatter_src", src_op.forward(mirror));
      write_tensor("gpu_scatter_dst", dst_op.forward(Xg));
      NtsVar gs = G2g.slice(1, 0, F).contiguous(), gd = G2g.slice(1, F, 2 * F).contiguous();
      write_tensor("gpu_scatter_src_bwd", src_op.backward(gs));
      write_tensor("gpu_scatter_dst_bwd", dst_op.backward(gd));
    }
    {
      NtsVar Mg = M.cuda(), M1g = M1.cuda(), GM1g = GM1.cuda();
      nts::op::DistGPUEdgeSoftMax op(pg, active);
      write_tensor("gpu_softmax", op.forward(Mg));
      nts::op::DistGPUEdgeSoftMax op1(pg, active);
      write_tensor("gpu_softmax1", op1.forward(M1g));
      write_tensor("gpu_softmax1_bwd", op1.backward(GM1g));
    }
    {
      NtsVar Eg = Emsg.cuda(), Xg = X.cuda();
      nts::op::DistGPUAggregateDst op(pg, active);
      write_tensor("gpu_agg", op.forward(Eg));
      write_tensor("gpu_agg_bwd", op.backward(Xg));
    }
    printf("reference GPU operators over libntship done\n");
  }
#else
  if (run_gpu) {
    fprintf(stderr, "this build has no GPU operators\n");
    return 2;
  }
#endif
  return 0;
}
