// Driver around the REFERENCE's own mini-batch path, compiled from the reference tree where it lies by
// oracle/build_toolkits.sh (it needs core/ntsSampler.hpp and core/ntsMiniBatchGraphOp.hpp, which include
// METIS: see that script).  INTEGRATION DEMONSTRATION ONLY; nothing here pins the oracle.
//
// With the configuration file of a GCNNEIGHBORGPU run it does what the toolkit does up to the first
// batches (toolkits/GCN_GPU_NEIGHBOR.hpp:116-131, 177-183, 1350-1378, 404-463): the reference's loader,
// its fully replicated graph, its own Sampler::sample_one with the reference's random neighbour pick,
// SampledSubgraph::trans_graph_to_gpu_async over the HIP veneer -- and then, for every layer of every
// sampled batch, runs the reference's two operator classes on the same input:
//   CPU  nts::op::MiniBatchFuseOp          (core/ntsMiniBatchGraphOp.hpp:145-245)
//   GPU  nts::op::SingleGPUSampleGraphOp   (core/ntsMiniBatchGraphOp.hpp:248-376) over libntship.so
// and prints, per layer and direction, the largest |gpu - cpu| / max(|gpu|, |cpu|, 1e-2 * sum|terms|)
// (sum|terms| from the CPU operator run on |input|; edge weights are positive) and how many output
// rows are equal bit for bit.
//
//   usage: ref_minibatch <cfg file> <batches> [time]
// With `time` nothing touches the device: after one untimed batch, the reference's Sampler::sample_one
// (neighbour pick, relabelling, CSR, weights: its whole host side) and its CPU operator MiniBatchFuseOp
// (forward and backward of every layer) are timed on <batches> batches and the totals printed -- the
// reference's own CPU cost of the steps this library moves to the GPU.
#include "core/neutronstar.hpp"  // what the toolkits include: graph, sampler, operators

#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstdio>
#include <string>
#include <vector>

static double worst_ratio(const NtsVar &gpu, const NtsVar &cpu, const NtsVar &scale, long *equal_rows) {
  NtsVar g = gpu.cpu().contiguous(), c = cpu.contiguous(), s = scale.contiguous();
  const float *pg = g.data_ptr<float>(), *pc = c.data_ptr<float>(), *ps = s.data_ptr<float>();
  const long rows = c.size(0), F = c.size(1);
  double worst = 0;
  long same = 0;
  for (long r = 0; r < rows; ++r) {
    bool eq = true;
    for (long f = 0; f < F; ++f) {
      const double a = pg[r * F + f], b = pc[r * F + f];
      const double den = std::max(std::max(std::fabs(a), std::fabs(b)), 1e-2 * std::fabs((double)ps[r * F + f]) + 1e-30);
      worst = std::max(worst, std::fabs(a - b) / den);
      eq = eq && pg[r * F + f] == pc[r * F + f];
    }
    same += eq;
  }
  *equal_rows = same;
  return worst;
}

int main(int argc, char **argv) {
  MPI_Instance mpi(&argc, &argv);
  if (argc < 3) {
    fprintf(stderr, "usage: %s cfg_file batches\n", argv[0]);
    return 2;
  }
  const int batches = std::stoi(argv[2]);
  Graph<Empty> *graph = new Graph<Empty>();
  graph->config->readFromCfgFile(argv[1]);
  graph->replication_threshold = graph->config->repthreshold;
  graph->load_directed(graph->config->edge_file, graph->config->vertices);
  graph->generate_backward_structure();
  // GCN_GPU_NEIGHBOR_impl's constructor and init_graph
  graph->init_gnnctx(graph->config->layer_string);
  graph->init_gnnctx_fanout(graph->gnnctx->fanout, graph->config->fanout_string);
  graph->init_gnnctx_fanout(graph->gnnctx->val_fanout, graph->config->val_fanout_string);
  std::reverse(graph->gnnctx->fanout.begin(), graph->gnnctx->fanout.end());
  std::reverse(graph->gnnctx->val_fanout.begin(), graph->gnnctx->val_fanout.end());
  graph->init_rtminfo();
  graph->rtminfo->process_local = graph->config->process_local;
  graph->rtminfo->reduce_comm = graph->config->process_local;
  graph->rtminfo->copy_data = false;
  graph->rtminfo->process_overlap = graph->config->overlap;
  graph->rtminfo->with_weight = true;
  graph->rtminfo->with_cuda = false;
  graph->rtminfo->lock_free = graph->config->lock_free;
  FullyRepGraph *fully_rep_graph = new FullyRepGraph(graph);
  fully_rep_graph->GenerateAll();
  fully_rep_graph->SyncAndLog("read_finish");

  std::vector<VertexId> train_nids;
  for (VertexId v = 0; v < graph->vertices; v += 2) train_nids.push_back(v);  // every other vertex trains
  Sampler *sampler = new Sampler(fully_rep_graph, train_nids, 1, false);
  if (argc > 3 && std::string(argv[3]) == "time") {
    auto now = [] { return std::chrono::duration<double>(std::chrono::steady_clock::now().time_since_epoch()).count(); };
    const int n_layers = graph->gnnctx->layer_size.size() - 1;
    double t_sample = 0, t_aggregate = 0;
    long edges = 0;
    int timed = 0;
    torch::manual_seed(1234);
    for (int b = 0; b < batches + 1 && sampler->work_offset < sampler->work_range[1]; ++b) {
      SampledSubgraph *ssg = sampler->subgraph_list[0];
      double t0 = now();
      sampler->sample_one(ssg, graph->config->batch_type, true);
      const double ts = now() - t0;
      double ta = 0;
      for (int l = 0; l < n_layers; ++l) {
        sampCSC *sg = ssg->sampled_sgs[l];
        const long F = graph->gnnctx->layer_size[l];
        NtsVar X = torch::randn({(long)sg->src_size, F});
        NtsVar G = torch::randn({(long)sg->v_size, F});
        nts::op::MiniBatchFuseOp op(ssg, graph, l);
        t0 = now();
        NtsVar Y = op.forward(X);
        NtsVar D = op.backward(G);
        ta += now() - t0;
        if (b > 0) edges += sg->e_size;
      }
      if (b > 0) {  // the first batch starts the thread pools and touches the buffers for the first time
        t_sample += ts;
        t_aggregate += ta;
        ++timed;
      }
      sampler->reverse_sgs(ssg);
    }
    printf("reference mini-batch cpu timing: batches=%d sample_s=%.6f aggregate_s=%.6f sampled_edges=%ld threads=%d\n", timed,
           t_sample, t_aggregate, edges, omp_get_max_threads());
    return 0;
  }
  Cuda_Stream *cs = new Cuda_Stream();
  const int layers = graph->gnnctx->layer_size.size() - 1;
  torch::manual_seed(1234);
  double worst_all = 0;
  for (int b = 0; b < batches && sampler->work_offset < sampler->work_range[1]; ++b) {
    SampledSubgraph *ssg = sampler->subgraph_list[0];
    sampler->sample_one(ssg, graph->config->batch_type, true);
    cudaStreamSynchronize(cs->stream);
    ssg->trans_graph_to_gpu_async(cs->stream, graph->config->mini_pull > 0);
    cudaStreamSynchronize(cs->stream);
    for (int l = 0; l < layers; ++l) {
      sampCSC *sg = ssg->sampled_sgs[l];
      const long F = graph->gnnctx->layer_size[l];
      NtsVar X = torch::randn({(long)sg->src_size, F});
      NtsVar G = torch::randn({(long)sg->v_size, F});
      nts::op::MiniBatchFuseOp cpu_op(ssg, graph, l), cpu_abs(ssg, graph, l);
      nts::op::SingleGPUSampleGraphOp gpu_op(ssg, graph, l, cs);
      NtsVar Xg = X.cuda(), Gg = G.cuda(), Xa = X.abs(), Ga = G.abs();
      NtsVar Yc = cpu_op.forward(X), Ys = cpu_abs.forward(Xa), Yg = gpu_op.forward(Xg);
      NtsVar Dc = cpu_op.backward(G), Ds = cpu_abs.backward(Ga), Dg = gpu_op.backward(Gg);
      long same_f = 0, same_b = 0;
      const double ef = worst_ratio(Yg, Yc, Ys, &same_f), eb = worst_ratio(Dg, Dc, Ds, &same_b);
      worst_all = std::max(worst_all, std::max(ef, eb));
      printf("reference operators: batch %d layer %d v_size %u e_size %u src_size %u F %ld forward_max_rel_err %.3e "
             "forward_equal_rows %ld backward_max_rel_err %.3e backward_equal_rows %ld\n",
             b, l, sg->v_size, sg->e_size, sg->src_size, F, ef, same_f, eb, same_b);
    }
    sampler->reverse_sgs(ssg);
  }
  printf("reference SingleGPUSampleGraphOp vs MiniBatchFuseOp: worst_max_rel_err %.3e\n", worst_all);
  return worst_all <= 1e-4 ? 0 : 1;
}
