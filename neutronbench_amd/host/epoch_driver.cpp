// One epoch of the sampled mini-batch path driven from C++ through the C ABI: the batch loop of
// toolkits/GCN_GPU_NEIGHBOR.hpp (run(): 386-500; the PIPELINES mode: 1350-1363) with this library's own
// sampler in place of the reference's CPU sampler, and without the dense layers.
//
// Per batch: nts_batch_builder_sample / _layers (all hops, relabelling, CSR, weights), the feature
// gather (zero-copy from mapped pinned host memory, or through the HBM cache of the top out-degree
// vertices), the label gather, and for every layer the aggregation forward (one launch: the hop's
// fanout bounds every destination's edges, nts_spmm_gather_bounded) and, in reverse order, backward
// (sources can be hubs: nts_spmm_gather cuts long rows on the device).  Outputs are written, not added
// to, so no buffer is cleared first.  With --heads H every
// layer is a GAT layer instead: fused attention (nts_gat_attention_fwd) and attention-weighted
// aggregation (nts_spmm_gather_heads) forward; backward the aggregation over the CSR, the per-edge
// gradient of alpha (nts_sddmm_heads), the fused attention backward and the sum of the edge
// gradients per source (nts_gather_edge_to_src).  Inputs of the layers after the first, the attention
// terms and the incoming gradients stand in for the dense layers' results: constant buffers of the
// right shape, filled once with pseudo-random values.
//
// --pipeline 1: everything on one stream.  --pipeline 2: the next batch is sampled on a second stream
// while this one is gathered and aggregated.  --pipeline P >= 3: P - 2 batches are sampled ahead, each
// chain of hops on a stream of its own, the next batch's features and labels are gathered on a gather
// stream, the current one is aggregated; events order a batch's gather before its aggregation and
// an arena's re-use after the aggregation that read it.  One host thread enqueues all of it.
// --graph g: how the builders replay their launches (nts_batch_builder_use_graph; with 3 the
// transposed structure is built beside the feature gather and joined before the first aggregation).
// --hw-queues n: hardware queues asked of the HIP runtime before it starts (default: 8 with
// --pipeline 4, see main()).
//
// The program reads raw arrays written by neutronbench_amd/epoch.py (--native): co.bin, ri.bin (uint32
// CSC of the whole graph), feat.bin (float32 [V, F]), labels.bin (int64 [V]), train.bin (uint32 ids),
// and prints one JSON line.  --verify 1 adds a checksum of every aggregation output (a device-side
// hash per batch, which waits for the stream: not for timing).  --dump-dir D [--dump-batch b]: after the
// timed epoch, batch b runs once more through the same calls and every array it produced -- the
// layers' structure, the gathered features and labels, each aggregation's input and output -- is
// written to D as raw files with a meta.json, for a checker to compare with the CPU oracle.
#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <chrono>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <numeric>
#include <string>
#include <vector>

#include "nts_hip.h"

namespace {

[[noreturn]] void die(const char *what) {
  fprintf(stderr, "nts_epoch: %s: %s\n", what, nts_last_error());
  exit(1);
}
#define NTS(call)                 \
  do {                            \
    if ((call) != NTS_OK) die(#call); \
  } while (0)
#define HIP(call)                                                              \
  do {                                                                         \
    hipError_t e_ = (call);                                                    \
    if (e_ != hipSuccess) {                                                    \
      fprintf(stderr, "nts_epoch: %s: %s\n", #call, hipGetErrorString(e_));    \
      exit(1);                                                                 \
    }                                                                          \
  } while (0)

double now() {
  return std::chrono::duration<double>(std::chrono::steady_clock::now().time_since_epoch()).count();
}

template <typename T>
std::vector<T> read_file(const std::string &path, size_t expect = 0) {
  FILE *f = fopen(path.c_str(), "rb");
  if (!f) {
    fprintf(stderr, "nts_epoch: cannot open %s\n", path.c_str());
    exit(1);
  }
  fseek(f, 0, SEEK_END);
  const size_t bytes = static_cast<size_t>(ftell(f));
  fseek(f, 0, SEEK_SET);
  std::vector<T> v(bytes / sizeof(T));
  if (fread(v.data(), sizeof(T), v.size(), f) != v.size() || (expect && v.size() != expect)) {
    fprintf(stderr, "nts_epoch: %s holds %zu elements, expected %zu\n", path.c_str(), v.size(), expect);
    exit(1);
  }
  fclose(f);
  return v;
}

template <typename T>
T *to_device(const std::vector<T> &v) {
  void *p = nullptr;
  NTS(nts_malloc_device(&p, std::max<size_t>(v.size() * sizeof(T), 256)));
  if (!v.empty()) NTS(nts_memcpy_h2d(p, v.data(), v.size() * sizeof(T), 1));
  return static_cast<T *>(p);
}

void *device_bytes(size_t bytes) {
  void *p = nullptr;
  NTS(nts_malloc_device(&p, std::max<size_t>(bytes, 256)));
  return p;
}

struct Args {
  std::string dir, dump_dir;
  uint32_t dump_batch = 0;
  std::vector<int32_t> fanout;
  uint32_t V = 0, F = 0, hidden = 128, batch = 1024, pipeline = 1, warmup = 2, max_batches = 0, heads = 0;
  double cache = 0.0;
  int graph = 1, verify = 0, stage_sync = 0;
  int hw_queues = -1;  // -1: 8 for --pipeline 4, else the runtime's own count
};

Args parse(int argc, char **argv) {
  Args a;
  for (int i = 1; i + 1 < argc; i += 2) {
    const std::string k = argv[i], v = argv[i + 1];
    if (k == "--dir") a.dir = v;
    else if (k == "--V") a.V = static_cast<uint32_t>(std::stoul(v));
    else if (k == "--F") a.F = static_cast<uint32_t>(std::stoul(v));
    else if (k == "--hidden") a.hidden = static_cast<uint32_t>(std::stoul(v));
    else if (k == "--batch") a.batch = static_cast<uint32_t>(std::stoul(v));
    else if (k == "--pipeline") a.pipeline = static_cast<uint32_t>(std::stoul(v));
    else if (k == "--warmup") a.warmup = static_cast<uint32_t>(std::stoul(v));
    else if (k == "--max-batches") a.max_batches = static_cast<uint32_t>(std::stoul(v));
    else if (k == "--heads") a.heads = static_cast<uint32_t>(std::stoul(v));
    else if (k == "--cache") a.cache = std::stod(v);
    else if (k == "--graph") a.graph = std::stoi(v);
    else if (k == "--verify") a.verify = std::stoi(v);
    else if (k == "--stage-sync") a.stage_sync = std::stoi(v);
    else if (k == "--hw-queues") a.hw_queues = std::stoi(v);
    else if (k == "--dump-dir") a.dump_dir = v;
    else if (k == "--dump-batch") a.dump_batch = static_cast<uint32_t>(std::stoul(v));
    else if (k == "--fanout") {
      size_t at = 0;
      while (at < v.size()) {
        size_t end = v.find(',', at);
        if (end == std::string::npos) end = v.size();
        a.fanout.push_back(std::stoi(v.substr(at, end - at)));
        at = end + 1;
      }
    } else {
      fprintf(stderr, "nts_epoch: unknown option %s\n", k.c_str());
      exit(2);
    }
  }
  if (a.dir.empty() || !a.V || !a.F || a.fanout.empty() || a.pipeline < 1 || a.pipeline > 8 ||
      (a.heads && a.hidden % a.heads)) {
    fprintf(stderr,
            "usage: nts_epoch --dir D --V n --F n --fanout a,b[,c] [--batch n] [--hidden n] [--heads n] [--pipeline 1..8]\n"
            "                 [--cache fraction] [--graph 0|1|2|3] [--warmup n] [--max-batches n] [--verify 0|1] [--stage-sync 0|1]\n"
            "                 [--hw-queues n] [--dump-dir D [--dump-batch b]]\n");
    exit(2);
  }
  return a;
}

struct Slot {  // one batch in flight
  nts_batch_builder_t *builder = nullptr;
  void *arena = nullptr;
  nts_sampled_layer_t layers[8];
  float *x = nullptr;       // gathered features [src_size of the input layer, F]
  int64_t *labels = nullptr;
  uint32_t *hits = nullptr;
  hipEvent_t gathered = nullptr, trained = nullptr;
  bool has_trained = false;
};

}  // namespace

int main(int argc, char **argv) {
  const Args a = parse(argc, argv);
  // Hardware queues of the process (the HIP runtime reads GPU_MAX_HW_QUEUES when it starts; its own count
  // is 4).  With four batches in flight the loop below feeds four streams -- training, gather and two
  // sampling chains -- beside the streams the library records its graphs on, and with four queues two of
  // them share one: a gather then waits behind a whole sampling chain.  Measured with 6 to 16 queues
  // against 4: four in flight 0.0226 -> 0.0174 s (Arxiv-shaped), 0.0255 -> 0.0212 s (Products-shaped),
  // 0.0151 -> 0.0157 s (GAT); five and six in flight get slower with them (GAT 0.019 -> 0.026-0.035 s), two
  // and three and the serial loop do not change.  So: 8 for --pipeline 4 unless --hw-queues says otherwise
  // (0 = leave the environment alone).
  {
    const int queues = a.hw_queues >= 0 ? a.hw_queues : (a.pipeline == 4 ? 8 : 0);
    if (queues > 0) setenv("GPU_MAX_HW_QUEUES", std::to_string(queues).c_str(), 1);
  }
  const uint32_t hops = static_cast<uint32_t>(a.fanout.size());
  const uint32_t V = a.V, F = a.F;
  std::vector<uint32_t> co = read_file<uint32_t>(a.dir + "/co.bin", static_cast<size_t>(V) + 1);
  std::vector<uint32_t> ri = read_file<uint32_t>(a.dir + "/ri.bin");
  const uint32_t E = static_cast<uint32_t>(ri.size());
  std::vector<int64_t> labels_h = read_file<int64_t>(a.dir + "/labels.bin", V);
  std::vector<uint32_t> train = read_file<uint32_t>(a.dir + "/train.bin");
  uint32_t *d_co = to_device(co), *d_ri = to_device(ri), *d_train = to_device(train);
  int64_t *d_labels = to_device(labels_h);

  // Feature table in mapped pinned host memory, read by the device over the link.
  float *table = nullptr;
  NTS(nts_malloc_pinned_mapped(reinterpret_cast<void **>(&table), static_cast<size_t>(V) * F * sizeof(float)));
  {
    std::vector<float> feat = read_file<float>(a.dir + "/feat.bin", static_cast<size_t>(V) * F);
    memcpy(table, feat.data(), feat.size() * sizeof(float));
  }
  // HBM cache of the top out-degree vertices (descending out-degree, ties by ascending id).
  const uint32_t n_cache = static_cast<uint32_t>(a.cache * V);
  float *d_cache = nullptr;
  uint32_t *d_hashmap = nullptr;
  if (n_cache) {
    std::vector<uint32_t> outdeg(V, 0);
    for (uint32_t s : ri) ++outdeg[s];
    std::vector<uint32_t> order(V);
    std::iota(order.begin(), order.end(), 0u);
    std::stable_sort(order.begin(), order.end(), [&](uint32_t x, uint32_t y) { return outdeg[x] > outdeg[y]; });
    std::vector<uint32_t> hashmap(V, 0xFFFFFFFFu);
    std::vector<float> rows(static_cast<size_t>(n_cache) * F);
    for (uint32_t k = 0; k < n_cache; ++k) {
      hashmap[order[k]] = k;
      memcpy(rows.data() + static_cast<size_t>(k) * F, table + static_cast<size_t>(order[k]) * F, F * sizeof(float));
    }
    d_cache = to_device(rows);
    d_hashmap = to_device(hashmap);
  }

  // Capacities: rows of a layer never exceed the graph or the product of the fanouts so far.
  uint64_t max_rows = a.batch;
  for (int32_t f : a.fanout) max_rows = f < 0 ? V : std::min<uint64_t>(V, max_rows * static_cast<uint32_t>(f));
  const uint32_t maxw = std::max(F, a.hidden);
  const uint32_t H = a.heads, Fh = H ? a.hidden / H : 0;
  // Edge capacity of every hop, as the builder lays it out (hop 0 = the batch's own hop).
  std::vector<uint64_t> e_cap(hops);
  {
    uint64_t vd = a.batch;
    for (uint32_t h = 0; h < hops; ++h) {
      uint64_t e = a.fanout[h] < 0 ? E : vd * static_cast<uint32_t>(a.fanout[h]);
      if (e > E && (h > 0 || a.fanout[h] < 0)) e = E;
      e_cap[h] = e;
      vd = std::min<uint64_t>(e, V);
    }
  }
  const uint64_t max_edges = *std::max_element(e_cap.begin(), e_cap.end());
  const uint32_t P = a.pipeline;
  std::vector<Slot> slots(P);
  const int want_perm = H ? 1 : 0;  // GAT layers walk the CSR through csr_to_csc
  const size_t arena_bytes = nts_batch_builder_arena_bytes(V, E, a.fanout.data(), hops, a.batch, want_perm);
  if (!arena_bytes) die("nts_batch_builder_arena_bytes");
  const uint32_t x_buffers = P >= 3 ? 2 : 1;  // the gather of the next batch overlaps this one's aggregation
  std::vector<float *> xbuf(x_buffers);
  std::vector<int64_t *> lbuf(x_buffers);
  std::vector<uint32_t *> hbufs(x_buffers);
  for (uint32_t k = 0; k < x_buffers; ++k) {
    xbuf[k] = static_cast<float *>(device_bytes(max_rows * F * sizeof(float)));
    lbuf[k] = static_cast<int64_t *>(device_bytes(static_cast<size_t>(a.batch) * sizeof(int64_t)));
    hbufs[k] = static_cast<uint32_t *>(device_bytes(256));
  }
  for (Slot &s : slots) {
    s.arena = device_bytes(arena_bytes);
    NTS(nts_batch_builder_create(&s.builder, d_co, d_ri, V, E, a.fanout.data(), hops, a.batch, want_perm, s.arena,
                                 arena_bytes));
    if (a.graph) NTS(nts_batch_builder_use_graph(s.builder, a.graph));
    HIP(hipEventCreateWithFlags(&s.gathered, hipEventDisableTiming));
    HIP(hipEventCreateWithFlags(&s.trained, hipEventDisableTiming));
  }
  // Stand-ins for what the dense layers would hand over, and the aggregation outputs.
  std::vector<float> ones(max_rows * maxw + 64);  // the stand-ins start a few (whole 16-byte) words apart
  {
    uint32_t state = 12345u;  // values in [-1, 1)
    for (float &v : ones) {
      state = state * 1664525u + 1013904223u;
      v = static_cast<float>(static_cast<int32_t>(state)) * (1.0f / 2147483648.0f);
    }
  }
  float *d_ones = to_device(ones);
  ones.clear();
  ones.shrink_to_fit();
  // GAT: alpha of every layer is kept until its backward; er is zero as in the Python loop
  std::vector<float *> d_alpha(hops, nullptr);
  float *d_er = nullptr, *d_galpha = nullptr, *d_gs = nullptr, *d_ger = nullptr, *d_gel = nullptr;
  if (H) {
    for (uint32_t l = 0; l < hops; ++l) d_alpha[l] = static_cast<float *>(device_bytes(e_cap[hops - 1 - l] * H * sizeof(float)));
    d_er = static_cast<float *>(device_bytes(max_rows * H * sizeof(float)));
    NTS(nts_memset_zero(d_er, max_rows * H * sizeof(float), nullptr));
    HIP(hipDeviceSynchronize());
    d_galpha = static_cast<float *>(device_bytes(max_edges * H * sizeof(float)));
    d_gs = static_cast<float *>(device_bytes(max_edges * H * sizeof(float)));
    d_ger = static_cast<float *>(device_bytes(max_rows * H * sizeof(float)));
    d_gel = static_cast<float *>(device_bytes(max_rows * H * sizeof(float)));
  }
  float *d_out = static_cast<float *>(device_bytes(max_rows * maxw * sizeof(float)));
  float *d_gin = static_cast<float *>(device_bytes(max_rows * maxw * sizeof(float)));

  hipStream_t main_stream = nullptr, gather_stream = nullptr;
  HIP(hipStreamCreateWithFlags(&main_stream, hipStreamNonBlocking));
  std::vector<hipStream_t> sample_streams;
  if (P >= 2) {
    const uint32_t chains = P >= 3 ? P - 2 : 1;
    sample_streams.resize(chains);
    for (hipStream_t &s : sample_streams) HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
  }
  if (P >= 3) HIP(hipStreamCreateWithFlags(&gather_stream, hipStreamNonBlocking));

  const uint32_t n_train = static_cast<uint32_t>(train.size());
  uint32_t n_batches = (n_train + a.batch - 1) / a.batch;
  if (a.max_batches && a.max_batches < n_batches) n_batches = a.max_batches;
  uint64_t edges_total = 0, rows_total = 0, checksum = 0;
  std::vector<uint32_t *> hit_words;  // device words read at the end of the epoch
  double t_sample = 0, t_gather = 0, t_fwd = 0, t_bwd = 0;

  auto sample = [&](Slot &s, uint32_t b, hipStream_t stream) {
    const uint32_t n = std::min(a.batch, n_train - b * a.batch);
    NTS(nts_batch_builder_sample(s.builder, d_train + static_cast<size_t>(b) * a.batch, n, 1000ull * b, stream));
  };
  auto gather = [&](Slot &s, uint32_t buffer, hipStream_t stream) {
    const nts_sampled_layer_t &in = s.layers[0], &top = s.layers[hops - 1];
    s.x = xbuf[buffer];
    s.labels = lbuf[buffer];
    s.hits = hbufs[buffer];
    if (n_cache)
      NTS(nts_gather_rows_cached_f32(s.x, table, d_cache, in.source, d_hashmap, in.src_size, F, s.hits, stream));
    else
      NTS(nts_gather_rows_f32(s.x, table, in.source, nullptr, nullptr, in.src_size, F, stream));
    NTS(nts_gather_labels_i64(s.labels, d_labels, top.destination, top.v_size, 1, stream));
  };
  uint64_t hits_total = 0;
  auto hash = [&](const float *p, uint64_t n, uint64_t salt, hipStream_t stream) {
    uint64_t fp = 0;
    NTS(nts_fingerprint_u32(&fp, reinterpret_cast<const uint32_t *>(p), n, nullptr, 0, stream));
    checksum ^= fp * (2 * salt + 1);
  };
  // Dump mode (after the timed epoch): every array of the batch goes to a file as the stages produce it.
  bool dumping = false;
  auto dump = [&](const std::string &name, const void *dev, size_t bytes, hipStream_t stream) {
    HIP(hipStreamSynchronize(stream));
    std::vector<char> host(bytes);
    if (bytes) HIP(hipMemcpy(host.data(), dev, bytes, hipMemcpyDeviceToHost));
    FILE *f = fopen((a.dump_dir + "/" + name).c_str(), "wb");
    if (!f || (bytes && fwrite(host.data(), 1, bytes, f) != bytes)) {
      fprintf(stderr, "nts_epoch: cannot write %s/%s\n", a.dump_dir.c_str(), name.c_str());
      exit(1);
    }
    fclose(f);
  };
  auto tag = [](const char *what, uint32_t layer) { return "L" + std::to_string(layer) + "_" + what + ".bin"; };
  auto aggregate_gat = [&](Slot &s, hipStream_t stream) {
    const float slope = 0.2f;
    double t0 = now();
    for (uint32_t l = 0; l < hops; ++l) {
      const nts_sampled_layer_t &L = s.layers[l];
      const float *x = d_ones;  // [src_size, H * Fh]: stands in for the projected features of the layer
      const float *el = d_ones + 8;  // [src_size, H]
      NTS(nts_gat_attention_fwd_bounded(d_alpha[l], el, d_er, L.column_offset, L.row_indices, L.v_size, H, slope,
                                        L.max_in_degree, stream));
      NTS(nts_spmm_gather_heads_bounded(x, d_out, d_alpha[l], nullptr, L.column_offset, L.row_indices, L.v_size, L.e_size,
                                        H, Fh, 0, L.max_in_degree, stream));
      if (a.verify) {
        hash(d_alpha[l], static_cast<uint64_t>(L.e_size) * H, 10 + l, stream);
        hash(d_out, static_cast<uint64_t>(L.v_size) * H * Fh, 20 + l, stream);
      }
      if (dumping) {
        dump(tag("x", l), x, static_cast<size_t>(L.src_size) * H * Fh * 4, stream);
        dump(tag("el", l), el, static_cast<size_t>(L.src_size) * H * 4, stream);
        dump(tag("er", l), d_er, static_cast<size_t>(L.v_size) * H * 4, stream);
        dump(tag("alpha", l), d_alpha[l], static_cast<size_t>(L.e_size) * H * 4, stream);
        dump(tag("out", l), d_out, static_cast<size_t>(L.v_size) * H * Fh * 4, stream);
      }
      if (a.stage_sync) HIP(hipStreamSynchronize(stream));
    }
    if (a.stage_sync) t_fwd += now() - t0;
    t0 = now();
    for (uint32_t k = hops; k-- > 0;) {
      const nts_sampled_layer_t &L = s.layers[k];
      const float *x = d_ones, *el = d_ones + 8, *g_out = d_ones + 4;  // g_out: [v_size, H * Fh]
      NTS(nts_spmm_gather_heads(g_out, d_gin, d_alpha[k], L.csr_to_csc, L.row_offset, L.column_indices, L.src_size,
                                L.e_size, H, Fh, 0, stream));
      NTS(nts_sddmm_heads(d_galpha, x, g_out, L.column_offset, L.row_indices, L.v_size, H, Fh, stream));
      NTS(nts_gat_attention_bwd_bounded(d_gs, d_ger, d_galpha, d_alpha[k], el, d_er, L.column_offset, L.row_indices,
                                        L.v_size, H, slope, L.max_in_degree, stream));
      NTS(nts_gather_edge_to_src(d_gel, d_gs, L.row_offset, L.csr_to_csc, L.src_size, H, 0, stream));
      if (a.verify) {
        hash(d_gin, static_cast<uint64_t>(L.src_size) * H * Fh, 30 + k, stream);
        hash(d_ger, static_cast<uint64_t>(L.v_size) * H, 40 + k, stream);
        hash(d_gel, static_cast<uint64_t>(L.src_size) * H, 50 + k, stream);
      }
      if (dumping) {
        dump(tag("gout", k), g_out, static_cast<size_t>(L.v_size) * H * Fh * 4, stream);
        dump(tag("gin", k), d_gin, static_cast<size_t>(L.src_size) * H * Fh * 4, stream);
        dump(tag("galpha", k), d_galpha, static_cast<size_t>(L.e_size) * H * 4, stream);
        dump(tag("gs", k), d_gs, static_cast<size_t>(L.e_size) * H * 4, stream);
        dump(tag("ger", k), d_ger, static_cast<size_t>(L.v_size) * H * 4, stream);
        dump(tag("gel", k), d_gel, static_cast<size_t>(L.src_size) * H * 4, stream);
      }
      if (a.stage_sync) HIP(hipStreamSynchronize(stream));
    }
    if (a.stage_sync) t_bwd += now() - t0;
  };
  auto aggregate = [&](Slot &s, hipStream_t stream) {
    // --graph 3: the transposed structure and the weights are still being built on the builder's own
    // stream while the features are gathered; the aggregation is the first to read them
    NTS(nts_batch_builder_join(s.builder, stream));
    if (H) return aggregate_gat(s, stream);
    double t0 = now();
    for (uint32_t l = 0; l < hops; ++l) {
      const nts_sampled_layer_t &L = s.layers[l];
      const uint32_t w = l == 0 ? F : a.hidden;
      const float *in = l == 0 ? s.x : d_ones;
      NTS(nts_spmm_gather_bounded(in, d_out, L.edge_weight_forward, L.column_offset, L.row_indices, 0, L.v_size, L.e_size,
                                  w, 0, L.max_in_degree, stream));
      if (a.verify) {
        uint64_t fp = 0;
        NTS(nts_fingerprint_u32(&fp, reinterpret_cast<const uint32_t *>(d_out), static_cast<uint64_t>(L.v_size) * w,
                                nullptr, 0, stream));
        checksum ^= fp * (2 * l + 1);
      }
      if (dumping) {
        dump(tag("in", l), in, static_cast<size_t>(L.src_size) * w * 4, stream);
        dump(tag("out", l), d_out, static_cast<size_t>(L.v_size) * w * 4, stream);
      }
      if (a.stage_sync) HIP(hipStreamSynchronize(stream));
    }
    if (a.stage_sync) t_fwd += now() - t0;
    t0 = now();
    for (uint32_t k = hops; k-- > 0;) {
      const nts_sampled_layer_t &L = s.layers[k];
      const uint32_t w = k == 0 ? F : a.hidden;
      NTS(nts_spmm_gather(d_ones, d_gin, L.edge_weight_backward, L.row_offset, L.column_indices, 0, L.src_size, L.e_size,
                          w, 0, stream));
      if (a.verify) {
        uint64_t fp = 0;
        NTS(nts_fingerprint_u32(&fp, reinterpret_cast<const uint32_t *>(d_gin), static_cast<uint64_t>(L.src_size) * w,
                                nullptr, 0, stream));
        checksum ^= fp * (2 * k + 2);
      }
      if (dumping) {
        dump(tag("gout", k), d_ones, static_cast<size_t>(L.v_size) * w * 4, stream);
        dump(tag("gin", k), d_gin, static_cast<size_t>(L.src_size) * w * 4, stream);
      }
      if (a.stage_sync) HIP(hipStreamSynchronize(stream));
    }
    if (a.stage_sync) t_bwd += now() - t0;
  };
  auto account = [&](Slot &s) {
    for (uint32_t l = 0; l < hops; ++l) edges_total += s.layers[l].e_size;
    rows_total += s.layers[0].src_size;
  };
  auto read_hits = [&](Slot &s, hipStream_t stream) {  // serial modes: after the gather has been waited for
    if (!n_cache) return;
    uint32_t h = 0;
    NTS(nts_memcpy_d2h_async(&h, s.hits, sizeof(h), stream));
    HIP(hipStreamSynchronize(stream));
    hits_total += h;
  };

  auto run_batches = [&](uint32_t count) {
    if (!count) return;
    if (P == 1) {
      Slot &s = slots[0];
      for (uint32_t b = 0; b < count; ++b) {
        double t0 = now();
        sample(s, b, main_stream);
        NTS(nts_batch_builder_layers(s.builder, s.layers));
        t_sample += now() - t0;
        t0 = now();
        gather(s, 0, main_stream);
        if (a.stage_sync) HIP(hipStreamSynchronize(main_stream));
        t_gather += now() - t0;
        account(s);
        aggregate(s, main_stream);
        if (a.stage_sync || a.verify) read_hits(s, main_stream);
      }
      return;
    }
    if (P == 2) {
      auto start = [&](uint32_t b) {
        Slot &s = slots[b % 2];
        if (s.has_trained) HIP(hipStreamWaitEvent(sample_streams[0], s.trained, 0));
        sample(s, b, sample_streams[0]);
      };
      start(0);
      for (uint32_t b = 0; b < count; ++b) {
        Slot &s = slots[b % 2];
        NTS(nts_batch_builder_layers(s.builder, s.layers));
        if (b + 1 < count) start(b + 1);
        gather(s, 0, main_stream);
        account(s);
        aggregate(s, main_stream);
        HIP(hipEventRecord(s.trained, main_stream));
        s.has_trained = true;
      }
      return;
    }
    const uint32_t chains = static_cast<uint32_t>(sample_streams.size());
    uint32_t started = 0;
    auto sample_through = [&](uint32_t last) {
      while (started <= std::min(last, count - 1)) {
        Slot &s = slots[started % P];
        hipStream_t stream = sample_streams[started % chains];
        if (s.has_trained) HIP(hipStreamWaitEvent(stream, s.trained, 0));  // the arena's last batch is still being read
        sample(s, started, stream);
        ++started;
      }
    };
    auto start_gather = [&](uint32_t b) {
      Slot &s = slots[b % P];
      NTS(nts_batch_builder_layers(s.builder, s.layers));
      // the x buffer this gather writes was read by the aggregation two batches back
      if (b >= 2 && slots[(b - 2) % P].has_trained) HIP(hipStreamWaitEvent(gather_stream, slots[(b - 2) % P].trained, 0));
      gather(s, b % 2, gather_stream);
      HIP(hipEventRecord(s.gathered, gather_stream));
    };
    sample_through(chains - 1);
    start_gather(0);
    sample_through(chains);
    for (uint32_t b = 0; b < count; ++b) {
      Slot &s = slots[b % P];
      if (b + 1 < count) start_gather(b + 1);
      sample_through(b + P - 1);
      HIP(hipStreamWaitEvent(main_stream, s.gathered, 0));
      account(s);
      aggregate(s, main_stream);
      HIP(hipEventRecord(s.trained, main_stream));
      s.has_trained = true;
    }
  };

  const uint32_t n_warm = std::min(a.warmup, n_batches);
  run_batches(n_warm);
  HIP(hipDeviceSynchronize());
  for (Slot &s : slots) s.has_trained = false;
  edges_total = rows_total = checksum = hits_total = 0;
  t_sample = t_gather = t_fwd = t_bwd = 0;
  const double t0 = now();
  run_batches(n_batches);
  HIP(hipDeviceSynchronize());
  const double epoch_s = now() - t0;
  const double stage_sample = t_sample, stage_gather = t_gather, stage_fwd = t_fwd, stage_bwd = t_bwd;

  if (!a.dump_dir.empty() && a.dump_batch < n_batches) {
    // The batch once more, through the same calls, with every array written out.
    Slot &s = slots[0];
    const uint32_t b = a.dump_batch;
    sample(s, b, main_stream);
    NTS(nts_batch_builder_layers(s.builder, s.layers));
    gather(s, 0, main_stream);
    NTS(nts_batch_builder_join(s.builder, main_stream));  // the transposed structure is written out below
    HIP(hipStreamSynchronize(main_stream));
    FILE *meta = fopen((a.dump_dir + "/meta.json").c_str(), "w");
    if (!meta) die("cannot write meta.json");
    fprintf(meta, "{\"batch\": %u, \"hops\": %u, \"F\": %u, \"hidden\": %u, \"heads\": %u, \"layers\": [", b, hops, F, a.hidden, H);
    for (uint32_t l = 0; l < hops; ++l) {
      const nts_sampled_layer_t &L = s.layers[l];
      fprintf(meta, "%s{\"v_size\": %u, \"e_size\": %u, \"src_size\": %u, \"max_in_degree\": %u, \"width\": %u}", l ? ", " : "",
              L.v_size, L.e_size, L.src_size, L.max_in_degree, H ? a.hidden : (l == 0 ? F : a.hidden));
      dump(tag("destination", l), L.destination, static_cast<size_t>(L.v_size) * 4, main_stream);
      dump(tag("source", l), L.source, static_cast<size_t>(L.src_size) * 4, main_stream);
      dump(tag("column_offset", l), L.column_offset, (static_cast<size_t>(L.v_size) + 1) * 4, main_stream);
      dump(tag("row_indices", l), L.row_indices, static_cast<size_t>(L.e_size) * 4, main_stream);
      dump(tag("row_offset", l), L.row_offset, (static_cast<size_t>(L.src_size) + 1) * 4, main_stream);
      dump(tag("column_indices", l), L.column_indices, static_cast<size_t>(L.e_size) * 4, main_stream);
      dump(tag("edge_weight_forward", l), L.edge_weight_forward, static_cast<size_t>(L.e_size) * 4, main_stream);
      dump(tag("edge_weight_backward", l), L.edge_weight_backward, static_cast<size_t>(L.e_size) * 4, main_stream);
      if (L.csr_to_csc) dump(tag("csr_to_csc", l), L.csr_to_csc, static_cast<size_t>(L.e_size) * 4, main_stream);
    }
    uint32_t hits = 0;
    if (n_cache) HIP(hipMemcpy(&hits, s.hits, sizeof(hits), hipMemcpyDeviceToHost));
    fprintf(meta, "], \"cache_rows\": %u, \"cache_hits\": %u}\n", n_cache, hits);
    fclose(meta);
    dump("x.bin", s.x, static_cast<size_t>(s.layers[0].src_size) * F * 4, main_stream);
    dump("labels.bin", s.labels, static_cast<size_t>(s.layers[hops - 1].v_size) * 8, main_stream);
    dumping = true;
    aggregate(s, main_stream);
    dumping = false;
    HIP(hipDeviceSynchronize());
  }

  printf("{\"driver\": \"native\", \"batches\": %u, \"batch_size\": %u, \"pipeline\": %u, \"hop_launches_as_graph\": %s, "
         "\"hop_graph_mode\": %d, \"stage_sync\": %s, \"epoch_s\": %.4f, \"sampled_edges\": %llu, \"gathered_rows\": %llu, \"cache_rows\": %u",
         n_batches, a.batch, P, a.graph ? "true" : "false", a.graph, a.stage_sync ? "true" : "false", epoch_s,
         static_cast<unsigned long long>(edges_total), static_cast<unsigned long long>(rows_total), n_cache);
  if (P == 1 && a.stage_sync)
    printf(", \"stage_s\": {\"sample\": %.4f, \"gather\": %.4f, \"aggregate_fwd\": %.4f, \"aggregate_bwd\": %.4f}", stage_sample,
           stage_gather, stage_fwd, stage_bwd);
  if (n_cache && P == 1 && (a.stage_sync || a.verify))
    printf(", \"cache_hit_rate\": %.4f", rows_total ? static_cast<double>(hits_total) / rows_total : 0.0);
  if (a.verify) printf(", \"checksum\": \"%016llx\"", static_cast<unsigned long long>(checksum));
  printf("}\n");

  for (Slot &s : slots) {
    NTS(nts_batch_builder_destroy(s.builder));
    NTS(nts_free_device(s.arena));
    HIP(hipEventDestroy(s.gathered));
    HIP(hipEventDestroy(s.trained));
  }
  NTS(nts_free_pinned(table));
  return 0;
}
