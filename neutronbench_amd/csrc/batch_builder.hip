// All layers of one sampled mini-batch built on the device in one stream-ordered sequence: the
// construction steps of Sampler::sample_one for every hop (core/ntsSampler.hpp:843-1106: init_dst,
// init_co, the neighbour pick, sampCSC::postprocessing, generate_csr_from_csc, update_degree,
// compute_weight_forward / backward; core/coocsc.hpp:136-450) without a host step in between.
//
// The reference sizes each hop's arrays on the host from the previous hop's result.  Here the sizes
// stay on the device: buffers are laid out once for the largest batch (hop h holds at most
// destinations x fanout edges and as many distinct sources), every kernel reads the live counts
// from a small device table written by the kernels before it, and the host reads that table back
// once per batch, after the last hop, to learn the shapes of the layers it then aggregates over.
// Results are identical to running the per-hop entry points with seeds seed, seed + 1, ...
#include <new>

#include "common.hpp"

namespace nts {
namespace {

constexpr uint32_t kMaxHops = 8;
constexpr uint32_t kSizeWords = 4;  // per hop: destinations, edges, sources, unused

inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

struct HopLayout {
  uint32_t vd_cap, e_cap, vs_cap;
  size_t co, ri_local, source, ro, ci, perm, ewf, ewb, owner;  // byte offsets into the arena
};

struct Layout {
  HopLayout hop[kMaxHops];
  size_t dst0, sizes, seed, ri_global, relabel_work, csr_work, scan_work, total;
  size_t relabel_bytes, csr_bytes, scan_bytes;
};

bool plan_layout(Layout *L, uint32_t V, uint32_t graph_edges, const int32_t *fanouts, uint32_t hops,
                 uint32_t max_batch, int want_perm) {
  size_t at = 0;
  auto take = [&at](size_t bytes) {
    const size_t here = at;
    at += align_up(bytes ? bytes : 1, 256);
    return here;
  };
  L->sizes = take((hops + 1) * kSizeWords * sizeof(uint32_t));
  L->seed = take(sizeof(uint64_t));
  L->dst0 = take(static_cast<size_t>(max_batch) * sizeof(uint32_t));
  uint32_t vd = max_batch;  // the caller's batch may repeat vertices, so it may be longer than V
  uint32_t e_max = 0;
  for (uint32_t h = 0; h < hops; ++h) {
    HopLayout &H = L->hop[h];
    const int32_t fan = fanouts[h];
    // Distinct destinations cannot have more in-edges than the graph holds; the caller's batch
    // (hop 0) may repeat a vertex, so there only the fanout bounds the edge count.
    uint64_t e = fan < 0 ? graph_edges : static_cast<uint64_t>(vd) * static_cast<uint32_t>(fan);
    if (e > graph_edges && (h > 0 || fan < 0)) e = graph_edges;
    if (e > 0xFFFFFFFFull) return false;
    H.vd_cap = vd;
    H.e_cap = static_cast<uint32_t>(e);
    H.vs_cap = H.e_cap < V ? H.e_cap : V;
    if (H.e_cap == 0) return false;
    const size_t eb = static_cast<size_t>(H.e_cap) * sizeof(uint32_t);
    H.co = take((static_cast<size_t>(H.vd_cap) + 1) * sizeof(uint32_t));
    H.ri_local = take(eb);
    H.source = take(static_cast<size_t>(H.vs_cap) * sizeof(uint32_t));
    H.ro = take((static_cast<size_t>(H.vs_cap) + 1) * sizeof(uint32_t));
    H.ci = take(eb);
    H.perm = want_perm ? take(eb) : 0;
    H.ewf = take(eb);
    H.ewb = take(eb);
    H.owner = take(eb);  // destination slot of every edge, recorded by the neighbour pick
    if (H.e_cap > e_max) e_max = H.e_cap;
    vd = H.vs_cap;
  }
  L->ri_global = take(static_cast<size_t>(e_max) * sizeof(uint32_t));
  L->relabel_bytes = nts_relabel_sources_work_bytes(V);
  // The sort and scan scratch is shared by the hops: the largest any of them asks for (a library
  // routine may pick another algorithm, with other needs, for a smaller input).
  L->csr_bytes = 0;
  L->scan_bytes = 0;
  for (uint32_t h = 0; h < hops; ++h) {
    const size_t c = csr_from_csc_bytes(L->hop[h].e_cap), sc = hop_scan_bytes(L->hop[h].vd_cap);
    if (!c || !sc) return false;
    if (c > L->csr_bytes) L->csr_bytes = c;
    if (sc > L->scan_bytes) L->scan_bytes = sc;
  }
  if (!L->relabel_bytes) return false;
  L->relabel_work = take(L->relabel_bytes);
  L->csr_work = take(L->csr_bytes);
  L->scan_work = take(L->scan_bytes);
  L->total = at;
  return true;
}

inline unsigned bits_for(uint32_t n) {  // bits needed to represent values in [0, n)
  unsigned b = 1;
  while (b < 32 && (1ull << b) < n) ++b;
  return b;
}

// The batch's vertex ids become hop 0's destinations; the live destination count of hop 0 is n.
// Everything that changes from batch to batch enters here -- the ids, their count and the seed go
// to fixed places in the arena -- so that the launches after this one are the same for every batch.
__global__ __launch_bounds__(256) void start_batch_kernel(uint32_t *__restrict__ dst0, const uint32_t *__restrict__ ids,
                                                          uint32_t n, uint32_t *__restrict__ sizes, uint32_t size_words,
                                                          uint64_t *__restrict__ seed_word, uint64_t seed) {
  const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < size_words) sizes[i] = i == 0 ? n : 0u;
  if (i == 0) *seed_word = seed;
  if (i < n) dst0[i] = ids[i];
}

}  // namespace
}  // namespace nts

using namespace nts;

struct nts_batch_builder {
  const uint32_t *graph_co, *graph_ri;
  uint32_t V, hops, max_batch;
  int32_t fanout[kMaxHops];
  int want_perm;
  Layout L;
  unsigned char *arena;
  uint32_t *host_sizes;  // page-locked
  hipEvent_t done;
  bool pending;
  bool bitmap_clean;  // the bitmap of sampled sources is all zero (each hop's last kernel leaves it so)
  bool use_graph;     // replay the hops' launches as one HIP graph, captured at the first batch
  bool fork_hops;     // in that graph, a hop's transposition and weights run on a branch beside the next hop's sampling
  bool defer;         // two graphs: sampling on the caller's stream, transpositions and weights on `side`
  hipGraph_t graph;
  hipGraphExec_t graph_exec;
  // defer only: the second graph, the builder's own stream that runs it, and the event recorded
  // after it (what nts_batch_builder_join makes a consumer's stream wait for)
  hipGraph_t structure_graph;
  hipGraphExec_t structure_exec;
  hipStream_t side;
  hipEvent_t structured;
  bool structure_pending;
};

namespace {

// Every launch of a batch after start_batch_kernel: the hops, then the copy of the size table to the
// host.  All arguments are addresses inside the arena, capacities and device-resident counts, so the
// sequence is the same for every batch of a builder.
// side (only while recording a graph): a second stream of the recording.  A hop's transposition and
// weights need nothing of the hops after it and the next hop's sampling needs only this hop's source
// list, so with `side` the chain forks after the relabelling: sort, CSR and weights of hop h go to the
// side stream (which takes them hop by hop: they share the sort scratch), the main stream goes on with
// hop h + 1, and the two join before the size table is copied.  The bitmap of sampled sources, which the
// weights launch otherwise clears on its way, is then cleared by a launch of its own on the main stream.
// phase: kAllOfABatch, or one half of it for a builder that defers the structure -- kSampling (offsets,
// pick, relabelling and bitmap clearing of every hop, then the size table) and kStructure (sort, CSR
// and weights of every hop), recorded as graphs of their own.
enum Phase { kAllOfABatch, kSampling, kStructure };
int enqueue_hops(nts_batch_builder *b, hipStream_t stream, hipStream_t side = nullptr, hipEvent_t *events = nullptr,
                 Phase phase = kAllOfABatch) {
  unsigned char *A = b->arena;
  uint32_t *sizes = reinterpret_cast<uint32_t *>(A + b->L.sizes);
  const uint64_t *seed_word = reinterpret_cast<const uint64_t *>(A + b->L.seed);
  uint32_t *dst = reinterpret_cast<uint32_t *>(A + b->L.dst0);
  uint32_t *ri_global = reinterpret_cast<uint32_t *>(A + b->L.ri_global);
  // where csr_from_csc leaves the sorted keys: the source of every CSR edge
  const uint32_t *csr_owner = reinterpret_cast<const uint32_t *>(A + b->L.csr_work);
  uint32_t *bits = reinterpret_cast<uint32_t *>(A + b->L.relabel_work);
  const uint32_t words = (b->V + 31) / 32;
  for (uint32_t h = 0; h < b->hops; ++h) {
    const HopLayout &H = b->L.hop[h];
    uint32_t *hop_sizes = sizes + h * kSizeWords;
    uint32_t *co = reinterpret_cast<uint32_t *>(A + H.co);
    uint32_t *ri = reinterpret_cast<uint32_t *>(A + H.ri_local);
    uint32_t *source = reinterpret_cast<uint32_t *>(A + H.source);
    uint32_t *ro = reinterpret_cast<uint32_t *>(A + H.ro);
    uint32_t *ci = reinterpret_cast<uint32_t *>(A + H.ci);
    uint32_t *perm = b->want_perm ? reinterpret_cast<uint32_t *>(A + H.perm) : nullptr;
    float *ewf = reinterpret_cast<float *>(A + H.ewf);
    float *ewb = reinterpret_cast<float *>(A + H.ewb);
    uint32_t *owner = reinterpret_cast<uint32_t *>(A + H.owner);
    const DevCount Vd = device_count(hop_sizes + 0, H.vd_cap);
    const DevCount Vs = device_count(hop_sizes + 2, H.vs_cap);
    const DevCount E = device_edge_count(co, hop_sizes + 0, H.vd_cap, H.e_cap);
    // the weights launch clears the bitmap on its way unless it runs apart from the sampling
    const bool clear_apart = side != nullptr || phase != kAllOfABatch;
    if (phase != kStructure) {
      if (int rc = hop_offsets(co, b->graph_co, dst, Vd, b->fanout[h], A + b->L.scan_work, b->L.scan_bytes, stream))
        return rc;
      if (int rc = hop_neighbors(ri_global, co, b->graph_co, b->graph_ri, dst, Vd, H.e_cap, b->fanout[h],
                                 device_seed(seed_word, h), bits, owner, stream))
        return rc;
      // Local ids; the unused tail of the edge array is padded with a key that sorts after every
      // source.
      if (int rc = relabel_sources(source, hop_sizes + 2, hop_sizes + kSizeWords, ri, ri_global, E, H.e_cap, H.vs_cap,
                                   hop_sizes + 1, b->V, A + b->L.relabel_work, true, stream))
        return rc;
      if (clear_apart)
        if (int rc = nts_memset_zero(bits, static_cast<size_t>(words) * sizeof(uint32_t), stream)) return rc;
    }
    hipStream_t rest = stream;
    if (side) {
      NTS_HIP_TRY(hipEventRecord(events[h], stream));
      NTS_HIP_TRY(hipStreamWaitEvent(side, events[h], 0));
      rest = side;
    }
    if (phase != kSampling) {
      if (int rc = csr_from_csc(ro, ci, perm, co, ri, Vd, Vs, E, H.e_cap, bits_for(H.vs_cap + 1), A + b->L.csr_work,
                                owner, rest))
        return rc;
      if (int rc = gcn_edge_weights(ewf, ewb, co, ri, ro, ci, Vd, Vs, clear_apart ? nullptr : bits,
                                    clear_apart ? 0u : words, owner, csr_owner, rest))
        return rc;
    }
    dst = source;  // the next hop's destinations are this hop's sources (init_dst)
  }
  if (side) {  // join
    NTS_HIP_TRY(hipEventRecord(events[b->hops], side));
    NTS_HIP_TRY(hipStreamWaitEvent(stream, events[b->hops], 0));
  }
  if (phase != kStructure) {
    const size_t size_bytes = (b->hops + 1) * kSizeWords * sizeof(uint32_t);
    NTS_HIP_TRY(hipMemcpyAsync(b->host_sizes, sizes, size_bytes, hipMemcpyDeviceToHost, stream));
  }
  return NTS_OK;
}

// Records enqueue_hops into a graph and instantiates it.  The recording runs on a stream created for
// it (the caller's may be the null stream, which cannot record; nothing executes while recording)
// in thread-local mode: other host threads keep using the device meanwhile.
int capture_hops(nts_batch_builder *b, Phase phase, hipGraph_t *graph_out, hipGraphExec_t *exec_out) {
  hipStream_t stream = nullptr;
  NTS_HIP_TRY(hipStreamCreateWithFlags(&stream, hipStreamNonBlocking));
  hipError_t begin = hipStreamBeginCapture(stream, hipStreamCaptureModeThreadLocal);
  if (begin != hipSuccess) {
    (void)hipStreamDestroy(stream);
    return fail_hip(begin, "nts_batch_builder_sample: hipStreamBeginCapture");
  }
  hipStream_t side = nullptr;
  hipEvent_t events[kMaxHops + 1] = {};
  int rc = NTS_OK;
  if (b->fork_hops && phase == kAllOfABatch) {
    if (hipStreamCreateWithFlags(&side, hipStreamNonBlocking) != hipSuccess)
      rc = fail(NTS_ERR_INVALID, "nts_batch_builder_sample: side stream");
    for (uint32_t h = 0; rc == NTS_OK && h <= b->hops; ++h)
      if (hipEventCreateWithFlags(&events[h], hipEventDisableTiming) != hipSuccess)
        rc = fail(NTS_ERR_INVALID, "nts_batch_builder_sample: event");
  }
  if (rc == NTS_OK) rc = enqueue_hops(b, stream, side, side ? events : nullptr, phase);
  hipGraph_t graph = nullptr;
  const hipError_t end = hipStreamEndCapture(stream, &graph);  // always ends the recording, also after an error
  (void)hipStreamDestroy(stream);
  if (side) (void)hipStreamDestroy(side);
  for (uint32_t h = 0; h <= kMaxHops; ++h)
    if (events[h]) (void)hipEventDestroy(events[h]);
  if (rc != NTS_OK) {
    if (graph) (void)hipGraphDestroy(graph);
    return rc;
  }
  if (end != hipSuccess) return fail_hip(end, "nts_batch_builder_sample: hipStreamEndCapture");
  hipGraphExec_t exec = nullptr;
  const hipError_t inst = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
  if (inst != hipSuccess) {
    (void)hipGraphDestroy(graph);
    return fail_hip(inst, "nts_batch_builder_sample: hipGraphInstantiate");
  }
  *graph_out = graph;
  *exec_out = exec;
  return NTS_OK;
}

// Drops the recorded graphs (after waiting for a structure graph still running): the next batch records again.
void drop_graphs(nts_batch_builder *b) {
  if (b->side) (void)hipStreamSynchronize(b->side);
  b->structure_pending = false;
  if (b->graph_exec) (void)hipGraphExecDestroy(b->graph_exec);
  if (b->graph) (void)hipGraphDestroy(b->graph);
  if (b->structure_exec) (void)hipGraphExecDestroy(b->structure_exec);
  if (b->structure_graph) (void)hipGraphDestroy(b->structure_graph);
  b->graph_exec = nullptr;
  b->graph = nullptr;
  b->structure_exec = nullptr;
  b->structure_graph = nullptr;
}

}  // namespace

extern "C" {

size_t nts_batch_builder_arena_bytes(uint32_t V, uint32_t graph_edges, const int32_t *fanouts, uint32_t hops,
                                     uint32_t max_batch, int want_perm) {
  if (!fanouts || hops == 0 || hops > kMaxHops || max_batch == 0 || V == 0 || graph_edges == 0) return 0;
  Layout L;
  if (!plan_layout(&L, V, graph_edges, fanouts, hops, max_batch, want_perm)) return 0;
  return L.total;
}

int nts_batch_builder_create(nts_batch_builder_t **out, const uint32_t *graph_co, const uint32_t *graph_ri, uint32_t V,
                             uint32_t graph_edges, const int32_t *fanouts, uint32_t hops, uint32_t max_batch,
                             int want_perm, void *arena, size_t arena_bytes) {
  NTS_TRACE_RANGE("nts_batch_builder_create");
  if (!out) return fail(NTS_ERR_INVALID, "nts_batch_builder_create: null out");
  *out = nullptr;
  if (!graph_co || !graph_ri || !fanouts || !arena) return fail(NTS_ERR_INVALID, "nts_batch_builder_create: null pointer");
  if (hops == 0 || hops > kMaxHops) return fail(NTS_ERR_INVALID, "nts_batch_builder_create: 1 to 8 hops");
  if (max_batch == 0 || V == 0 || graph_edges == 0)
    return fail(NTS_ERR_INVALID, "nts_batch_builder_create: empty graph or batch");
  for (uint32_t h = 0; h < hops; ++h) {
    if (fanouts[h] == 0) return fail(NTS_ERR_INVALID, "nts_batch_builder_create: fanout 0");
  }
  if (!aligned_to(arena, 256)) return fail(NTS_ERR_INVALID, "nts_batch_builder_create: arena must be 256-byte aligned");
  nts_batch_builder *b = new (std::nothrow) nts_batch_builder();
  if (!b) return fail(NTS_ERR_INVALID, "nts_batch_builder_create: out of host memory");
  if (!plan_layout(&b->L, V, graph_edges, fanouts, hops, max_batch, want_perm) || b->L.total > arena_bytes) {
    delete b;
    return fail(NTS_ERR_INVALID, "nts_batch_builder_create: arena smaller than nts_batch_builder_arena_bytes");
  }
  b->graph_co = graph_co;
  b->graph_ri = graph_ri;
  b->V = V;
  b->hops = hops;
  b->max_batch = max_batch;
  b->want_perm = want_perm;
  for (uint32_t h = 0; h < hops; ++h) b->fanout[h] = fanouts[h];
  b->arena = static_cast<unsigned char *>(arena);
  b->host_sizes = nullptr;
  b->pending = false;
  b->bitmap_clean = false;
  b->use_graph = false;
  b->fork_hops = false;
  b->defer = false;
  b->graph = nullptr;
  b->graph_exec = nullptr;
  b->structure_graph = nullptr;
  b->structure_exec = nullptr;
  b->side = nullptr;
  b->structured = nullptr;
  b->structure_pending = false;
  hipError_t err = hipHostMalloc(reinterpret_cast<void **>(&b->host_sizes), (hops + 1) * kSizeWords * sizeof(uint32_t),
                                 hipHostMallocDefault);
  if (err == hipSuccess) {
    err = hipEventCreateWithFlags(&b->done, hipEventDisableTiming);
    if (err != hipSuccess) (void)hipHostFree(b->host_sizes);
  }
  if (err != hipSuccess) {
    delete b;
    return fail_hip(err, "nts_batch_builder_create");
  }
  *out = b;
  return NTS_OK;
}

int nts_batch_builder_destroy(nts_batch_builder_t *b) {
  NTS_TRACE_RANGE("nts_batch_builder_destroy");
  if (!b) return NTS_OK;
  drop_graphs(b);
  if (b->structured) (void)hipEventDestroy(b->structured);
  if (b->side) (void)hipStreamDestroy(b->side);
  hipError_t e1 = hipEventDestroy(b->done);
  hipError_t e2 = hipHostFree(b->host_sizes);
  delete b;
  if (e1 != hipSuccess) return fail_hip(e1, "nts_batch_builder_destroy: hipEventDestroy");
  if (e2 != hipSuccess) return fail_hip(e2, "nts_batch_builder_destroy: hipHostFree");
  return NTS_OK;
}

int nts_batch_builder_sample(nts_batch_builder_t *b, const uint32_t *batch_ids, uint32_t n, uint64_t seed,
                             nts_stream_t stream) {
  NTS_TRACE_RANGE("nts_batch_builder_sample");
  if (!b) return fail(NTS_ERR_INVALID, "nts_batch_builder_sample: null builder");
  if (n > b->max_batch) return fail(NTS_ERR_INVALID, "nts_batch_builder_sample: batch larger than max_batch");
  if (n && !batch_ids) return fail(NTS_ERR_INVALID, "nts_batch_builder_sample: null batch_ids");
  unsigned char *A = b->arena;
  uint32_t *sizes = reinterpret_cast<uint32_t *>(A + b->L.sizes);
  uint32_t *dst = reinterpret_cast<uint32_t *>(A + b->L.dst0);
  uint64_t *seed_word = reinterpret_cast<uint64_t *>(A + b->L.seed);
  const uint32_t size_words = (b->hops + 1) * kSizeWords;
  // The neighbour pick sets the bits of the sources it emits, the relabelling reads them, and the
  // hop's last kernel clears them again; only a first or an interrupted batch clears them up front.
  uint32_t *bits = reinterpret_cast<uint32_t *>(A + b->L.relabel_work);
  const uint32_t words = (b->V + 31) / 32;
  // the structure graph of the batch before reads what this batch's sampling overwrites
  if (b->structure_pending) NTS_HIP_TRY(hipStreamWaitEvent(stream, b->structured, 0));
  if (!b->bitmap_clean)
    if (int rc = nts_memset_zero(bits, static_cast<size_t>(words) * sizeof(uint32_t), stream)) return rc;
  b->bitmap_clean = false;
  const uint32_t start_threads = n > size_words ? n : size_words;
  hipLaunchKernelGGL(start_batch_kernel, dim3(ceil_div(start_threads, 256)), dim3(256), 0, stream, dst, batch_ids, n,
                     sizes, size_words, seed_word, seed);
  NTS_LAUNCH_CHECK("start_batch_kernel");
  if (b->use_graph) {
    if (!b->graph_exec)
      if (int rc = capture_hops(b, b->defer ? kSampling : kAllOfABatch, &b->graph, &b->graph_exec)) return rc;
    if (b->defer && !b->structure_exec)
      if (int rc = capture_hops(b, kStructure, &b->structure_graph, &b->structure_exec)) return rc;
    NTS_HIP_TRY(hipGraphLaunch(b->graph_exec, stream));
  } else {
    if (int rc = enqueue_hops(b, stream)) return rc;
  }
  NTS_HIP_TRY(hipEventRecord(b->done, stream));
  b->pending = true;
  b->bitmap_clean = true;
  if (b->use_graph && b->defer) {
    NTS_HIP_TRY(hipStreamWaitEvent(b->side, b->done, 0));
    NTS_HIP_TRY(hipGraphLaunch(b->structure_exec, b->side));
    NTS_HIP_TRY(hipEventRecord(b->structured, b->side));
    b->structure_pending = true;
  }
  return NTS_OK;
}

int nts_batch_builder_use_graph(nts_batch_builder_t *b, int enable) {
  if (!b) return fail(NTS_ERR_INVALID, "nts_batch_builder_use_graph: null builder");
  if (b->use_graph != (enable != 0) || b->fork_hops != (enable == 2) || b->defer != (enable == 3))
    drop_graphs(b);  // another shape of graph than the one recorded: record again at the next batch
  if (enable == 3 && !b->side) {
    NTS_HIP_TRY(hipStreamCreateWithFlags(&b->side, hipStreamNonBlocking));
    const hipError_t err = hipEventCreateWithFlags(&b->structured, hipEventDisableTiming);
    if (err != hipSuccess) {
      (void)hipStreamDestroy(b->side);
      b->side = nullptr;
      return fail_hip(err, "nts_batch_builder_use_graph: hipEventCreateWithFlags");
    }
  }
  b->use_graph = enable != 0;
  b->fork_hops = enable == 2;
  b->defer = enable == 3;
  return NTS_OK;
}

int nts_batch_builder_join(nts_batch_builder_t *b, nts_stream_t stream) {
  if (!b) return fail(NTS_ERR_INVALID, "nts_batch_builder_join: null builder");
  if (b->structure_pending) NTS_HIP_TRY(hipStreamWaitEvent(stream, b->structured, 0));
  return NTS_OK;
}

int nts_batch_builder_layers(nts_batch_builder_t *b, nts_sampled_layer_t *layers) {
  NTS_TRACE_RANGE("nts_batch_builder_layers");
  if (!b || !layers) return fail(NTS_ERR_INVALID, "nts_batch_builder_layers: null pointer");
  if (!b->pending) return fail(NTS_ERR_INVALID, "nts_batch_builder_layers: no batch has been sampled");
  NTS_HIP_TRY(hipEventSynchronize(b->done));
  unsigned char *A = b->arena;
  for (uint32_t h = 0; h < b->hops; ++h) {
    const HopLayout &H = b->L.hop[h];
    const uint32_t *s = b->host_sizes + h * kSizeWords;
    nts_sampled_layer_t &out = layers[b->hops - 1 - h];  // index 0 = the input-side layer, as sampled_sgs
    out.v_size = s[0];
    out.e_size = s[1];
    out.src_size = s[2];
    out.max_in_degree = b->fanout[h] > 0 ? static_cast<uint32_t>(b->fanout[h]) : 0u;
    out.destination = reinterpret_cast<uint32_t *>(A + (h == 0 ? b->L.dst0 : b->L.hop[h - 1].source));
    out.source = reinterpret_cast<uint32_t *>(A + H.source);
    out.column_offset = reinterpret_cast<uint32_t *>(A + H.co);
    out.row_indices = reinterpret_cast<uint32_t *>(A + H.ri_local);
    out.row_offset = reinterpret_cast<uint32_t *>(A + H.ro);
    out.column_indices = reinterpret_cast<uint32_t *>(A + H.ci);
    out.csr_to_csc = b->want_perm ? reinterpret_cast<uint32_t *>(A + H.perm) : nullptr;
    out.edge_weight_forward = reinterpret_cast<float *>(A + H.ewf);
    out.edge_weight_backward = reinterpret_cast<float *>(A + H.ewb);
  }
  return NTS_OK;
}

}  // extern "C"
