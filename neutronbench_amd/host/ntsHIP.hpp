// ntsHIP.hpp -- C++ host veneer over libntship's C ABI with the names and signatures the
// NeutronBench tree already uses (cuda/ntsCUDA.hpp:26-211): the free allocation / copy helpers,
// deviceCSC and the Cuda_Stream class.  Including this header instead of cuda/ntsCUDA.hpp lets
// core/ and toolkits/ compile unchanged against the HIP library; nothing here launches a kernel
// itself.
//
// Error behaviour follows the reference (cuda/ntsCUDAGraphOP.cu:11-20): a failing call prints the
// library's error text and exits with status 1.  Callers that want status codes use nts_hip.h
// directly.
#ifndef NTS_HIP_VENEER_HPP
#define NTS_HIP_VENEER_HPP

#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

#include <map>
#include <mutex>

#include "nts_hip.h"

typedef uint32_t VertexId_CUDA;
// The stream type of the reference's interfaces.  hipStream_t and this typedef are the same
// pointer type, so streams taken from libtorch-ROCm's pool can be passed straight in.
typedef nts_stream_t cudaStream_t;

const int CUDA_NUM_THREADS = 512;  // kept for source compatibility; launch shapes are chosen by the library
const int CUDA_NUM_BLOCKS = 128;
const int CUDA_NUM_THREADS_SOFTMAX = 32;
const int CUDA_NUM_BLOCKS_SOFTMAX = 512;

enum graph_type { CSR, CSC, PAIR };
enum weight_type { NULL_TYPE, SCALA_TYPE, TENSOR_TYPE };

#define NTS_VENEER_CHECK(call_expr)                                                        \
  do {                                                                                     \
    int nts_rc__ = (call_expr);                                                            \
    if (nts_rc__ != NTS_OK) {                                                              \
      printf("HIP call on line %d returned error %d: %s\n", __LINE__, nts_rc__, nts_last_error()); \
      exit(1);                                                                             \
    }                                                                                      \
  } while (0)

// ---- aggregation schedules for static graphs, kept behind the reference's call signatures --------
//
// The reference calls Gather_By_Dst_From_Src / Gather_By_Src_From_Dst with bare device pointers.
// For a whole-graph chunk those arrays never change after CopyGraphToDevice, and a schedule built
// once (nts_spmm_plan_create_slabs) makes every later pass about 1.5x faster than the per-call
// balancing of nts_spmm_gather.
// When to build one is a heuristic: every write the tree makes to device memory it allocated goes
// through the helpers of this header, so each allocation made here is a region with a generation
// number that every upload, zeroing or kernel output into it advances; a call whose offsets and
// indices both lie in such regions, names its source range, has at least 2^22 edges and repeats with
// unchanged generations for the third time gets a schedule (built once, blocking: the arrays are read
// back and the rows scheduled on the host, 0.4 s for 115 M edges).  Mini-batch layers are re-uploaded
// every batch and never qualify.
// Whether a schedule may be used is verified, not inferred: other code can write those arrays without
// this header seeing it (a libtorch operator, a kernel of the caller's own).  The schedule remembers a
// checksum of offsets and indices taken on the device when it was built, and every later call takes it
// again first (nts_fingerprint_u32: 0.1 ms for 115 M indices, and a wait for the stream, which the
// reference's operators end with anyway); when it differs, the schedule is dropped and the call runs
// through nts_spmm_gather on what the arrays hold now.
// NTS_VENEER_PLAN_CACHE=0 in the environment switches the mechanism off.
namespace nts_veneer {

struct Region {
  size_t bytes;
  unsigned long long generation;
};
struct CachedPlan {
  nts_spmm_plan_t *plan;
  const void *indices;
  uint32_t rows, edges, n_index, index_base;
  unsigned long long gen_offsets, gen_indices;
  int seen;
  uint64_t fingerprint;  // checksum of offsets and indices when the schedule was built
};
struct State {
  std::mutex mu;
  std::map<uintptr_t, Region> regions;
  std::map<uintptr_t, CachedPlan> plans;  // keyed by the offsets pointer
  unsigned long long clock = 1;
  long plans_built = 0;
  long planned_calls = 0;
  long plans_dropped_by_checksum = 0;
  long deferred_checks = 0;
  int enabled = -1;
  // A checksum taken on a side stream while the scheduled aggregation it guards runs (see plan_for):
  // at most one is outstanding; it is settled at the next call through this header.
  nts_stream_t verify_stream = NULL;
  nts_event_t verify_fork = NULL;
  uint64_t *pinned_sum = NULL;
  int async_verify = -1;
  struct Pending {
    bool active;
    uintptr_t key;
    const float *input, *weight;
    float *output;
    const uint32_t *offsets, *indices;
    uint32_t index_base, rows, edges, F;
    nts_stream_t stream;
  } pending = {false, 0, NULL, NULL, NULL, NULL, NULL, 0, 0, 0, 0, NULL};
};
inline State &state() {
  static State s;
  return s;
}
const uint32_t kPlanMinEdges = 1u << 22;

// The buffer this host thread cleared last through zero_buffer, until anything else is written through
// this header: the reference clears an output and then aggregates into it (Nts->ZeroVarMem + GatherBy*,
// core/graph.hpp:3443-3445, 3469-3471); an aggregation that finds its output in this record writes the
// sums instead of adding them to the zeros -- the same values, without reading the output back.  Only
// writes made through this header are seen: a caller that clears a buffer here, fills it by other means
// and then aggregates into it must switch this off (NTS_VENEER_ZERO_TRACKING=0 in the environment).
struct ZeroRecord {
  const void *ptr;
  size_t floats;
};
inline ZeroRecord &zero_record() {
  static thread_local ZeroRecord r = {NULL, 0};
  return r;
}
inline bool zero_tracking_enabled() {
  static const int on = [] {
    const char *e = getenv("NTS_VENEER_ZERO_TRACKING");
    return (e && e[0] == '0') ? 0 : 1;
  }();
  return on != 0;
}
inline void note_zeroed(const void *p, size_t floats) {
  ZeroRecord &r = zero_record();
  r.ptr = p;
  r.floats = floats;
}
// True when `p` is exactly the buffer cleared last and `floats` of it are still known to be zero.
inline bool take_zeroed(const void *p, size_t floats) {
  ZeroRecord &r = zero_record();
  const bool hit = zero_tracking_enabled() && r.ptr != NULL && r.ptr == p && floats <= r.floats;
  r.ptr = NULL;
  r.floats = 0;
  return hit;
}

inline void settle_pending_locked(State &st);
inline std::map<uintptr_t, Region>::iterator region_of(State &st, const void *p) {
  const uintptr_t a = (uintptr_t)p;
  std::map<uintptr_t, Region>::iterator it = st.regions.upper_bound(a);
  if (it == st.regions.begin()) return st.regions.end();
  --it;
  return a < it->first + it->second.bytes ? it : st.regions.end();
}
inline void note_alloc(void *p, size_t bytes) {
  if (!p) return;
  State &st = state();
  std::lock_guard<std::mutex> lock(st.mu);
  Region r = {bytes, st.clock++};
  st.regions[(uintptr_t)p] = r;
}
inline void drop_plans_touching(State &st, uintptr_t base, size_t bytes) {
  for (std::map<uintptr_t, CachedPlan>::iterator it = st.plans.begin(); it != st.plans.end();) {
    const uintptr_t o = it->first, i = (uintptr_t)it->second.indices;
    if ((o >= base && o < base + bytes) || (i >= base && i < base + bytes)) {
      if (it->second.plan) nts_spmm_plan_destroy(it->second.plan);
      it = st.plans.erase(it);
    } else {
      ++it;
    }
  }
}
inline void note_free(void *p) {
  if (!p) return;
  State &st = state();
  std::lock_guard<std::mutex> lock(st.mu);
  settle_pending_locked(st);
  std::map<uintptr_t, Region>::iterator it = st.regions.find((uintptr_t)p);
  if (it == st.regions.end()) return;
  drop_plans_touching(st, it->first, it->second.bytes);
  st.regions.erase(it);
}
// Settles the outstanding side-stream checksum, if any: waits for it, and when the arrays no longer
// hold what the schedule was built from, drops the schedule and computes the aggregation again without
// one (the output had been cleared before the call, so it is cleared again and rewritten).  Caller
// holds st.mu.  Every entry of this header that writes, synchronises or copies results out comes
// through here first, so a result computed with a stale schedule never leaves this header.
inline void settle_pending_locked(State &st) {
  if (!st.pending.active) return;
  State::Pending p = st.pending;
  st.pending.active = false;
  bool stale = nts_stream_sync(st.verify_stream) != NTS_OK;
  std::map<uintptr_t, CachedPlan>::iterator it = st.plans.find(p.key);
  if (!stale && it != st.plans.end() && it->second.plan)
    stale = nts_fingerprint_finish(*st.pinned_sum, (uint64_t)p.rows + 1, p.edges) != it->second.fingerprint;
  if (!stale) return;
  if (it != st.plans.end() && it->second.plan) {
    nts_stream_sync(p.stream);  // the call that used the schedule has finished before the schedule goes
    nts_spmm_plan_destroy(it->second.plan);
    it->second.plan = NULL;
    it->second.seen = 1;
  }
  ++st.plans_dropped_by_checksum;
  --st.planned_calls;  // the call is not one that a schedule served
  if (nts_spmm_gather(p.input, p.output, p.weight, p.offsets, p.indices, p.index_base, p.rows, p.edges, p.F, 0,
                      p.stream) != NTS_OK) {
    printf("HIP call while recomputing an aggregation returned an error: %s\n", nts_last_error());
    exit(1);
  }
}
inline void settle_pending() {
  State &st = state();
  std::lock_guard<std::mutex> lock(st.mu);
  settle_pending_locked(st);
}
// A write into device memory at p (an upload, a zeroing, a kernel output).
inline void note_write(const void *p) {
  if (!p) return;
  zero_record().ptr = NULL;  // something was written through this header since the last zero_buffer
  State &st = state();
  std::lock_guard<std::mutex> lock(st.mu);
  settle_pending_locked(st);
  std::map<uintptr_t, Region>::iterator it = region_of(st, p);
  if (it != st.regions.end()) it->second.generation = st.clock++;
}
// The schedule for this (offsets, indices) pair if the structure has proved static, else NULL.
// may_defer: the caller's output is known to be all zeros, so the call can be computed again if needed;
// then the checksum runs on a side stream next to the aggregation and *deferred is set -- the caller
// registers the call with defer_check once it is enqueued.
inline nts_spmm_plan_t *plan_for(const uint32_t *offsets, const uint32_t *indices, uint32_t index_base,
                                 uint32_t n_index, uint32_t rows, uint32_t edges, nts_stream_t stream,
                                 bool may_defer = false, bool *deferred = NULL) {
  if (deferred) *deferred = false;
  if (edges < kPlanMinEdges || n_index == 0) return NULL;
  State &st = state();
  std::lock_guard<std::mutex> lock(st.mu);
  settle_pending_locked(st);
  if (st.enabled < 0) {
    const char *e = getenv("NTS_VENEER_PLAN_CACHE");
    st.enabled = (e && e[0] == '0') ? 0 : 1;
  }
  if (!st.enabled) return NULL;
  std::map<uintptr_t, Region>::iterator ro = region_of(st, offsets), ri = region_of(st, indices);
  if (ro == st.regions.end() || ri == st.regions.end()) return NULL;
  CachedPlan &c = st.plans[(uintptr_t)offsets];
  const bool same = c.indices == indices && c.rows == rows && c.edges == edges && c.n_index == n_index &&
                    c.index_base == index_base && c.gen_offsets == ro->second.generation &&
                    c.gen_indices == ri->second.generation;
  if (!same) {
    if (c.plan) nts_spmm_plan_destroy(c.plan);
    CachedPlan fresh = {NULL, indices, rows, edges, n_index, index_base, ro->second.generation, ri->second.generation, 1,
                        0};
    c = fresh;
    return NULL;
  }
  uint64_t now = 0;
  if (!c.plan) {
    if (++c.seen < 3) return NULL;
    // checksum first: the schedule is then made from arrays that are at least as new as the checksum
    if (nts_fingerprint_u32(&c.fingerprint, offsets, (uint64_t)rows + 1, indices, edges, stream) != NTS_OK ||
        nts_spmm_plan_create_slabs(&c.plan, offsets, indices, index_base, n_index, rows, edges, 0, 0, stream) != NTS_OK) {
      c.plan = NULL;
      c.seen = -1000000;  // do not try again for this structure
      return NULL;
    }
    ++st.plans_built;
  }
  if (may_defer && deferred) {
    if (st.async_verify < 0) {
      const char *e = getenv("NTS_VENEER_ASYNC_VERIFY");
      st.async_verify = (e && e[0] == '0') ? 0 : 1;
      if (st.async_verify && (nts_stream_create(&st.verify_stream) != NTS_OK || nts_event_create(&st.verify_fork) != NTS_OK ||
                              nts_malloc_pinned_mapped((void **)&st.pinned_sum, 64) != NTS_OK))
        st.async_verify = 0;
    }
    // the side stream sees the arrays as the caller's stream has left them so far
    if (st.async_verify && nts_event_record(st.verify_fork, stream) == NTS_OK &&
        nts_stream_wait_event(st.verify_stream, st.verify_fork) == NTS_OK &&
        nts_fingerprint_u32_async(st.pinned_sum, offsets, (uint64_t)rows + 1, indices, edges, st.verify_stream) == NTS_OK) {
      *deferred = true;
      ++st.planned_calls;
      ++st.deferred_checks;
      return c.plan;
    }
  }
  if (nts_fingerprint_u32(&now, offsets, (uint64_t)rows + 1, indices, edges, stream) != NTS_OK || now != c.fingerprint) {
    // the arrays were written behind this header's back: forget the schedule and start counting again
    nts_spmm_plan_destroy(c.plan);
    c.plan = NULL;
    c.seen = 1;
    ++st.plans_dropped_by_checksum;
    return NULL;
  }
  ++st.planned_calls;
  return c.plan;
}
// Registers the scheduled call that was just enqueued on `stream` with the side-stream checksum started
// by plan_for: settled at the next entry of this header.
inline void defer_check(const uint32_t *offsets, const uint32_t *indices, uint32_t index_base, uint32_t rows,
                        uint32_t edges, uint32_t F, const float *input, float *output, const float *weight,
                        nts_stream_t stream) {
  State &st = state();
  std::lock_guard<std::mutex> lock(st.mu);
  State::Pending p = {true, (uintptr_t)offsets, input, weight, output, offsets, indices, index_base, rows, edges, F, stream};
  st.pending = p;
}
inline long deferred_checks() { return state().deferred_checks; }
inline long plans_built() { return state().plans_built; }
inline long planned_calls() { return state().planned_calls; }
inline long plans_dropped_by_checksum() { return state().plans_dropped_by_checksum; }

}  // namespace nts_veneer

// ---- allocation and copies ---------------------------------------------------------------------

inline void *cudaMallocPinned(long size_of_bytes) {
  void *p = NULL;
  NTS_VENEER_CHECK(nts_malloc_pinned_mapped(&p, (size_t)size_of_bytes));
  return p;
}
inline void *getDevicePointer(void *host_data_to_device) {
  void *d = NULL;
  NTS_VENEER_CHECK(nts_host_get_device_ptr(&d, host_data_to_device));
  return d;
}
inline void *cudaMallocGPU(long size_of_bytes) {
  void *p = NULL;
  NTS_VENEER_CHECK(nts_malloc_device(&p, (size_t)size_of_bytes));
  nts_veneer::note_alloc(p, (size_t)size_of_bytes);
  return p;
}
inline void ntsFreeHost(void *buffer) { NTS_VENEER_CHECK(nts_free_pinned(buffer)); }
inline void FreeBuffer(float *buffer) {
  nts_veneer::note_free(buffer);
  NTS_VENEER_CHECK(nts_free_device(buffer));
}
inline void FreeEdge(VertexId_CUDA *buffer) {
  nts_veneer::note_free(buffer);
  NTS_VENEER_CHECK(nts_free_device(buffer));
}
inline void FreeBufferAsync(float *buffer, cudaStream_t cs) {
  nts_veneer::note_free(buffer);
  NTS_VENEER_CHECK(nts_free_device_async(buffer, cs));
}
inline void FreeEdgeAsync(VertexId_CUDA *buffer, cudaStream_t cs) {
  nts_veneer::note_free(buffer);
  NTS_VENEER_CHECK(nts_free_device_async(buffer, cs));
}
template <typename T>
inline void free_gpu_data(T *data) {
  nts_veneer::note_free(data);
  NTS_VENEER_CHECK(nts_free_device(data));
}
template <typename T>
inline void alloc_gpu_data(T **input, int size) {
  NTS_VENEER_CHECK(nts_malloc_device((void **)input, sizeof(T) * (size_t)size));
  nts_veneer::note_alloc(*input, sizeof(T) * (size_t)size);
}
inline void allocate_gpu_buffer(float **input, int size) {
  NTS_VENEER_CHECK(nts_malloc_device((void **)input, sizeof(float) * (size_t)size));
  nts_veneer::note_alloc(*input, sizeof(float) * (size_t)size);
}
inline void allocate_gpu_edge(VertexId_CUDA **input, int size) {
  NTS_VENEER_CHECK(nts_malloc_device((void **)input, sizeof(VertexId_CUDA) * (size_t)size));
  nts_veneer::note_alloc(*input, sizeof(VertexId_CUDA) * (size_t)size);
}
inline void allocate_gpu_buffer_async(float **input, int size, cudaStream_t cs) {
  NTS_VENEER_CHECK(nts_malloc_device_async((void **)input, sizeof(float) * (size_t)size, cs));
  nts_veneer::note_alloc(*input, sizeof(float) * (size_t)size);
}
inline void allocate_gpu_edge_async(VertexId_CUDA **input, int size, cudaStream_t cs) {
  NTS_VENEER_CHECK(nts_malloc_device_async((void **)input, sizeof(VertexId_CUDA) * (size_t)size, cs));
  nts_veneer::note_alloc(*input, sizeof(VertexId_CUDA) * (size_t)size);
}
inline void move_result_out(float *output, float *input, int src, int dst, int feature_size, bool sync = true) {
  nts_veneer::settle_pending();
  NTS_VENEER_CHECK(nts_memcpy_d2h(output, input, (size_t)(dst - src) * feature_size * sizeof(float), sync));
}
inline void move_data_in(float *d_pointer, float *h_pointer, int start, int end, int feature_size, bool sync = true) {
  nts_veneer::note_write(d_pointer);
  NTS_VENEER_CHECK(nts_memcpy_h2d(d_pointer, h_pointer, (size_t)(end - start) * feature_size * sizeof(float), sync));
}
inline void move_edge_in(VertexId_CUDA *d_pointer, VertexId_CUDA *h_pointer, VertexId_CUDA start, VertexId_CUDA end,
                         int feature_size, bool sync = true) {
  nts_veneer::note_write(d_pointer);
  NTS_VENEER_CHECK(
      nts_memcpy_h2d(d_pointer, h_pointer, (size_t)(end - start) * feature_size * sizeof(VertexId_CUDA), sync));
}
inline void move_bytes_in(void *d_pointer, void *h_pointer, long bytes, bool sync = true) {
  nts_veneer::note_write(d_pointer);
  NTS_VENEER_CHECK(nts_memcpy_h2d(d_pointer, h_pointer, (size_t)bytes, sync));
}
inline void move_bytes_in_async(void *d_pointer, void *h_pointer, long bytes, cudaStream_t cs) {
  nts_veneer::note_write(d_pointer);
  NTS_VENEER_CHECK(nts_memcpy_h2d_async(d_pointer, h_pointer, (size_t)bytes, cs));
}
inline void zero_buffer(float *buffer, int size) {
  nts_veneer::note_write(buffer);
  NTS_VENEER_CHECK(nts_memset_zero(buffer, sizeof(float) * (size_t)size, (cudaStream_t)0));
  NTS_VENEER_CHECK(nts_device_sync());
  nts_veneer::note_zeroed(buffer, (size_t)size);
}
inline void CUDA_DEVICE_SYNCHRONIZE() {
  nts_veneer::settle_pending();
  NTS_VENEER_CHECK(nts_device_sync());
}
// The few raw runtime names that core/ and comm/ call outside cuda/ (core/ntsMiniBatchGraphOp.hpp:283,
// core/coocsc.hpp:673-773, comm/network.cpp:53, 84).
inline int cudaFree(void *p) {
  nts_veneer::note_free(p);
  return nts_free_device(p);
}
inline int cudaFreeHost(void *p) { return nts_free_pinned(p); }
inline int cudaStreamSynchronize(cudaStream_t s) {
  nts_veneer::settle_pending();
  return nts_stream_sync(s);
}

// cudaMallocManaged as the data loader uses it (core/ntsDataloador.hpp:66-73): memory that both the
// host and the device address.  Page-locked mapped host memory has that property; the device reads
// it in place (zero-copy), which is how the feature table is consumed anyway.
template <typename T>
inline int cudaMallocManaged(T **ptr, size_t bytes) {
  return nts_malloc_pinned_mapped((void **)ptr, bytes);
}

// ---- deviceCSC (cuda/ntsCUDA.hpp:54-97) ----------------------------------------------------------

class deviceCSC {
 public:
  VertexId_CUDA *column_offset = NULL;
  VertexId_CUDA *row_indices = NULL;
  VertexId_CUDA *mirror_index = NULL;
  VertexId_CUDA v_size = 0;
  VertexId_CUDA e_size = 0;
  VertexId_CUDA mirror_size = 0;
  bool require_mirror = false;

  void init(VertexId_CUDA v_size_, VertexId_CUDA e_size_, bool require_mirror_ = false,
            VertexId_CUDA mirror_size_ = 0) {
    v_size = v_size_;
    e_size = e_size_;
    column_offset = (VertexId_CUDA *)cudaMallocGPU((long)(v_size_ + 1) * sizeof(VertexId_CUDA));
    row_indices = (VertexId_CUDA *)cudaMallocGPU((long)e_size_ * sizeof(VertexId_CUDA));
    require_mirror = require_mirror_;
    if (require_mirror_) {
      mirror_size = mirror_size_;
      mirror_index = (VertexId_CUDA *)cudaMallocGPU((long)mirror_size_ * sizeof(VertexId_CUDA));
    }
  }
  void load_from_host(VertexId_CUDA *h_column_offset, VertexId_CUDA *h_row_indices, VertexId_CUDA *h_mirror_index) {
    load_from_host(h_column_offset, h_row_indices);
    move_bytes_in(mirror_index, h_mirror_index, (long)mirror_size * sizeof(VertexId_CUDA));
  }
  void load_from_host(VertexId_CUDA *h_column_offset, VertexId_CUDA *h_row_indices) {
    move_bytes_in(column_offset, h_column_offset, (long)(v_size + 1) * sizeof(VertexId_CUDA));
    move_bytes_in(row_indices, h_row_indices, (long)e_size * sizeof(VertexId_CUDA));
  }
  void release() {
    FreeEdge(column_offset);
    FreeEdge(row_indices);
    if (require_mirror) FreeEdge(mirror_index);
    column_offset = row_indices = mirror_index = NULL;
  }
};

// ---- Cuda_Stream (cuda/ntsCUDA.hpp:99-211) -------------------------------------------------------

class Cuda_Stream {
 public:
  cudaStream_t stream = NULL;
  bool owns_stream = false;

  Cuda_Stream() {
    NTS_VENEER_CHECK(nts_stream_create(&stream));
    owns_stream = true;
  }
  ~Cuda_Stream() { destory_Stream(); }
  void destory_Stream() {
    if (owns_stream && stream) NTS_VENEER_CHECK(nts_stream_destroy(stream));
    stream = NULL;
    owns_stream = false;
  }
  cudaStream_t getStream() { return stream; }
  // Adopts a stream owned by someone else (a libtorch pool stream); the previous own stream is destroyed.
  void setNewStream(cudaStream_t cudaStream) {
    destory_Stream();
    stream = cudaStream;
  }
  void CUDA_DEVICE_SYNCHRONIZE() {
    nts_veneer::settle_pending();
    NTS_VENEER_CHECK(nts_stream_sync(stream));
  }

  void move_result_out(float *output, float *input, VertexId_CUDA src, VertexId_CUDA dst, int feature_size,
                       bool sync = true) {
    (void)sync;
    nts_veneer::settle_pending();
    NTS_VENEER_CHECK(nts_memcpy_d2h_async(output, input, (size_t)(dst - src) * feature_size * sizeof(float), stream));
  }
  void move_data_in(float *d_pointer, float *h_pointer, VertexId_CUDA start, VertexId_CUDA end, int feature_size,
                    bool sync = true) {
    (void)sync;
    nts_veneer::note_write(d_pointer);
    NTS_VENEER_CHECK(
        nts_memcpy_h2d_async(d_pointer, h_pointer, (size_t)(end - start) * feature_size * sizeof(float), stream));
  }
  void move_edge_in(VertexId_CUDA *d_pointer, VertexId_CUDA *h_pointer, VertexId_CUDA start, VertexId_CUDA end,
                    int feature_size, bool sync = true) {
    (void)sync;
    nts_veneer::note_write(d_pointer);
    NTS_VENEER_CHECK(nts_memcpy_h2d_async(d_pointer, h_pointer,
                                          (size_t)(end - start) * feature_size * sizeof(VertexId_CUDA), stream));
  }

  // Aggregation.  The *_end and dst_start / src_start arguments that the reference's kernels never
  // read are accepted and ignored.  Semantics: output += sum (output is pre-zeroed by the caller).
  void Gather_By_Dst_From_Src(float *input, float *output, float *weight_forward, VertexId_CUDA *row_indices,
                              VertexId_CUDA *column_offset, VertexId_CUDA src_start, VertexId_CUDA src_end,
                              VertexId_CUDA dst_start, VertexId_CUDA dst_end, VertexId_CUDA edges,
                              VertexId_CUDA batch_size, VertexId_CUDA feature_size, bool with_weight = false,
                              bool tensor_weight = false) {
    (void)dst_start; (void)dst_end;
    reject_tensor_weight(with_weight && tensor_weight);
    // output += sum; on an output this thread has just cleared with zero_buffer that is output = sum
    const int accumulate = nts_veneer::take_zeroed(output, (size_t)batch_size * feature_size) ? 0 : 1;
    nts_veneer::note_write(output);
    bool deferred = false;
    nts_spmm_plan_t *plan =
        nts_veneer::plan_for(column_offset, row_indices, src_start, src_end > src_start ? src_end - src_start : 0,
                             batch_size, edges, stream, accumulate == 0, &deferred);
    if (plan) {
      NTS_VENEER_CHECK(nts_spmm_gather_planned(plan, input, output, with_weight ? weight_forward : NULL, column_offset,
                                               row_indices, src_start, feature_size, accumulate, stream));
      if (deferred)
        nts_veneer::defer_check(column_offset, row_indices, src_start, batch_size, edges, feature_size, input, output,
                                with_weight ? weight_forward : NULL, stream);
    } else
      NTS_VENEER_CHECK(nts_spmm_gather(input, output, with_weight ? weight_forward : NULL, column_offset, row_indices,
                                       src_start, batch_size, edges, feature_size, accumulate, stream));
  }
  void Gather_By_Dst_From_Src_Optim(float *input, float *output, float *weight_forward, VertexId_CUDA *row_indices,
                                    VertexId_CUDA *column_offset, VertexId_CUDA src_start, VertexId_CUDA src_end,
                                    VertexId_CUDA dst_start, VertexId_CUDA dst_end, VertexId_CUDA edges,
                                    VertexId_CUDA batch_size, VertexId_CUDA feature_size, bool with_weight = false,
                                    bool tensor_weight = false) {
    Gather_By_Dst_From_Src(input, output, weight_forward, row_indices, column_offset, src_start, src_end, dst_start,
                           dst_end, edges, batch_size, feature_size, with_weight, tensor_weight);
  }
  void Gather_By_Src_From_Dst(float *input, float *output, float *weight_backward, VertexId_CUDA *row_offset,
                              VertexId_CUDA *column_indices, VertexId_CUDA src_start, VertexId_CUDA src_end,
                              VertexId_CUDA dst_start, VertexId_CUDA dst_end, VertexId_CUDA edges,
                              VertexId_CUDA batch_size, VertexId_CUDA feature_size, bool with_weight = false,
                              bool tensor_weight = false) {
    (void)src_start; (void)src_end;
    reject_tensor_weight(with_weight && tensor_weight);
    const int accumulate = nts_veneer::take_zeroed(output, (size_t)batch_size * feature_size) ? 0 : 1;
    nts_veneer::note_write(output);
    bool deferred = false;
    nts_spmm_plan_t *plan =
        nts_veneer::plan_for(row_offset, column_indices, dst_start, dst_end > dst_start ? dst_end - dst_start : 0,
                             batch_size, edges, stream, accumulate == 0, &deferred);
    if (plan) {
      NTS_VENEER_CHECK(nts_spmm_gather_planned(plan, input, output, with_weight ? weight_backward : NULL, row_offset,
                                               column_indices, dst_start, feature_size, accumulate, stream));
      if (deferred)
        nts_veneer::defer_check(row_offset, column_indices, dst_start, batch_size, edges, feature_size, input, output,
                                with_weight ? weight_backward : NULL, stream);
    } else
      NTS_VENEER_CHECK(nts_spmm_gather(input, output, with_weight ? weight_backward : NULL, row_offset, column_indices,
                                       dst_start, batch_size, edges, feature_size, accumulate, stream));
  }
  void Gather_By_Src_From_Dst_Optim(float *input, float *output, float *weight_backward, VertexId_CUDA *row_offset,
                                    VertexId_CUDA *column_indices, VertexId_CUDA src_start, VertexId_CUDA src_end,
                                    VertexId_CUDA dst_start, VertexId_CUDA dst_end, VertexId_CUDA edges,
                                    VertexId_CUDA batch_size, VertexId_CUDA feature_size, bool with_weight = false,
                                    bool tensor_weight = false) {
    Gather_By_Src_From_Dst(input, output, weight_backward, row_offset, column_indices, src_start, src_end, dst_start,
                           dst_end, edges, batch_size, feature_size, with_weight, tensor_weight);
  }
  void Scatter_Grad_Back_To_Message(float *input, float *message_grad, VertexId_CUDA *row_indices,
                                    VertexId_CUDA *column_offset, VertexId_CUDA src_start, VertexId_CUDA src_end,
                                    VertexId_CUDA dst_start, VertexId_CUDA dst_end, VertexId_CUDA edges,
                                    VertexId_CUDA batch_size, VertexId_CUDA feature_size, bool with_weight = true) {
    (void)row_indices; (void)src_start; (void)src_end; (void)dst_start; (void)dst_end; (void)edges;
    if (with_weight) {
      printf("tensor_weight Scatter_Grad_Back_To_Weight not implemented\n");
      exit(0);
    }
    nts_veneer::note_write(message_grad);
    NTS_VENEER_CHECK(nts_scatter_grad_to_edge(message_grad, input, column_offset, batch_size, feature_size, stream));
  }

  // Edge <-> vertex.
  void Scatter_Src_Mirror_to_Msg(float *message, float *src_mirror_feature, VertexId_CUDA *row_indices,
                                 VertexId_CUDA *column_offset, VertexId_CUDA *mirror_index, VertexId_CUDA batch_size,
                                 VertexId_CUDA feature_size) {
    nts_veneer::note_write(message);
    NTS_VENEER_CHECK(nts_scatter_src_to_edge(message, src_mirror_feature, row_indices, column_offset, mirror_index,
                                             batch_size, feature_size, stream));
  }
  void Scatter_Dst_to_Msg(float *message, float *dst_feature, VertexId_CUDA *row_indices,
                          VertexId_CUDA *column_offset, VertexId_CUDA batch_size, VertexId_CUDA feature_size) {
    (void)row_indices;
    nts_veneer::note_write(message);
    NTS_VENEER_CHECK(nts_scatter_dst_to_edge(message, dst_feature, column_offset, batch_size, feature_size, stream));
  }
  void Gather_Msg_to_Dst(float *dst_feature, float *message, VertexId_CUDA *row_indices, VertexId_CUDA *column_offset,
                         VertexId_CUDA batch_size, VertexId_CUDA feature_size) {
    (void)row_indices;
    nts_veneer::note_write(dst_feature);
    NTS_VENEER_CHECK(nts_gather_edge_to_dst(dst_feature, message, column_offset, batch_size, feature_size, 1, stream));
  }
  // Reference argument list; deterministic, but sorts the edges by target row on every call.
  void Gather_Msg_To_Src_Mirror(float *src_mirror_feature, float *message, VertexId_CUDA *row_indices,
                                VertexId_CUDA *column_offset, VertexId_CUDA *mirror_index, VertexId_CUDA batch_size,
                                VertexId_CUDA feature_size) {
    nts_veneer::note_write(src_mirror_feature);
    NTS_VENEER_CHECK(nts_gather_edge_to_src_unsorted(src_mirror_feature, message, row_indices, column_offset,
                                                     mirror_index, batch_size, feature_size, stream));
  }
  // Cheaper deterministic form of the same operation: takes the transposed structure
  // (row_offset [src_size+1], csr_to_csc [E]) instead of (row_indices, column_offset, mirror_index).
  void Gather_Msg_To_Src(float *src_feature, float *message, VertexId_CUDA *row_offset, VertexId_CUDA *csr_to_csc,
                         VertexId_CUDA src_size, VertexId_CUDA feature_size) {
    nts_veneer::note_write(src_feature);
    NTS_VENEER_CHECK(nts_gather_edge_to_src(src_feature, message, row_offset, csr_to_csc, src_size, feature_size, 1,
                                            stream));
  }
  void Edge_Softmax_Forward_Block(float *msg_output, float *msg_input, float *msg_cached, VertexId_CUDA *row_indices,
                                  VertexId_CUDA *column_offset, VertexId_CUDA batch_size,
                                  VertexId_CUDA feature_size) {
    (void)row_indices;
    nts_veneer::note_write(msg_output);
    NTS_VENEER_CHECK(nts_edge_softmax_fwd(msg_output, msg_input, column_offset, batch_size, feature_size, stream));
    if (msg_cached && msg_cached != msg_output) {
      // The edge count is only known on the device: copy column_offset[batch_size] back once.
      VertexId_CUDA edges = 0;
      NTS_VENEER_CHECK(nts_memcpy_d2h_async(&edges, column_offset + batch_size, sizeof(edges), stream));
      NTS_VENEER_CHECK(nts_stream_sync(stream));
      NTS_VENEER_CHECK(
          nts_memcpy_d2d_async(msg_cached, msg_output, (size_t)edges * feature_size * sizeof(float), stream));
    }
  }
  void Edge_Softmax_Backward_Block(float *msg_input_grad, float *msg_output_grad, float *msg_cached,
                                   VertexId_CUDA *row_indices, VertexId_CUDA *column_offset, VertexId_CUDA batch_size,
                                   VertexId_CUDA feature_size) {
    (void)row_indices;
    nts_veneer::note_write(msg_input_grad);
    NTS_VENEER_CHECK(nts_edge_softmax_bwd(msg_input_grad, msg_output_grad, msg_cached, column_offset, batch_size,
                                          feature_size, stream));
  }

  // Declared by the reference but never defined there (cuda/ntsCUDA.hpp:180-187); kept so that
  // core/NtsScheduler.hpp parses.  Calling them is a link error, as it is in the reference.
  void Gather_By_Dst_From_Message(float *input, float *output, VertexId_CUDA *src, VertexId_CUDA *dst,
                                  VertexId_CUDA src_start, VertexId_CUDA src_end, VertexId_CUDA dst_start,
                                  VertexId_CUDA dst_end, VertexId_CUDA edges, VertexId_CUDA batch_size,
                                  VertexId_CUDA feature_size, bool with_weight = false, bool tensor_weight = false);
  void zero_copy_embedding_move_gpu(float *dev_feature, float *pinned_host_feature, VertexId_CUDA feature_size,
                                    VertexId_CUDA vertex_size);
  // Rows that arrive as message records {vertex id, F floats} (cuda/ntsCUDATransferKernel.cuh:43-93): the
  // full-graph operators ForwardGPUfuseOp / DistGPUGetDepNbrOp exchange rows this way, also when the
  // one partition of a single-GPU run sends to itself (core/NtsScheduler.hpp:300-314).
  void aggregate_comm_result_debug(float *aggregate_buffer, float *input_buffer, VertexId_CUDA data_size,
                                   VertexId_CUDA feature_size, VertexId_CUDA partition_start,
                                   VertexId_CUDA partition_end, bool sync) {
    (void)sync;
    nts_veneer::note_write(aggregate_buffer);
    NTS_VENEER_CHECK(nts_message_rows_add(aggregate_buffer, input_buffer, data_size, feature_size, partition_start,
                                          partition_end, stream));
  }
  void deSerializeToGPU(float *input_gpu_buffer, float *input_buffer, VertexId_CUDA data_size,
                        VertexId_CUDA feature_size, VertexId_CUDA partition_start, VertexId_CUDA partition_end,
                        bool sync) {
    (void)sync;
    nts_veneer::note_write(input_gpu_buffer);
    NTS_VENEER_CHECK(nts_message_rows_unpack(input_gpu_buffer, input_buffer, data_size, feature_size, partition_start,
                                             partition_end, stream));
  }
  // The reference's kernel behind this one adds the message buffer to itself and prints
  // (cuda/ntsCUDATransferKernel.cuh:30-41); nothing in core/ calls it.  It fails loudly.
  void aggregate_comm_result(float *, float *, VertexId_CUDA, int, int, bool = true) { dist_unsupported(); }

  // Mini-batch assembly; like the reference these return with the result complete.
  void zero_copy_feature_move_gpu(float *dev_feature, float *pinned_host_feature, VertexId_CUDA *src_vertex,
                                  VertexId_CUDA feature_size, VertexId_CUDA vertex_size) {
    nts_veneer::note_write(dev_feature);
    NTS_VENEER_CHECK(nts_gather_rows_f32(dev_feature, pinned_host_feature, src_vertex, NULL, NULL, vertex_size,
                                         feature_size, stream));
    CUDA_DEVICE_SYNCHRONIZE();
  }
  void zero_copy_feature_move_gpu_cache(float *dev_feature, float *host_pinned_feature, VertexId_CUDA *src_vertex,
                                        VertexId_CUDA feature_size, VertexId_CUDA vertex_size,
                                        VertexId_CUDA *local_idx) {
    nts_veneer::note_write(dev_feature);
    NTS_VENEER_CHECK(nts_gather_rows_f32(dev_feature, host_pinned_feature, src_vertex, local_idx, NULL, vertex_size,
                                         feature_size, stream));
    CUDA_DEVICE_SYNCHRONIZE();
  }
  void gather_feature_from_gpu_cache(float *dev_feature, float *dev_cache_feature, VertexId_CUDA *src_vertex,
                                     VertexId_CUDA feature_size, VertexId_CUDA vertex_size,
                                     VertexId_CUDA *local_idx_cache, VertexId_CUDA *cache_node_hashmap) {
    nts_veneer::note_write(dev_feature);
    NTS_VENEER_CHECK(nts_gather_rows_f32(dev_feature, dev_cache_feature, src_vertex, local_idx_cache,
                                         cache_node_hashmap, vertex_size, feature_size, stream));
    CUDA_DEVICE_SYNCHRONIZE();
  }
  void global_copy_label_move_gpu(long *dev_label, long *global_dev_label, VertexId_CUDA *dst_vertex,
                                  VertexId_CUDA vertex_size) {
    nts_veneer::note_write(dev_label);
    NTS_VENEER_CHECK(nts_gather_labels_i64((int64_t *)dev_label, (const int64_t *)global_dev_label, dst_vertex,
                                           vertex_size, 1, stream));
    CUDA_DEVICE_SYNCHRONIZE();
  }
  void global_copy_mulilabel_move_gpu(long *dev_label, long *global_dev_label, VertexId_CUDA *dst_vertex,
                                      VertexId_CUDA vertex_size, VertexId_CUDA label_size) {
    nts_veneer::note_write(dev_label);
    NTS_VENEER_CHECK(nts_gather_labels_i64((int64_t *)dev_label, (const int64_t *)global_dev_label, dst_vertex,
                                           vertex_size, label_size, stream));
    CUDA_DEVICE_SYNCHRONIZE();
  }

 private:
  static void dist_unsupported() {
    printf("Cuda_Stream::aggregate_comm_result has no defined result in the reference and is not implemented\n");
    exit(1);
  }
  static void reject_tensor_weight(bool tensor) {
    if (tensor) {
      printf("tensor-weight aggregation is a legacy implementation\n");
      exit(0);
    }
  }
};

#endif  // NTS_HIP_VENEER_HPP
