/*
 * nts_hip.h -- C ABI of libntship.so, the gfx950 (MI355X, wave64) replacement for the
 * single-GPU graph-operator kernels of NeutronBench.
 *
 * Every entry point is `extern "C"`, takes plain pointers and sizes, receives the HIP stream
 * explicitly, returns an int status (0 = NTS_OK) and never prints or exits.  State that outlives a
 * call is either in a handle the caller owns (a schedule, a batch builder: calls on one handle are
 * serialised by the library, see each) or one of four items that are safe to share: a per-device
 * pool that keeps freed scratch (thread-safe, stream-ordered), the per-thread last-error text, a
 * stream per host thread and device on which the softmax / attention entry points run the block
 * kernels of their hub rows beside their other launches (forked from and joined to the caller's
 * stream inside the call; never while that stream records a graph), and the fixed scratch array of
 * nts_spmm_gather_static_scratch (whose calls a caller must serialise).  Calls on different streams and host threads are otherwise independent, which is what
 * the reference's pipelined mini-batch loop needs (one Cuda_Stream per host thread,
 * toolkits/GCN_GPU_NEIGHBOR.hpp:1350-1363).
 *
 * Conventions: indices are uint32 (VertexId_CUDA, cuda/cuda_type.h:21), values are fp32, labels
 * are int64.  Dense operands are row-major and contiguous: a [n, F] tensor has row stride F.
 * All pointers are device pointers unless a comment says "mapped host" (pinned host memory that
 * the device reads through its device alias).
 *
 * Each declaration cites the reference interface it replaces (file:line relative to the
 * NeutronBench source tree).
 */
#ifndef NTS_HIP_H
#define NTS_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* hipStream_t is `struct ihipStream_t *`; spelled out so that C callers need no HIP headers. */
typedef struct ihipStream_t *nts_stream_t;

enum nts_status {
  NTS_OK = 0,
  NTS_ERR_INVALID = 1,     /* null pointer, zero width, size overflow, inconsistent arguments */
  NTS_ERR_HIP = 2,         /* a HIP runtime call failed; see nts_last_error() */
  NTS_ERR_UNSUPPORTED = 3, /* argument combination the reference also rejects (tensor weights) */
  NTS_ERR_NOMEM = 4        /* allocation failed */
};

/* Text of the last error raised on the calling thread ("" if none).  Replaces the reference's
 * CHECK_CUDA_RESULT print-and-exit (cuda/ntsCUDAGraphOP.cu:11-20). */
const char *nts_last_error(void);
/* ABI version: bumped when a signature changes. */
int nts_abi_version(void);
/* Profiler ranges.  With NTS_TRACE_RANGES=1 in the environment (read when the first traced entry
 * point runs) the compute, layout, sampling and reader entry points below push a rocTX range named
 * after themselves on entry and pop it on return, so that `rocprofv3 --marker-trace --kernel-trace`
 * attributes kernels to calls; the rocTX library is loaded at run time only then.  The reference
 * brackets its stages with wall-clock accumulators instead (toolkits/GCN_GPU_NEIGHBOR.hpp:617-705).
 * nts_trace_ranges_emitted: ranges pushed so far by this process (0 when ranges are off). */
long nts_trace_ranges_emitted(void);
/* Scratch memory.  A few entry points need device memory beyond their arguments (stated with each
 * of them: calls of nts_spmm_gather / nts_spmm_gather_heads that cut hub rows, the lists of hub rows
 * of the edge operators, nts_gather_edge_to_src_unsorted).  It is allocated and freed in stream
 * order from a memory pool of the library's own, one per device, which keeps freed blocks for the
 * next call instead of returning them to the driver at every synchronisation: the pool holds on to
 * the largest scratch any call has needed (the reference allocates such buffers with cudaMalloc per
 * call, cuda/ntsCUDAGraphOP.cu:595-653).  nts_scratch_trim returns the current device's unused
 * scratch to the driver; work queued earlier is not affected. */
int nts_scratch_trim(void);
/* Scratch blocks the library has taken from its pool so far in this process (every call that needs
 * scratch takes one or two): lets a caller check that a code path allocates nothing. */
long nts_scratch_alloc_count(void);

/* ---------------------------------------------------------------------------------------------
 * Memory, copies, streams
 * ------------------------------------------------------------------------------------------- */

/* cudaMallocGPU (cuda/ntsCUDAGraphOP.cu:45-55), allocate_gpu_buffer / allocate_gpu_edge /
 * alloc_gpu_data (:603-629).  Sizes are bytes in size_t: the reference's `int size` element
 * counts overflow above 2^31 elements. */
int nts_malloc_device(void **ptr, size_t bytes);
/* FreeBuffer / FreeEdge / free_gpu_data (:557-601).  NULL is accepted (the reference's ~sampCSC
 * frees pointers it never initialised, core/coocsc.hpp:100-116). */
int nts_free_device(void *ptr);
/* allocate_gpu_buffer_async / allocate_gpu_edge_async (:631-651): stream-ordered allocation. */
int nts_malloc_device_async(void **ptr, size_t bytes, nts_stream_t stream);
/* FreeBufferAsync / FreeEdgeAsync (:566-592). */
int nts_free_device_async(void *ptr, nts_stream_t stream);
/* cudaMallocPinned (:34-43): page-locked host memory mapped into the device address space. */
int nts_malloc_pinned_mapped(void **host_ptr, size_t bytes);
/* ntsFreeHost (:548-555). */
int nts_free_pinned(void *host_ptr);
/* getDevicePointer (:23-32): device alias of a mapped pinned host allocation. */
int nts_host_get_device_ptr(void **dev_ptr, void *host_ptr);
/* move_data_in / move_edge_in / move_bytes_in (:487-522): blocking host-to-device copy; when
 * `sync` is non-zero the whole device is synchronised afterwards as the reference does. */
int nts_memcpy_h2d(void *dst_dev, const void *src_host, size_t bytes, int sync);
/* move_bytes_in_async (:524-531), Cuda_Stream::move_data_in / move_edge_in (:132-152). */
int nts_memcpy_h2d_async(void *dst_dev, const void *src_host, size_t bytes, nts_stream_t stream);
/* move_result_out (:476-485): blocking device-to-host copy. */
int nts_memcpy_d2h(void *dst_host, const void *src_dev, size_t bytes, int sync);
/* Cuda_Stream::move_result_out (:121-130). */
int nts_memcpy_d2h_async(void *dst_host, const void *src_dev, size_t bytes, nts_stream_t stream);
/* Device-to-device copy on a stream (the reference has none: its edge-softmax kernel writes the
 * output and the cached copy itself, cuda/ntsCUDADistKernel.cuh:207-209). */
int nts_memcpy_d2d_async(void *dst_dev, const void *src_dev, size_t bytes, nts_stream_t stream);
/* zero_buffer (:594-601) / NtsScheduler::ZeroVarMem (core/NtsScheduler.hpp:321-336).  Done with a
 * fill kernel on `stream` (safe under graph capture); does not synchronise. */
int nts_memset_zero(void *dev_ptr, size_t bytes, nts_stream_t stream);
/* Cuda_Stream::Cuda_Stream / ~Cuda_Stream / destory_Stream (:57-93). Default priority only. */
int nts_stream_create(nts_stream_t *stream);
int nts_stream_destroy(nts_stream_t stream);
/* Cuda_Stream::CUDA_DEVICE_SYNCHRONIZE (:111-119) -- which is a *stream* synchronise. */
int nts_stream_sync(nts_stream_t stream);
/* cudaDeviceSynchronize as used by zero_buffer / move_* with sync=true. */
int nts_device_sync(void);
/* get_gpu_mem / show_gpu_mem (utils/cuda_memory.hpp:6-68): free and total device bytes. */
int nts_mem_info(size_t *free_bytes, size_t *total_bytes);

/* 64-bit checksum of one or two uint32 device arrays (position-dependent: moving or changing any
 * element changes it, up to hash collisions), computed on the device and read back: the call waits
 * for `stream`.  Either array may be empty.  For callers that keep something derived from device
 * arrays they do not own -- the host veneer verifies with it, before every call through a schedule it
 * built by itself, that offsets and indices still hold what the schedule was made from.  No
 * counterpart in the reference.  About 0.1 ms for 115 M indices (one multiply-add per element, one atomic per block). */
int nts_fingerprint_u32(uint64_t *fingerprint, const uint32_t *a, uint64_t n_a, const uint32_t *b, uint64_t n_b,
                        nts_stream_t stream);
/* The same checksum without waiting: the kernels and the copy of the raw sum into *pinned_sum (page-locked
 * host memory, e.g. nts_malloc_pinned_mapped) are enqueued on `stream`; once the stream has reached
 * that point, nts_fingerprint_finish(*pinned_sum, n_a, n_b) is the value nts_fingerprint_u32 returns.
 * Lets a caller take the checksum on a side stream while the work it guards runs (the host veneer
 * does: it checks the value when the reference's operator synchronises, and recomputes the
 * aggregation without its schedule if the arrays turn out to have changed). */
int nts_fingerprint_u32_async(uint64_t *pinned_sum, const uint32_t *a, uint64_t n_a, const uint32_t *b, uint64_t n_b,
                              nts_stream_t stream);
uint64_t nts_fingerprint_finish(uint64_t sum, uint64_t n_a, uint64_t n_b);

/* Device-side timers (the reference only has host wall clocks, dep/gemini/time.hpp:20-26, around
 * synchronised calls).  An event is an opaque handle; elapsed time is in milliseconds between two
 * recorded events and synchronises on `stop`. */
typedef struct ihipEvent_t *nts_event_t;
int nts_event_create(nts_event_t *event);
int nts_event_destroy(nts_event_t event);
int nts_event_record(nts_event_t event, nts_stream_t stream);
/* Work enqueued on `stream` after this call starts only when `event`, as last recorded, has completed
 * (hipStreamWaitEvent): orders streams without blocking the host. */
int nts_stream_wait_event(nts_stream_t stream, nts_event_t event);
int nts_event_elapsed_ms(float *ms, nts_event_t start, nts_event_t stop);

/* ---------------------------------------------------------------------------------------------
 * Aggregation (weighted / unweighted SpMM as a row gather)
 *
 *   out[r, :] (+)= sum_{e in [offsets[r], offsets[r+1])} w[e] * in[indices[e] - index_base, :]
 *
 * Forward = CSC arrays (column_offset, row_indices, edge_weight_forward), rows = destinations.
 * Backward = CSR arrays (row_offset, column_indices, edge_weight_backward), rows = sources: the
 * gradient scatter is executed as the transposed gather, so no float atomics are used and the
 * result is bit-reproducible run to run.
 * ------------------------------------------------------------------------------------------- */

/* Cuda_Stream::Gather_By_Dst_From_Src[_Optim] and Gather_By_Src_From_Dst[_Optim]
 * (cuda/ntsCUDA.hpp:124-143; launches cuda/ntsCUDAGraphOP.cu:186-292; kernels
 * cuda/ntsCUDAFuseKernel.cuh:147-290, 327-487).
 *   w           NULL = unweighted (with_weight=false)
 *   index_base  src_start (forward) or dst_start (backward); 0 for sampled layers
 *   accumulate  0: out = sum (out need not be initialised);  non-zero: out += sum, the
 *               reference's semantics on a pre-zeroed output
 * Works without any preprocessing; one wavefront (or a sub-wavefront group for narrow F) per row,
 * its edges added in order with one fused multiply-add each.  Calls of 65,536 edges or more do not
 * leave long rows to one wavefront: rows of more than P edges are cut into P-edge pieces on the
 * device (no copy to the host), the pieces write partial sums and a second stage adds them in
 * order -- still deterministic, but a long row's sum is then associated piece by piece.  P = 256
 * edges; from 2^22 edges up the pieces are also issued in source order.  That path takes stream-ordered scratch
 * from the library's pool (see nts_scratch_trim; about (E/P + min(rows, E/P) + 1) * (F * 4 + 48)
 * bytes plus 4 bytes per row, released in stream order before the call returns); a caller that
 * must not allocate, or that runs the same structure many times, uses a plan (below), which also
 * orders the pieces for the L2. */
int nts_spmm_gather(const float *in, float *out, const float *w, const uint32_t *offsets,
                    const uint32_t *indices, uint32_t index_base, uint32_t rows, uint32_t edges,
                    uint32_t F, int accumulate, nts_stream_t stream);

/* nts_spmm_gather with a bound the caller knows: no row has more than max_row_edges edges (a sampled
 * layer's forward pass: a destination keeps at most `fanout` neighbours, core/ntsSampler.hpp:936-1042;
 * nts_batch_builder_layers reports the bound as nts_sampled_layer_t::max_in_degree).  With
 * 0 < max_row_edges <= 256 the call is ONE launch -- a wavefront or lane group per row, nothing to cut,
 * no scratch -- whatever the edge count; with 0 (unknown) or a larger bound it is nts_spmm_gather.
 * The bound only selects the launch: a row longer than stated is still summed correctly, by one
 * wavefront.  Replaces the same reference calls as nts_spmm_gather (cuda/ntsCUDA.hpp:124-143), as
 * reached from SingleGPUSampleGraphOp::forward (core/ntsMiniBatchGraphOp.hpp:288-318). */
int nts_spmm_gather_bounded(const float *in, float *out, const float *w, const uint32_t *offsets,
                            const uint32_t *indices, uint32_t index_base, uint32_t rows, uint32_t edges,
                            uint32_t F, int accumulate, uint32_t max_row_edges, nts_stream_t stream);

/* nts_spmm_gather for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.
 * Same arguments, same kernels and bit-identical results; the scratch of calls that cut long rows
 * lives in a fixed array inside the library's code object (NTS_SPMM_STATIC_SCRATCH_BYTES, held by
 * every device that loads the library until the process ends) instead of the stream-ordered pool.
 * The call itself allocates and frees nothing (the first call on a device looks the array's address
 * up once; do that call before a capture).  A call whose scratch, by the formula given with
 * nts_spmm_gather plus the scan / sort work area, exceeds the array returns NTS_ERR_INVALID with
 * both sizes in nts_last_error() and launches nothing; calls below 65,536 edges need no scratch.
 * Every call on a device uses the same array: calls that overlap on one device (two streams, two
 * host threads) race, so a caller serialises them.  Nothing in the array has to be zero on entry:
 * each call writes every word before it reads it.  Under stream capture: calls below 2^22 edges record
 * kernel launches only; from 2^22 edges up the pieces are ordered with the runtime library's radix sort,
 * which may record fill nodes, so such a call is not for capture. */
#define NTS_SPMM_STATIC_SCRATCH_BYTES ((size_t)64 << 20)
int nts_spmm_gather_static_scratch(const float *in, float *out, const float *w, const uint32_t *offsets,
                                   const uint32_t *indices, uint32_t index_base, uint32_t rows,
                                   uint32_t edges, uint32_t F, int accumulate, nts_stream_t stream);

/* Degree-bucketed schedule for a fixed offsets array (full-graph chunks: CSC_segment_pinned,
 * core/GraphSegment.h:54-133).  Rows are ordered by descending degree class; rows longer than
 * `chunk_edges` are split into chunks whose partial sums are combined by a second kernel in a
 * fixed order (deterministic).  chunk_edges = 0 selects the default.  The call reads `offsets`
 * back to the host once and synchronises `stream`. */
typedef struct nts_spmm_plan nts_spmm_plan_t;
int nts_spmm_plan_create(nts_spmm_plan_t **plan, const uint32_t *offsets, uint32_t rows,
                         uint32_t edges, uint32_t chunk_edges, nts_stream_t stream);
/* The same schedule, made cache-aware: `indices` (the gather index array that belongs to `offsets`)
 * is read back once as well, and the pieces of split rows whose indices ascend are cut at the
 * boundaries of `n_slabs` equal ranges of [index_base, index_base + n_index) and issued slab by slab,
 * so that concurrently running wavefronts gather from the same range of source rows (each XCD's
 * L2 then holds that range's hot rows).  n_slabs = 0 and chunk_edges = 0 select the defaults (32
 * ranges, 512 edges, tuned on a 114.8 M-edge power-law graph at F = 602).  A row that is cut but
 * whose indices do not ascend (an edge file in arbitrary order; the reference's loader leaves CSR
 * rows in thread-arrival order) is cut in a copy of the index array, owned by the plan, in which
 * it is sorted (stably); the plan then gathers through that copy (E * 8 more bytes on the device)
 * and such a row's sum is associated in source order.  With 8 or more ranges, rows of at most
 * 4 * chunk_edges edges are cut at n_slabs / 2 ranges of twice the width, and rows of more
 * than chunk_edges / 4 edges are cut as well, at the boundaries of n_slabs / 4 four-times-wider
 * ranges (their pieces run next to the long rows' pieces of the same sources); such a row stays
 * whole when all its edges fall into one wide range.  Results differ from nts_spmm_plan_create only
 * in which rows are cut and where; rows of at most chunk_edges / 4 edges are never cut. */
int nts_spmm_plan_create_slabs(nts_spmm_plan_t **plan, const uint32_t *offsets, const uint32_t *indices,
                               uint32_t index_base, uint32_t n_index, uint32_t rows, uint32_t edges,
                               uint32_t chunk_edges, uint32_t n_slabs, nts_stream_t stream);
/* The schedule the two calls above would build, computed from HOST copies of the arrays and
 * returned instead of uploaded (no device needed; indices_host NULL = nts_spmm_plan_create's
 * schedule, chunk_edges / n_slabs 0 = that call's defaults).  items_out (nullable) receives up to
 * items_cap items of four words each, in issue order: (row, first edge, end edge, partial-sum slot
 * or 0xFFFFFFFF for a row that is summed whole).  For tests and for inspecting a schedule. */
int nts_spmm_plan_schedule_host(const uint32_t *offsets_host, const uint32_t *indices_host, uint32_t n_index,
                                uint32_t rows, uint32_t chunk_edges, uint32_t n_slabs, uint32_t *items_out,
                                uint64_t items_cap, uint32_t *n_items, uint32_t *n_split_rows,
                                uint32_t *n_partials);
int nts_spmm_plan_destroy(nts_spmm_plan_t *plan);
/* Copies a plan's schedule to the host: items_out (nullable; items_cap items of four words, as
 * nts_spmm_plan_schedule_host writes them) and splits_out (nullable; splits_cap entries of four words:
 * row, first partial slot, slot count, 0 -- the split rows in the order the second stage visits them).
 * For tests and for inspecting a schedule; the counts come from nts_spmm_plan_info. */
int nts_spmm_plan_copy_schedule(const nts_spmm_plan_t *plan, uint32_t *items_out, uint64_t items_cap,
                                uint32_t *splits_out, uint64_t splits_cap);
/* Number of work items, split rows and partial-sum slots of a plan (for tests and reports). */
int nts_spmm_plan_info(const nts_spmm_plan_t *plan, uint32_t *items, uint32_t *split_rows,
                       uint32_t *partials);
/* What a call of width F through this plan keeps in the plan's scratch, and what the schedule found:
 * bytes of partial sums, bytes of the padded input copy (0 when the call gathers from `in` itself),
 * the number of edges that repeat the gather index of the edge before them in their row, and whether
 * calls load a source row once per run of such edges.  Any out-pointer may be NULL. */
int nts_spmm_plan_scratch_info(nts_spmm_plan_t *plan, uint32_t F, size_t *partial_bytes, size_t *padded_input_bytes,
                               uint64_t *repeated_edges, int *loads_once_per_run);
/* Grow the plan's scratch (partial sums of split rows; for a schedule with runs of equal indices
 * also a copy of the input with padded rows, see below) so that a later call of width F allocates
 * nothing. */
int nts_spmm_plan_reserve(nts_spmm_plan_t *plan, uint32_t F);
/* NtsScheduler::GatherByDstFromSrc / GatherBySrcFromDst on a full-graph chunk
 * (core/NtsScheduler.hpp:146-178, 239-271; core/graph.hpp:3432-3478).  `offsets` must be the
 * array the plan was built from.
 * Parallel edges.  When at least 1 edge in 20 repeats the gather index of the edge before it (a
 * multigraph with sorted rows; nts_spmm_plan_create_slabs counts them), the call loads a source row
 * once per run of equal indices and still adds it once per edge, with that edge's weight and in edge
 * order, so every sum keeps its bits.  Such a schedule also gathers rows that are wider than 128
 * floats and not a multiple of four floats wide from a copy of `in` whose rows are padded to whole
 * 128-byte lines (made by the call, in the plan's scratch, n_index * 4 * ceil(F / 32) * 32 bytes), so
 * that the row loads are 16 bytes per lane.
 * Concurrency.  A plan's scratch is shared by all calls on it.  The host side of a call is
 * serialised per plan, and a call on another stream than the previous one first waits, on the
 * device, for that call's last kernel; calls on one plan therefore never overlap on the device,
 * from however many streams or host threads they come (use one plan per stream for overlap).  The
 * caller must not destroy a plan while a call on it is being made.  A call on a stream that is being
 * captured is recorded without that ordering (no event is waited for or recorded under capture): the
 * caller orders replays of the captured call against eager calls and other streams that use the plan.
 * `in` must hold all n_index rows the plan was built for: a plan that gathers from a padded copy of
 * the input (see below) copies every row of `in` on each call. */
int nts_spmm_gather_planned(nts_spmm_plan_t *plan, const float *in, float *out, const float *w,
                            const uint32_t *offsets, const uint32_t *indices, uint32_t index_base,
                            uint32_t F, int accumulate, nts_stream_t stream);
/* Profiling hook: when both events are non-NULL, every later nts_spmm_gather_planned on this plan
 * records `start` immediately before and `stop` immediately after its main gather kernel (the
 * partial-sum reduction of split rows follows `stop`).  NULL, NULL switches it off. */
int nts_spmm_plan_set_events(nts_spmm_plan_t *plan, nts_event_t start, nts_event_t stop);

/* ---------------------------------------------------------------------------------------------
 * Edge <-> vertex data movement (GAT building blocks).  `co` = column_offset [Vd+1],
 * `ri` = row_indices [E] (source row of each edge), edge tensors are [E, F] in CSC edge order.
 * ------------------------------------------------------------------------------------------- */

/* Cuda_Stream::Scatter_Src_Mirror_to_Msg (cuda/ntsCUDA.hpp:145-147; kernel
 * cuda/ntsCUDADistKernel.cuh:23-44): msg[e,:] = feat[mirror[ri[e]], :]; mirror NULL = identity. */
int nts_scatter_src_to_edge(float *msg, const float *feat, const uint32_t *ri, const uint32_t *co,
                            const uint32_t *mirror, uint32_t Vd, uint32_t F, nts_stream_t stream);
/* Cuda_Stream::Scatter_Dst_to_Msg (cuda/ntsCUDA.hpp:153-155; kernel :65-79):
 * msg[e,:] = feat[d,:] for e in CSC(d). */
int nts_scatter_dst_to_edge(float *msg, const float *feat, const uint32_t *co, uint32_t Vd,
                            uint32_t F, nts_stream_t stream);
/* Cuda_Stream::Scatter_Grad_Back_To_Message (cuda/ntsCUDA.hpp:192-196; kernel
 * cuda/ntsCUDAFuseKernel.cuh:492-506): msg_grad[e,:] += gout[d,:] for e in CSC(d). */
int nts_scatter_grad_to_edge(float *msg_grad, const float *gout, const uint32_t *co, uint32_t Vd,
                             uint32_t F, nts_stream_t stream);
/* Cuda_Stream::Gather_Msg_to_Dst (cuda/ntsCUDA.hpp:157-159; kernel
 * cuda/ntsCUDADistKernel.cuh:81-95): out[d,:] (+)= sum_{e in CSC(d)} msg[e,:].  Rows of at most
 * 1,024 edges are summed in edge order (the running fp32 sum); longer rows are spread over the
 * slices of a block (and, above 16,384 edges, over several blocks) whose partial sums are added in
 * a fixed order: the same bits on every call, within rounding of the edge-order sum.  accumulate as
 * in nts_spmm_gather. */
int nts_gather_edge_to_dst(float *out, const float *msg, const uint32_t *co, uint32_t Vd,
                           uint32_t F, int accumulate, nts_stream_t stream);
/* Cuda_Stream::Gather_Msg_To_Src_Mirror (cuda/ntsCUDA.hpp:149-151; kernel :46-63), made
 * deterministic: out[s,:] (+)= sum_{k in CSR(s)} msg[perm[k], :] where `ro` = row_offset [Vs+1]
 * and perm[k] is the CSC edge id of the k-th CSR edge (see nts_csr_from_csc). */
int nts_gather_edge_to_src(float *out, const float *msg, const uint32_t *ro, const uint32_t *perm,
                           uint32_t Vs, uint32_t F, int accumulate, nts_stream_t stream);

/* The reference's own argument list of Gather_Msg_To_Src_Mirror (cuda/ntsCUDA.hpp:149-151), for
 * callers that have no transposed structure: out[mirror ? mirror[ri[e]] : ri[e], :] += msg[e, :] for
 * every CSC edge e.  Deterministic (edges of one target row are added in ascending edge order): the
 * call sorts the edges by target row in stream-ordered temporary memory, so it costs a sort per
 * call and reads co[Vd] back (synchronises `stream`).  Prefer nts_gather_edge_to_src. */
int nts_gather_edge_to_src_unsorted(float *out, const float *msg, const uint32_t *ri, const uint32_t *co,
                                    const uint32_t *mirror, uint32_t Vd, uint32_t F, nts_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * Edge softmax and fused GAT attention.  H = number of heads (columns); edge tensors [E, H].
 * ------------------------------------------------------------------------------------------- */

/* Cuda_Stream::Edge_Softmax_Forward_Block (cuda/ntsCUDA.hpp:161-163; kernel
 * cuda/ntsCUDADistKernel.cuh:166-213) with the semantics of the CPU operator SingleEdgeSoftMax
 * (core/ntsSingleCPUGraphOp.hpp:297-319): per destination segment and per column,
 * y = softmax(x), computed with the segment maximum subtracted.  `y` is also the cache the
 * backward needs.  Empty segments write nothing.  The exponential is the hardware's 2^(x log2 e):
 * measured against a float64 softmax, relative error at most 2e-6 on terms above 1e-6 and
 * absolute error at most 5e-7 (the operators are held to 1e-4). */
int nts_edge_softmax_fwd(float *y, const float *x, const uint32_t *co, uint32_t Vd, uint32_t H,
                         nts_stream_t stream);
/* Cuda_Stream::Edge_Softmax_Backward_Block (cuda/ntsCUDA.hpp:165-167; kernel :216-260;
 * SingleEdgeSoftMax::backward core/ntsSingleCPUGraphOp.hpp:321-341):
 * gx[e,h] = y[e,h] * (gy[e,h] - sum_{e' in seg} gy[e',h] * y[e',h]). */
int nts_edge_softmax_bwd(float *gx, const float *gy, const float *y, const uint32_t *co,
                         uint32_t Vd, uint32_t H, nts_stream_t stream);

/* Fused attention forward.  Replaces the chain scatter-src / scatter-dst / sum / leaky_relu /
 * edge-softmax of toolkits/GAT_CPU_DIST_OPTM.hpp:186-228 (algebraically equal to
 * toolkits/GAT_CPU.hpp:178-204):
 *   s[e,h]     = el[ri[e], h] + er[d, h]              for e in CSC(d)
 *   alpha[e,:] = softmax over CSC(d) of leaky_relu(s[e,:], slope)
 * el: [Vs, H] per-source scalars (a_l . h_src), er: [Vd, H] per-destination scalars. */
int nts_gat_attention_fwd(float *alpha, const float *el, const float *er, const uint32_t *co,
                          const uint32_t *ri, uint32_t Vd, uint32_t H, float slope,
                          nts_stream_t stream);
/* Fused attention backward, destination side: from galpha [E,H] and the cached alpha computes
 *   gs[e,h]  = leaky'(s[e,h]) * alpha[e,h] * (galpha[e,h] - sum_seg galpha*alpha)   (edge tensor)
 *   ger[d,h] = sum_{e in CSC(d)} gs[e,h]
 * The source-side gradient gel[s,h] = sum_{e: src(e)=s} gs[e,h] is nts_gather_edge_to_src(gs). */
int nts_gat_attention_bwd(float *gs, float *ger, const float *galpha, const float *alpha,
                          const float *el, const float *er, const uint32_t *co, const uint32_t *ri,
                          uint32_t Vd, uint32_t H, float slope, nts_stream_t stream);

/* nts_gat_attention_fwd / _bwd with the caller's bound on a destination's edges (a sampled layer: the
 * hop's fanout, nts_sampled_layer_t::max_in_degree).  When max_degree * H is at most 128 (and H a power
 * of two up to 16) the call is ONE launch, a lane group per destination with the segment in registers;
 * up to 32,768 values the launches that look for hub destinations and handle them are left out (three
 * launches instead of eleven for a layer of 16,384 destinations or more); 0 = no bound known = the calls
 * above.  The bound only selects the launches: a longer segment than stated is still computed -- by one
 * lane group or wavefront, slowly. */
int nts_gat_attention_fwd_bounded(float *alpha, const float *el, const float *er, const uint32_t *co,
                                  const uint32_t *ri, uint32_t Vd, uint32_t H, float slope,
                                  uint32_t max_degree, nts_stream_t stream);
int nts_gat_attention_bwd_bounded(float *gs, float *ger, const float *galpha, const float *alpha,
                                  const float *el, const float *er, const uint32_t *co, const uint32_t *ri,
                                  uint32_t Vd, uint32_t H, float slope, uint32_t max_degree,
                                  nts_stream_t stream);

/* Attention-weighted aggregation, multi-head (DistAggregateDstFuseWeight::forward,
 * core/ntsDistCPUGraphOp.hpp:401-440; composition E_msg*alpha -> SingleCPUDstAggregateOp of
 * toolkits/GAT_CPU.hpp:196-201):
 *   out[r, h*Fh + f] (+)= sum_{e in [offsets[r], offsets[r+1])} alpha[eid(e), h] * in[indices[e], h*Fh + f]
 * eid(e) = e when perm is NULL (forward over CSC) or perm[e] (backward over CSR, alpha kept in
 * CSC edge order).  `edges` = offsets[rows]; as in nts_spmm_gather, calls of 65,536 edges or more
 * cut long rows into pieces on the device (same piece length). */
int nts_spmm_gather_heads(const float *in, float *out, const float *alpha, const uint32_t *perm,
                          const uint32_t *offsets, const uint32_t *indices, uint32_t rows,
                          uint32_t edges, uint32_t H, uint32_t Fh, int accumulate, nts_stream_t stream);
/* nts_spmm_gather_heads with the caller's bound on the longest row, as nts_spmm_gather_bounded: one
 * launch when 0 < max_row_edges <= 256 (a sampled GAT layer's forward pass). */
int nts_spmm_gather_heads_bounded(const float *in, float *out, const float *alpha, const uint32_t *perm,
                                  const uint32_t *offsets, const uint32_t *indices, uint32_t rows,
                                  uint32_t edges, uint32_t H, uint32_t Fh, int accumulate,
                                  uint32_t max_row_edges, nts_stream_t stream);
/* The same through a schedule built by nts_spmm_plan_create[_slabs] for `offsets` (full-graph GAT:
 * hub rows are split and the sum order of split rows is the plan's). */
int nts_spmm_gather_heads_planned(nts_spmm_plan_t *plan, const float *in, float *out, const float *alpha,
                                  const uint32_t *perm, const uint32_t *offsets, const uint32_t *indices,
                                  uint32_t H, uint32_t Fh, int accumulate, nts_stream_t stream);
/* Gradient of the aggregation with respect to alpha (get_additional_grad of
 * DistAggregateDstFuseWeight, core/ntsDistCPUGraphOp.hpp:442-472):
 *   galpha[e,h] = < in[ri[e], h*Fh : (h+1)*Fh], gout[d, h*Fh : (h+1)*Fh] >   for e in CSC(d) */
int nts_sddmm_heads(float *galpha, const float *in, const float *gout, const uint32_t *co,
                    const uint32_t *ri, uint32_t Vd, uint32_t H, uint32_t Fh, nts_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * Mini-batch assembly
 * ------------------------------------------------------------------------------------------- */

/* One kernel for the three feature-gather launches of the reference:
 *   Cuda_Stream::zero_copy_feature_move_gpu        (cuda/ntsCUDA.hpp:168-169; kernel
 *       cuda/ntsCUDATransferKernel.cuh:96-108)      sel = NULL, remap = NULL, table = mapped host
 *   Cuda_Stream::zero_copy_feature_move_gpu_cache  (:170-172; kernel :153-166)   sel = local_idx
 *   Cuda_Stream::gather_feature_from_gpu_cache     (:173-175; kernel :168-182)   sel = local_idx_cache,
 *                                                                                  remap = cache_node_hashmap
 * For k < n:  i = sel ? sel[k] : k;  g = row_ids[i];  if (remap) g = remap[g];
 *             out[i, :] = table[g, :]          (bit-exact copy)
 * `table`, `sel`, `remap` may be device memory or mapped host memory.  A gather from a table in host
 * memory is bound by the link and is launched with a small fixed grid (128 blocks, which keep the
 * link full), so that work on other streams keeps the rest of the chip; the library learns where
 * `table` lives from hipPointerGetAttributes. */
int nts_gather_rows_f32(float *out, const float *table, const uint32_t *row_ids,
                        const uint32_t *sel, const uint32_t *remap, uint32_t n, uint32_t F,
                        nts_stream_t stream);
/* Device-side split-and-gather that needs no host loop: for every i < n,
 *   slot = hashmap[row_ids[i]];  out[i,:] = (slot != 0xFFFFFFFF) ? cache[slot,:] : table[row_ids[i],:]
 * Same result as the reference's host split (core/ntsSampler.hpp:424-469) followed by its two
 * kernels.  hits, if not NULL, receives the number of cache hits (device uint32, zeroed by the call). */
int nts_gather_rows_cached_f32(float *out, const float *table, const float *cache,
                               const uint32_t *row_ids, const uint32_t *hashmap, uint32_t n,
                               uint32_t F, uint32_t *hits, nts_stream_t stream);
/* Cuda_Stream::global_copy_label_move_gpu (classes == 1) and global_copy_mulilabel_move_gpu
 * (cuda/ntsCUDA.hpp:176-179; kernels cuda/ntsCUDATransferKernel.cuh:184-203):
 * out[i, :] = table[ids[i], :] with `classes` int64 values per row. */
int nts_gather_labels_i64(int64_t *out, const int64_t *table, const uint32_t *ids, uint32_t n,
                          uint32_t classes, nts_stream_t stream);

/* Vertex rows that arrive as message records.  The reference's full-graph GPU operators
 * (ForwardGPUfuseOp, core/ntsDistGPUFusedGraphOp.hpp:49-91; scheduler calls core/NtsScheduler.hpp:300-314)
 * exchange rows between partitions as records {uint32 vertex id, F floats} in a pinned host buffer --
 * also when the one partition of a single-GPU run sends to itself.  `records` (device memory or mapped
 * host memory) holds n_records records of 4 * (F + 1) bytes; records whose id lies outside
 * [id_begin, id_end) are skipped.
 *   nts_message_rows_unpack  Cuda_Stream::deSerializeToGPU (cuda/ntsCUDA.hpp:118-121; kernel
 *                            cuda/ntsCUDATransferKernel.cuh:66-93): rows[id - id_begin, :] = record values
 *   nts_message_rows_add     Cuda_Stream::aggregate_comm_result_debug (cuda/ntsCUDA.hpp:113-117; kernel
 *                            :43-64): rows[id - id_begin, :] += record values, without the reference's
 *                            float atomics: records that name distinct rows are added in parallel,
 *                            and a buffer that names a row twice is added in record order, so the
 *                            result is reproducible either way.  Takes 4 * (id_end - id_begin + 1) bytes
 *                            of stream-ordered scratch (see nts_scratch_trim). */
int nts_message_rows_unpack(float *rows, const float *records, uint32_t n_records, uint32_t F, uint32_t id_begin,
                            uint32_t id_end, nts_stream_t stream);
int nts_message_rows_add(float *rows, const float *records, uint32_t n_records, uint32_t F, uint32_t id_begin,
                         uint32_t id_end, nts_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * Sampled-layer index construction on the device (sampCSC, core/coocsc.hpp)
 * ------------------------------------------------------------------------------------------- */

/* One hop of neighbour sampling over a whole-graph CSC in HBM (Sampler::sample_one's construction
 * steps, core/ntsSampler.hpp:843-1106).  graph_co [V+1] / graph_ri [E_graph] are the whole graph's
 * column_offset / row_indices (global source ids), dst [n] the hop's destinations (global ids).
 *   nts_sample_hop_offsets   co[i+1]-co[i] = fanout < 0 ? deg(dst[i]) : min(deg(dst[i]), fanout), co[n] = number
 *                            of sampled edges (init_co, core/FullyRepGraph.hpp:199-209; bit-exact).  `work` is
 *                            nts_sample_hop_work_bytes(n) bytes of 256-byte-aligned device scratch.
 *   nts_sample_hop_neighbors ri_global[co[i] .. co[i+1]) = all in-neighbours of dst[i] in CSC order when none is
 *                            dropped, otherwise that many DISTINCT positions of its CSC segment chosen uniformly
 *                            from a hash of (seed, i, dst[i]), in ascending position order.  Any fanout, as the
 *                            reference's sampler (core/ntsSampler.hpp:936-1042): up to 64 by Floyd's sampling inside
 *                            a lane group, up to 1,024 by a keyed permutation of the positions, above that the
 *                            positions with the `fanout` smallest keyed hashes (a radix select per destination).
 * Which neighbours the reference picks depends on its RNG, thread count and container iteration
 * order, so the pick is specified here by these properties, not by equality with the reference. */
size_t nts_sample_hop_work_bytes(uint32_t n);
int nts_sample_hop_offsets(uint32_t *co, const uint32_t *graph_co, const uint32_t *dst, uint32_t n, int32_t fanout,
                           void *work, nts_stream_t stream);
int nts_sample_hop_neighbors(uint32_t *ri_global, const uint32_t *co, const uint32_t *graph_co,
                             const uint32_t *graph_ri, const uint32_t *dst, uint32_t n, int32_t fanout,
                             uint64_t seed, nts_stream_t stream);

/* All layers of one mini-batch in one stream-ordered sequence, with no host step between the hops:
 * for every hop init_dst, init_co, the neighbour pick, sampCSC::postprocessing,
 * generate_csr_from_csc, update_degree and compute_weight_forward / backward (Sampler::sample_one,
 * core/ntsSampler.hpp:843-1106; core/coocsc.hpp:136-450).  The reference sizes each hop's arrays on
 * the host from the previous hop's result and copies eight arrays per layer to the device
 * (core/coocsc.hpp:737-773); here the arrays live in one caller-provided device arena laid out for
 * the largest batch, the kernels read the live counts from the device, and the host learns the
 * layer shapes from ONE read-back per batch.  Every array equals what the per-hop entry points
 * above give with seeds seed, seed + 1, ... for hops 0, 1, ... (hop 0 = the batch's own hop).
 *
 *   fanouts[h]   fanout of hop h, hop 0 first (the output-side hop); < 0 = whole neighbourhood, in
 *                which case the batch must not repeat a vertex
 *   arena        nts_batch_builder_arena_bytes(...) bytes of 256-byte-aligned device memory, owned by
 *                the caller, in use until nts_batch_builder_destroy; graph_co / graph_ri likewise.
 *                The size includes the scratch of the library's scan and sort routines for the
 *                current device, so the call needs a device; 0 = unsupported arguments (no hop,
 *                more than 8 hops, a fanout of 0, an empty graph or batch).
 *   nts_batch_builder_sample  enqueues everything on `stream` and returns; n <= max_batch
 *   nts_batch_builder_layers  waits for that batch and fills layers[0 .. hops): index 0 is the
 *                input-side layer (its `source` indexes the feature gather), index hops-1 the
 *                layer whose `destination` is the batch -- the order of SampledSubgraph::sampled_sgs.
 *                Pointers address the arena and stay valid until the next nts_batch_builder_sample
 *                on the same builder; a pipeline that samples batch k+1 while batch k trains uses
 *                one builder per stage in flight, as the reference uses one SampledSubgraph each.
 *   nts_batch_builder_use_graph  enable != 0: nts_batch_builder_sample records the launches of the
 *                hops (and the copy of the layer shapes to the host) once, at the builder's next
 *                batch, as a HIP graph, and replays that graph for every later batch; only one small
 *                launch that stores the batch's ids, their count and the seed stays outside.  The
 *                arrays are the same bit for bit (every launch reads counts and the seed from the
 *                arena, none is a memset node); what changes is the host time per batch.  The
 *                recording is thread-local and runs on a stream the library creates for it; the
 *                graph is then launched on the caller's stream.  Off by default.
 *                enable == 2: the same, and in the recorded graph each hop's transposition and edge
 *                weights run on a side branch beside the next hop's sampling (same arrays; a batch
 *                built on an otherwise idle device gets shorter, one built beside other batches in
 *                flight does not -- use 1 there).
 *                enable == 3: two graphs.  The first holds the sampling and relabelling of every hop
 *                and the copy of the layer shapes and runs on the caller's stream; the second holds
 *                every hop's transposition and edge weights and runs after it on a stream that the
 *                builder owns.  nts_batch_builder_layers then returns as soon as the FIRST has
 *                finished: destination, source, column_offset and row_indices of every layer are
 *                complete, and the feature gather can start, while row_offset, column_indices,
 *                csr_to_csc and both weight arrays are still being written.  A stream that reads
 *                those must be passed to nts_batch_builder_join first (the host must wait for that
 *                stream before it reads them itself).  The next nts_batch_builder_sample of the
 *                builder waits for the second graph by itself.  Same arrays bit for bit.
 *                Any other non-zero value means 1.  Changing the value after a graph was recorded
 *                discards it (waiting for a second graph still running); the next batch records again.
 *   nts_batch_builder_join  makes `stream` wait (on the device; the call returns at once) until every
 *                array of the builder's current batch is complete.  Needed with enable == 3 only;
 *                otherwise the arrays are complete when nts_batch_builder_layers returns and the call
 *                does nothing.  `stream` must not be recording a graph (the event it waits for is
 *                recorded outside any recording).
 * Calls on one builder must not overlap: consecutive nts_batch_builder_sample calls go to the same
 * stream, or the earlier batch is waited for first (nts_batch_builder_layers does). */
typedef struct nts_batch_builder nts_batch_builder_t;
typedef struct nts_sampled_layer {
  uint32_t v_size, e_size, src_size;           /* destinations, edges, distinct sources */
  uint32_t max_in_degree;                      /* no destination has more edges than this (the hop's
                                                  fanout); 0 = no bound known (fanout -1)          */
  uint32_t *destination;                       /* [v_size]   global ids                        */
  uint32_t *source;                            /* [src_size] global ids, ascending             */
  uint32_t *column_offset;                     /* [v_size+1]                                   */
  uint32_t *row_indices;                       /* [e_size]   LOCAL source index                */
  uint32_t *row_offset;                        /* [src_size+1]                                 */
  uint32_t *column_indices;                    /* [e_size]   local destination index           */
  uint32_t *csr_to_csc;                        /* [e_size]   CSC position of CSR edge k, or NULL */
  float *edge_weight_forward;                  /* [e_size]   CSC order                         */
  float *edge_weight_backward;                 /* [e_size]   CSR order                         */
} nts_sampled_layer_t;
size_t nts_batch_builder_arena_bytes(uint32_t V, uint32_t graph_edges, const int32_t *fanouts, uint32_t hops,
                                     uint32_t max_batch, int want_perm);
int nts_batch_builder_create(nts_batch_builder_t **builder, const uint32_t *graph_co, const uint32_t *graph_ri,
                             uint32_t V, uint32_t graph_edges, const int32_t *fanouts, uint32_t hops,
                             uint32_t max_batch, int want_perm, void *arena, size_t arena_bytes);
int nts_batch_builder_sample(nts_batch_builder_t *builder, const uint32_t *batch_ids, uint32_t n, uint64_t seed,
                             nts_stream_t stream);
int nts_batch_builder_use_graph(nts_batch_builder_t *builder, int enable);
int nts_batch_builder_join(nts_batch_builder_t *builder, nts_stream_t stream);
int nts_batch_builder_layers(nts_batch_builder_t *builder, nts_sampled_layer_t *layers);
int nts_batch_builder_destroy(nts_batch_builder_t *builder);

/* sampCSC::postprocessing (core/coocsc.hpp:338-424): the sampled edges' GLOBAL source ids
 * (values < V) are marked in a bitmap; `source` receives the set bits in ascending order (the
 * distinct sampled sources), *n_source (device) their count, and local[e] the position of
 * global_ids[e] in `source` (local may alias global_ids).  `source` needs room for min(E, V) ids;
 * `work` is nts_relabel_sources_work_bytes(V) bytes of 256-byte-aligned device scratch.  Bit-exact
 * with the host bitmap scan. */
size_t nts_relabel_sources_work_bytes(uint32_t V);
int nts_relabel_sources(uint32_t *source, uint32_t *n_source, uint32_t *local, const uint32_t *global_ids,
                        uint32_t E, uint32_t V, void *work, nts_stream_t stream);
/* sampCSC::generate_csr_from_csc (core/coocsc.hpp:243-309): stable counting sort of the CSC edges
 * by local source.  Outputs ro [Vs+1], ci [E] (local destination of each CSR edge, ascending
 * within a source) and, if perm is not NULL, perm [E] (CSC edge id of each CSR edge).
 * `work` is caller-provided device scratch of nts_csr_from_csc_work_bytes(Vd, Vs, E) bytes.
 * Bit-exact with the host algorithm. */
size_t nts_csr_from_csc_work_bytes(uint32_t Vd, uint32_t Vs, uint32_t E);
int nts_csr_from_csc(uint32_t *ro, uint32_t *ci, uint32_t *perm, const uint32_t *co,
                     const uint32_t *ri, uint32_t Vd, uint32_t Vs, uint32_t E, void *work,
                     nts_stream_t stream);
/* sampCSC::update_degree + compute_weight_forward / compute_weight_backward
 * (core/coocsc.hpp:136-216) with nts_norm_degree (core/ntsBaseOp.hpp:183-186) evaluated from the
 * layer's own degrees: in_deg(d) = co[d+1]-co[d], out_deg(s) = ro[s+1]-ro[s],
 *   ewf[e] = 1 / ((float)sqrt((double)out_deg(ri[e])) * (float)sqrt((double)in_deg(d)))  e in CSC(d)
 *   ewb[k] = same value for the k-th CSR edge.
 * Either output may be NULL.  Bit-exact with the host computation. */
int nts_gcn_edge_weights(float *ewf, float *ewb, const uint32_t *co, const uint32_t *ri,
                         const uint32_t *ro, const uint32_t *ci, uint32_t Vd, uint32_t Vs,
                         nts_stream_t stream);

/* PartitionedGraph::generatePartitionedSubgraph + PartitionToChunks for one partition
 * (core/PartitionedGraph.hpp:281-388; device arrays of CSC_segment_pinned, core/GraphSegment.h:54-133):
 * from the edge list `pairs` (device, E records {src, dst} as the .edge file holds them, all ids < V)
 * builds on the device
 *   CSR  ro [V+1], ci [E]: edges ordered by source, input order kept inside a source,
 *   CSC  co [V+1], ri [E]: that list re-ordered by destination, stably (sources ascend in a row),
 * and, unless both are NULL, ewf [E] / ewb [E] = nts_norm_degree(out_deg(src), in_deg(dst)) in CSC /
 * CSR order, degrees being the edge counts of the list (duplicates and self loops count).
 * `work` is nts_chunk_from_edges_work_bytes(V, E) bytes of 256-byte-aligned device scratch.
 * Integer outputs and weights are bit-exact with the host construction fed the same list. */
size_t nts_chunk_from_edges_work_bytes(uint32_t V, uint32_t E);
int nts_chunk_from_edges(uint32_t *co, uint32_t *ri, float *ewf, uint32_t *ro, uint32_t *ci, float *ewb,
                         const uint32_t *pairs, uint32_t E, uint32_t V, void *work, nts_stream_t stream);

/* ---- on-disk dataset formats (host side; all buffers are host memory) ------------------------- */

/* Binary edge list: packed records {uint32 src, uint32 dst} in host byte order, no header
 * (EdgeUnit<Empty>, dep/gemini/type.hpp:99-106; Graph::load_directed takes file bytes / 8 as the
 * edge count, core/graph.hpp:1050-1061; written by data/generate_nts_dataset.py:340-345).
 * nts_edge_file_read copies records [first, first+n) into pairs [2n] and, if max_id is not NULL,
 * stores the largest vertex id among them (callers check it against their vertex count). */
int nts_edge_file_count(const char *path, uint64_t *edges);
int nts_edge_file_read(const char *path, uint32_t *pairs, uint64_t first, uint64_t n, uint32_t *max_id);

/* GNNDatum::readFeature_Label_Mask for a partition that owns every vertex
 * (core/ntsDataloador.hpp:264-395; readFtrFrom1, :209-262, reads the same feature and label text).
 * All three files are white-space separated tokens.
 *   feature file: records of 1 + F tokens "id f0 .. fF-1"; the values go to local_feature[id*F ..]
 *     ([V, F]); a value is the nearest float of its decimal text, as `istream >> float` yields;
 *     records whose id is >= V are skipped like vertices outside the reader's partition.
 *   label file: records "id label" (classes <= 1, tables [V]) or "id count idx_1 .. idx_count"
 *     (classes > 1, tables [V, classes], the named entries are set to 1).
 *   mask file: records "id word"; train -> 0, eval / val -> 1, test -> 2, anything else -> 3.
 * local_label / local_mask: the k-th label / mask record is stored at the vertex named by the k-th
 * FEATURE record (the files are read in step and the id column of the label / mask file is
 * ignored); global_label / global_mask: records are stored at their own id.  Entries the files do
 * not name keep their value, so tables come in zeroed as the reference's constructor leaves them
 * (:78-88).  Any of the four label / mask tables may be NULL.  Parsing runs on `threads` host
 * threads (<= 0: all); it fails with NTS_ERR_INVALID on an unreadable file, a malformed token or an
 * incomplete last feature record. */
int nts_read_feature_label_mask(const char *path_f, const char *path_l, const char *path_m, uint32_t V,
                                uint32_t F, uint32_t classes, float *local_feature, int64_t *local_label,
                                int32_t *local_mask, int64_t *global_label, int32_t *global_mask,
                                int threads);
/* Writes the feature file nts_read_feature_label_mask reads, in the form the reference's data
 * preparation produces (data/generate_nts_dataset.py:308, 356-359: "%.4f" after the id): record r is
 * "id f0 .. fF-1" with id = ids[r] (ids NULL: r) and every value printed with `decimals` (0..9) digits
 * after the point.  Formatting runs on `threads` host threads (<= 0: all). */
int nts_feature_text_write(const char *path, const float *table, const uint32_t *ids, uint32_t V, uint32_t F,
                           int decimals, int threads);
/* Comma-separated feature file of readFeature_Label_Mask_OGB (core/ntsDataloador.hpp:397-437): line k
 * holds the F values of vertex k; each field is converted with atof and narrowed to float. */
int nts_feature_csv_read(const char *path, float *table, uint32_t V, uint32_t F, int threads);
/* White-space separated integers (the label column and the train / valid / test id lists of
 * readFeature_Label_Mask_OGB, core/ntsDataloador.hpp:432, 461-469): stores the first `capacity` of them
 * in out (may be NULL) and the number found in *count; reading ends at the first non-integer token. */
int nts_int_list_text_read(const char *path, int64_t *out, uint64_t capacity, uint64_t *count);
/* Binary table (no counterpart in the reference, which only reads text): a 32-byte little-endian
 * header {"NTSTABLE", uint64 rows, uint64 cols, uint32 elem_bytes, uint32 0} followed by the
 * row-major data.  nts_table_bin_read copies rows [row_begin, row_begin+rows) into out, e.g.
 * straight into the pinned feature table. */
int nts_table_bin_write(const char *path, const void *data, uint64_t rows, uint64_t cols, uint32_t elem_bytes);
int nts_table_bin_info(const char *path, uint64_t *rows, uint64_t *cols, uint32_t *elem_bytes);
int nts_table_bin_read(const char *path, void *out, uint64_t row_begin, uint64_t rows);

#ifdef __cplusplus
}
#endif
#endif /* NTS_HIP_H */
