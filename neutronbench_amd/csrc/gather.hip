// Mini-batch assembly kernels: feature-row gather from mapped pinned host memory and / or an HBM
// feature cache, and label gather (replaces cuda/ntsCUDATransferKernel.cuh:96-203 and the
// launchers cuda/ntsCUDAGraphOP.cu:379-447).  Pure copies: results are bit-exact.
//
// A group of G lanes (G chosen so that G*VEC*4 bytes covers a row with little idle width) moves
// one row with 4/8/16-byte accesses; 64/G rows per wavefront.  Wide accesses matter most on the
// zero-copy path, where every wave load becomes PCIe read requests.
#include <algorithm>

#include "common.hpp"

namespace nts {
namespace {

constexpr uint32_t kMiss = 0xFFFFFFFFu;

template <typename V, int G>
__global__ __launch_bounds__(256) void gather_rows_kernel(V *__restrict__ out, const V *__restrict__ table,
                                                          const uint32_t *__restrict__ row_ids,
                                                          const uint32_t *__restrict__ sel,
                                                          const uint32_t *__restrict__ remap, uint32_t n,
                                                          uint32_t Fv) {
  constexpr uint32_t kRowsPerBlock = 256 / G;
  const uint32_t gl = threadIdx.x & (G - 1);
  for (uint64_t k = static_cast<uint64_t>(blockIdx.x) * kRowsPerBlock + threadIdx.x / G; k < n;
       k += static_cast<uint64_t>(gridDim.x) * kRowsPerBlock) {
    const uint32_t i = sel ? sel[k] : static_cast<uint32_t>(k);
    uint32_t g = row_ids[i];
    if (remap) g = remap[g];
    const V *src = table + static_cast<size_t>(g) * Fv;
    V *dst = out + static_cast<size_t>(i) * Fv;
    for (uint32_t c = gl; c < Fv; c += G) dst[c] = src[c];
  }
}

// Cached gather: a row comes from the HBM cache when its id has a slot, else from the (mapped host)
// table.  Blocks stride over the rows and count their hits locally; one integer atomic per block
// adds the block's count (one atomic per hit row on a single address was measured at 1.3 ms of a
// 1.9 ms launch for 337 k rows).
// miss_blocks > 0 (table in host memory): the first miss_blocks blocks copy only the rows that miss
// the cache -- they wait for the link -- and the blocks after them only the rows that hit, from HBM;
// every block walks all row ids of its stride and skips the rows of the other kind.  The few blocks
// that keep the link full are then not also the ones that move the (many more) cached rows.
template <typename V, int G>
__global__ __launch_bounds__(256) void gather_rows_cached_kernel(V *__restrict__ out, const V *__restrict__ table,
                                                                 const V *__restrict__ cache,
                                                                 const uint32_t *__restrict__ row_ids,
                                                                 const uint32_t *__restrict__ hashmap, uint32_t n,
                                                                 uint32_t Fv, uint32_t *__restrict__ hits,
                                                                 uint32_t miss_blocks) {
  constexpr uint32_t kRowsPerBlock = 256 / G;
  const uint32_t gl = threadIdx.x & (G - 1);
  uint32_t my_hits = 0;
  // blocks of this block's kind, and its rank among them
  const bool split = miss_blocks != 0, miss_side = blockIdx.x < miss_blocks;
  const uint32_t peers = !split ? gridDim.x : (miss_side ? miss_blocks : gridDim.x - miss_blocks);
  const uint32_t rank = (!split || miss_side) ? blockIdx.x : blockIdx.x - miss_blocks;
  for (uint64_t i = static_cast<uint64_t>(rank) * kRowsPerBlock + threadIdx.x / G; i < n;
       i += static_cast<uint64_t>(peers) * kRowsPerBlock) {
    const uint32_t g = row_ids[i];
    const uint32_t slot = hashmap[g];
    const bool hit = slot != kMiss;
    if (split && hit == miss_side) continue;  // the other kind of block copies this row
    const V *src = hit ? cache + static_cast<size_t>(slot) * Fv : table + static_cast<size_t>(g) * Fv;
    V *dst = out + static_cast<size_t>(i) * Fv;
    for (uint32_t c = gl; c < Fv; c += G) dst[c] = src[c];
    my_hits += (hit && gl == 0) ? 1u : 0u;
  }
  if (!hits) return;  // uniform across the block
  __shared__ uint32_t wave_hits[256 / kWave];
#pragma unroll
  for (int m = kWave / 2; m >= 1; m >>= 1) my_hits += __shfl_xor(my_hits, m, kWave);
  if ((threadIdx.x & (kWave - 1)) == 0) wave_hits[threadIdx.x / kWave] = my_hits;
  __syncthreads();
  if (threadIdx.x == 0) {
    uint32_t total = 0;
#pragma unroll
    for (int k = 0; k < 256 / kWave; ++k) total += wave_hits[k];
    if (total) atomicAdd(hits, total);  // integer count: order-independent
  }
}

__global__ __launch_bounds__(256) void gather_labels_kernel(int64_t *__restrict__ out,
                                                            const int64_t *__restrict__ table,
                                                            const uint32_t *__restrict__ ids, uint32_t n,
                                                            uint32_t classes) {
  const size_t total = static_cast<size_t>(n) * classes;
  for (size_t t = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; t < total;
       t += static_cast<size_t>(gridDim.x) * blockDim.x) {
    const uint32_t i = static_cast<uint32_t>(t / classes);
    const uint32_t c = static_cast<uint32_t>(t - static_cast<size_t>(i) * classes);
    out[t] = table[static_cast<size_t>(ids[i]) * classes + c];
  }
}

__global__ void zero_u32_kernel(uint32_t *p) { *p = 0u; }

// Lanes per row for a row of Fv vector elements: the smallest power of two >= Fv, clamped to [4, 64].
inline int group_for(uint32_t Fv) {
  int g = 4;
  while (g < 64 && static_cast<uint32_t>(g) < Fv) g <<= 1;
  return g;
}

struct RowsArgs {
  float *out;
  const float *table;
  const float *cache;  // null: plain gather
  const uint32_t *row_ids;
  const uint32_t *sel;
  const uint32_t *remap;  // plain gather: optional remap; cached gather: hashmap
  uint32_t n;
  uint32_t F;
  uint32_t *hits;
  hipStream_t stream;
};

// Blocks of a gather whose table lies in host memory.  Such a launch is bound by the PCIe link
// (about 57 GB/s here).  Where every row crosses the link, 32 blocks of four wavefronts, one row in
// flight per lane group, keep it full: the same time as with 128 blocks or 16,384.  In the cached
// gather the blocks that copy the missed rows also look up, one after the other, the rows that they
// then skip, and need 128 blocks for the same (32: three times the time; a variant in which a
// wavefront looks 64 rows up at once and 32 blocks suffice gathered 4-6 % faster and changed no
// epoch: what runs beside it slowed down by as much).  What the small grid buys is the rest of the
// chip and of the memory path: kernels that run beside a gather slow down several times over while
// their requests queue behind outstanding reads of host memory, and the fewer of those a gather keeps
// in flight beyond what the link needs, the less they do (a sampled batch's sort, CSR and weight
// kernels beside a plain 128-block gather: 5 to 18 times their usual time; beside 32 blocks: unchanged).
constexpr uint32_t kHostTableBlocks = 32;   // every row over the link
constexpr uint32_t kHostMissBlocks = 128;   // the missed rows of a cached gather
// NTS_GATHER_HOST_BLOCKS in the environment overrides both counts (for measurements).
uint32_t host_table_blocks(bool cached) {
  static const uint32_t forced = [] {
    const char *env = getenv("NTS_GATHER_HOST_BLOCKS");
    const long n = env ? atol(env) : 0;
    return n > 0 ? static_cast<uint32_t>(n) : 0u;
  }();
  return forced ? forced : (cached ? kHostMissBlocks : kHostTableBlocks);
}
constexpr uint32_t kCachedBlocks = 16384;  // table in device memory: fill the chip several times over
constexpr uint32_t kHitBlocks = 1024;      // table in host memory: blocks that copy the rows the HBM cache holds

// Whether `p` is host memory the device reads over the link.  The answer for the last table asked
// about is kept per thread (one query costs microseconds, and a caller gathers from the same table
// batch after batch); a stale answer could only pick the other grid size.
bool table_in_host_memory(const void *p) {
  thread_local const void *last_ptr = nullptr;
  thread_local bool last_host = false;
  if (p == last_ptr) return last_host;
  hipPointerAttribute_t attr;
  bool host = false;
  if (hipPointerGetAttributes(&attr, p) == hipSuccess)
    host = attr.type == hipMemoryTypeHost;
  else
    (void)hipGetLastError();  // an address the runtime does not know is not an error here
  last_ptr = p;
  last_host = host;
  return host;
}

template <typename V, int G>
void launch_rows(const RowsArgs &a, uint32_t Fv) {
  const uint32_t per_block = 256 / G;
  uint32_t blocks = ceil_div(a.n, per_block);
  const bool host_table = table_in_host_memory(a.table);
  // Both kernels stride over the rows, so any grid covers them.
  const uint32_t cap = host_table ? host_table_blocks(a.cache != nullptr) : (a.cache ? kCachedBlocks : blocks);
  const uint32_t wanted = blocks;
  if (blocks > cap) blocks = cap;
  if (a.cache) {
    // table in host memory: kHostMissBlocks blocks for the rows that miss, and beside them blocks for
    // the rows the cache holds (enough to move them at HBM speed, still a fraction of the chip)
    const uint32_t miss_blocks = (host_table && wanted > host_table_blocks(true)) ? host_table_blocks(true) : 0u;
    const uint32_t hit_blocks = miss_blocks ? std::min<uint32_t>(wanted, kHitBlocks) : 0u;
    hipLaunchKernelGGL((gather_rows_cached_kernel<V, G>), dim3(blocks + hit_blocks), dim3(256), 0, a.stream,
                       reinterpret_cast<V *>(a.out), reinterpret_cast<const V *>(a.table),
                       reinterpret_cast<const V *>(a.cache), a.row_ids, a.remap, a.n, Fv, a.hits, miss_blocks);
    return;
  }
  const dim3 grid(blocks);
    hipLaunchKernelGGL((gather_rows_kernel<V, G>), grid, dim3(256), 0, a.stream, reinterpret_cast<V *>(a.out),
                       reinterpret_cast<const V *>(a.table), a.row_ids, a.sel, a.remap, a.n, Fv);
}

template <typename V>
void launch_rows_v(const RowsArgs &a, uint32_t Fv) {
  switch (group_for(Fv)) {
    case 4: launch_rows<V, 4>(a, Fv); break;
    case 8: launch_rows<V, 8>(a, Fv); break;
    case 16: launch_rows<V, 16>(a, Fv); break;
    case 32: launch_rows<V, 32>(a, Fv); break;
    default: launch_rows<V, 64>(a, Fv); break;
  }
}

void launch_rows_any(const RowsArgs &a) {
  const bool c16 = !a.cache || aligned_to(a.cache, 16);
  const bool c8 = !a.cache || aligned_to(a.cache, 8);
  if (a.F % 4 == 0 && aligned_to(a.out, 16) && aligned_to(a.table, 16) && c16) return launch_rows_v<float4>(a, a.F / 4);
  if (a.F % 2 == 0 && aligned_to(a.out, 8) && aligned_to(a.table, 8) && c8) return launch_rows_v<float2>(a, a.F / 2);
  return launch_rows_v<float>(a, a.F);
}

// ---- rows that arrive as message records -----------------------------------------------------------
// The reference's full-graph GPU operators (ForwardGPUfuseOp, core/ntsDistGPUFusedGraphOp.hpp:49-91) move
// vertex rows between partitions as records {uint32 vertex id, F floats} in a pinned host buffer, also
// when the one partition sends to itself.  A wavefront takes one record at a time; its lanes cover
// the columns (records are 4 * (F + 1) bytes long, so rows are only 4-byte aligned).

__global__ __launch_bounds__(256) void message_rows_unpack_kernel(float *__restrict__ rows,
                                                                  const float *__restrict__ records, uint32_t n,
                                                                  uint32_t F, uint32_t id_begin, uint32_t id_end) {
  const uint32_t lane = threadIdx.x & (kWave - 1);
  const uint64_t waves = static_cast<uint64_t>(gridDim.x) * (blockDim.x / kWave);
  for (uint64_t k = static_cast<uint64_t>(blockIdx.x) * (blockDim.x / kWave) + threadIdx.x / kWave; k < n; k += waves) {
    const float *rec = records + k * (static_cast<uint64_t>(F) + 1);
    const uint32_t id = __float_as_uint(rec[0]);
    if (id < id_begin || id >= id_end) continue;
    float *dst = rows + static_cast<size_t>(id - id_begin) * F;
    for (uint32_t c = lane; c < F; c += kWave) dst[c] = rec[1 + c];
  }
}

// Counts how many records name each row; *repeated becomes non-zero when some row is named twice.
__global__ __launch_bounds__(256) void message_rows_claim_kernel(uint32_t *__restrict__ claims,
                                                                 uint32_t *__restrict__ repeated,
                                                                 const float *__restrict__ records, uint32_t n,
                                                                 uint32_t F, uint32_t id_begin, uint32_t id_end) {
  const uint64_t k = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (k >= n) return;
  const uint32_t id = __float_as_uint(records[k * (static_cast<uint64_t>(F) + 1)]);
  if (id < id_begin || id >= id_end) return;
  if (atomicAdd(&claims[id - id_begin], 1u) != 0u) atomicOr(repeated, 1u);
}

// rows[id - id_begin, :] += record values.  Records that name distinct rows (what the reference's
// operators send: one record per vertex and buffer) are added in parallel, each row by one
// wavefront, without atomics.  If two records of the buffer name the same row, the additions run in
// record order instead (one thread per column walks the buffer), so the result does not depend on
// scheduling either way.
__global__ __launch_bounds__(256) void message_rows_add_kernel(float *__restrict__ rows,
                                                               const float *__restrict__ records, uint32_t n,
                                                               uint32_t F, uint32_t id_begin, uint32_t id_end,
                                                               const uint32_t *__restrict__ repeated) {
  const uint64_t stride = static_cast<uint64_t>(F) + 1;
  if (*repeated) {
    const uint64_t c = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (c >= F) return;
    for (uint64_t k = 0; k < n; ++k) {
      const uint32_t id = __float_as_uint(records[k * stride]);
      if (id < id_begin || id >= id_end) continue;
      rows[static_cast<size_t>(id - id_begin) * F + c] += records[k * stride + 1 + c];
    }
    return;
  }
  const uint32_t lane = threadIdx.x & (kWave - 1);
  const uint64_t waves = static_cast<uint64_t>(gridDim.x) * (blockDim.x / kWave);
  for (uint64_t k = static_cast<uint64_t>(blockIdx.x) * (blockDim.x / kWave) + threadIdx.x / kWave; k < n; k += waves) {
    const float *rec = records + k * stride;
    const uint32_t id = __float_as_uint(rec[0]);
    if (id < id_begin || id >= id_end) continue;
    float *dst = rows + static_cast<size_t>(id - id_begin) * F;
    for (uint32_t c = lane; c < F; c += kWave) dst[c] += rec[1 + c];
  }
}

}  // namespace
}  // namespace nts

using namespace nts;

extern "C" {

int nts_message_rows_unpack(float *rows, const float *records, uint32_t n_records, uint32_t F, uint32_t id_begin,
                            uint32_t id_end, nts_stream_t stream) {
  NTS_TRACE_RANGE("nts_message_rows_unpack");
  if (F == 0) return fail(NTS_ERR_INVALID, "nts_message_rows_unpack: F is 0");
  if (n_records == 0 || id_end <= id_begin) return NTS_OK;
  if (!rows || !records) return fail(NTS_ERR_INVALID, "nts_message_rows_unpack: null pointer");
  const uint32_t blocks = static_cast<uint32_t>(std::min<uint64_t>((static_cast<uint64_t>(n_records) + 3) / 4, 16384));
  hipLaunchKernelGGL(message_rows_unpack_kernel, dim3(blocks), dim3(256), 0, stream, rows, records, n_records, F,
                     id_begin, id_end);
  NTS_LAUNCH_CHECK("nts_message_rows_unpack");
  return NTS_OK;
}

int nts_message_rows_add(float *rows, const float *records, uint32_t n_records, uint32_t F, uint32_t id_begin,
                         uint32_t id_end, nts_stream_t stream) {
  NTS_TRACE_RANGE("nts_message_rows_add");
  if (F == 0) return fail(NTS_ERR_INVALID, "nts_message_rows_add: F is 0");
  if (n_records == 0 || id_end <= id_begin) return NTS_OK;
  if (!rows || !records) return fail(NTS_ERR_INVALID, "nts_message_rows_add: null pointer");
  const size_t words = static_cast<size_t>(id_end - id_begin) + 1;  // claims per row, then the flag
  uint32_t *claims = nullptr;
  NTS_HIP_TRY(scratch_alloc(reinterpret_cast<void **>(&claims), words * sizeof(uint32_t), stream));
  int rc = nts_memset_zero(claims, words * sizeof(uint32_t), stream);
  if (rc == NTS_OK) {
    uint32_t *repeated = claims + (words - 1);
    hipLaunchKernelGGL(message_rows_claim_kernel, dim3((n_records + 255) / 256), dim3(256), 0, stream, claims, repeated,
                       records, n_records, F, id_begin, id_end);
    // enough blocks for one wavefront per record and for one thread per column
    const uint64_t want = std::max<uint64_t>((static_cast<uint64_t>(n_records) + 3) / 4, (static_cast<uint64_t>(F) + 255) / 256);
    const uint32_t blocks = static_cast<uint32_t>(std::min<uint64_t>(want, 16384));
    hipLaunchKernelGGL(message_rows_add_kernel, dim3(std::max(blocks, (F + 255) / 256)), dim3(256), 0, stream, rows,
                       records, n_records, F, id_begin, id_end, repeated);
    const hipError_t err = hipGetLastError();
    if (err != hipSuccess) rc = fail_hip(err, "nts_message_rows_add");
  }
  const hipError_t ferr = scratch_free(claims, stream);
  if (rc == NTS_OK && ferr != hipSuccess) rc = fail_hip(ferr, "nts_message_rows_add: scratch_free");
  return rc;
}

int nts_gather_rows_f32(float *out, const float *table, const uint32_t *row_ids, const uint32_t *sel,
                        const uint32_t *remap, uint32_t n, uint32_t F, nts_stream_t stream) {
  NTS_TRACE_RANGE("nts_gather_rows_f32");
  if (F == 0) return fail(NTS_ERR_INVALID, "nts_gather_rows_f32: F is 0");
  if (n == 0) return NTS_OK;
  if (!out || !table || !row_ids) return fail(NTS_ERR_INVALID, "nts_gather_rows_f32: null pointer");
  RowsArgs a{out, table, nullptr, row_ids, sel, remap, n, F, nullptr, stream};
  launch_rows_any(a);
  NTS_LAUNCH_CHECK("nts_gather_rows_f32");
  return NTS_OK;
}

int nts_gather_rows_cached_f32(float *out, const float *table, const float *cache, const uint32_t *row_ids,
                               const uint32_t *hashmap, uint32_t n, uint32_t F, uint32_t *hits,
                               nts_stream_t stream) {
  NTS_TRACE_RANGE("nts_gather_rows_cached_f32");
  if (F == 0) return fail(NTS_ERR_INVALID, "nts_gather_rows_cached_f32: F is 0");
  if (hits) {
    hipLaunchKernelGGL(zero_u32_kernel, dim3(1), dim3(1), 0, stream, hits);
    NTS_LAUNCH_CHECK("zero_u32_kernel");
  }
  if (n == 0) return NTS_OK;
  if (!out || !table || !cache || !row_ids || !hashmap)
    return fail(NTS_ERR_INVALID, "nts_gather_rows_cached_f32: null pointer");
  RowsArgs a{out, table, cache, row_ids, nullptr, hashmap, n, F, hits, stream};
  launch_rows_any(a);
  NTS_LAUNCH_CHECK("nts_gather_rows_cached_f32");
  return NTS_OK;
}

int nts_gather_labels_i64(int64_t *out, const int64_t *table, const uint32_t *ids, uint32_t n, uint32_t classes,
                          nts_stream_t stream) {
  NTS_TRACE_RANGE("nts_gather_labels_i64");
  if (classes == 0) return fail(NTS_ERR_INVALID, "nts_gather_labels_i64: classes is 0");
  if (n == 0) return NTS_OK;
  if (!out || !table || !ids) return fail(NTS_ERR_INVALID, "nts_gather_labels_i64: null pointer");
  const size_t total = static_cast<size_t>(n) * classes;
  size_t blocks = (total + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  hipLaunchKernelGGL(gather_labels_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream, out, table, ids,
                     n, classes);
  NTS_LAUNCH_CHECK("nts_gather_labels_i64");
  return NTS_OK;
}

}  // extern "C"
