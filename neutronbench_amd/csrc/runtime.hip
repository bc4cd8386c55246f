// Memory, copy and stream entry points of libntship (replaces the free functions and the
// Cuda_Stream plumbing of cuda/ntsCUDAGraphOP.cu:23-119, 476-653 and utils/cuda_memory.hpp).
#include <string.h>

#include <dlfcn.h>
#include <stdlib.h>

#include <atomic>
#include <algorithm>
#include <mutex>

#include "common.hpp"

namespace nts {

namespace {
thread_local char g_last_error[512] = "";
}

int fail(int code, const char *msg) {
  snprintf(g_last_error, sizeof(g_last_error), "%s", msg);
  return code;
}

int fail_hip(hipError_t err, const char *what) {
  snprintf(g_last_error, sizeof(g_last_error), "%s: %s (%d)", what, hipGetErrorString(err), static_cast<int>(err));
  return err == hipErrorOutOfMemory ? NTS_ERR_NOMEM : NTS_ERR_HIP;
}

namespace {

// 16-byte stores over the aligned body, byte stores over the ragged head and tail.
__global__ __launch_bounds__(256) void fill_zero_kernel(unsigned char *p, size_t head, size_t body16, size_t tail) {
  const size_t tid = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
  uint4 *body = reinterpret_cast<uint4 *>(p + head);
  for (size_t i = tid; i < body16; i += stride) body[i] = make_uint4(0u, 0u, 0u, 0u);
  if (tid < head) p[tid] = 0;
  if (tid < tail) p[head + body16 * 16 + tid] = 0;
}

// Position-dependent 64-bit checksum of a uint32 array: the sum over i of (a[i] + c) * k(salt + i) in
// 64 bits, k an odd 32-bit word hashed from the position -- one 32 x 32 -> 64 multiply-add per element,
// so the kernel runs at the rate the array can be read.  An element that changes changes the sum (an odd
// multiplier times a non-zero 32-bit difference is never 0 mod 2^64); elements that move change it unless
// their multipliers collide.  A sum, so that blocks can add their shares in any order (integer atomics).
__device__ __forceinline__ unsigned long long checksum_term(uint32_t v, unsigned long long pos) {
  uint32_t k = static_cast<uint32_t>(pos) * 0x9E3779B1u + static_cast<uint32_t>(pos >> 32) * 0x85EBCA77u;
  k ^= k >> 15;
  k *= 0x2C1B3C6Du;
  k ^= k >> 12;
  return static_cast<unsigned long long>(v + 0x632BE5ABu) * (k | 1u);
}

__global__ __launch_bounds__(256) void fingerprint_kernel(unsigned long long *__restrict__ out,
                                                          const uint32_t *__restrict__ a, unsigned long long n,
                                                          unsigned long long salt) {
  unsigned long long acc = 0;
  const unsigned long long tid = static_cast<unsigned long long>(blockIdx.x) * blockDim.x + threadIdx.x;
  const unsigned long long stride = static_cast<unsigned long long>(gridDim.x) * blockDim.x;
  // elements before the first 16-byte boundary, then 16-byte loads, then the rest
  unsigned long long head = ((16 - (reinterpret_cast<uintptr_t>(a) & 15)) & 15) / 4;
  if (head > n) head = n;
  const unsigned long long quads = (n - head) / 4;
  const uint4 *body = reinterpret_cast<const uint4 *>(a + head);
  for (unsigned long long q = tid; q < quads; q += stride) {
    const uint4 v = body[q];
    const unsigned long long at = salt + head + 4 * q;
    acc += checksum_term(v.x, at) + checksum_term(v.y, at + 1) + checksum_term(v.z, at + 2) + checksum_term(v.w, at + 3);
  }
  if (tid < head) acc += checksum_term(a[tid], salt + tid);
  const unsigned long long tail0 = head + 4 * quads;
  if (tid < n - tail0) acc += checksum_term(a[tail0 + tid], salt + tail0 + tid);
#pragma unroll
  for (int m = kWave / 2; m >= 1; m >>= 1) acc += __shfl_xor(acc, m, kWave);
  // one atomic per block: thousands of atomics on one word would take longer than reading the array
  __shared__ unsigned long long wave_sum[256 / kWave];
  if ((threadIdx.x & (kWave - 1)) == 0) wave_sum[threadIdx.x / kWave] = acc;
  __syncthreads();
  if (threadIdx.x == 0) {
    unsigned long long total = 0;
    for (int k = 0; k < 256 / kWave; ++k) total += wave_sum[k];
    if (total) atomicAdd(out, total);
  }
}

}  // namespace
namespace {
std::atomic<long> g_trace_ranges{0};
}

const TraceApi *trace_api() {
  static const TraceApi *api = []() -> const TraceApi * {
    const char *e = getenv("NTS_TRACE_RANGES");
    if (!e || e[0] != '1') return nullptr;
    void *lib = dlopen("librocprofiler-sdk-roctx.so", RTLD_NOW | RTLD_GLOBAL);
    if (!lib) lib = dlopen("libroctx64.so", RTLD_NOW | RTLD_GLOBAL);
    if (!lib) return nullptr;
    static TraceApi found;
    found.push = reinterpret_cast<int (*)(const char *)>(dlsym(lib, "roctxRangePushA"));
    found.pop = reinterpret_cast<int (*)()>(dlsym(lib, "roctxRangePop"));
    return (found.push && found.pop) ? &found : nullptr;
  }();
  return api;
}

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_pool_mutex;
hipMemPool_t g_scratch_pool[kMaxDevices] = {};

hipError_t scratch_pool(hipMemPool_t *pool) {
  int dev = 0;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) return err;
  if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
  std::lock_guard<std::mutex> lock(g_pool_mutex);
  if (!g_scratch_pool[dev]) {
    hipMemPoolProps props = {};
    props.allocType = hipMemAllocationTypePinned;
    props.handleTypes = hipMemHandleTypeNone;
    props.location.type = hipMemLocationTypeDevice;
    props.location.id = dev;
    hipMemPool_t created = nullptr;
    err = hipMemPoolCreate(&created, &props);
    if (err != hipSuccess) return err;
    uint64_t keep = UINT64_MAX;  // never trim at synchronisation points
    err = hipMemPoolSetAttribute(created, hipMemPoolAttrReleaseThreshold, &keep);
    if (err != hipSuccess) {
      (void)hipMemPoolDestroy(created);
      return err;
    }
    g_scratch_pool[dev] = created;
  }
  *pool = g_scratch_pool[dev];
  return hipSuccess;
}
}  // namespace

namespace {
std::atomic<long> g_scratch_allocs{0};
}
long scratch_alloc_count() { return g_scratch_allocs.load(); }

hipError_t scratch_alloc(void **ptr, size_t bytes, hipStream_t stream) {
  g_scratch_allocs.fetch_add(1);
  hipMemPool_t pool = nullptr;
  if (scratch_pool(&pool) != hipSuccess) {
    (void)hipGetLastError();                   // a device without pool support: the device's default pool
    return hipMallocAsync(ptr, bytes, stream);
  }
  return hipMallocFromPoolAsync(ptr, bytes, pool, stream);
}

hipError_t scratch_free(void *ptr, hipStream_t stream) { return hipFreeAsync(ptr, stream); }

hipError_t scratch_trim() {
  int dev = 0;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) return err;
  if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
  std::lock_guard<std::mutex> lock(g_pool_mutex);
  return g_scratch_pool[dev] ? hipMemPoolTrimTo(g_scratch_pool[dev], 0) : hipSuccess;
}

void count_trace_range() { g_trace_ranges.fetch_add(1, std::memory_order_relaxed); }
long trace_ranges_emitted() { return g_trace_ranges.load(std::memory_order_relaxed); }

}  // namespace nts

using nts::fail;

extern "C" {

const char *nts_last_error(void) { return nts::g_last_error; }
long nts_trace_ranges_emitted(void) { return nts::trace_ranges_emitted(); }
long nts_scratch_alloc_count(void) { return nts::scratch_alloc_count(); }

int nts_scratch_trim(void) {
  hipError_t err = nts::scratch_trim();
  return err == hipSuccess ? NTS_OK : nts::fail_hip(err, "nts_scratch_trim");
}

int nts_abi_version(void) { return 1; }

int nts_malloc_device(void **ptr, size_t bytes) {
  if (!ptr) return fail(NTS_ERR_INVALID, "nts_malloc_device: null out-pointer");
  *ptr = nullptr;
  if (bytes == 0) return NTS_OK;
  NTS_HIP_TRY(hipMalloc(ptr, bytes));
  return NTS_OK;
}

int nts_free_device(void *ptr) {
  if (!ptr) return NTS_OK;
  NTS_HIP_TRY(hipFree(ptr));
  return NTS_OK;
}

int nts_malloc_device_async(void **ptr, size_t bytes, nts_stream_t stream) {
  if (!ptr) return fail(NTS_ERR_INVALID, "nts_malloc_device_async: null out-pointer");
  *ptr = nullptr;
  if (bytes == 0) return NTS_OK;
  NTS_HIP_TRY(hipMallocAsync(ptr, bytes, stream));
  return NTS_OK;
}

int nts_free_device_async(void *ptr, nts_stream_t stream) {
  if (!ptr) return NTS_OK;
  NTS_HIP_TRY(hipFreeAsync(ptr, stream));
  return NTS_OK;
}

int nts_malloc_pinned_mapped(void **host_ptr, size_t bytes) {
  if (!host_ptr) return fail(NTS_ERR_INVALID, "nts_malloc_pinned_mapped: null out-pointer");
  *host_ptr = nullptr;
  if (bytes == 0) return NTS_OK;
  NTS_HIP_TRY(hipHostMalloc(host_ptr, bytes, hipHostMallocMapped));
  return NTS_OK;
}

int nts_free_pinned(void *host_ptr) {
  if (!host_ptr) return NTS_OK;
  NTS_HIP_TRY(hipHostFree(host_ptr));
  return NTS_OK;
}

int nts_host_get_device_ptr(void **dev_ptr, void *host_ptr) {
  if (!dev_ptr || !host_ptr) return fail(NTS_ERR_INVALID, "nts_host_get_device_ptr: null pointer");
  NTS_HIP_TRY(hipHostGetDevicePointer(dev_ptr, host_ptr, 0));
  return NTS_OK;
}

int nts_memcpy_h2d(void *dst_dev, const void *src_host, size_t bytes, int sync) {
  if (bytes == 0) return NTS_OK;
  if (!dst_dev || !src_host) return fail(NTS_ERR_INVALID, "nts_memcpy_h2d: null pointer");
  NTS_HIP_TRY(hipMemcpy(dst_dev, src_host, bytes, hipMemcpyHostToDevice));
  if (sync) NTS_HIP_TRY(hipDeviceSynchronize());
  return NTS_OK;
}

int nts_memcpy_h2d_async(void *dst_dev, const void *src_host, size_t bytes, nts_stream_t stream) {
  if (bytes == 0) return NTS_OK;
  if (!dst_dev || !src_host) return fail(NTS_ERR_INVALID, "nts_memcpy_h2d_async: null pointer");
  NTS_HIP_TRY(hipMemcpyAsync(dst_dev, src_host, bytes, hipMemcpyHostToDevice, stream));
  return NTS_OK;
}

int nts_memcpy_d2h(void *dst_host, const void *src_dev, size_t bytes, int sync) {
  if (bytes == 0) return NTS_OK;
  if (!dst_host || !src_dev) return fail(NTS_ERR_INVALID, "nts_memcpy_d2h: null pointer");
  NTS_HIP_TRY(hipMemcpy(dst_host, src_dev, bytes, hipMemcpyDeviceToHost));
  if (sync) NTS_HIP_TRY(hipDeviceSynchronize());
  return NTS_OK;
}

int nts_memcpy_d2h_async(void *dst_host, const void *src_dev, size_t bytes, nts_stream_t stream) {
  if (bytes == 0) return NTS_OK;
  if (!dst_host || !src_dev) return fail(NTS_ERR_INVALID, "nts_memcpy_d2h_async: null pointer");
  NTS_HIP_TRY(hipMemcpyAsync(dst_host, src_dev, bytes, hipMemcpyDeviceToHost, stream));
  return NTS_OK;
}

int nts_memcpy_d2d_async(void *dst_dev, const void *src_dev, size_t bytes, nts_stream_t stream) {
  if (bytes == 0) return NTS_OK;
  if (!dst_dev || !src_dev) return fail(NTS_ERR_INVALID, "nts_memcpy_d2d_async: null pointer");
  NTS_HIP_TRY(hipMemcpyAsync(dst_dev, src_dev, bytes, hipMemcpyDeviceToDevice, stream));
  return NTS_OK;
}

int nts_memset_zero(void *dev_ptr, size_t bytes, nts_stream_t stream) {
  if (bytes == 0) return NTS_OK;
  if (!dev_ptr) return fail(NTS_ERR_INVALID, "nts_memset_zero: null pointer");
  unsigned char *p = static_cast<unsigned char *>(dev_ptr);
  size_t head = (16 - (reinterpret_cast<uintptr_t>(p) & 15)) & 15;
  if (head > bytes) head = bytes;
  const size_t body16 = (bytes - head) / 16;
  const size_t tail = bytes - head - body16 * 16;
  size_t blocks = (body16 + 255) / 256;
  if (blocks < 1) blocks = 1;
  if (blocks > 16384) blocks = 16384;
  hipLaunchKernelGGL(nts::fill_zero_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream, p, head,
                     body16, tail);
  NTS_LAUNCH_CHECK("fill_zero_kernel");
  return NTS_OK;
}

namespace {
// Enqueues the checksum kernels for (a, b) on `stream`, accumulating into the zeroed device word `word`.
int enqueue_fingerprint(unsigned long long *word, const uint32_t *a, uint64_t n_a, const uint32_t *b, uint64_t n_b,
                        hipStream_t stream) {
  if (int rc = nts_memset_zero(word, 16, stream)) return rc;
  const uint64_t lens[2] = {n_a, n_b};
  const uint32_t *arrays[2] = {a, b};
  for (int k = 0; k < 2; ++k) {
    if (!lens[k]) continue;
    const unsigned blocks = static_cast<unsigned>(std::min<uint64_t>((lens[k] / 4 + 255) / 256 + 1, 2048));
    hipLaunchKernelGGL(nts::fingerprint_kernel, dim3(blocks), dim3(256), 0, stream, word, arrays[k],
                       static_cast<unsigned long long>(lens[k]), k ? 0x5851F42D4C957F2Dull + n_a : 0ull);
    const hipError_t err = hipGetLastError();
    if (err != hipSuccess) return nts::fail_hip(err, "fingerprint_kernel");
  }
  return NTS_OK;
}
// lengths are part of the value, so that a prefix of an array does not collide with the array
inline uint64_t fingerprint_value(uint64_t sum, uint64_t n_a, uint64_t n_b) {
  return sum ^ (n_a * 0xD6E8FEB86659FD93ull) ^ (n_b * 0xA0761D6478BD642Full);
}
}  // namespace

int nts_fingerprint_u32(uint64_t *fingerprint, const uint32_t *a, uint64_t n_a, const uint32_t *b, uint64_t n_b,
                        nts_stream_t stream) {
  if (!fingerprint) return fail(NTS_ERR_INVALID, "nts_fingerprint_u32: null out-pointer");
  if ((n_a && !a) || (n_b && !b)) return fail(NTS_ERR_INVALID, "nts_fingerprint_u32: null array");
  unsigned long long *word = nullptr;
  NTS_HIP_TRY(nts::scratch_alloc(reinterpret_cast<void **>(&word), 16, stream));
  int rc = enqueue_fingerprint(word, a, n_a, b, n_b, stream);
  unsigned long long host = 0;
  if (rc == NTS_OK) {
    hipError_t err = hipMemcpyAsync(&host, word, sizeof(host), hipMemcpyDeviceToHost, stream);
    if (err == hipSuccess) err = hipStreamSynchronize(stream);
    if (err != hipSuccess) rc = nts::fail_hip(err, "nts_fingerprint_u32: read-back");
  }
  const hipError_t ferr = nts::scratch_free(word, stream);
  if (rc == NTS_OK && ferr != hipSuccess) rc = nts::fail_hip(ferr, "nts_fingerprint_u32: scratch_free");
  *fingerprint = fingerprint_value(host, n_a, n_b);
  return rc;
}

int nts_fingerprint_u32_async(uint64_t *pinned_sum, const uint32_t *a, uint64_t n_a, const uint32_t *b, uint64_t n_b,
                              nts_stream_t stream) {
  if (!pinned_sum) return fail(NTS_ERR_INVALID, "nts_fingerprint_u32_async: null out-pointer");
  if ((n_a && !a) || (n_b && !b)) return fail(NTS_ERR_INVALID, "nts_fingerprint_u32_async: null array");
  unsigned long long *word = nullptr;
  NTS_HIP_TRY(nts::scratch_alloc(reinterpret_cast<void **>(&word), 16, stream));
  int rc = enqueue_fingerprint(word, a, n_a, b, n_b, stream);
  if (rc == NTS_OK) {
    const hipError_t err = hipMemcpyAsync(pinned_sum, word, sizeof(uint64_t), hipMemcpyDeviceToHost, stream);
    if (err != hipSuccess) rc = nts::fail_hip(err, "nts_fingerprint_u32_async: read-back");
  }
  const hipError_t ferr = nts::scratch_free(word, stream);
  if (rc == NTS_OK && ferr != hipSuccess) rc = nts::fail_hip(ferr, "nts_fingerprint_u32_async: scratch_free");
  return rc;
}

uint64_t nts_fingerprint_finish(uint64_t sum, uint64_t n_a, uint64_t n_b) { return fingerprint_value(sum, n_a, n_b); }

int nts_stream_create(nts_stream_t *stream) {
  if (!stream) return fail(NTS_ERR_INVALID, "nts_stream_create: null out-pointer");
  NTS_HIP_TRY(hipStreamCreate(stream));
  return NTS_OK;
}

int nts_stream_destroy(nts_stream_t stream) {
  if (!stream) return NTS_OK;
  NTS_HIP_TRY(hipStreamDestroy(stream));
  return NTS_OK;
}

int nts_stream_sync(nts_stream_t stream) {
  NTS_HIP_TRY(hipStreamSynchronize(stream));
  return NTS_OK;
}

int nts_device_sync(void) {
  NTS_HIP_TRY(hipDeviceSynchronize());
  return NTS_OK;
}

int nts_event_create(nts_event_t *event) {
  if (!event) return fail(NTS_ERR_INVALID, "nts_event_create: null out-pointer");
  NTS_HIP_TRY(hipEventCreate(event));
  return NTS_OK;
}

int nts_event_destroy(nts_event_t event) {
  if (!event) return NTS_OK;
  NTS_HIP_TRY(hipEventDestroy(event));
  return NTS_OK;
}

int nts_event_record(nts_event_t event, nts_stream_t stream) {
  if (!event) return fail(NTS_ERR_INVALID, "nts_event_record: null event");
  NTS_HIP_TRY(hipEventRecord(event, stream));
  return NTS_OK;
}

int nts_stream_wait_event(nts_stream_t stream, nts_event_t event) {
  if (!event) return fail(NTS_ERR_INVALID, "nts_stream_wait_event: null event");
  NTS_HIP_TRY(hipStreamWaitEvent(stream, event, 0));
  return NTS_OK;
}

int nts_event_elapsed_ms(float *ms, nts_event_t start, nts_event_t stop) {
  if (!ms || !start || !stop) return fail(NTS_ERR_INVALID, "nts_event_elapsed_ms: null argument");
  NTS_HIP_TRY(hipEventSynchronize(stop));
  NTS_HIP_TRY(hipEventElapsedTime(ms, start, stop));
  return NTS_OK;
}

int nts_mem_info(size_t *free_bytes, size_t *total_bytes) {
  if (!free_bytes || !total_bytes) return fail(NTS_ERR_INVALID, "nts_mem_info: null pointer");
  NTS_HIP_TRY(hipMemGetInfo(free_bytes, total_bytes));
  return NTS_OK;
}

}  // extern "C"
