// Rates of the memory path of one GPU by working-set size, for reading the library's roofline figures
// against what the machine delivers (lib/nts_membw, no arguments):
//   read_sum    every wavefront streams the set with 16-byte loads (four in flight per lane), nothing
//               is written: sets inside the L2s, inside the Infinity Cache, and beyond both
//   gather_sum  every wavefront reads 512 rows of 602 floats picked by a hash from a table of the given
//               size with 4-byte lanes, ten loads per row and four rows in flight -- the access pattern
//               of the F = 602 aggregation without its arithmetic, indices or output
//   gather16    every lane reads 16-byte rows picked by a hash from a table of the given size, eight in
//               flight per lane, either one row per lane (16-byte loads) or one row per four lanes (4-byte
//               loads) -- the el[src] reads of the fused attention kernels without anything else
// Prints GB/s per case.  A measuring tool: nothing in the library calls it.
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#include <vector>
#define CK(x) do{hipError_t e=(x); if(e!=hipSuccess){printf("%s: %s\n",#x,hipGetErrorString(e)); exit(1);} }while(0)
__global__ __launch_bounds__(256) void read_sum(const float4* __restrict__ p, size_t n, float* out, int passes) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  float4 a = make_float4(0,0,0,0), b = a, c = a, d = a;
  for (int pass = 0; pass < passes; ++pass) {  // small sets are read several times per launch, so that the launch itself does not count
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  for (; i + 3 * stride < n; i += 4 * stride) {
    float4 v0 = p[i], v1 = p[i + stride], v2 = p[i + 2 * stride], v3 = p[i + 3 * stride];
    a.x += v0.x; a.y += v0.y; a.z += v0.z; a.w += v0.w;
    b.x += v1.x; b.y += v1.y; b.z += v1.z; b.w += v1.w;
    c.x += v2.x; c.y += v2.y; c.z += v2.z; c.w += v2.w;
    d.x += v3.x; d.y += v3.y; d.z += v3.z; d.w += v3.w;
  }
  for (; i < n; i += stride) { float4 v = p[i]; a.x += v.x; a.y += v.y; a.z += v.z; a.w += v.w; }
  }
  float s = a.x + a.y + a.z + a.w + b.x + b.y + b.z + b.w + c.x + c.y + c.z + c.w + d.x + d.y + d.z + d.w;
  if (s == 12345.678f) out[0] = s;
}
// random row gather: each wave reads `rows_per_wave` rows of row_floats floats picked by a hash from a table of n_rows rows
__global__ __launch_bounds__(256) void gather_sum(const float* __restrict__ p, uint32_t n_rows, uint32_t row_floats, uint32_t rows_per_wave, float* out) {
  const uint32_t lane = threadIdx.x & 63, wave = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
  float acc[10]; for (int k = 0; k < 10; ++k) acc[k] = 0.f;
  uint32_t state = wave * 2654435761u + 12345u;
  for (uint32_t r = 0; r < rows_per_wave; r += 4) {
    const float* src[4];
    for (int u = 0; u < 4; ++u) { state = state * 1664525u + 1013904223u; uint32_t row = __builtin_amdgcn_readfirstlane((uint32_t)(((uint64_t)(state >> 4) * n_rows) >> 28)); src[u] = p + (size_t)row * row_floats; }
    float v[4][10];
    for (int u = 0; u < 4; ++u) for (int k = 0; k < 10; ++k) { uint32_t c = lane + 64 * k; if (c >= row_floats) c = row_floats - 1; v[u][k] = src[u][c]; }
    for (int u = 0; u < 4; ++u) for (int k = 0; k < 10; ++k) acc[k] += v[u][k];
  }
  float s = 0; for (int k = 0; k < 10; ++k) s += acc[k];
  if (s == 12345.678f) out[0] = s;
}
// random 16-byte rows: QUAD = false: one row per lane; true: one row per four adjacent lanes, 4 bytes each
template <bool QUAD>
__global__ __launch_bounds__(256) void gather16(const float* __restrict__ p, uint32_t n_rows, uint32_t per_lane, float* out) {
  const uint32_t t = blockIdx.x * blockDim.x + threadIdx.x;
  uint32_t state = (QUAD ? t >> 2 : t) * 2654435761u + 12345u;
  float acc = 0.f;
  for (uint32_t r = 0; r < per_lane; r += 8) {
    uint32_t row[8];
    for (int u = 0; u < 8; ++u) { state = state * 1664525u + 1013904223u; row[u] = (uint32_t)(((uint64_t)(state >> 4) * n_rows) >> 28); }
    if (QUAD) {
      float v[8];
      for (int u = 0; u < 8; ++u) v[u] = p[(size_t)row[u] * 4 + (t & 3)];
      for (int u = 0; u < 8; ++u) acc += v[u];
    } else {
      float4 v[8];
      for (int u = 0; u < 8; ++u) v[u] = reinterpret_cast<const float4*>(p)[row[u]];
      for (int u = 0; u < 8; ++u) acc += v[u].x + v[u].y + v[u].z + v[u].w;
    }
  }
  if (acc == 12345.678f) out[0] = acc;
}
int main() {
  float* out; CK(hipMalloc(&out, 256));
  size_t sizes[] = {2ull<<20, 8ull<<20, 24ull<<20, 64ull<<20, 128ull<<20, 200ull<<20, 512ull<<20, 2048ull<<20, 8192ull<<20};
  hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
  for (size_t bytes : sizes) {
    float4* p; CK(hipMalloc(&p, bytes)); CK(hipMemset(p, 0, bytes));
    const size_t n = bytes / 16;
    for (int blocks : {2048, 8192}) {
      int passes = (int)((512ull << 20) / bytes); if (passes < 1) passes = 1;
      int reps = (int)((8ull << 30) / (bytes * passes)); if (reps < 3) reps = 3;
      for (int w = 0; w < 2; ++w) hipLaunchKernelGGL(read_sum, dim3(blocks), dim3(256), 0, 0, p, n, out, passes);
      CK(hipEventRecord(e0));
      for (int r = 0; r < reps; ++r) hipLaunchKernelGGL(read_sum, dim3(blocks), dim3(256), 0, 0, p, n, out, passes);
      CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1));
      float ms; CK(hipEventElapsedTime(&ms, e0, e1));
      printf("read_sum  set %7.0f MiB blocks %5d: %8.1f GB/s (%.3f ms per pass over the set)\n", bytes / 1048576.0, blocks, bytes * (double)reps * passes / ms / 1e6, ms / reps / passes);
      fflush(stdout);
    }
    CK(hipFree(p));
  }
  // random gathers of 602-float rows from tables of different sizes: 114.8M/32 rows per launch equivalent
  const uint32_t F = 602;
  for (uint32_t n_rows : {1024u, 1700u, 7280u, 29120u, 100000u, 232965u}) {
    float* p; size_t bytes = (size_t)n_rows * F * 4; CK(hipMalloc(&p, bytes)); CK(hipMemset(p, 0, bytes));
    const uint32_t waves = 256 * 16 * 8, rpw = 512;  // 16.8 M row reads = 40 GB
    for (int w = 0; w < 1; ++w) hipLaunchKernelGGL(gather_sum, dim3(waves / 4), dim3(256), 0, 0, p, n_rows, F, rpw, out);
    CK(hipEventRecord(e0));
    for (int r = 0; r < 3; ++r) hipLaunchKernelGGL(gather_sum, dim3(waves / 4), dim3(256), 0, 0, p, n_rows, F, rpw, out);
    CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1));
    float ms; CK(hipEventElapsedTime(&ms, e0, e1));
    double gb = (double)waves * rpw * F * 4 / 1e9;
    printf("gather_sum table %6u rows (%7.1f MiB): %8.1f GB/s (%.3f ms per %.1f GB)\n", n_rows, bytes / 1048576.0, gb * 3 / ms * 1e3, ms / 3, gb);
    fflush(stdout);
    CK(hipFree(p));
  }
  // random gathers of 16-byte rows (2.449 M rows = the el table of a Products-shaped graph with four heads)
  for (uint32_t n_rows : {65536u, 262144u, 2449029u, 16777216u, 134217728u}) {
    float* p; size_t bytes = (size_t)n_rows * 16; CK(hipMalloc(&p, bytes)); CK(hipMemset(p, 0, bytes));
    for (int quad = 0; quad < 2; ++quad) {
      const uint32_t lanes = 256 * 2048 * (quad ? 4 : 1), per_lane = 256;  // 134 M row reads per launch
      auto launch = [&] {
        if (quad) hipLaunchKernelGGL(gather16<true>, dim3(lanes / 256), dim3(256), 0, 0, p, n_rows, per_lane, out);
        else hipLaunchKernelGGL(gather16<false>, dim3(lanes / 256), dim3(256), 0, 0, p, n_rows, per_lane, out);
      };
      launch();
      CK(hipEventRecord(e0));
      for (int r = 0; r < 3; ++r) launch();
      CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1));
      float ms; CK(hipEventElapsedTime(&ms, e0, e1));
      const double rows = 256.0 * 2048 * per_lane;
      printf("gather16 table %9u rows (%7.1f MiB) %s: %7.1f G rows/s = %7.1f GB/s of rows (%.3f ms per %.0f M rows)\n", n_rows,
             bytes / 1048576.0, quad ? "4-byte lanes, 4 per row" : "16-byte lanes, 1 per row", rows * 3 / ms / 1e6,
             rows * 16 * 3 / ms / 1e6, ms / 3, rows / 1e6);
      fflush(stdout);
    }
    CK(hipFree(p));
  }
  return 0;
}
