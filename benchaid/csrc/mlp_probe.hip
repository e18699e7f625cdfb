// Memory-level-parallelism probe: rows at uniformly random addresses of a 4 GiB table, fetched
// with 16-byte vector loads and dropped.  Answers two questions about the device that the design
// of the fused embedding kernel rests on:
//   * is the rate of a gather without reuse bounded per compute unit (miss slots of its L1) or by
//     the memory side?  -- the grid sweep at the end: 1, 8, 32 ... 512 workgroups;
//   * can a wavefront get more misses in flight by also prefetching through the scalar data
//     cache (reads only)?
//       mode 0: plain vector loads
//       mode 1: + a scalar load of both 64-byte halves of every line of the next iteration
//       mode 2: + one scalar load per line of the next iteration
//       mode 3: + s_atc_probe of every line of the next iteration
// Measurement aid (python -m benchaid.mlp_probe); no counterpart in the reference, and the
// product path never runs it.
// Build: hipcc --offload-arch=gfx950 -O3 mlp_probe.hip -o mlp_probe
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <vector>
#include <algorithm>
#include <string>

#define CHECK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("HIP error %s at %s:%d\n", hipGetErrorString(e_), __FILE__, __LINE__); exit(1);} } while (0)

typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ void sprefetch(const char *p, unsigned &dummy) {
  asm volatile("s_load_dword %0, %1, 0x0" : "+s"(dummy) : "s"(p));
}
__device__ __forceinline__ void sprefetch2(const char *p, unsigned &dummy) {
  asm volatile("s_load_dword %0, %1, 0x0\n\ts_load_dword %0, %1, 0x40" : "+s"(dummy) : "s"(p));
}
__device__ __forceinline__ void sprobe(const char *p) {
  asm volatile("s_atc_probe 0, %0, 0x0" :: "s"(p));
}
__device__ __forceinline__ void swait(unsigned &dummy) {
  asm volatile("s_waitcnt lgkmcnt(0)" : "+s"(dummy));
}

// LPR = lanes per row (row bytes = LPR*16), U = loads in flight per lane
template <int MODE, int U, int LPR>
__global__ void __launch_bounds__(256)
gather(const char *__restrict__ table, const int *__restrict__ idx, const long long n_idx,
       const int per_wave, float *__restrict__ sink) {
  constexpr int RPI = 64 / LPR;            // rows per load instruction
  constexpr int ROWB = LPR * 16;
  const int lane = threadIdx.x & 63;
  const long long wave = (long long)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const long long beg = wave * per_wave;
  if (beg >= n_idx) return;
  const int *my = idx + beg;
  const int r = lane / LPR, x = lane % LPR;
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  unsigned dummy = 0;
  int cur[U];
#pragma unroll
  for (int u = 0; u < U; ++u) cur[u] = my[u * RPI + r];
  for (int base = 0; base < per_wave; base += U * RPI) {
    f32x4 buf[U];
#pragma unroll
    for (int u = 0; u < U; ++u)
      buf[u] = *reinterpret_cast<const f32x4 *>(table + (long long)cur[u] * ROWB + x * 16);
    int nxt[U];
    const int nb = base + U * RPI < per_wave ? base + U * RPI : base;
#pragma unroll
    for (int u = 0; u < U; ++u) nxt[u] = my[nb + u * RPI + r];
    if constexpr (MODE != 0) {
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int k = 0; k < RPI; ++k) {
          const int i = __builtin_amdgcn_readlane(nxt[u], k * LPR);
          const char *p = table + (long long)i * ROWB;
#pragma unroll
          for (int l = 0; l < ROWB; l += 128) {
            if constexpr (MODE == 1) sprefetch2(p + l, dummy);
            if constexpr (MODE == 2) sprefetch(p + l, dummy);
            if constexpr (MODE == 3) sprobe(p + l);
          }
          if constexpr (ROWB < 128 && MODE != 3) { /* one s_load covers the row */ }
        }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) acc += buf[u];
    if constexpr (MODE == 1 || MODE == 2) swait(dummy);
#pragma unroll
    for (int u = 0; u < U; ++u) cur[u] = nxt[u];
  }
  if (acc.x + acc.y + acc.z + acc.w + (float)dummy == 1.2345e38f) sink[threadIdx.x] = acc.x;
}

template <int MODE, int U, int LPR>
float run(const char *table, const int *idx, long long n_idx, int grid, float *sink, int reps) {
  const long long waves = (long long)grid * 4;
  int per_wave = (int)(n_idx / waves);
  per_wave = per_wave / (U * (64 / LPR)) * (U * (64 / LPR));
  hipEvent_t a, b;
  CHECK(hipEventCreate(&a)); CHECK(hipEventCreate(&b));
  std::vector<float> ts;
  for (int i = 0; i < reps + 2; ++i) {
    CHECK(hipEventRecord(a));
    gather<MODE, U, LPR><<<grid, 256>>>(table, idx, n_idx, per_wave, sink);
    CHECK(hipEventRecord(b));
    CHECK(hipEventSynchronize(b));
    float ms; CHECK(hipEventElapsedTime(&ms, a, b));
    if (i >= 2) ts.push_back(ms);
  }
  CHECK(hipGetLastError());
  std::sort(ts.begin(), ts.end());
  const float ms = ts[ts.size() / 2];
  const double bytes = (double)per_wave * waves * LPR * 16;
  printf("mode %d U %d rowbytes %4d grid %5d (%.2f wg/cu): %8.1f us  %7.1f GB/s  %6.2f Grows/s\n", MODE, U, LPR * 16,
         grid, grid / 256.0, ms * 1e3, bytes / ms / 1e6, (double)per_wave * waves / ms / 1e6);
  fflush(stdout);
  return ms;
}

int main(int argc, char **argv) {
  const long long table_bytes = 4LL << 30;
  const long long n_idx = 16LL << 20;
  char *table; int *idx; float *sink;
  CHECK(hipMalloc(&table, table_bytes));
  CHECK(hipMemset(table, 0, table_bytes));
  CHECK(hipMalloc(&idx, n_idx * 4));
  CHECK(hipMalloc(&sink, 1024));
  std::string dist = argc > 1 ? argv[1] : "uniform";
  // indices in units of 512-byte rows at most: keep below table_bytes / 512 rows so every row size fits
  const long long rows = table_bytes / 512;
  std::vector<int> h(n_idx);
  uint64_t s = 0x9E3779B97F4A7C15ull;
  for (long long i = 0; i < n_idx; ++i) {
    s ^= s << 13; s ^= s >> 7; s ^= s << 17;
    h[i] = (int)(s % (uint64_t)rows);
  }
  CHECK(hipMemcpy(idx, h.data(), n_idx * 4, hipMemcpyHostToDevice));
  printf("table %.1f GiB, %lld lookups, rows %lld (dist %s)\n", table_bytes / 1073741824.0, n_idx, rows, dist.c_str());
  const int reps = 5;
  // 1. chip-wide, 128-byte rows
  for (int grid : {1024, 2048}) {
    run<0, 4, 8>(table, idx, n_idx, grid, sink, reps);
    run<0, 8, 8>(table, idx, n_idx, grid, sink, reps);
    run<1, 4, 8>(table, idx, n_idx, grid, sink, reps);
    run<2, 4, 8>(table, idx, n_idx, grid, sink, reps);
    run<3, 4, 8>(table, idx, n_idx, grid, sink, reps);
    run<1, 2, 8>(table, idx, n_idx, grid, sink, reps);
    run<1, 8, 8>(table, idx, n_idx, grid, sink, reps);
  }
  // 2. 512-byte rows and 32-byte rows
  run<0, 4, 32>(table, idx, n_idx, 1024, sink, reps);
  run<1, 4, 32>(table, idx, n_idx, 1024, sink, reps);
  run<2, 4, 32>(table, idx, n_idx, 1024, sink, reps);
  run<0, 4, 2>(table, idx, n_idx, 1024, sink, reps);
  run<2, 4, 2>(table, idx, n_idx, 1024, sink, reps);
  // 3. is the limit per CU?  few workgroups (one per CU at most), small slice of the lookups
  for (int grid : {1, 8, 32, 64, 128, 256, 512}) {
    run<0, 8, 8>(table, idx, (long long)grid * 4 * 4096, grid, sink, reps);
    run<1, 4, 8>(table, idx, (long long)grid * 4 * 4096, grid, sink, reps);
  }
  return 0;
}
