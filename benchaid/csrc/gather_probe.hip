// Gather probe: reads exactly the table rows a batch looks up -- same tables, same index
// streams, 16-byte loads -- and does nothing else (no bags, no sums, no output).  Its run time is
// the floor the memory system sets for any kernel that has to fetch those rows, hot rows served
// by the caches included; bench.py reports the fused kernel's time beside it.  On request it
// also writes as many bytes as the pooled output has, in the friendliest way there is (each
// wavefront stores a contiguous run of whole cache lines after each chunk of lookups): the
// floor for fetching the rows and writing an output of that size.
//
// No counterpart in the reference.  Measurement aid only: the product path never calls it.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));

// a run of consecutive lookups of one feature
struct Chunk {
  int32_t feat;
  int32_t begin;   // first position in the feature's index array
  int32_t count;
  int32_t log2x;   // lanes per row = 1 << log2x (a power of two >= 16-byte vectors per row, <= 64)
};

template <typename T> __device__ __forceinline__ const T *global_ptr(int64_t addr) {
  typedef const T __attribute__((address_space(1))) * gptr_t;
  return (const T *)reinterpret_cast<gptr_t>(addr);
}

constexpr int kXcds = 8;

// U row loads in flight per lane.  The chunk space (feature-ordered) is cut into 8 * segments
// equal parts, part s belongs to the workgroups of XCD s % 8 (workgroup i runs on XCD i % 8), as
// in the fused kernel's tile walk; segments == 0: workgroup i takes chunks 4i.., stride 4 * grid.
template <int U>
__global__ void __launch_bounds__(256)
gather_probe_knl(const Chunk *__restrict__ chunks, const int n_chunks, const int segments,
                 const int64_t *__restrict__ table_ptrs, const int64_t *__restrict__ index_ptrs,
                 const int32_t *__restrict__ row_strides, const int32_t *__restrict__ row_vectors,
                 float *__restrict__ sink, f32x4 *__restrict__ out, const int64_t out_f4) {
  const int lane = threadIdx.x & 63;
  const int wave_in_wg = threadIdx.x >> 6;
  const int groups = (n_chunks + 3) / 4;              // a workgroup takes four chunks at a time
  int first = blockIdx.x, last = groups, step = gridDim.x;
  int xcd = 0, seg_len = 1;
  const bool by_xcd = segments > 0 && gridDim.x % kXcds == 0;
  if (by_xcd) {
    seg_len = (groups + kXcds * segments - 1) / (kXcds * segments);
    xcd = blockIdx.x % kXcds;
    first = blockIdx.x / kXcds;
    last = seg_len * segments;
    step = gridDim.x / kXcds;
  }
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  for (int walk = first; walk < last; walk += step) {
    int group = walk;
    if (by_xcd) {
      const int seg = walk / seg_len;
      group = (seg * kXcds + xcd) * seg_len + (walk - seg * seg_len);
    }
    const int c = group * 4 + wave_in_wg;
    if (group >= groups || c >= n_chunks) continue;
    const Chunk ch = chunks[c];
    const char *table = global_ptr<char>(table_ptrs[ch.feat]);
    const int *idx = global_ptr<int>(index_ptrs[ch.feat]) + ch.begin;
    const int64_t stride = row_strides[ch.feat];
    const int vecs = row_vectors[ch.feat];
    const int x = lane & ((1 << ch.log2x) - 1);   // vector of the row this lane reads first
    const int row_in_instr = lane >> ch.log2x;
    const int rows_per_instr = 64 >> ch.log2x;
    for (int base = 0; base < ch.count; base += rows_per_instr * U) {
      int ids[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int p = base + u * rows_per_instr + row_in_instr;
        ids[u] = p < ch.count ? idx[p] : -1;
      }
      for (int v = x; v < vecs; v += 64) {     // rows wider than 64 vectors take several passes
        f32x4 buf[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          buf[u] = f32x4{0.f, 0.f, 0.f, 0.f};
          if (ids[u] >= 0)
            buf[u] = *reinterpret_cast<const f32x4 *>(table + ids[u] * stride + v * 16);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) acc += buf[u];
      }
    }
    if (out_f4 > 0) {
      // this chunk's share of the output-sized buffer
      const int64_t per = (out_f4 + n_chunks - 1) / n_chunks;
      const int64_t lo = c * per;
      const int64_t hi = lo + per < out_f4 ? lo + per : out_f4;
      for (int64_t i = lo + lane; i < hi; i += 64) __builtin_nontemporal_store(acc, out + i);
    }
  }
  // keeps the loads alive; never true for finite table values
  if (acc.x + acc.y + acc.z + acc.w == 1.2345e38f) sink[threadIdx.x] = acc.x;
}

// Plain copy of n 16-byte vectors, grid-stride.  Its HBM traffic is known (n * 16 bytes read,
// n * 16 written), so a counter run that holds one launch of it yields the bytes one unit of a
// memory counter stands for.  The name is unique on purpose: a counter file is searched for it.
__global__ void __launch_bounds__(256)
CalibrationCopyKnl(const f32x4 *__restrict__ src, f32x4 *__restrict__ dst, const int64_t n) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += stride)
    dst[i] = src[i];
}

} // namespace

// Copies `bytes` (a multiple of 16; both pointers 16-byte aligned, buffers disjoint) from src to
// dst on `stream` with CalibrationCopyKnl.  Returns the hipError_t of the launch.
extern "C" int calibration_copy_launch(const void *src, void *dst, int64_t bytes, int grid_blocks,
                                       void *stream) {
  if (!src || !dst || bytes < 0 || bytes % 16 != 0 || grid_blocks <= 0 ||
      reinterpret_cast<uintptr_t>(src) % 16 != 0 || reinterpret_cast<uintptr_t>(dst) % 16 != 0)
    return static_cast<int>(hipErrorInvalidValue);
  if (bytes == 0) return 0;
  hipLaunchKernelGGL(CalibrationCopyKnl, dim3(grid_blocks), dim3(256), 0,
                     static_cast<hipStream_t>(stream), static_cast<const f32x4 *>(src),
                     static_cast<f32x4 *>(dst), bytes / 16);
  return static_cast<int>(hipGetLastError());
}

// Launches the probe on `stream` (asynchronous).  chunks: device array of n_chunks records
// {int32 feat, begin, count, log2x}; table_ptrs / index_ptrs: device int64[F]; row_strides /
// row_vectors: device int32[F] (bytes between rows, 16-byte vectors per row); sink: device
// float[256]; in_flight: 2, 4 or 8 row loads per lane; segments: chunk-space segments per XCD
// (0 = flat); out / out_bytes: device buffer (16-byte aligned) that is written once, spread over
// the chunks, or NULL / 0 for the bare gather.  Returns the hipError_t of the launch.
extern "C" int gather_probe_launch(const void *chunks, int n_chunks, const int64_t *table_ptrs,
                                   const int64_t *index_ptrs, const int32_t *row_strides,
                                   const int32_t *row_vectors, float *sink, int grid_blocks,
                                   int in_flight, int segments, void *stream, void *out,
                                   int64_t out_bytes) {
  if (!chunks || !table_ptrs || !index_ptrs || !row_strides || !row_vectors || !sink ||
      n_chunks < 0 || grid_blocks <= 0 || segments < 0)
    return static_cast<int>(hipErrorInvalidValue);
  if ((out_bytes > 0 && !out) || out_bytes < 0 || reinterpret_cast<uintptr_t>(out) % 16 != 0)
    return static_cast<int>(hipErrorInvalidValue);
  if (n_chunks == 0) return 0;
  f32x4 *out4 = static_cast<f32x4 *>(out);
  const int64_t out_f4 = out_bytes / 16;
  const dim3 grid(grid_blocks), block(256);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const Chunk *ch = static_cast<const Chunk *>(chunks);
  switch (in_flight) {
  case 2:
    hipLaunchKernelGGL(gather_probe_knl<2>, grid, block, 0, s, ch, n_chunks, segments, table_ptrs,
                       index_ptrs, row_strides, row_vectors, sink, out4, out_f4);
    break;
  case 4:
    hipLaunchKernelGGL(gather_probe_knl<4>, grid, block, 0, s, ch, n_chunks, segments, table_ptrs,
                       index_ptrs, row_strides, row_vectors, sink, out4, out_f4);
    break;
  case 8:
    hipLaunchKernelGGL(gather_probe_knl<8>, grid, block, 0, s, ch, n_chunks, segments, table_ptrs,
                       index_ptrs, row_strides, row_vectors, sink, out4, out_f4);
    break;
  default:
    return static_cast<int>(hipErrorInvalidValue);
  }
  return static_cast<int>(hipGetLastError());
}
