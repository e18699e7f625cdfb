// Host-side launch helpers shared by every generated librecom.so: occupancy query, the
// dynamic-LDS pad that pins the number of resident workgroups per CU, and the per-device cache
// of both.
//
// Reference counterparts: get_max_concurrent_blocks / get_dyn_smem_size
// (RecFlex/sched_basic_csrc/include/utils.cuh:6-58).  HIP has no
// cudaOccupancyAvailableDynamicSMemPerBlock, so the pad is searched with
// hipOccupancyMaxActiveBlocksPerMultiprocessor starting from the LDS size of a CU divided by
// (occupancy + 1).
#pragma once
#include <hip/hip_runtime.h>
#include <mutex>
#include <stdint.h>

namespace rfx {

struct LaunchState {
  bool ready = false;
  int cus = 0;            // compute units of the device
  int occupancy = 0;      // resident workgroups per CU with dyn_lds bytes of dynamic LDS
  int dyn_lds = 0;        // dynamic LDS pad per workgroup (bytes)
  int natural_occupancy = 0;  // resident workgroups per CU without the pad
};

constexpr int kMaxDevices = 64;

template <typename K>
inline hipError_t occupancy_of(K kernel, int block_threads, size_t dyn_lds, int *out) {
  return hipOccupancyMaxActiveBlocksPerMultiprocessor(out, kernel, block_threads, dyn_lds);
}

// Fills `st` for the current device.  want_occupancy <= 0: take what the kernel reaches.
template <typename K>
inline hipError_t init_launch_state(K kernel, int block_threads, int want_occupancy,
                                    LaunchState *st) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  int cus = 0, lds_cu = 0;
  e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
  if (e != hipSuccess) return e;
  e = hipDeviceGetAttribute(&lds_cu, hipDeviceAttributeMaxSharedMemoryPerMultiprocessor, dev);
  if (e != hipSuccess) return e;
  hipFuncAttributes attr;
  e = hipFuncGetAttributes(&attr, reinterpret_cast<const void *>(kernel));
  if (e != hipSuccess) return e;

  int occ0 = 0;
  e = occupancy_of(kernel, block_threads, 0, &occ0);
  if (e != hipSuccess) return e;
  st->cus = cus;
  st->natural_occupancy = occ0;
  st->occupancy = occ0;
  st->dyn_lds = 0;

  if (want_occupancy > 0 && occ0 > want_occupancy) {
    // smallest pad (in 256-byte steps) with which want_occupancy + 1 workgroups no longer fit
    int64_t dyn = lds_cu / (want_occupancy + 1) + 1 - static_cast<int64_t>(attr.sharedSizeBytes);
    if (dyn < 0) dyn = 0;
    dyn = (dyn + 255) / 256 * 256;
    const int64_t dyn_max = static_cast<int64_t>(lds_cu) - static_cast<int64_t>(attr.sharedSizeBytes);
    for (;;) {
      if (dyn > dyn_max) dyn = dyn_max;
      if (dyn > attr.maxDynamicSharedSizeBytes) {
        e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(dyn));
        if (e != hipSuccess) return e;
      }
      int occ = 0;
      e = occupancy_of(kernel, block_threads, static_cast<size_t>(dyn), &occ);
      if (e != hipSuccess) return e;
      if (occ <= want_occupancy || dyn >= dyn_max) {
        if (occ >= 1) {
          st->occupancy = occ;
          st->dyn_lds = static_cast<int>(dyn);
        }
        break;
      }
      dyn += 1024;
    }
  }
  st->ready = true;
  return hipSuccess;
}

// One cache per generated library (the template is instantiated with that library's kernel).
template <typename K>
inline hipError_t get_launch_state(K kernel, int block_threads, int want_occupancy,
                                   const LaunchState **out) {
  static LaunchState states[kMaxDevices];
  static std::mutex mu;
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
  std::lock_guard<std::mutex> lock(mu);
  if (!states[dev].ready) {
    e = init_launch_state(kernel, block_threads, want_occupancy, &states[dev]);
    if (e != hipSuccess) return e;
  }
  *out = &states[dev];
  return hipSuccess;
}

} // namespace rfx
