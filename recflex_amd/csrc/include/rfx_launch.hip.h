// Host-side launch helpers shared by every generated librecom.so: occupancy query, the
// dynamic-LDS pad that pins the number of resident workgroups per CU, and the per-device cache
// of both.
//
// Reference counterparts: get_max_concurrent_blocks / get_dyn_smem_size
// (RecFlex/sched_basic_csrc/include/utils.cuh:6-58).  HIP has no
// cudaOccupancyAvailableDynamicSMemPerBlock, so the pad is computed from the LDS size of a CU:
// a little more than 1/(occupancy + 1) of it per workgroup.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <mutex>
#include <stdint.h>

namespace rfx {

struct LaunchState {
  bool ready = false;
  int cus = 0;            // compute units of the device
  int occupancy = 0;      // workgroups per CU the persistent grid is sized for
  int dyn_lds = 0;        // dynamic LDS pad per workgroup (bytes)
  int natural_occupancy = 0;  // workgroups per CU the kernel's registers and static LDS allow
  int api_occupancy = 0;  // hipOccupancyMaxActiveBlocksPerMultiprocessor without a pad
  int num_vgprs = 0;      // vector registers per lane of the kernel
  int static_lds = 0;     // static LDS of the kernel (bytes)
  int lds_per_cu = 0;     // LDS of one compute unit (bytes)
  int padded_api_occupancy = 0;  // the occupancy API's answer with the pad
};

// gfx950: 4 SIMDs per CU, 512 vector registers per lane and SIMD (allocated in blocks of 8),
// at most 8 wavefronts per SIMD
constexpr int kVgprsPerSimd = 512;
constexpr int kVgprGranule = 8;
constexpr int kMaxWavesPerSimd = 8;
constexpr int kSimdsPerCu = 4;

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

  int occ_api = 0;
  e = occupancy_of(kernel, block_threads, 0, &occ_api);
  if (e != hipSuccess) return e;

  // Workgroups per CU the hardware can hold: register file and LDS, computed from the kernel's
  // own resource use.  (The occupancy API is kept as a cross-check only: it has been seen to
  // report half of what a 56-register kernel reaches on this device.)
  const int waves_per_wg = (block_threads + 63) / 64;
  const int vgprs = attr.numRegs > 0 ? (attr.numRegs + kVgprGranule - 1) / kVgprGranule * kVgprGranule
                                     : kVgprGranule;
  int waves_per_simd = kVgprsPerSimd / vgprs;
  if (waves_per_simd > kMaxWavesPerSimd) waves_per_simd = kMaxWavesPerSimd;
  int occ_regs = waves_per_simd * kSimdsPerCu / waves_per_wg;
  const int static_lds = static_cast<int>(attr.sharedSizeBytes);
  int occ_lds = static_lds > 0 ? lds_cu / static_lds : kMaxWavesPerSimd * kSimdsPerCu;
  int natural = occ_regs < occ_lds ? occ_regs : occ_lds;
  if (natural < 1) natural = 1;

  st->cus = cus;
  st->api_occupancy = occ_api;
  st->natural_occupancy = natural;
  st->num_vgprs = attr.numRegs;
  st->static_lds = static_lds;
  st->lds_per_cu = lds_cu;
  st->occupancy = natural;
  st->dyn_lds = 0;

  if (want_occupancy > 0 && natural > want_occupancy) {
    // smallest pad (in 512-byte steps) with which want_occupancy + 1 workgroups no longer fit
    // into the LDS of a CU
    int64_t dyn = lds_cu / (want_occupancy + 1) + 1 - static_lds;
    if (dyn < 0) dyn = 0;
    dyn = (dyn + 511) / 512 * 512;
    const int64_t dyn_max = static_cast<int64_t>(lds_cu) - static_lds;
    if (dyn > dyn_max) dyn = dyn_max;
    if (dyn > attr.maxDynamicSharedSizeBytes) {
      e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                              hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(dyn));
      if (e != hipSuccess) return e;
    }
    st->occupancy = want_occupancy;
    st->dyn_lds = static_cast<int>(dyn);
  }
  st->padded_api_occupancy = occ_api;
  if (st->dyn_lds > 0) {
    e = occupancy_of(kernel, block_threads, static_cast<size_t>(st->dyn_lds), &st->padded_api_occupancy);
    if (e != hipSuccess) return e;
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
