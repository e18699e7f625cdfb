// The arrival protocol by which several workgroups ("parts") of one bag combine their partial
// sums without waiting for each other (split bags, outlier tiles):
//
//   every part:   store its D partial sums to its slot        (Mem::store_slot)
//                 make them visible before it announces       (Mem::release)
//                 add 1 to the bag's arrival counter          (Mem::arrive -> the old value)
//   the part that read parts - 1 (the last to arrive, whoever that is):
//                 load all slots, add them in part order      (Mem::load_slot)
//                 put the counter back to zero                (Mem::reset)
//
// The memory operations come from a policy type, so that the very same steps run on the device
// (rfx::DeviceMem in rfx_schedules.hip.h: device-scope atomic stores and loads, the memory
// counter drained as the release, a relaxed device-scope add whose returned value every slot load
// depends on as the acquire) and on the CPU (tests: plain stores and loads around a
// release/acquire counter, one thread per part, under ThreadSanitizer -- which reports a data
// race the moment a step is moved out of this order).
//
// Reference counterpart: task_sync (RecFlex/sched_basic_csrc/include/task_sync.cuh:4-50), whose
// blocks spin on the counter until all have arrived; here nobody waits.
#pragma once

#if defined(__HIPCC__)
#define RFX_ARRIVAL_FN __device__ __forceinline__
#else
#define RFX_ARRIVAL_FN inline
#endif

namespace rfx {

// This part's value of column j.  Mem::store_slot must be the only kind of store a slot ever sees.
template <class Mem>
RFX_ARRIVAL_FN void arrival_store(unsigned int *slots, const int part, const int slot_stride,
                                  const int j, const float v) {
  Mem::store_slot(slots + static_cast<long long>(part) * slot_stride + j, v);
}

// After every store of this part has been released (and, in a workgroup, after the barrier that
// puts all its lanes' stores before this call): true for exactly one of the bag's parts, the one
// that may now read all slots.
template <class Mem> RFX_ARRIVAL_FN bool arrival_is_last(int *counter, const int parts) {
  return Mem::arrive(counter) == parts - 1;
}

// Column j of the bag: the parts' values added in part order, whoever arrived last.  The slot
// loads are issued eight at a time and only then added: one after the other, each a round trip to
// the device's coherence point, they made the last arrival of every bag the tail of the kernel.
template <class Mem>
RFX_ARRIVAL_FN float arrival_combine(const unsigned int *slots, const int parts,
                                     const int slot_stride, const int j) {
  constexpr int kBurst = 8;
  float t = 0.f;
  int p = 0;
  for (; p + kBurst <= parts; p += kBurst) {
    float v[kBurst];
#pragma unroll
    for (int k = 0; k < kBurst; ++k)
      v[k] = Mem::load_slot(slots + static_cast<long long>(p + k) * slot_stride + j);
#pragma unroll
    for (int k = 0; k < kBurst; ++k) t += v[k];
  }
  for (; p < parts; ++p) t += Mem::load_slot(slots + static_cast<long long>(p) * slot_stride + j);
  return t;
}

} // namespace rfx
