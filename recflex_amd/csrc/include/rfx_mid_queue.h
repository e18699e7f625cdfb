// The list on which a workgroup keeps bags that wait for a wavefront ("mid-size bags": beyond
// their schedule's reach, too small to be cut into parts for several workgroups).
//
// A wavefront whose team meets such a bag puts {feature, bag} here instead of summing it on the
// spot, and every wavefront of the workgroup takes bags from the list between its tiles:
// whichever wavefront is ahead sums them, and the four finish together.  (Summed on the spot, a
// wavefront that met several such bags -- each a chain of up to 32 dependent round trips -- fell
// 60-80 us behind the others of its workgroup in a 180 us kernel, and a workgroup's block-wide
// work waits for its last wavefront.)
//
// The list is filled once: CAP entries for the whole launch, no wrap-around; when it is full a
// bag is summed where it was met.
//   count    entries reserved so far (may run past CAP: those were not stored)
//   taken    entries handed out
//   walking  wavefronts of the workgroup that still have regular tiles (and may add entries):
//            one that has none left keeps taking bags until this is zero and the list is empty,
//            so that the last wavefront's finds are shared as well
//   e[i]     feature << 32 | bag, kEmpty until its producer has written it
//
//   producer:  reserve (count++), then store the entry               (push)
//   consumer:  claim (taken++ by compare and swap while taken < min(count, CAP)), then wait for
//              the entry, which its producer stores right after reserving                 (pop)
//   finishing: walking-- after the wavefront's last push; a wavefront that reads walking == 0
//              and then finds nothing to claim has seen every entry there will ever be
// Producers never wait for anything, so a consumer's wait is short and cannot lock up.
//
// The memory operations come from a policy type: on the device rfx::LdsMem (rfx_schedules.hip.h,
// workgroup-scope atomics on LDS, one lane acting for its wavefront), on the CPU std::atomic with
// one thread per wavefront (tests, under ThreadSanitizer).
#pragma once

#if defined(__HIPCC__)
#define RFX_QUEUE_FN __device__ __forceinline__
#else
#define RFX_QUEUE_FN inline
#endif

namespace rfx {

template <int CAP> struct MidQueue {
  static constexpr int kCap = CAP;
  static constexpr unsigned long long kEmpty = ~0ull;
  int count, taken, walking;
  unsigned long long e[CAP];
};

// One caller (for a wavefront: one lane); false: the list is full.
template <class Mem, int CAP>
RFX_QUEUE_FN bool mid_queue_push_one(MidQueue<CAP> *q, const int feat, const int bag) {
  const int i = Mem::fetch_add(&q->count, 1);
  if (i >= CAP) return false;
  Mem::store_entry(&q->e[i], (static_cast<unsigned long long>(static_cast<unsigned int>(feat)) << 32) |
                                 static_cast<unsigned int>(bag));
  return true;
}

// One caller; true: *entry is the caller's to sum.
template <class Mem, int CAP>
RFX_QUEUE_FN bool mid_queue_pop_one(MidQueue<CAP> *q, unsigned long long *entry) {
  int t = Mem::load(&q->taken);
  for (;;) {
    int c = Mem::load(&q->count);
    c = c < CAP ? c : CAP;
    if (t >= c) return false;
    if (Mem::compare_exchange(&q->taken, &t, t + 1)) break;      // t: the current value on failure
  }
  unsigned long long v;
  do {
    v = Mem::load_entry(&q->e[t]);
  } while (v == MidQueue<CAP>::kEmpty);
  *entry = v;
  return true;
}

// anything to take?  (a cheap look before a call of the routine that sums the bags)
template <class Mem, int CAP> RFX_QUEUE_FN bool mid_queue_pending(MidQueue<CAP> *q) {
  const int c = Mem::load(&q->count);
  const int t = Mem::load(&q->taken);
  return t < (c < CAP ? c : CAP);
}

// The caller has made its last push.
template <class Mem, int CAP> RFX_QUEUE_FN void mid_queue_walk_done_one(MidQueue<CAP> *q) {
  Mem::release_add(&q->walking, -1);
}

// true while somebody may still push (look at the list again after a false: what the last
// producer pushed before it finished is visible by then)
template <class Mem, int CAP> RFX_QUEUE_FN bool mid_queue_open(MidQueue<CAP> *q) {
  return Mem::acquire_load(&q->walking) > 0;
}

} // namespace rfx
