// Long bags taken out of the teams' hands (optional part of the fused embedding kernel, for data
// whose bag lengths are skewed).
//
// A bag far longer than its feature's schedule was chosen for keeps one team -- at best one
// wavefront (rfx::wave_bag) -- busy long after the rest of the grid has finished, and the
// wavefront that meets it in the middle of its tiles falls behind the others of its workgroup.
// A library emitted with outliers=True deals with such bags at two levels.
//   * Outliers: find_outliers, launched ahead of the fused kernel, walks all offsets of the
//     batch, and every bag longer than its feature's outlier threshold (beyond its schedule's
//     reach, rfx::long_bag_threshold, and at least 128 KiB of traffic) becomes an entry
//     {feature, bag, first part, parts} of a list in the caller's workspace, parts = its
//     traffic / kOutlierUnit (1..kOutlierMaxParts; 128, 256 and 512 KiB per part give 227, 219
//     and 234 us on a 100-feature model with lognormal bag lengths).  The teams of the fused
//     kernel leave those bags alone.  When a workgroup has run its share of the regular tiles it
//     draws parts from a ticket counter until none is left, so that the workgroups whose
//     regular tiles were cheap take more of them (dealt out like the regular tiles, three parts
//     of 10-30 us to one workgroup and one to another, the same model spent a third of the
//     kernel in its tail: 224 us against 192 with the parts drawn).  A part runs like a part of
//     a split bag (rfx::split_part: the workgroup sums its share, partial sums in a slot,
//     arrival counter, the last one adds the slots in part order and writes the output).  If
//     the list overflows (more than CAP bags or 4 * CAP parts) the launch does without it.
//     The workgroup that finishes last puts the list header back to zero for the next launch.
//   * Mid-size bags (beyond the schedule's reach, below the outlier threshold) are summed by one
//     wavefront, but not necessarily the one that met them: it puts them on a list of its
//     workgroup in LDS (MidQueue), and every wavefront of the workgroup takes bags from that
//     list between its tiles, so that the four wavefronts of a workgroup finish together.
//
// Reference counterpart: the role of rbk::SparseSegmentReduce
// (examples/csrc/include/reduce_by_key_kernel.cuh), load balance under skewed bag lengths.
#pragma once
#include "rfx_binding.hip.h"

namespace rfx {

// The list holds CAP entries and 4 * CAP parts; the emitter sizes it by the model (4 096 entries
// up to 128 features, 16 384 beyond).
constexpr int kOutlierUnit = 256 * 1024;     // traffic of one part
constexpr int kOutlierMaxParts = 64;

struct OutlierHeader {
  unsigned long long pack;                   // entries << 32 | parts, both as reserved so far
  int finished;                              // workgroups of the fused kernel that are done
  int last_entries, last_parts;              // what the previous launch found (for the caller)
  int next_part;                             // ticket counter: the next part nobody has taken yet
  int pad[26];
};
struct OutlierEntry {
  int feat, bag, first, parts;
};

// MAXD: largest embedding dimension among the features that can have outliers, rounded up to 4
template <int MAXD, int CAP> struct OutlierSpace {
  static constexpr int kCap = CAP;           // entries
  static constexpr int kPartCap = 4 * CAP;   // parts of all entries together
  OutlierHeader hdr;
  OutlierEntry entries[kCap];
  int counters[kCap];                        // arrival counters, zero between launches
  int partmap[kPartCap];                     // part -> entry
  unsigned int slots[kPartCap][MAXD];        // partial sums
};

// One thread per (feature, bag); grid (x: bags, y: features), any size.
template <int F, typename Space>
__device__ __forceinline__ void
find_outliers(Space *__restrict__ sp, const IoView &io,
              const int *__restrict__ long_thr, const int *__restrict__ lookup_bytes) {
  for (int f = blockIdx.y; f < F; f += gridDim.y) {
    const int thr = long_thr[f];
    if (thr <= 0) continue;                  // a schedule that handles long bags itself
    const int *offs = io.offsets(f);
    for (int b = blockIdx.x * blockDim.x + threadIdx.x; b < io.batch; b += gridDim.x * blockDim.x) {
      const int len = offs[b + 1] - offs[b];
      if (len <= thr) continue;
      const long long cost = static_cast<long long>(len) * lookup_bytes[f];
      long long want = (cost + kOutlierUnit - 1) / kOutlierUnit;
      const int parts = want < 1 ? 1 : (want > kOutlierMaxParts ? kOutlierMaxParts : static_cast<int>(want));
      const unsigned long long old =
          atomicAdd(&sp->hdr.pack, (1ull << 32) | static_cast<unsigned long long>(parts));
      const long long q = static_cast<long long>(old >> 32);
      const long long first = static_cast<long long>(old & 0xffffffffull);
      if (q < Space::kCap && first + parts <= Space::kPartCap) {
        sp->entries[q] = OutlierEntry{f, b, static_cast<int>(first), parts};
        for (int p = 0; p < parts; ++p) sp->partmap[first + p] = static_cast<int>(q);
      }
    }
  }
}

// What the fused kernel reads when it starts: the number of outlier parts to draw, 0 if
// there are none or the list overflowed (then the teams sum every bag themselves).
template <typename Space>
__device__ __forceinline__ int outlier_parts(const Space *sp) {
  const unsigned long long pack =
      __hip_atomic_load(&sp->hdr.pack, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  const unsigned long long entries = pack >> 32, parts = pack & 0xffffffffull;
  return entries <= Space::kCap && parts <= Space::kPartCap ? static_cast<int>(parts) : 0;
}

// The next outlier part for the calling workgroup (one thread draws); at or beyond
// the number of parts when all are taken.
template <typename Space> __device__ __forceinline__ int draw_outlier_part(Space *sp) {
  return __hip_atomic_fetch_add(&sp->hdr.next_part, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Called by every workgroup of the fused kernel when it has run out of tiles (by one thread):
// the last one clears the header for the next launch.
template <typename Space> __device__ __forceinline__ void outliers_done(Space *sp) {
  const int done = __hip_atomic_fetch_add(&sp->hdr.finished, 1, __ATOMIC_RELAXED,
                                          __HIP_MEMORY_SCOPE_AGENT);
  if (done == static_cast<int>(gridDim.x) - 1) {
    const unsigned long long pack =
        __hip_atomic_load(&sp->hdr.pack, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    sp->hdr.last_entries = static_cast<int>(pack >> 32);
    sp->hdr.last_parts = static_cast<int>(pack & 0xffffffffull);
    __hip_atomic_store(&sp->hdr.finished, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(&sp->hdr.next_part, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(&sp->hdr.pack, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

// ---------------------------------------------------------------------------------------------
// The drawn end of the tile walk (emit option drawn_tail = N): the last N passes of a workgroup
// over the tile space are not dealt out by the stride; the workgroups of an XCD draw them from a
// ticket counter of that XCD (one cache line each), so that a workgroup whose tiles were cheap
// takes over from one whose tiles were dear.  It pays together with a tile order that puts the
// cheap tiles last (a model of a thousand small features, five tiles per workgroup: 70.2 ->
// 67.8 us; alone, or on a model of 100 features with ten tiles per workgroup, nothing).  One
// thread draws, the next ticket is requested before the current tile runs, the workgroup agrees
// through LDS; the last workgroup to finish puts the counters back to zero.
// ---------------------------------------------------------------------------------------------
struct TailTickets {
  int next[8][32];                           // per XCD, each on a cache line of its own
  int finished;                              // workgroups that are done
  int pad[31];
};

__device__ __forceinline__ int draw_tail_ticket(TailTickets *t, const int xcd) {
  return __hip_atomic_fetch_add(&t->next[xcd][0], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// by one thread of every workgroup when it has drawn its last ticket
__device__ __forceinline__ void tail_tickets_done(TailTickets *t) {
  const int done = __hip_atomic_fetch_add(&t->finished, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  if (done == static_cast<int>(gridDim.x) - 1) {
    for (int x = 0; x < 8; ++x)
      __hip_atomic_store(&t->next[x][0], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(&t->finished, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

} // namespace rfx
