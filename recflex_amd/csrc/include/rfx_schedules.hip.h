// The per-feature schedule bodies of the fused embedding kernel, written for 64-lane
// wavefronts: every bag (one sample's lookups of one feature) is summed by a "team" of
// T = X*Y lanes.  X lanes split the row into 16-byte vectors (column lanes), Y lanes split the
// bag's lookups (lookup lanes) and are combined by a DPP / ds_swizzle / permlane butterfly.
//
//   T == 1          thread-per-bag          (team_bags)
//   1 < T < 64      sub-wavefront-per-bag   (team_bags)
//   T == 64         wavefront-per-bag       (team_bags)
//   T == BT (256)   block-per-bag           (block_bags: indices staged in LDS, partial sums
//                                            of the 4 wavefronts combined through LDS)
//   T == parts*BT   several workgroups per bag (split_bags: block_bags on a share of the bag's
//                                            lookups, partial sums combined through a workspace
//                                            by the workgroup that finishes last)
//
// Reference counterparts: ws::SparseSegmentReduce
// (examples/csrc/include/warp_per_sample_kernel.cuh:10-82), obms::SparseSegmentReduce
// (examples/csrc/include/one_block_multi_sample_kernel.cuh:9-126) and onehot::GatherSegments
// (examples/csrc/include/onehot_kernel.cuh:14-87).  Semantics kept: sum pooling, empty bag ->
// zeros, output row-major [batch, EMBED_DIM_SUM] with this feature at column embed_dim_offset.
// Differences: 64-bit row addressing, tables may be fp32 / fp16 / int8 row-wise, the work unit
// is a range of bags [bag_begin, bag_end) chosen at run time, and U lookups x UB bags x VPP
// vectors are kept in flight per lane.
#pragma once
#include "rfx_arrival.h"
#include "rfx_mid_queue.h"
#include "rfx_binding.hip.h"
#include "rfx_crosslane.hip.h"
#include "rfx_rows.hip.h"

namespace rfx {

// LDS staging of a team's output.  A lane of an fp16 (int8) team ends a bag with 8 (16)
// consecutive output columns per row vector, i.e. 2 (4) float4 -- written straight from the
// registers, each store instruction would put 16 bytes every 32 (64) bytes, four partial writes
// per 128-byte line (measured: 3.6 TB/s against 4.9-6.1 TB/s for whole lines).  The team
// therefore passes the segment through LDS and stores it with consecutive float4 per lane.
// Every wavefront owns a fixed slice (the wavefronts of a workgroup drift apart and may be in
// tiles of different features at the same time); fp32 teams never touch it.
constexpr int kStageF4PerLane = 4;      // int8: 16 floats per lane and row vector
#ifndef RFX_STAGE_MIN_F4
#define RFX_STAGE_MIN_F4 2              // stage from this many float4 per lane and vector on
#endif
template <int BT> struct TeamStage {
  f32x4 seg[BT / 64][64 * kStageF4PerLane];
};

// threadIdx.x for a schedule body.  The fused kernel inlines some twenty bodies into one tile
// loop; given the plain thread index the compiler computes every body's lane decomposition (team,
// x, y and what follows from them) once before that loop and keeps all of it in registers
// throughout: 128 registers and a spill for the 100-feature model, against 94 when each body
// derives its values per tile.  The lane number therefore passes through an empty asm statement,
// which nothing can be moved across.  The wavefront number stays a scalar and both ranges stay
// visible to the compiler (the masks), which the straight-line paths of the bodies rely on.
template <int BT> __device__ __forceinline__ int body_thread_id() {
  static_assert(BT % 64 == 0 && ((BT / 64) & (BT / 64 - 1)) == 0, "1, 2, 4, 8 or 16 wavefronts");
  int lane = threadIdx.x & 63;
  asm volatile("" : "+v"(lane));
  return (__builtin_amdgcn_readfirstlane(threadIdx.x >> 6) & (BT / 64 - 1)) * 64 + (lane & 63);
}

// ---------------------------------------------------------------------------------------------
// The workgroup's list of mid-size bags (rfx_mid_queue.h) in LDS: workgroup-scope atomics, and
// one lane acting for its wavefront.
// ---------------------------------------------------------------------------------------------
struct LdsMem {
  static __device__ __forceinline__ int fetch_add(int *p, int v) {
    return __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  }
  static __device__ __forceinline__ int load(int *p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  }
  static __device__ __forceinline__ bool compare_exchange(int *p, int *expected, int desired) {
    return __hip_atomic_compare_exchange_strong(p, expected, desired, __ATOMIC_RELAXED,
                                                __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  }
  static __device__ __forceinline__ void store_entry(unsigned long long *p, unsigned long long v) {
    __hip_atomic_store(p, v, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
  }
  static __device__ __forceinline__ unsigned long long load_entry(unsigned long long *p) {
    return __hip_atomic_load(p, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP);
  }
  static __device__ __forceinline__ void release_add(int *p, int v) {
    __hip_atomic_fetch_add(p, v, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
  }
  static __device__ __forceinline__ int acquire_load(int *p) {
    return __hip_atomic_load(p, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP);
  }
};

constexpr int kMidQueueCap = 192;
using MidBagQueue = MidQueue<kMidQueueCap>;

// by all threads of the workgroup, before a barrier that precedes the first use
template <int BT> __device__ __forceinline__ void mid_queue_init(MidBagQueue *q) {
  for (int i = threadIdx.x; i < kMidQueueCap; i += BT) q->e[i] = MidBagQueue::kEmpty;
  if (threadIdx.x == 0) {
    q->count = 0;
    q->taken = 0;
    q->walking = BT / 64;
  }
}

// Called by a whole wavefront with uniform arguments; false: the list is full.
__device__ __forceinline__ bool mid_queue_push(MidBagQueue *q, const int feat, const int bag) {
  int ok = 0;
  if ((threadIdx.x & 63) == 0) ok = mid_queue_push_one<LdsMem>(q, feat, bag) ? 1 : 0;
  return __builtin_amdgcn_readfirstlane(ok) != 0;
}

// Called by a whole wavefront; true: {feat, bag} is the calling wavefront's to sum.
__device__ __forceinline__ bool mid_queue_pop(MidBagQueue *q, int *feat, int *bag) {
  unsigned int lo = 0, hi = 0;
  int got = 0;
  if ((threadIdx.x & 63) == 0) {
    unsigned long long v = 0;
    got = mid_queue_pop_one<LdsMem>(q, &v) ? 1 : 0;
    lo = static_cast<unsigned int>(v);
    hi = static_cast<unsigned int>(v >> 32);
  }
  if (!__builtin_amdgcn_readfirstlane(got)) return false;
  *bag = static_cast<int>(__builtin_amdgcn_readfirstlane(lo));
  *feat = static_cast<int>(__builtin_amdgcn_readfirstlane(hi));
  return true;
}

__device__ __forceinline__ bool mid_queue_pending(MidBagQueue *q) {
  return mid_queue_pending<LdsMem>(q);
}

// The calling wavefront has run its last regular tile.
__device__ __forceinline__ void mid_queue_walk_done(MidBagQueue *q) {
  if ((threadIdx.x & 63) == 0) mid_queue_walk_done_one<LdsMem>(q);
}

__device__ __forceinline__ bool mid_queue_open(MidBagQueue *q) { return mid_queue_open<LdsMem>(q); }

// ---------------------------------------------------------------------------------------------
// wave_bag: one bag summed by a whole wavefront, whatever the feature's schedule -- the way out
// for a bag far longer than its feature's schedule was chosen for.  A team of T lanes with U
// lookups in flight per lookup lane walks a bag of n lookups in n / (U*Y) dependent rounds of a
// memory round trip each: a single bag of 2 000 lookups among one-lookup bags (16 lanes per bag,
// one lookup in flight) held one wavefront for 1.2 ms in a kernel of 124 us, one of 20 000 for
// 10 ms.  Here all 64 lanes work on the bag: as many column lanes as the row has vectors (at
// most 64), the rest lookup lanes, four lookups in flight each (eight would push the
// 100-feature kernel, which inlines this into twenty bodies, over its 96 registers: 8 spills),
// indices fetched a round ahead, butterfly over the lookup lanes at the end.
// No LDS and no barrier: only the wavefront that met the bag is involved.
// ---------------------------------------------------------------------------------------------
// a bag of more lookups than this is an outlier for a team with U lookups in flight on each of
// Y lookup lanes: more than sixteen dependent rounds (at least 64 lookups)
__host__ __device__ constexpr int long_bag_threshold(int u, int y) {
  return 16 * u * y > 64 ? 16 * u * y : 64;
}

__host__ __device__ constexpr int pow2_at_least(int n) {
  int p = 1;
  while (p < n) p <<= 1;
  return p;
}

template <int DT, int D, int OVEC>
__device__ __forceinline__ void
wave_bag(const char *__restrict__ table, const int *__restrict__ indices, const int beg,
         const int end, float *__restrict__ dst, const int lane) {
  using R = Row<DT, D>;
  constexpr int XW = R::V >= 64 ? 64 : pow2_at_least(R::V);
  constexpr int YW = 64 / XW;
  constexpr int VPL = ceil_div(R::V, XW);
  constexpr int VB = R::VB;
  constexpr int EPV = R::EPV;
  constexpr int UW = 4;

  const int y = lane / XW;
  const int x = lane - y * XW;
  float acc[VPL][EPV];
  float bias_acc = 0.f;
#pragma unroll
  for (int v = 0; v < VPL; ++v)
#pragma unroll
    for (int e = 0; e < EPV; ++e) acc[v][e] = 0.f;

  int idx[UW];
#pragma unroll
  for (int u = 0; u < UW; ++u) {
    const int p = beg + u * YW + y;
    idx[u] = p < end ? indices[p] : -1;
  }
  for (int base = beg; base < end; base += UW * YW) {
    Vec<VB> buf[UW][VPL];
    f32x2 sb[UW];
#pragma unroll
    for (int u = 0; u < UW; ++u)
      if (idx[u] >= 0) {
        const char *row = table + static_cast<int64_t>(idx[u]) * R::STRIDE;
#pragma unroll
        for (int v = 0; v < VPL; ++v) {
          const int c = x + v * XW;
          if (c < R::V) buf[u][v] = load_vec<VB>(row + c * VB);
        }
        if constexpr (DT == I8) sb[u] = load_scale_bias<D>(row);
      }
    int nidx[UW];
#pragma unroll
    for (int u = 0; u < UW; ++u) {
      const int p = base + (UW + u) * YW + y;
      nidx[u] = p < end ? indices[p] : -1;
    }
#pragma unroll
    for (int u = 0; u < UW; ++u)
      if (idx[u] >= 0) {
#pragma unroll
        for (int v = 0; v < VPL; ++v) {
          const int c = x + v * XW;
          if (c < R::V) accumulate<DT, VB>(acc[v], buf[u][v], DT == I8 ? sb[u].x : 1.f);
        }
        if constexpr (DT == I8) bias_acc += sb[u].y;
      }
#pragma unroll
    for (int u = 0; u < UW; ++u) idx[u] = nidx[u];
  }
  if constexpr (XW < 64) {
    if constexpr (DT == I8) bias_acc = reduce_over_y<XW, 64>(bias_acc);
#pragma unroll
    for (int v = 0; v < VPL; ++v)
#pragma unroll
      for (int e = 0; e < EPV; ++e) acc[v][e] = reduce_over_y<XW, 64>(acc[v][e]);
  }
  if (y == 0) {
#pragma unroll
    for (int v = 0; v < VPL; ++v) {
      const int c = x + v * XW;
      if (c < R::V) {
        if constexpr (DT == I8) {
#pragma unroll
          for (int e = 0; e < EPV; ++e) acc[v][e] += bias_acc;
        }
        store_floats<EPV, OVEC>(dst + c * EPV, acc[v]);
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------
// team_bags: teams of T <= 64 lanes; a workgroup of BT threads holds BT/T teams; team t sums
// bags bag_begin + (t + k*TEAMS)*UB + [0, UB).
//   U   lookups of one bag in flight per lookup lane
//   UB  bags in flight per team (for short bags)
//   VPP row vectors per lane per pass (a lane owns ceil(V/X) vectors; if that exceeds VPP the
//       bag's index list is walked again for the next VPP vectors)
// A bag of more than kLong = max(64, 16*U*Y) lookups (teams of fewer than 64 lanes) is not
// walked by its team: the team's wavefront sums it with all its lanes first (wave_bag).
// ---------------------------------------------------------------------------------------------
template <int BT, int DT, int D, int X, int Y, int U, int UB, int VPP, int OVEC>
__device__ __forceinline__ void
team_bags(f32x4 *__restrict__ stage, const char *__restrict__ table,
          const int *__restrict__ indices,
          const int *__restrict__ offsets, float *__restrict__ out, const int esum,
          const int col_off, const int bag_begin, const int bag_end,
          const int skip_longer_than = 0x7fffffff, MidBagQueue *mid_queue = nullptr,
          const int feat = 0) {
  using R = Row<DT, D>;
  constexpr int T = X * Y;
  static_assert(T >= 1 && T <= 64 && (T & (T - 1)) == 0, "team must be a power of two <= 64");
  static_assert(BT % T == 0 && BT % 64 == 0, "workgroup must hold whole teams");
  constexpr int TEAMS = BT / T;
  constexpr int VPL = ceil_div(R::V, X);
  static_assert(VPP >= 1 && VPP <= VPL, "vectors per pass");
  constexpr int VB = R::VB;
  constexpr int EPV = R::EPV;

  const int tid = body_thread_id<BT>();
  const int team = tid / T;
  const int lt = tid - team * T;
  const int y = lt / X;
  const int x = lt - y * X;

  // Teams of fewer than 64 lanes: the wavefront stays together until its last team has run out
  // of bags (teams beyond bag_end see empty bags), because a long bag needs all of its lanes.
  auto more_bags = [&](const int bag0) {
    if constexpr (T < 64) return __builtin_amdgcn_ballot_w64(bag0 < bag_end) != 0;
    else return bag0 < bag_end;
  };
  for (int bag0 = bag_begin + team * UB; more_bags(bag0); bag0 += TEAMS * UB) {
    int beg[UB], end[UB];
    {
      int prev = offsets[bag0 < bag_end ? bag0 : bag_end];
#pragma unroll
      for (int i = 0; i < UB; ++i) {
        const int b = bag0 + i + 1;
        const int next = offsets[b < bag_end ? b : bag_end];
        beg[i] = prev;
        end[i] = (bag0 + i < bag_end) ? next : prev;
        prev = next;
      }
    }
    // bags far longer than this schedule suits: the whole wavefront sums them, one at a time;
    // their teams then see an empty bag and leave the output alone
    // (bags of more than skip_longer_than lookups were found ahead of the kernel and are summed
    // by several workgroups as tiles of their own, rfx::find_outliers; nobody touches them here)
    int done_mask = 0;
    constexpr int kLong = long_bag_threshold(U, Y);
    if constexpr (T < 64) {
#pragma unroll
      for (int i = 0; i < UB; ++i) {
        const bool skip = end[i] - beg[i] > skip_longer_than;
        const bool is_long = end[i] - beg[i] > kLong;
        unsigned long long pending = __builtin_amdgcn_ballot_w64(is_long && !skip && lt == 0);
        while (pending) {                         // the same in every lane of the wavefront
          const int src = __builtin_ctzll(pending);
          pending &= pending - 1;
          const int b = __builtin_amdgcn_readlane(bag0 + i, src);
          // left to whichever wavefront of the workgroup has time, if there is such a list
          if (mid_queue && mid_queue_push(mid_queue, feat, b)) continue;
          wave_bag<DT, D, OVEC>(table, indices, __builtin_amdgcn_readlane(beg[i], src),
                                __builtin_amdgcn_readlane(end[i], src),
                                out + static_cast<int64_t>(b) * esum + col_off, tid & 63);
        }
        if (is_long) {
          done_mask |= 1 << i;
          end[i] = beg[i];
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < UB; ++i) {
        const int len = end[i] - beg[i];
        // beyond this schedule's reach: another wavefront may have time for it sooner
        if (len > skip_longer_than ||
            (mid_queue && len > kLong && mid_queue_push(mid_queue, feat, bag0 + i))) {
          done_mask |= 1 << i;
          end[i] = beg[i];
        }
      }
    }
    int len_max = 0;
#pragma unroll
    for (int i = 0; i < UB; ++i) len_max = max(len_max, end[i] - beg[i]);

#pragma unroll
    for (int v0 = 0; v0 < VPL; v0 += VPP) {
      float acc[UB][VPP][EPV];
      float bias_acc[UB];
#pragma unroll
      for (int i = 0; i < UB; ++i) {
        bias_acc[i] = 0.f;
#pragma unroll
        for (int v = 0; v < VPP; ++v)
#pragma unroll
          for (int e = 0; e < EPV; ++e) acc[i][v][e] = 0.f;
      }

      // index of the lookup each (bag, unroll slot) will read next; -1 = none
      int idx[UB][U];
#pragma unroll
      for (int i = 0; i < UB; ++i)
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int p = beg[i] + u * Y + y;
          idx[i][u] = p < end[i] ? indices[p] : -1;
        }

      for (int base = 0; base < len_max; base += U * Y) {
        Vec<VB> buf[UB][U][VPP];
        f32x2 sb[UB][U];
        const int nbase = base + U * Y;

        // A round in which every lane of the wavefront has all its U lookups: straight-line
        // code, every load issued before the first add.
        bool full = true;
#pragma unroll
        for (int i = 0; i < UB; ++i) full = full && (beg[i] + nbase <= end[i]);
        if (__builtin_amdgcn_ballot_w64(!full) == 0) {
#pragma unroll
          for (int i = 0; i < UB; ++i)
#pragma unroll
            for (int u = 0; u < U; ++u) {
              const char *row = table + static_cast<int64_t>(idx[i][u]) * R::STRIDE;
#pragma unroll
              for (int v = 0; v < VPP; ++v) {
                const int c = x + (v0 + v) * X;
                if (v0 + v < VPL && c < R::V) buf[i][u][v] = load_vec<VB>(row + c * VB);
              }
              if constexpr (DT == I8) sb[i][u] = load_scale_bias<D>(row);
            }
          // next round's indices: the address is clamped into the bag, the value dropped if
          // the position lies beyond it
          int nidx[UB][U];
#pragma unroll
          for (int i = 0; i < UB; ++i)
#pragma unroll
            for (int u = 0; u < U; ++u) {
              const int p = beg[i] + nbase + u * Y + y;
              nidx[i][u] = indices[p < end[i] ? p : end[i] - 1];
            }
#pragma unroll
          for (int i = 0; i < UB; ++i)
#pragma unroll
            for (int u = 0; u < U; ++u) {
#pragma unroll
              for (int v = 0; v < VPP; ++v) {
                const int c = x + (v0 + v) * X;
                if (v0 + v < VPL && c < R::V)
                  accumulate<DT, VB>(acc[i][v], buf[i][u][v], DT == I8 ? sb[i][u].x : 1.f);
              }
              if constexpr (DT == I8) bias_acc[i] += sb[i][u].y;
            }
#pragma unroll
          for (int i = 0; i < UB; ++i)
#pragma unroll
            for (int u = 0; u < U; ++u) {
              const int p = beg[i] + nbase + u * Y + y;
              idx[i][u] = p < end[i] ? nidx[i][u] : -1;
            }
          continue;
        }

#pragma unroll
        for (int i = 0; i < UB; ++i)
#pragma unroll
          for (int u = 0; u < U; ++u)
            if (idx[i][u] >= 0) {
              const char *row = table + static_cast<int64_t>(idx[i][u]) * R::STRIDE;
#pragma unroll
              for (int v = 0; v < VPP; ++v) {
                const int c = x + (v0 + v) * X;
                if (v0 + v < VPL && c < R::V) buf[i][u][v] = load_vec<VB>(row + c * VB);
              }
              if constexpr (DT == I8) sb[i][u] = load_scale_bias<D>(row);
            }

        // fetch the next round of indices while the rows are in flight
        int nidx[UB][U];
#pragma unroll
        for (int i = 0; i < UB; ++i)
#pragma unroll
          for (int u = 0; u < U; ++u) {
            const int p = beg[i] + nbase + u * Y + y;
            nidx[i][u] = p < end[i] ? indices[p] : -1;
          }

#pragma unroll
        for (int i = 0; i < UB; ++i)
#pragma unroll
          for (int u = 0; u < U; ++u)
            if (idx[i][u] >= 0) {
#pragma unroll
              for (int v = 0; v < VPP; ++v) {
                const int c = x + (v0 + v) * X;
                if (v0 + v < VPL && c < R::V)
                  accumulate<DT, VB>(acc[i][v], buf[i][u][v], DT == I8 ? sb[i][u].x : 1.f);
              }
              if constexpr (DT == I8) bias_acc[i] += sb[i][u].y;
            }

#pragma unroll
        for (int i = 0; i < UB; ++i)
#pragma unroll
          for (int u = 0; u < U; ++u) idx[i][u] = nidx[i][u];
      }

      if constexpr (Y > 1) {
#pragma unroll
        for (int i = 0; i < UB; ++i) {
          if constexpr (DT == I8) bias_acc[i] = reduce_over_y<X, T>(bias_acc[i]);
#pragma unroll
          for (int v = 0; v < VPP; ++v)
#pragma unroll
            for (int e = 0; e < EPV; ++e) acc[i][v][e] = reduce_over_y<X, T>(acc[i][v][e]);
        }
      }

      if constexpr (OVEC == 4 && EPV / 4 >= RFX_STAGE_MIN_F4) {
        // several float4 of consecutive columns per lane: through LDS, so that each store
        // instruction of the team writes consecutive memory
        constexpr int Q = EPV / 4;
        static_assert(Q <= kStageF4PerLane, "stage slice too small");
        // this team's part of its wavefront's slice
        f32x4 *seg = stage + (tid >> 6) * (64 * kStageF4PerLane) + ((tid & 63) / T) * (X * Q);
#pragma unroll
        for (int i = 0; i < UB; ++i) {
          const int bag = bag0 + i;
          const bool live = y == 0 && bag < bag_end && !((done_mask >> i) & 1);
          float *dst = out + static_cast<int64_t>(bag) * esum + col_off;
#pragma unroll
          for (int v = 0; v < VPP; ++v) {
            if (v0 + v < VPL) {
              const int first = (v0 + v) * X;                 // first row vector of the segment
              const int nvec = R::V - first < X ? R::V - first : X;
              if (live && x < nvec) {
#pragma unroll
                for (int q = 0; q < Q; ++q) {
                  f32x4 t;
                  t.x = acc[i][v][4 * q + 0]; t.y = acc[i][v][4 * q + 1];
                  t.z = acc[i][v][4 * q + 2]; t.w = acc[i][v][4 * q + 3];
                  if constexpr (DT == I8) t += bias_acc[i];
                  seg[x * Q + q] = t;
                }
              }
              // the lanes of a team sit in one wavefront: order its LDS writes before its reads
              __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
              __builtin_amdgcn_wave_barrier();
              __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
              if (live) {
#pragma unroll
                for (int k = 0; k < Q; ++k) {
                  const int j = k * X + x;                    // float4 of the segment
                  if (j < nvec * Q)
                    store_streaming(reinterpret_cast<f32x4 *>(dst + first * EPV + j * 4), seg[j]);
                }
              }
              // ... and these reads before the next segment's writes
              __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
              __builtin_amdgcn_wave_barrier();
              __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            }
          }
        }
      } else if (y == 0) {
#pragma unroll
        for (int i = 0; i < UB; ++i) {
          const int bag = bag0 + i;
          if (bag < bag_end && !((done_mask >> i) & 1)) {
            float *dst = out + static_cast<int64_t>(bag) * esum + col_off;
#pragma unroll
            for (int v = 0; v < VPP; ++v) {
              const int c = x + (v0 + v) * X;
              if (v0 + v < VPL && c < R::V) {
                if constexpr (DT == I8) {
#pragma unroll
                  for (int e = 0; e < EPV; ++e) acc[i][v][e] += bias_acc[i];
                }
                store_floats<EPV, OVEC>(dst + c * EPV, acc[i][v]);
              }
            }
          }
        }
      }
    }
  }
  (void)stage;
}

// ---------------------------------------------------------------------------------------------
// onehot_bags: bags of at most one lookup (the pooled output row is a copy of a table row, or
// zeros), X column lanes per bag, no lookup lanes.  Such a feature costs latencies, not
// arithmetic: offsets -> index -> row -> store is a chain of three round trips to memory per
// pass, so a wavefront takes UB bags per team at once (64 / X teams: (64 / X) * UB bags and as
// many row loads in flight per pass) and, when the binding found exactly as many lookups as
// bags in the batch (one_per_bag), fetches indices[bag] together with the offsets instead of
// after them -- right whenever offsets[bag] == bag, which is then checked.  A wavefront that
// meets a longer bag in its pass hands that pass to team_bags.
//
// Wavefront w of the workgroup owns the bags [bag_begin + (w + k * BT/64) * WB, + WB), WB =
// (64 / X) * UB; within it team t takes bags t, t + 64/X, ...: consecutive lanes of an offsets or
// index load read consecutive words.
//
// Reference counterpart: onehot::GatherSegments (examples/csrc/include/onehot_kernel.cuh:14-87),
// which copies rows with 4-byte accesses and takes the bag length of 1 for granted.
// ---------------------------------------------------------------------------------------------
template <int BT, int DT, int D, int X, int UB, int OVEC>
__device__ __forceinline__ void
onehot_bags(f32x4 *__restrict__ stage, const char *__restrict__ table,
            const int *__restrict__ indices, const int *__restrict__ offsets,
            float *__restrict__ out, const int esum, const int col_off, const int bag_begin,
            const int bag_end, const int skip_longer_than, const int one_per_bag) {
  using R = Row<DT, D>;
  static_assert(X >= 1 && X <= 64 && (X & (X - 1)) == 0, "column lanes: a power of two <= 64");
  constexpr int TEAMS_W = 64 / X;               // teams per wavefront
  constexpr int WB = TEAMS_W * UB;              // bags per wavefront and pass
  constexpr int WAVES = BT / 64;
  constexpr int VPL = ceil_div(R::V, X);
  constexpr int VB = R::VB;
  constexpr int EPV = R::EPV;

  const int tid = body_thread_id<BT>();
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int team = lane / X;
  const int x = lane - team * X;

  for (int pass0 = bag_begin + wave * WB; pass0 < bag_end; pass0 += WAVES * WB) {
    const int pass_end = min(pass0 + WB, bag_end);
    int bag[UB], beg[UB], len[UB], spec[UB];
    // first round trip: the bags' bounds, and on the hint the index each would have
#pragma unroll
    for (int u = 0; u < UB; ++u) {
      bag[u] = pass0 + u * TEAMS_W + team;
      const int b = min(bag[u], bag_end - 1);
      beg[u] = offsets[b];
      len[u] = bag[u] < pass_end ? offsets[b + 1] - beg[u] : 0;
      spec[u] = one_per_bag ? indices[b] : 0;   // exactly `batch` lookups exist: in bounds
    }
    bool mine = true;         // every bag of this lane has zero or one lookup
    bool guessed = true;      // ... and the one lookup is where the hint says
#pragma unroll
    for (int u = 0; u < UB; ++u) {
      mine = mine && len[u] <= 1;
      guessed = guessed && (len[u] == 0 || beg[u] == bag[u]);
    }
    if (__builtin_amdgcn_ballot_w64(!mine) != 0) {
      // the general routine for this wavefront's bags (it also knows what to do with very long ones)
      team_bags<64, DT, D, X, 1, 2, 1, VPL, OVEC>(
          stage ? stage + wave * (64 * kStageF4PerLane) : nullptr, table, indices, offsets, out,
          esum, col_off, pass0, pass_end, skip_longer_than);
      continue;
    }
    int idx[UB];
    if (one_per_bag && __builtin_amdgcn_ballot_w64(!guessed) == 0) {
#pragma unroll
      for (int u = 0; u < UB; ++u) idx[u] = len[u] == 1 ? spec[u] : -1;
    } else {
#pragma unroll
      for (int u = 0; u < UB; ++u) idx[u] = len[u] == 1 ? indices[beg[u]] : -1;
    }
    // the rows
    Vec<VB> buf[UB][VPL];
    f32x2 sb[UB];
#pragma unroll
    for (int u = 0; u < UB; ++u)
      if (idx[u] >= 0) {
        const char *row = table + static_cast<int64_t>(idx[u]) * R::STRIDE;
#pragma unroll
        for (int v = 0; v < VPL; ++v) {
          const int c = x + v * X;
          if (c < R::V) buf[u][v] = load_vec<VB>(row + c * VB);
        }
        if constexpr (DT == I8) sb[u] = load_scale_bias<D>(row);
      }
    // 0 + row, as the sum of a bag of one lookup is formed everywhere else (an empty bag: zeros)
#pragma unroll
    for (int u = 0; u < UB; ++u) {
      if (bag[u] >= pass_end) continue;
      float *dst = out + static_cast<int64_t>(bag[u]) * esum + col_off;
#pragma unroll
      for (int v = 0; v < VPL; ++v) {
        const int c = x + v * X;
        if (c >= R::V) continue;
        float acc[EPV];
#pragma unroll
        for (int e = 0; e < EPV; ++e) acc[e] = 0.f;
        if (idx[u] >= 0) {
          accumulate<DT, VB>(acc, buf[u][v], DT == I8 ? sb[u].x : 1.f);
          if constexpr (DT == I8) {
#pragma unroll
            for (int e = 0; e < EPV; ++e) acc[e] += sb[u].y;
          }
        }
        store_floats<EPV, OVEC>(dst + c * EPV, acc);
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------
// block_bags: the whole workgroup sums one bag at a time (long bags).  The bag's indices are
// staged in LDS in chunks of CHUNK with coalesced loads; lane (y, x) reads index y + k*Y of the
// chunk and vector(s) x of the row; the Y lookup lanes inside a wavefront are combined with the
// cross-lane butterfly, the BT/64 wavefronts through LDS, and the result is written with
// coalesced 4-byte stores.
// ---------------------------------------------------------------------------------------------
template <int BT, int DT, int D, int X, int CHUNK> struct BlockBagStorage {
  using R = Row<DT, D>;
  static constexpr int VPL = ceil_div(R::V, X);
  static constexpr int COLS = X * VPL * R::EPV; // >= D
  int idx[2][CHUNK];                            // two chunks of indices: one summed, one arriving
  float part[BT / 64][COLS];
  float part_bias[BT / 64];
  int last;                                     // split_bags: this workgroup finishes the bag
};

// The workgroup sums the lookups [beg, end) of one bag: afterwards s.part[w][j] holds wavefront
// w's share of column j (and s.part_bias[w] its share of the int8 biases), and a barrier has
// made them visible to every thread.  Starts with a barrier that orders an earlier use of
// s.part / s.idx before this one.
template <int BT, int DT, int D, int X, int U, int CHUNK>
__device__ __forceinline__ void
block_sum_range(BlockBagStorage<BT, DT, D, X, CHUNK> &s, const char *__restrict__ table,
                const int *__restrict__ indices, const int beg, const int end, const int tid) {
  using R = Row<DT, D>;
  static_assert(X >= 1 && X <= 64 && (X & (X - 1)) == 0, "column lanes");
  static_assert(BT % 64 == 0 && CHUNK % BT == 0, "chunk must be whole workgroup loads");
  constexpr int Y = BT / X;
  constexpr int VPL = ceil_div(R::V, X);
  constexpr int VB = R::VB;
  constexpr int EPV = R::EPV;

  const int y = tid / X;
  const int x = tid - y * X;
  const int wave = tid / 64;
  const int lane = tid - wave * 64;

  float acc[VPL][EPV];
  float bias_acc = 0.f;
#pragma unroll
  for (int v = 0; v < VPL; ++v)
#pragma unroll
    for (int e = 0; e < EPV; ++e) acc[v][e] = 0.f;

  // The bag's indices pass through LDS in chunks, two buffers taking turns: while the rows of
  // one chunk are summed, the next chunk's indices are already on their way into registers, and
  // they are written to the other buffer once this chunk's rows are done.  One barrier per chunk:
  // a wavefront that writes buffer b for chunk k + 1 has passed the barrier of chunk k, which
  // every wavefront reaches only after its last read of chunk k - 1 (the earlier tenant of b).
  constexpr int IPT = CHUNK / BT;               // indices per thread and chunk
  int arriving[IPT];
  auto request_chunk = [&](const int c0) {
#pragma unroll
    for (int i = 0; i < IPT; ++i) {
      const int p = c0 + i * BT + tid;
      arriving[i] = indices[p < end ? p : end - 1];      // beyond the bag: a dummy, never used
    }
  };
  if (beg < end) request_chunk(beg);
  __syncthreads();
  int cur = 0;
  for (int c0 = beg; c0 < end; c0 += CHUNK, cur ^= 1) {
    const int n = min(CHUNK, end - c0);
    const int *__restrict__ chunk = s.idx[cur];
#pragma unroll
    for (int i = 0; i < IPT; ++i) s.idx[cur][i * BT + tid] = arriving[i];
    if (c0 + CHUNK < end) request_chunk(c0 + CHUNK);
    __syncthreads();

    for (int base = 0; base < n; base += U * Y) {
      Vec<VB> buf[U][VPL];
      f32x2 sb[U];
      bool ok[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int p = base + u * Y + y;
        ok[u] = p < n;
        if (ok[u]) {
          const char *row = table + static_cast<int64_t>(chunk[p]) * R::STRIDE;
#pragma unroll
          for (int v = 0; v < VPL; ++v) {
            const int c = x + v * X;
            if (c < R::V) buf[u][v] = load_vec<VB>(row + c * VB);
          }
          if constexpr (DT == I8) sb[u] = load_scale_bias<D>(row);
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u)
        if (ok[u]) {
#pragma unroll
          for (int v = 0; v < VPL; ++v) {
            const int c = x + v * X;
            if (c < R::V) accumulate<DT, VB>(acc[v], buf[u][v], DT == I8 ? sb[u].x : 1.f);
          }
          if constexpr (DT == I8) bias_acc += sb[u].y;
        }
    }
  }

  // combine the lookup lanes that share a wavefront
  if constexpr (X < 64) {
    if constexpr (DT == I8) bias_acc = reduce_over_y<X, 64>(bias_acc);
#pragma unroll
    for (int v = 0; v < VPL; ++v)
#pragma unroll
      for (int e = 0; e < EPV; ++e) acc[v][e] = reduce_over_y<X, 64>(acc[v][e]);
  }
  if (lane < X) {
#pragma unroll
    for (int v = 0; v < VPL; ++v)
#pragma unroll
      for (int e = 0; e < EPV; ++e) s.part[wave][(x + v * X) * EPV + e] = acc[v][e];
    if (lane == 0) s.part_bias[wave] = bias_acc;
  }
  __syncthreads();
}

// column j of what block_sum_range left in LDS: the wavefronts' shares in wavefront order
template <int BT, int DT, int D, int X, int CHUNK>
__device__ __forceinline__ float
block_column(const BlockBagStorage<BT, DT, D, X, CHUNK> &s, const int j) {
  constexpr int WAVES = BT / 64;
  float t = 0.f;
#pragma unroll
  for (int w = 0; w < WAVES; ++w) t += s.part[w][j];
  if constexpr (DT == I8) {
#pragma unroll
    for (int w = 0; w < WAVES; ++w) t += s.part_bias[w];
  }
  return t;
}

template <int BT, int DT, int D, int X, int U, int CHUNK>
__device__ __forceinline__ void
block_bags(BlockBagStorage<BT, DT, D, X, CHUNK> &s, const char *__restrict__ table,
           const int *__restrict__ indices, const int *__restrict__ offsets,
           float *__restrict__ out, const int esum, const int col_off, const int bag_begin,
           const int bag_end) {
  const int tid = body_thread_id<BT>();
  for (int bag = bag_begin; bag < bag_end; ++bag) {
    block_sum_range<BT, DT, D, X, U, CHUNK>(s, table, indices, offsets[bag], offsets[bag + 1], tid);
    float *dst = out + static_cast<int64_t>(bag) * esum + col_off;
    for (int j = tid; j < D; j += BT) store_streaming(dst + j, block_column(s, j));
  }
}

// ---------------------------------------------------------------------------------------------
// split_bags: one bag summed by `parts` workgroups (a batch of few, very long bags: fewer bags
// than the device has workgroups).  Tile (bag, part) sums lookups
// [beg + part*per, beg + (part+1)*per) of the bag, per = ceil(length / parts), like block_bags,
// and writes its D partial sums to slot bag*parts + part of the feature's workspace region.
// The workgroup that finds the bag's arrival counter at parts-1 adds the slots in part order --
// the result does not depend on which workgroup came last -- writes the output row slice and
// puts the counter back to zero for the next launch.  No workgroup ever waits for another.
//
// The feature's region of the caller's workspace: kSplitMaxTiles slots of D floats, then
// kSplitMaxTiles arrival counters (int), which must be zero when the kernel starts.
// The binding keeps batch*parts <= kSplitMaxTiles.
//
// Reference counterparts: mbs::SparseSegmentReduce, which adds the blocks' partial sums onto
// the output with atomics (examples/csrc/include/multi_block_per_sample_kernel.cuh), and
// rbk::SparseSegmentReduce (examples/csrc/include/reduce_by_key_kernel.cuh); the arrival
// counter has the role of task_sync (RecFlex/sched_basic_csrc/include/task_sync.cuh:4-50)
// without its waiting loop.
// ---------------------------------------------------------------------------------------------
constexpr int kSplitMaxTiles = kBindMaxSplitTiles;      // what the binding keeps to

// floats of workspace a feature of dimension D needs when one of its schedules splits bags
__host__ __device__ constexpr int64_t split_region_floats(int d) {
  return static_cast<int64_t>(kSplitMaxTiles) * (d + 1);
}

// Memory operations of the arrival protocol on the device.  Partial sums and counters are read
// and written with device-scope atomic loads and stores: the workgroups of one bag run on
// different XCDs, whose L2 caches do not see each other's lines otherwise.  A device-scope fence
// would order them, but it writes back and invalidates the whole L2 of the XCD -- every table row
// cached there -- for each tile (measured: 6 to 15 times the kernel time of unsplit bags).
// Device-scope stores are performed at device scope when the memory counter has drained, so
// waiting for it before the arrival is announced orders the slots before the counter (the
// release); the finishing workgroup loads the slots only after its arrival has returned (the
// acquire: every slot load depends on the returned count through the branch on it).
struct DeviceMem {
  static __device__ __forceinline__ void store_slot(unsigned int *p, const float v) {
    __hip_atomic_store(p, __float_as_uint(v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  static __device__ __forceinline__ float load_slot(const unsigned int *p) {
    return __uint_as_float(__hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
  }
  static __device__ __forceinline__ void release() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
  static __device__ __forceinline__ int arrive(int *counter) {
    return __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  static __device__ __forceinline__ void reset(int *counter) {
    __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
};

// Part `part` of `parts` of bag `bag`: slot p of the bag is slots + p * slot_stride (D values),
// counter its arrival counter.
template <int BT, int DT, int D, int X, int U, int CHUNK>
__device__ __forceinline__ void
split_part(BlockBagStorage<BT, DT, D, X, CHUNK> &s, const char *__restrict__ table,
           const int *__restrict__ indices, const int *__restrict__ offsets,
           float *__restrict__ out, const int esum, const int col_off, const int bag,
           const int part, const int parts, unsigned int *__restrict__ slots,
           const int slot_stride, int *__restrict__ counter) {
  const int tid = body_thread_id<BT>();
  const int beg = offsets[bag];
  const int end = offsets[bag + 1];
  const int per = (end - beg + parts - 1) / parts;
  const int pbeg = min(end, beg + part * per);
  const int pend = min(end, pbeg + per);
  block_sum_range<BT, DT, D, X, U, CHUNK>(s, table, indices, pbeg, pend, tid);
  if (parts == 1) {                 // the whole bag: nothing to combine
    float *dst = out + static_cast<int64_t>(bag) * esum + col_off;
    for (int j = tid; j < D; j += BT) store_streaming(dst + j, block_column(s, j));
    return;
  }

  // The arrival protocol of rfx_arrival.h with the device's memory operations (DeviceMem above).
  for (int j = tid; j < D; j += BT)
    arrival_store<DeviceMem>(slots, part, slot_stride, j, block_column(s, j));
  DeviceMem::release();
  __syncthreads();
  if (tid == 0) s.last = arrival_is_last<DeviceMem>(counter, parts);
  __syncthreads();
  if (!s.last) return;              // the same for the whole workgroup
  float *dst = out + static_cast<int64_t>(bag) * esum + col_off;
  for (int j = tid; j < D; j += BT)
    store_streaming(dst + j, arrival_combine<DeviceMem>(slots, parts, slot_stride, j));
  if (tid == 0) DeviceMem::reset(counter);
}

template <int BT, int DT, int D, int X, int U, int CHUNK>
__device__ __forceinline__ void
split_bags(BlockBagStorage<BT, DT, D, X, CHUNK> &s, const char *__restrict__ table,
           const int *__restrict__ indices, const int *__restrict__ offsets,
           float *__restrict__ out, const int esum, const int col_off, const int bag_begin,
           const int bag_end, const int part, const int parts, float *__restrict__ region) {
  if (parts <= 1) {
    block_bags<BT, DT, D, X, U, CHUNK>(s, table, indices, offsets, out, esum, col_off, bag_begin,
                                       bag_end);
    return;
  }
  const int bag = bag_begin;
  unsigned int *slots = reinterpret_cast<unsigned int *>(region) +
                        static_cast<int64_t>(bag) * parts * D;
  int *counter = reinterpret_cast<int *>(region + static_cast<int64_t>(kSplitMaxTiles) * D) + bag;
  split_part<BT, DT, D, X, U, CHUNK>(s, table, indices, offsets, out, esum, col_off, bag, part,
                                     parts, slots, D, counter);
}

} // namespace rfx
