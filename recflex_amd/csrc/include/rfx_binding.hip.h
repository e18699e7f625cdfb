// Run-time thread binding of the fused embedding kernel, computed on the device.
//
// Every workgroup of the persistent grid derives, from the live offsets of the batch, how many
// tiles (ranges of consecutive bags worth about `tile_bytes` of memory traffic) each feature
// gets, exclusive-scans these counts in LDS and then walks the global tile space
// [0, total_tiles) with stride gridDim.x, finding the owning feature of a tile by binary search
// in the LDS prefix array.  A feature with long bags therefore gets many small bag ranges, a
// feature with short bags few large ones, and no host-side mapping or read-back is needed.
//
// Reference counterparts: the host-built (feature, block) list GetTaskMapping
// (RecFlex/sched_basic_csrc/task_mapping.cu:6-18), the per-feature num_tiles/num_blocks
// computed in the host preprocessors (examples/csrc/warp_per_sample_preprocess.cu:34-37) and
// the lookup `d_task_mapping[blockIdx.x]` at the top of the generated kernel
// (RecFlex/code_emitter/codegen.py:331-336).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace rfx {

// A device address read from memory, as a pointer the compiler knows to be global memory (so
// that accesses become global_load/global_store instead of flat ones).
template <typename T> __device__ __forceinline__ const T *global_ptr(int64_t addr) {
  typedef const T __attribute__((address_space(1))) * gptr_t;
  return (const T *)reinterpret_cast<gptr_t>(addr);
}

// 128-byte alignment of the vectors inside a packed argument buffer
// (RecFlex/sched_basic_csrc/include/utils.cuh:60-62)
__host__ __device__ constexpr int64_t alignmem(int64_t x) { return (x + 127) / 128 * 128; }

// Where a feature's int32 offsets[batch+1] and indices[] live.  Two forms are accepted:
//  * pointer table: io_ptrs[2f] = indices, io_ptrs[2f+1] = offsets (device addresses);
//  * packed buffer: feature f starts at arg_base + arg_offsets[f] (bytes) with its offsets,
//    padded to 128 B, followed by its indices.
struct IoView {
  const int64_t *__restrict__ io_ptrs;
  const char *__restrict__ arg_base;
  const int64_t *__restrict__ arg_offsets;
  int batch;

  __device__ __forceinline__ const int *offsets(int f) const {
    if (io_ptrs) return global_ptr<int>(io_ptrs[2 * f + 1]);
    return global_ptr<int>(reinterpret_cast<int64_t>(arg_base) + arg_offsets[f]);
  }
  __device__ __forceinline__ const int *indices(int f) const {
    if (io_ptrs) return global_ptr<int>(io_ptrs[2 * f]);
    return global_ptr<int>(reinterpret_cast<int64_t>(arg_base) + arg_offsets[f] +
                           alignmem((static_cast<int64_t>(batch) + 1) * 4));
  }
};

// Schedules that split a bag over several workgroups (rfx::split_bags) announce themselves with
// a granularity of kSplitGran.  A bag is worth splitting when it alone would keep its workgroup
// busy for a good part of the kernel: the unit is a quarter of a workgroup's fair share of the
// batch's traffic (total / grid), at least one tile and kSplitMinUnit; when the mean bag of such a feature
// carries more than two units, the feature gets batch * parts tiles, parts = bag / unit, tile t
// being part t % parts of bag t / parts, and bags_per_tile holds -parts.  (A part costs some
// 20 us of dependent memory round trips besides its rows, and with two to five tiles per
// workgroup the time moves in steps of whole tiles: a unit of half a share gave 150 / 162 /
// 161 us where a quarter gives 177 / 109 / 160 us on 16 x 20 000, 64 x 4 000 and 128 x 2 500
// lookups; the finer one is kept, it also evens out bags of unequal length.)
// Always parts <= kBindMaxParts and batch * parts <= kBindMaxSplitTiles (the slots of the feature's
// workspace region).  Otherwise -- many bags, or a small grid -- the feature is bound like any
// other with one bag per workgroup pass.  (Measured on 8 features of 16 bags of 20 000 lookups:
// 968 us unsplit, 177 us split; 64 bags of 4 000: 204 and 109 us; 512 bags of 1 000 stay
// unsplit at 185 us.)
// Smallest part: 256 KiB of traffic (with 128 KiB parts the three shapes above take 175 / 108 /
// 161 us at four workgroups per CU, with 256 KiB parts 142 / 103 / 122 us; at eight workgroups
// per CU, which these light kernels allow, 138 / 76 / 83 us and 107 / 83 / 96 us).
constexpr int kSplitMinUnit = 256 * 1024;
constexpr int kSplitGran = -1;
constexpr int kBindMaxParts = 64;
constexpr int kBindMaxSplitTiles = 2048;

// a tile is rounded up to one whole workgroup pass of its schedule only if that pass carries at
// most this many times the target traffic per tile
constexpr int kMaxTileFactor = 8;

template <int F> struct BindingStorage {
  int prefix[F + 1];      // prefix[f] = first global tile id of feature f
  int bags_per_tile[F];
  int cand[F];            // index (into the candidate tables) of the schedule feature f runs
  long long partial[16];  // per-wavefront sums of the batch's traffic (automatic tile size)
};

// Automatic tile size (tile_bytes <= 0): the batch's traffic divided by kAutoTilesPerWorkgroup
// tiles for each workgroup of the grid, within [kAutoTileMin, kAutoTileMax], in steps of 4 KiB.
// Small batches keep 64 KiB tiles; a batch of tens of GB with bags of hundreds of wide rows gets
// 256 KiB, several bags per tile instead of one (measured on the 400-feature fp16 model with its
// default schedules: 7.1 ms with 64 KiB tiles, 5.0 ms with 256 KiB).
constexpr int kAutoTilesPerWorkgroup = 64;
constexpr int kAutoTileMin = 64 * 1024;
constexpr int kAutoTileMax = 256 * 1024;

__device__ __forceinline__ int wave_inclusive_scan(int v, int lane) {
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const int t = __shfl_up(v, d, 64);
    if (lane >= d) v += t;
  }
  return v;
}

// lookup_bytes[f]: bytes fetched per lookup (row + index); bag_bytes[f]: bytes per bag that do
// not depend on its length (output row slice + offset).
// Feature f owns the candidate schedules cand_begin[f] .. cand_begin[f+1]-1 (exactly one in a
// production build, the whole candidate list in a tuning build); choice[f] (clamped; 0 if
// choice is null) selects the one this launch runs, and cand_gran[] gives the bags a workgroup
// of that schedule handles per pass (tiles are whole multiples of it unless a pass is too large).
// tile_bytes: traffic a tile should carry; <= 0 lets the workgroup size the tiles from the batch
// (see kAutoTilesPerWorkgroup above).
// fixed_tiles: if non-null, the tile count per feature is taken from it instead of from the
// live offsets (static thread binding, for the ablation).
// grid_blocks: workgroups of the fused kernel's grid (for the automatic tile size).
// Returns the total number of tiles.  Ends with a barrier.
template <int F, int BT, bool SPLIT = false>
__device__ __forceinline__ int
bind_tiles(BindingStorage<F> &s, const IoView &io, const int tile_bytes,
           const int *__restrict__ lookup_bytes, const int *__restrict__ bag_bytes,
           const int *__restrict__ cand_begin, const int *__restrict__ cand_gran,
           const int *__restrict__ choice, const int *__restrict__ fixed_tiles,
           const int grid_blocks) {
  static_assert(BT <= 16 * 64, "partial sums: at most 16 wavefronts");
  const int tid = threadIdx.x;
  const int B = io.batch;

  // tiles of every feature this thread is responsible for (tid, tid + BT, ...) at the given
  // tile size; returns the traffic of those features
  // split_unit: traffic per part of a split bag (0: no bag is split)
  auto bind_features = [&](const int tile_size, const long long split_unit) {
    long long traffic = 0;
    for (int f = tid; f < F; f += BT) {
      const int first = cand_begin[f];
      const int ncand = cand_begin[f + 1] - first;
      int pick = choice ? choice[f] : 0;
      pick = pick < 0 ? 0 : (pick >= ncand ? ncand - 1 : pick);
      s.cand[f] = first + pick;
      int g = cand_gran[first + pick];
      const bool may_split = g == kSplitGran && !fixed_tiles;
      if (g == kSplitGran) g = 1;
      int64_t want;
      int64_t bag_cost = 0;       // mean traffic of one bag of this feature
      if (fixed_tiles) {
        want = fixed_tiles[f];
      } else {
        const int *offs = io.offsets(f);
        const int64_t lookups = static_cast<int64_t>(offs[B]) - offs[0];
        const int64_t cost = lookups * lookup_bytes[f] + static_cast<int64_t>(B) * bag_bytes[f];
        traffic += cost;
        want = (cost + tile_size - 1) / tile_size;
        bag_cost = B > 0 ? cost / B : 0;
      }
      int tiles = want < 1 ? 1 : (want > B ? B : static_cast<int>(want));
      int bpt = 0;
      int64_t parts = 1;
      if (SPLIT && may_split && B > 0 && split_unit > 0 && bag_cost > 2 * split_unit) {
        parts = (bag_cost + split_unit - 1) / split_unit;
        if (parts > kBindMaxParts) parts = kBindMaxParts;
        if (parts * B > kBindMaxSplitTiles) parts = kBindMaxSplitTiles / B;
      }
      if (parts > 1) {
        tiles = B * static_cast<int>(parts);
        bpt = -static_cast<int>(parts);
      } else if (B > 0) {
        bpt = (B + tiles - 1) / tiles;
        // Tiles are whole workgroup passes (g bags) -- unless one pass of this schedule is more
        // than kMaxTileFactor times the traffic a tile should carry: then the tile keeps its
        // share of the traffic and some of the schedule's teams idle.
        const int whole = (bpt + g - 1) / g * g;
        if (fixed_tiles || bpt >= g ||
            static_cast<int64_t>(whole) * bag_cost <= static_cast<int64_t>(kMaxTileFactor) * tile_size)
          bpt = whole;
        tiles = (B + bpt - 1) / bpt;
      } else {
        tiles = 0;
      }
      s.bags_per_tile[f] = bpt;
      s.prefix[f + 1] = tiles;
    }
    return traffic;
  };

  // Automatic tile size: bind with the smallest size and add up the batch's traffic on the
  // way; only a batch large enough for bigger tiles is bound a second time.
  const bool automatic = tile_bytes <= 0 && !fixed_tiles;
  const bool need_total = automatic || (SPLIT && !fixed_tiles);
  long long traffic = bind_features(automatic ? kAutoTileMin : tile_bytes, 0);
  if (need_total) {
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) traffic += __shfl_xor(traffic, d, 64);
    if ((tid & 63) == 0) s.partial[tid >> 6] = traffic;
  }
  if (tid == 0) s.prefix[0] = 0;
  __syncthreads();
  if (need_total) {
    long long total = 0;
    for (int w = 0; w < BT / 64; ++w) total += s.partial[w];
    int tile_size = tile_bytes;
    if (automatic) {
      long long t = total / (static_cast<long long>(grid_blocks) * kAutoTilesPerWorkgroup);
      t = t < kAutoTileMin ? kAutoTileMin : (t > kAutoTileMax ? kAutoTileMax : t);
      tile_size = static_cast<int>(t) & ~4095;
    }
    long long split_unit = 0;
    if (SPLIT) {
      split_unit = total / (4ll * (grid_blocks > 0 ? grid_blocks : 1));
      if (split_unit < tile_size) split_unit = tile_size;
      if (split_unit < kSplitMinUnit) split_unit = kSplitMinUnit;
    }
    // the same decision in every thread of the grid
    if (SPLIT || tile_size != kAutoTileMin) {
      bind_features(tile_size, split_unit);
      __syncthreads();
    }
  }
  if (tid < 64) {
    int carry = 0;
    for (int c = 0; c < F; c += 64) {
      const int i = c + tid;
      int v = i < F ? s.prefix[i + 1] : 0;
      v = wave_inclusive_scan(v, tid) + carry;
      if (i < F) s.prefix[i + 1] = v;
      carry = __shfl(v, 63, 64);
    }
  }
  __syncthreads();
  return s.prefix[F];
}

// feature owning global tile id `tile` (0 <= tile < prefix[F]): largest f with prefix[f] <= tile
template <int F>
__device__ __forceinline__ int find_feature(const int *prefix, const int tile) {
  int lo = 0, hi = F;
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (prefix[mid] <= tile) lo = mid; else hi = mid;
  }
  return lo;
}
template <int F>
__device__ __forceinline__ int find_feature(const BindingStorage<F> &s, const int tile) {
  return find_feature<F>(s.prefix, tile);
}

// ---------------------------------------------------------------------------------------------
// Binding computed once per launch, for models of thousands of features.  The binding costs
// every workgroup some 10 us per thousand features and 12 bytes of LDS per feature; at 10 000
// features that is 100 us per workgroup and 120 KB, which leaves one workgroup per CU.  Such a
// model is bound by one workgroup of a small kernel launched ahead of the fused one
// (bind_once), into a table in device memory; the workgroups of the fused kernel copy only the
// prefix array into LDS (load_prefix) and read the two other entries of a tile's feature from
// the table.
// ---------------------------------------------------------------------------------------------
template <int F> struct BoundTables {       // in device memory
  int prefix[F + 1];
  int bags_per_tile[F];
  int cand[F];
};

template <int F> struct PrefixStorage {     // what a workgroup of the fused kernel keeps in LDS
  int prefix[F + 1];
};

template <int F, int BT, bool SPLIT = false>
__device__ __forceinline__ void
bind_once(BindingStorage<F> &s, BoundTables<F> *__restrict__ out, const IoView &io,
          const int tile_bytes, const int *__restrict__ lookup_bytes,
          const int *__restrict__ bag_bytes, const int *__restrict__ cand_begin,
          const int *__restrict__ cand_gran, const int *__restrict__ choice,
          const int *__restrict__ fixed_tiles, const int grid_blocks) {
  bind_tiles<F, BT, SPLIT>(s, io, tile_bytes, lookup_bytes, bag_bytes, cand_begin, cand_gran,
                           choice, fixed_tiles, grid_blocks);
  for (int f = threadIdx.x; f < F; f += BT) {
    out->bags_per_tile[f] = s.bags_per_tile[f];
    out->cand[f] = s.cand[f];
  }
  for (int f = threadIdx.x; f <= F; f += BT) out->prefix[f] = s.prefix[f];
}

// Returns the total number of tiles.  Ends with a barrier.
template <int F, int BT>
__device__ __forceinline__ int load_prefix(PrefixStorage<F> &s,
                                           const BoundTables<F> *__restrict__ bound) {
  for (int f = threadIdx.x; f <= F; f += BT) s.prefix[f] = bound->prefix[f];
  __syncthreads();
  return s.prefix[F];
}

} // namespace rfx
