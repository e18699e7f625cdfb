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
  // optional: the lookups of every feature in this batch as the caller knows them (a hint for
  // the binding, which otherwise reads offsets[batch] of every feature)
  const int *__restrict__ counts = nullptr;
  // optional: the caller's number of every feature of the kernel.  A kernel emitted with a tile
  // order lays the features out in its tile space in an order of its own and numbers them by
  // their place there; whatever the caller passes per feature -- addresses, counts, tables -- is
  // found through this table (null: the kernel's numbers are the caller's).
  const int *__restrict__ ext = nullptr;

  __device__ __forceinline__ int ext_of(int f) const { return ext ? ext[f] : f; }
  __device__ __forceinline__ int count(int f) const { return counts[ext_of(f)]; }
  __device__ __forceinline__ int64_t offsets_addr(int f) const {
    f = ext_of(f);
    if (io_ptrs) return io_ptrs[2 * f + 1];
    return reinterpret_cast<int64_t>(arg_base) + arg_offsets[f];
  }
  __device__ __forceinline__ int64_t indices_addr(int f) const {
    f = ext_of(f);
    if (io_ptrs) return io_ptrs[2 * f];
    return reinterpret_cast<int64_t>(arg_base) + arg_offsets[f] +
           alignmem((static_cast<int64_t>(batch) + 1) * 4);
  }
  // Both addresses of feature f from two independent loads of one cache line, whichever form the
  // inputs have (no branch: the binding issues these loads for all features at once).
  __device__ __forceinline__ void addrs(int f, int64_t &indices_at, int64_t &offsets_at) const {
    addrs_at(ext_of(f), indices_at, offsets_at);
  }
  // ... of the feature the caller numbers f
  __device__ __forceinline__ void addrs_at(const int f, int64_t &indices_at, int64_t &offsets_at) const {
    typedef long long pair_t __attribute__((ext_vector_type(2), aligned(8)));
    const bool ptrs = io_ptrs != nullptr;
    // pointer table: {indices, offsets} of f; packed form: {byte offset of f, of f + 1}
    const int64_t *src = ptrs ? io_ptrs + 2 * f : arg_offsets + f;
    const pair_t ab = *reinterpret_cast<const pair_t *>(src);
    const int64_t a = ab.x, b = ab.y;
    const int64_t base = reinterpret_cast<int64_t>(arg_base);
    offsets_at = ptrs ? b : base + a;
    indices_at = ptrs ? a : base + a + alignmem((static_cast<int64_t>(batch) + 1) * 4);
  }
  __device__ __forceinline__ const int *offsets(int f) const { return global_ptr<int>(offsets_addr(f)); }
  __device__ __forceinline__ const int *indices(int f) const { return global_ptr<int>(indices_addr(f)); }
};

// Schedules that split a bag over several workgroups (rfx::split_bags) announce themselves with
// a granularity of kSplitGran.  A bag is worth splitting when it alone would keep its workgroup
// busy for a good part of the kernel: the unit is a quarter of a workgroup's fair share of the
// batch's traffic (total / grid), at least one tile and kSplitMinUnit; when the mean bag of such a feature
// carries more than 1.25 units, the feature gets batch * parts tiles, parts = bag / unit, tile t
// being part t % parts of bag t / parts, and bags_per_tile holds -parts.  (A part costs some
// 6 us of dependent memory round trips besides its rows, and with two to five tiles per
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
// ... unless the batch is so small that parts of that size leave the workgroups with one or two
// tiles each: then the part size is chosen so that the tiles come out as a whole number per
// workgroup, down to kSplitFloorUnit (16 x 20 000 lookups on 2 048 workgroups: 2 880 parts of
// 256 KiB are 1.4 tiles per workgroup, i.e. two rounds with the second a third full, 94 us;
// 3 872 parts of 199 KiB are 1.9, 88 us).
constexpr int kSplitFloorUnit = 128 * 1024;
constexpr int kSplitGran = -1;
constexpr int kBindMaxParts = 64;
constexpr int kBindMaxSplitTiles = 2048;

// a tile is rounded up to one whole workgroup pass of its schedule only if that pass carries at
// most this many times the target traffic per tile
constexpr int kMaxTileFactor = 8;
// ... or, whatever it carries, if whole passes still give the grid this many tiles per workgroup
// (estimated from the feature at hand: its whole passes times the number of features)
constexpr int kPlentyTilesPerWorkgroup = 2;

// Models of up to this many features also keep, per feature, the three addresses a tile needs
// (table, indices, offsets) in LDS: the binding reads them anyway, and a tile then starts with
// an LDS read instead of a round trip to memory for its pointers.
constexpr int kBindKeepAddrs = 512;

template <int F> struct BindingStorage {
  static constexpr bool kKeepAddrs = F <= kBindKeepAddrs;
  int prefix[F + 1];      // prefix[f] = first global tile id of feature f
  int bags_per_tile[F];
  int cand[F];            // index (into the candidate tables) of the schedule feature f runs
  long long partial[16];  // per-wavefront sums of the batch's traffic (automatic tile size)
  int chunk_sum[(F + 63) / 64];   // tiles of every 64 features (the prefix sum's second level)
  int64_t table_addr[kKeepAddrs ? F : 1];
  int64_t indices_addr[kKeepAddrs ? F : 1];
  int64_t offsets_addr[kKeepAddrs ? F : 1];
  // 1: the batch holds exactly as many lookups of this feature as bags (every bag may have
  // exactly one: bodies for bags of one lookup then fetch indices[bag] without waiting for the
  // bag's offsets, and check afterwards)
  unsigned char one_per_bag[kKeepAddrs ? F : 1];
};

// a 64-bit value that is the same in every lane, as a scalar
__device__ __forceinline__ int64_t uniform64(const int64_t v) {
  const unsigned lo = __builtin_amdgcn_readfirstlane(static_cast<int>(v));
  const unsigned hi = __builtin_amdgcn_readfirstlane(static_cast<int>(v >> 32));
  return static_cast<int64_t>((static_cast<unsigned long long>(hi) << 32) | lo);
}

// Automatic tile size (tile_bytes <= 0): the batch's traffic divided by kAutoTilesPerWorkgroup
// tiles for each workgroup of the grid, within [kAutoTileMin, kAutoTileMax], in steps of 4 KiB.
// Small batches keep 64 KiB tiles; a batch of tens of GB with bags of hundreds of wide rows gets
// 256 KiB, several bags per tile instead of one (measured on the 400-feature fp16 model with its
// default schedules: 7.1 ms with 64 KiB tiles, 5.0 ms with 256 KiB).
// A batch too small for that (less than kAutoTileMin of traffic per workgroup of the grid) gets
// about two tiles per workgroup instead, down to kAutoTileFloor: its launch is a matter of
// latencies -- every pass of a workgroup over a tile is a chain of dependent round trips to
// memory -- so the passes are spread over all workgroups as evenly as their number allows
// (measured on 26 features x 4 096 one-lookup bags, 1 024 workgroups: 9.0 us with 54 KiB tiles
// of two passes each, 8.3 us with 32 KiB tiles of one).
constexpr int kAutoTilesPerWorkgroup = 64;
constexpr int kAutoTileMin = 64 * 1024;
constexpr int kAutoTileMax = 256 * 1024;
constexpr int kAutoTileFloor = 4 * 1024;

__host__ __device__ inline int auto_tile_size(const long long total, const int grid_blocks) {
  const long long grid = grid_blocks > 0 ? grid_blocks : 1;
  long long t = total / (grid * kAutoTilesPerWorkgroup);
  if (t >= kAutoTileMin) return static_cast<int>(t > kAutoTileMax ? kAutoTileMax : t) & ~4095;
  t = total / (2 * grid);
  t = t < kAutoTileFloor ? kAutoTileFloor : (t > kAutoTileMin ? kAutoTileMin : t);
  return static_cast<int>(t) & ~1023;
}

// Inclusive prefix sum over the 64 lanes of a wavefront with DPP moves (no LDS traffic): shifts
// by 1, 2, 4 and 8 inside each row of 16 lanes (lanes shifted in from outside the row read 0),
// then lane 15 of a row broadcast to the next row (rows 1 and 3), then lane 31 to rows 2 and 3.
template <int CTRL, int ROW_MASK> __device__ __forceinline__ int dpp_or_zero(const int v) {
  return __builtin_amdgcn_update_dpp(0, v, CTRL, ROW_MASK, 0xf, false);
}
__device__ __forceinline__ int wave_inclusive_scan(int v, int lane) {
  (void)lane;
  v += dpp_or_zero<0x111, 0xf>(v);   // row_shr:1
  v += dpp_or_zero<0x112, 0xf>(v);   // row_shr:2
  v += dpp_or_zero<0x114, 0xf>(v);   // row_shr:4
  v += dpp_or_zero<0x118, 0xf>(v);   // row_shr:8
  v += dpp_or_zero<0x142, 0xa>(v);   // row_bcast:15 -> rows 1, 3
  v += dpp_or_zero<0x143, 0xc>(v);   // row_bcast:31 -> rows 2, 3
  return v;
}
// Sum of v over the wavefront, the same value in every lane (the same steps on floats; the order
// of the additions is fixed, so every wavefront of every workgroup gets the same bits).
__device__ __forceinline__ float wave_sum(float v) {
  v += __int_as_float(dpp_or_zero<0x111, 0xf>(__float_as_int(v)));
  v += __int_as_float(dpp_or_zero<0x112, 0xf>(__float_as_int(v)));
  v += __int_as_float(dpp_or_zero<0x114, 0xf>(__float_as_int(v)));
  v += __int_as_float(dpp_or_zero<0x118, 0xf>(__float_as_int(v)));
  v += __int_as_float(dpp_or_zero<0x142, 0xa>(__float_as_int(v)));
  v += __int_as_float(dpp_or_zero<0x143, 0xc>(__float_as_int(v)));
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
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
// table_ptrs: the tables' base addresses, kept in LDS beside the input addresses for models of
// up to kBindKeepAddrs features (required for those, not read otherwise).
// ONE_CAND: every feature has exactly one candidate (a production build): feature f runs
// candidate f and the candidate tables are not read to find that out.
// Returns the total number of tiles.  Ends with a barrier.
//
// A feature's traffic and the tile counts that follow from it are single-precision figures (a
// 64-bit integer division costs some hundred instructions, and every workgroup of every launch
// pays for the binding before its first load: at four features per thread and four workgroups
// per CU the binding's 740 vector instructions kept every SIMD busy for 5 us).  Being off by
// one tile near a boundary changes nothing but the balance, and every workgroup computes the
// same figures.  The divisions that decide which bags a tile holds stay exact.
//
// a / b, exact, for 0 <= a < 2^22 and b >= 1: a single-precision quotient and one step of
// correction either way, a third of the instructions of the 32-bit integer division.  The
// binding takes four quotients per feature that decide which bags a tile holds and must be
// exact; every workgroup of every launch computes them for all features before its first load.
__device__ __forceinline__ int div_small(const int a, const int b) {
  int q = static_cast<int>(static_cast<float>(a) * __builtin_amdgcn_rcpf(static_cast<float>(b)));
  const int r = a - q * b;
  q += r >= b ? 1 : 0;
  q -= r < 0 ? 1 : 0;
  return q;
}
// batches up to which div_small serves (its dividends stay below twice the batch)
constexpr int kSmallDivBatch = 1 << 21;

template <int F, int BT, bool SPLIT = false, bool ONE_CAND = false>
__device__ __forceinline__ int
bind_tiles(BindingStorage<F> &s, const IoView &io, const int tile_bytes,
           const int *__restrict__ lookup_bytes, const int *__restrict__ bag_bytes,
           const int *__restrict__ cand_begin, const int *__restrict__ cand_gran,
           const int *__restrict__ choice, const int *__restrict__ fixed_tiles,
           const int grid_blocks, const int64_t *__restrict__ table_ptrs = nullptr) {
  static_assert(BT <= 16 * 64, "partial sums: at most 16 wavefronts");
  const int tid = threadIdx.x;
  const int B = io.batch;
  // this thread is responsible for features tid, tid + BT, ...
  constexpr int K = (F + BT - 1) / BT;
  // up to 64 features: all of them sit in the first wavefront, which then needs no LDS and no
  // barrier to add up the traffic and to scan the tile counts
  constexpr bool ONE_WAVE = F <= 64;
  float cost[K];            // traffic of the feature in this batch (sizes tiles: 24 bits serve)
  int gran[K];              // bags per workgroup pass of the feature's schedule (kSplitGran: splits)

  // Step 1, the only one that reads memory, in rounds of loads that do not wait for each other
  // (every condition that is the same for all features stands outside the loops over them: a
  // branch inside made the compiler wait for one feature's loads before it issued the next
  // one's, eight round trips in a row where two do): the caller's numbers of the features (a
  // kernel with a tile order); the addresses, the schedule and the per-lookup / per-bag bytes
  // of every feature; then its live lookup count.  Surplus threads repeat the last feature,
  // stores included.
  int64_t offs_at[K], idx_at[K], table_at[K];
  int lookup_b[K], bag_b[K], cand[K], ext_f[K];
  if (io.ext) {
#pragma unroll
    for (int k = 0; k < K; ++k) ext_f[k] = io.ext[min(tid + k * BT, F - 1)];
  } else {
#pragma unroll
    for (int k = 0; k < K; ++k) ext_f[k] = min(tid + k * BT, F - 1);
  }
  // (a model that finds its addresses per tile and gets the lookup counts needs none here)
  if (BindingStorage<F>::kKeepAddrs || !io.counts) {
#pragma unroll
    for (int k = 0; k < K; ++k) io.addrs_at(ext_f[k], idx_at[k], offs_at[k]);
  } else {
#pragma unroll
    for (int k = 0; k < K; ++k) idx_at[k] = offs_at[k] = 0;
  }
  // (the once-per-launch binding kernel has no use for the tables' addresses and passes none)
  if (BindingStorage<F>::kKeepAddrs && table_ptrs) {
#pragma unroll
    for (int k = 0; k < K; ++k) table_at[k] = table_ptrs[ext_f[k]];
  } else {
#pragma unroll
    for (int k = 0; k < K; ++k) table_at[k] = 0;
  }
#pragma unroll
  for (int k = 0; k < K; ++k) {
    const int f = min(tid + k * BT, F - 1);
    cand[k] = f;
    if constexpr (!ONE_CAND) {
      const int first = cand_begin[f];
      const int ncand = cand_begin[f + 1] - first;
      int pick = choice ? choice[f] : 0;
      pick = pick < 0 ? 0 : (pick >= ncand ? ncand - 1 : pick);
      cand[k] = first + pick;
    }
    gran[k] = cand_gran[cand[k]];
    lookup_b[k] = lookup_bytes[f];
    bag_b[k] = bag_bytes[f];
  }
  int lookups[K], first_lookup[K];
  if (fixed_tiles) {
#pragma unroll
    for (int k = 0; k < K; ++k) lookups[k] = first_lookup[k] = 0;
  } else if (io.counts) {                     // one array for all features instead of a line each
#pragma unroll
    for (int k = 0; k < K; ++k) {
      lookups[k] = io.counts[ext_f[k]];
      first_lookup[k] = 0;
    }
  } else {
#pragma unroll
    for (int k = 0; k < K; ++k) {
      const int *offs = global_ptr<int>(offs_at[k]);
      first_lookup[k] = offs[0];
      lookups[k] = offs[B] - first_lookup[k];
    }
  }
  float traffic = 0.f;
#pragma unroll
  for (int k = 0; k < K; ++k) {
    const bool real = tid + k * BT < F;
    const int f = min(tid + k * BT, F - 1);
    cost[k] = 0.f;
    bool one_per_bag = false;
    if (!fixed_tiles) {
      cost[k] = static_cast<float>(lookups[k]) * static_cast<float>(lookup_b[k]) +
                static_cast<float>(B) * static_cast<float>(bag_b[k]);
      traffic += real ? cost[k] : 0.f;
      one_per_bag = lookups[k] == B && first_lookup[k] == 0;
    }
    s.cand[f] = cand[k];
    if constexpr (BindingStorage<F>::kKeepAddrs) {
      s.offsets_addr[f] = offs_at[k];
      s.indices_addr[f] = idx_at[k];
      s.table_addr[f] = table_at[k];
      s.one_per_bag[f] = one_per_bag;
    }
  }

  // Step 2 (only where the tile size or the split unit depend on it): the batch's traffic, in
  // single precision -- it sizes tiles in steps of kilobytes.
  const bool automatic = tile_bytes <= 0 && !fixed_tiles;
  const bool need_total = automatic || (SPLIT && !fixed_tiles);
  int tile_size = tile_bytes;
  long long split_unit = 0;
  if (need_total) {
    float total = wave_sum(traffic);
    if constexpr (!ONE_WAVE) {
      float *partial = reinterpret_cast<float *>(s.partial);
      if ((tid & 63) == 0) partial[tid >> 6] = total;
      __syncthreads();
      total = 0.f;
      for (int w = 0; w < BT / 64; ++w) total += partial[w];
    }
    // the same in every lane: what follows from it is scalar arithmetic
    total = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(total)));
    const long long total_bytes = static_cast<long long>(total);
    if (automatic) tile_size = auto_tile_size(total_bytes, grid_blocks);
    if (SPLIT) {
      const long long grid = grid_blocks > 0 ? grid_blocks : 1;
      split_unit = total_bytes / (4ll * grid);
      if (split_unit < tile_size) split_unit = tile_size;
      if (split_unit < kSplitMinUnit) {
        // whole tiles per workgroup at about the minimum part size, and 6 % of slack for the
        // rounding up of every feature's parts per bag
        const long long per_workgroup = (total_bytes + grid * kSplitMinUnit - 1) / (grid * kSplitMinUnit);
        split_unit = total_bytes / (grid * (per_workgroup > 0 ? per_workgroup : 1));
        split_unit += split_unit >> 4;
        if (split_unit > kSplitMinUnit) split_unit = kSplitMinUnit;
        if (split_unit < kSplitFloorUnit) split_unit = kSplitFloorUnit;
        if (split_unit < tile_size) split_unit = tile_size;
      }
    }
  }

  // Step 3: tiles of every feature, from registers.  Traffic figures in single precision;
  // the quotients that decide which bags a tile holds exact.
  const float tile_f = static_cast<float>(tile_size);
  const float inv_tile = __builtin_amdgcn_rcpf(tile_f);
  const float inv_batch = B > 0 ? __builtin_amdgcn_rcpf(static_cast<float>(B)) : 0.f;
  const float split_unit_f = static_cast<float>(split_unit);
  const bool small = B < kSmallDivBatch;
  // "tiles in plenty" below: (B / g) * F >= kPlentyTilesPerWorkgroup * grid  <=>  B >= g * need
  const int plenty_need = grid_blocks > 0
      ? static_cast<int>((static_cast<long long>(kPlentyTilesPerWorkgroup) * grid_blocks + F - 1) / F) : 0;
  int tiles_of[K];
#pragma unroll
  for (int k = 0; k < K; ++k) {
    const bool real = tid + k * BT < F;
    const int f = min(tid + k * BT, F - 1);
    int g = gran[k];
    const bool may_split = g == kSplitGran && !fixed_tiles;
    if (g == kSplitGran) g = 1;
    // mean traffic of one bag of this feature
    const float bag_cost = cost[k] * inv_batch;
    int tiles;
    if (fixed_tiles) {
      const int want = fixed_tiles[f];
      tiles = want < 1 ? 1 : (want > B ? B : want);
    } else {
      const float want = ceilf(cost[k] * inv_tile);
      tiles = static_cast<int>(fminf(fmaxf(want, 1.f), static_cast<float>(B)));
    }
    int bpt = 0;
    int parts = 1;
    // a bag is split from 1.25 units on (128 x 2 500 lookups: 102.8 us with bags of 1.7 units left
    // whole beside split ones, 89.3 us with those in two parts)
    if (SPLIT && may_split && B > 0 && split_unit > 0 && 4.f * bag_cost > 5.f * split_unit_f) {
      parts = static_cast<int>(fminf(ceilf(bag_cost / split_unit_f), static_cast<float>(kBindMaxParts)));
      if (static_cast<long long>(parts) * B > kBindMaxSplitTiles) parts = kBindMaxSplitTiles / B;
    }
    if (parts > 1) {
      tiles = B * parts;
      bpt = -parts;
    } else if (B > 0) {
      bpt = small ? div_small(B + tiles - 1, tiles) : (B + tiles - 1) / tiles;
      // Tiles are whole workgroup passes (g bags) -- unless one pass of this schedule is more
      // than kMaxTileFactor times the traffic a tile should carry AND whole passes would leave
      // the grid short of tiles: then the tile keeps its share of the traffic and some of the
      // schedule's teams idle (a small batch is spread over more workgroups that way).  With
      // tiles in plenty -- this feature's whole passes times the number of features is at
      // least kPlentyTilesPerWorkgroup tiles per workgroup of the grid -- idle teams are a pure
      // loss: a batch whose bags are twice as long as the tile size was chosen for ran 262 us
      // with a quarter of the wavefronts busy in the long-bag features, 197 us with whole passes.
      const int passes = small ? div_small(bpt + g - 1, g) : (bpt + g - 1) / g;
      const int whole = passes * g;
      const bool plenty = grid_blocks > 0 &&
                          static_cast<long long>(B) >= static_cast<long long>(g) * plenty_need;
      if (fixed_tiles || bpt >= g || plenty ||
          static_cast<float>(whole) * bag_cost <= static_cast<float>(kMaxTileFactor) * tile_f)
        bpt = whole;
      tiles = small ? div_small(B + bpt - 1, bpt) : (B + bpt - 1) / bpt;
    } else {
      tiles = 0;
    }
    // (a surplus thread may have sized its tiles from another wavefront's view of the total)
    if (real) s.bags_per_tile[f] = bpt;
    tiles_of[k] = real ? tiles : 0;
  }

  // Step 4: prefix[f] = first tile of feature f.
  if constexpr (ONE_WAVE) {
    if (tid < 64) {
      const int incl = wave_inclusive_scan(tiles_of[0], tid);
      if (tid < F) s.prefix[tid + 1] = incl;
      if (tid == 0) s.prefix[0] = 0;
    }
  } else {
#pragma unroll
    for (int k = 0; k < K; ++k) {
      const int f = tid + k * BT;
      if (f < F) s.prefix[f + 1] = tiles_of[k];
    }
    if (tid == 0) s.prefix[0] = 0;
    __syncthreads();
    // Two levels, so that no wavefront walks the whole array: every wavefront scans the chunks
    // of 64 features that fall to it, the first wavefront scans the chunks' totals, and every
    // thread adds its chunk's offset.  (One wavefront over all chunks took 0.1 us per chunk:
    // 4 us of a 12 us binding kernel at 2 500 features, 1.6 us of every workgroup's 6 us at
    // 1 000.)
    static_assert(BT % 64 == 0, "whole wavefronts");
    constexpr int CHUNKS = (F + 63) / 64;
    const int lane = tid & 63;
    for (int c = tid >> 6; c < CHUNKS; c += BT / 64) {
      const int i = c * 64 + lane;
      int v = i < F ? s.prefix[i + 1] : 0;
      v = wave_inclusive_scan(v, lane);
      if (i < F) s.prefix[i + 1] = v;
      if (lane == 63) s.chunk_sum[c] = v;
    }
    __syncthreads();
    if (tid < 64) {
      int carry = 0;
      for (int c = 0; c < CHUNKS; c += 64) {
        const int i = c + tid;
        const int v = i < CHUNKS ? s.chunk_sum[i] : 0;
        const int incl = wave_inclusive_scan(v, tid) + carry;
        if (i < CHUNKS) s.chunk_sum[i] = incl - v;       // tiles before the chunk
        carry = __shfl(incl, 63, 64);
      }
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < K; ++k) {
      const int f = tid + k * BT;
      if (f >= 64 && f < F) s.prefix[f + 1] += s.chunk_sum[f >> 6];
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

// The same for a whole wavefront at once (`tile` the same in all its lanes; every lane gets the
// answer): the number of features whose first tile is at or before `tile`, counted 64 features
// at a time with independent LDS reads and ballots instead of log2(F) dependent ones.  Beyond
// 512 features in two levels: the chunk of 64 features (counted the same way over every 64th
// entry), then the feature within it -- two dependent reads where the binary search takes ten
// to fourteen, at the head of every tile.
template <int F>
__device__ __forceinline__ int find_feature_wave(const int *prefix, const int tile) {
  const int lane = threadIdx.x & 63;
  if constexpr (F > 512) {
    constexpr int CHUNKS = (F + 63) / 64;
    int chunk = 0;
#pragma unroll
    for (int base = 0; base < CHUNKS; base += 64) {
      const int c = base + lane + 1;            // prefix[64 c] <= tile: chunk c starts at or before it
      const bool at_or_before = c <= CHUNKS - 1 && prefix[c * 64] <= tile;
      chunk += __builtin_popcountll(__builtin_amdgcn_ballot_w64(at_or_before));
    }
    // lanes 0..62: features 1..63 of the chunk (the next chunk's first feature starts after the tile)
    const int f = chunk * 64 + lane + 1;
    const bool at_or_before = lane < 63 && f <= F - 1 && prefix[f] <= tile;
    return chunk * 64 + __builtin_popcountll(__builtin_amdgcn_ballot_w64(at_or_before));
  } else {
    int count = 0;
#pragma unroll
    for (int base = 0; base < F; base += 64) {
      const int f = base + lane + 1;            // prefix[f] <= tile: feature f starts at or before it
      const bool at_or_before = f <= F - 1 && prefix[f] <= tile;
      count += __builtin_popcountll(__builtin_amdgcn_ballot_w64(at_or_before));
    }
    return count;
  }
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
