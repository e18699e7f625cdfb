"""Feature-specific schedule fusion for gfx950: emits ``process.hip`` (the fused kernel
``FusedKnl`` plus its C-ABI entry points), ``preprocess.cpp`` (the host text front end) and a
``CMakeLists.txt`` that builds both with hipcc / g++.

Keeps the interface of the reference's ``CodeEmitter``
(``RecFlex/code_emitter/codegen.py:20-568``: ``emit``, ``emit_host``, ``emit_cmake_list``,
``serialize_config``, ``emit_if_updated``, de-duplication of identical schedule bodies
``:233-243``, per-feature ``__device__`` tables ``:279-299``, in-kernel timers ``:301-316``).
What is emitted is new:

* The kernel is a persistent grid.  Every workgroup computes the thread binding itself from
  the live offsets (``rfx::bind_tiles``), then walks the tile space with stride ``gridDim.x``
  and dispatches each tile to its feature's schedule body through a ``switch`` (``inline``)
  or through calls to ``__noinline__`` functions.  There is no host-built task mapping.
* Entry points are plain C (``include/recflex_hip.h``), loaded with ``ctypes``; several
  emitted libraries can live in one process.
* Timing builds add each tile's ``s_memtime`` ticks to a per-feature accumulator instead of
  storing one stamp per block.
"""

import json
import os
from typing import Any, Dict, List, NamedTuple, Tuple

from .schedule_base import ScheduleBase, ScheduleVars, PreprocessVars, SPLIT_MAX_TILES, SPLIT_GRANULARITY
from .build_basic import BasicBuilder

# memory traffic (bytes) the run-time binding aims at per tile
DEFAULT_TILE_BYTES = 64 * 1024
SIMDS_PER_CU = 4
MAX_WAVES_PER_SIMD = 8


def waves_per_simd(occupancy: int, block_threads: int) -> int:
    """Wavefronts each SIMD of a CU holds when ``occupancy`` workgroups of ``block_threads``
    threads are resident on it."""
    waves = occupancy * ((block_threads + 63) // 64)
    return max(1, min(MAX_WAVES_PER_SIMD, -(-waves // SIMDS_PER_CU)))


# XCDs (L2 slices) of an MI355X; workgroup i of a launch runs on XCD i % 8
XCD_COUNT = 8
# ``drawn_tail`` of a library all of whose tiles are drawn: more passes than any walk has
DRAWN_ALL = 100000
# per-bag traffic that does not depend on the bag length, besides the output slice: one offset
BAG_FIXED_BYTES = 4
INDEX_BYTES = 4
# The binding sizes tiles by cost = lookups * (row bytes + index + this) + bags * (output + offset):
# a lookup costs time that does not shrink with the row (address arithmetic, a memory round
# trip), expressed here as extra bytes so that tiles of narrow-row features do not run longer
# than tiles of wide-row features.
LOOKUP_OVERHEAD_BYTES = 0
# Models of more features than this, or whose binding tables would not fit into LDS beside the
# build's workgroups per CU, are bound once per launch by a small kernel instead of by every
# workgroup of the fused kernel (rfx::bind_once), unless the emitter is told otherwise
# (``bind_once=``).  Measured on models of 256-bag batches of small features at four workgroups
# per CU, rotated batches, per workgroup against once per launch: 1 000 features 64.7 against
# 69.6 us, 2 500 features 174.1 against 178.7 us (the binding kernel takes 7.2 us there and the
# workgroups still copy the prefix array, 2.9 us; every workgroup binding for itself takes 10).
# Before the binding's arithmetic and loads were trimmed it cost every workgroup 10 us per
# thousand features and the limit stood at 2 048.
BIND_ONCE_MIN_FEATS = 3072
# LDS of a CU, and what a workgroup's binding tables take per feature (prefix, bags per tile,
# schedule; the second level of the prefix sum) beside an allowance for the schedules' own
LDS_BYTES_PER_CU = 160 * 1024
BIND_LDS_ALLOWANCE = 4096


def binds_once_by_default(num_feats: int, occupancy: int = None) -> bool:
    if num_feats > BIND_ONCE_MIN_FEATS:
        return True
    tables = (num_feats + 1) * 4 + num_feats * 8 + (num_feats + 63) // 64 * 4 + 128
    return tables + BIND_LDS_ALLOWANCE > LDS_BYTES_PER_CU // (occupancy or 4)
# a bag becomes tiles of its own (libraries emitted with outliers=True) from this much traffic
OUTLIER_MIN_BYTES = 128 * 1024


def outlier_capacity(num_feats: int) -> int:
    """Entries of the outlier list of a library emitted with outlier tiles (four parts each)."""
    return 4096 if num_feats <= 128 else 16384


def _c_array(ctype: str, name: str, values: List[int], per_line: int = 16) -> str:
    lines = []
    for i in range(0, len(values), per_line):
        lines.append("    " + ", ".join(str(v) for v in values[i:i + per_line]))
    body = ",\n".join(lines) if lines else "    0"
    return f"__constant__ {ctype} {name}[] = {{\n{body}\n}};\n\n"


class CodeEmitter:
    def __init__(self, feat_schedules: List[Tuple[ScheduleBase, NamedTuple]],
                 feat_candidates: List[List[Tuple[ScheduleBase, NamedTuple]]] = None):
        """``feat_schedules[f]`` is the schedule of feature ``f``.  A tuning build may instead
        give ``feat_candidates[f]``, the list of schedules feature ``f`` can run; the launch then
        picks one per feature at run time (``d_schedule_choice``), and ``feat_schedules`` is
        taken to be each list's first entry."""
        if feat_candidates is not None:
            assert all(len(c) > 0 for c in feat_candidates)
            feat_schedules = [tuple(c[0]) for c in feat_candidates]
        self.feat_schedules: List[Tuple[ScheduleBase, NamedTuple]] = feat_schedules
        self.feat_candidates = ([[tuple(sp) for sp in c] for c in feat_candidates]
                                if feat_candidates is not None
                                else [[tuple(sp)] for sp in feat_schedules])
        if len(self.feat_schedules) > 0:
            self.block_threads: int = feat_schedules[0][0].block_threads
            for cands in self.feat_candidates:
                for schedule, params in cands:
                    assert self.block_threads == schedule.block_threads
                    assert schedule.meta == cands[0][0].meta, "candidates of a feature share its table"

    # ------------------------------------------------------------------ configuration dump

    def serialize_config(self) -> List[Dict[str, Any]]:
        return [
            {
                "schedule": schedule.__class__.__name__,
                "params": params._asdict(),
                "embed_dim": schedule.meta.embed_dim,
                "data_type": schedule.meta.data_type,
            }
            for schedule, params in self.feat_schedules
        ]

    def serialize_candidates(self) -> List[List[Dict[str, Any]]]:
        return [CodeEmitter(cands).serialize_config() for cands in self.feat_candidates]

    def dump_key(self, fname: str) -> None:
        with open(fname, "w") as f:
            json.dump(self.serialize_config(), fp=f, indent=1)

    # ------------------------------------------------------------------ derived tables

    def embed_dims(self) -> List[int]:
        return [sched.meta.embed_dim for sched, _ in self.feat_schedules]

    def embed_dim_offsets(self) -> List[int]:
        offsets = [0]
        for d in self.embed_dims():
            offsets.append(offsets[-1] + d)
        return offsets

    def out_vec(self) -> int:
        """Widest output store (floats) that is aligned for every feature's column offset."""
        offs = self.embed_dim_offsets()
        for w in (4, 2):
            if all(o % w == 0 for o in offs):
                return w
        return 1

    def flat_candidates(self) -> Tuple[List[Tuple[ScheduleBase, NamedTuple]], List[int]]:
        """All candidates in feature order, and ``begin[f]`` = index of feature f's first one."""
        flat, begin = [], [0]
        for cands in self.feat_candidates:
            flat.extend(cands)
            begin.append(len(flat))
        return flat, begin

    def split_regions(self) -> Tuple[List[int], int]:
        """Workspace of the schedules that split bags over workgroups: the first float of each
        feature's region (-1 for a feature none of whose candidates needs one; a feature's
        candidates share its region, only one of them runs in a launch) and the total floats."""
        regions, total = [], 0
        for cands in self.feat_candidates:
            need = max(schedule.WorkspaceFloats(params) for schedule, params in cands)
            need = (need + 31) // 32 * 32          # regions start on 128-byte boundaries
            regions.append(total if need else -1)
            total += need
        return regions, total

    def long_bag_tables(self) -> Tuple[List[int], List[Tuple[int, int]], List[int]]:
        """For a build with outlier tiles: per feature the bag length beyond which a bag is run
        as tiles of its own (beyond its schedule's threshold and carrying at least
        OUTLIER_MIN_BYTES of traffic; 0 = none), the distinct
        (element type, dim) pairs of the features that have one, and per feature the index of
        its pair (-1 = none)."""
        thr, keys, body_of = [], [], []
        for cands in self.feat_candidates:
            t = self._schedule_reach(cands)
            if t > 0:
                per_lookup = cands[0][0].meta.row_bytes + INDEX_BYTES
                t = max(t, -(-OUTLIER_MIN_BYTES // per_lookup))
            thr.append(t)
            key = (cands[0][0].meta.dtype_id, cands[0][0].meta.embed_dim)
            if t > 0 and key not in keys:
                keys.append(key)
            body_of.append(keys.index(key) if t > 0 else -1)
        return thr, keys, body_of

    @staticmethod
    def _schedule_reach(cands) -> int:
        """The bag length beyond which the feature's schedule hands a bag to a whole wavefront
        (0 = a schedule that handles long bags itself)."""
        t = [schedule.LongBagThreshold(params) for schedule, params in cands]
        return 0 if min(t) <= 0 else max(t)

    @staticmethod
    def _meta_of(dtype_id: int, dim: int):
        from .schedule_base import MetaData
        return MetaData(dim, ("float", "half", "int8")[dtype_id])

    def dedup(self) -> Tuple[Dict[int, int], List[int]]:
        """candidate index -> index of the first candidate with the same (LDS type, body); list
        of those first indices.  With one schedule per feature, candidate index == feature."""
        seen: Dict[str, int] = {}
        id_map: Dict[int, int] = {}
        flat, _ = self.flat_candidates()
        for idx, (schedule, params) in enumerate(flat):
            key = schedule.EmitShmemType(params) + "\n" + schedule.EmitScheduleBody(params)
            if key not in seen:
                seen[key] = idx
            id_map[idx] = seen[key]
        return id_map, list(seen.values())

    # ------------------------------------------------------------------ device code

    def emit_headers(self) -> str:
        headers = {"<hip/hip_runtime.h>", "<stdint.h>", '"recflex_hip.h"', '"rfx_binding.hip.h"',
                   '"rfx_launch.hip.h"', '"rfx_outliers.hip.h"', '"rfx_schedules.hip.h"'}
        for schedule, params in self.feat_schedules:
            headers = headers.union(schedule.EmitHeaders())
        return ''.join(sorted(f"#include {header}\n" for header in headers)) + '\n'

    def emit_kernel(self, occupancy: int = None, inline: bool = True, timing: bool = False,
                    timing_branch: bool = False, fixed_task_block_nums: List[int] = None,
                    tile_bytes: int = None, xcd_aware: bool = False,
                    lookup_overhead_bytes: int = None, xcd_segments: int = 8,
                    outliers: bool = False, bind_once: bool = None,
                    tile_order: List[int] = None, drawn_tail: int = 0) -> str:
        num_feats = len(self.feat_schedules)
        if lookup_overhead_bytes is None:
            lookup_overhead_bytes = LOOKUP_OVERHEAD_BYTES
        assert num_feats > 0, "cannot emit a fused kernel for zero features"
        vars_ = ScheduleVars()
        id_map, body_ids = self.dedup()
        flat, cand_begin = self.flat_candidates()
        embed_dim_offsets = self.embed_dim_offsets()
        if bind_once is None:
            bind_once = binds_once_by_default(num_feats, occupancy)
        split_regions, workspace_floats = self.split_regions()
        has_split = workspace_floats > 0
        assert not (outliers and (timing or fixed_task_block_nums)), \
            "outlier tiles are for production builds (no per-feature timers, no frozen binding)"
        # the list of outliers is made with one threshold per feature, which the feature's body
        # must share: one schedule per feature
        assert not outliers or all(len(c) == 1 for c in self.feat_candidates)
        long_thr, long_keys, long_body_of = self.long_bag_tables() if outliers else ([], [], [])
        outliers = outliers and len(long_keys) > 0
        # Tile order: place p of the kernel's tile space holds feature tile_order[p] of the model.
        # Inside the kernel a feature's number is its place: every per-feature table below is
        # emitted in that order, and what the caller passes per feature is found through
        # c_ext_feat (rfx::IoView::ext).  Everything the library says about itself to the host
        # (recom_get_feature_tables ...) stays in the model's order.
        if tile_order is not None:
            tile_order = [int(f) for f in tile_order]
            assert sorted(tile_order) == list(range(num_feats)), "tile_order must be a permutation of the features"
            assert all(len(c) == 1 for c in self.feat_candidates) and not timing and not fixed_task_block_nums, \
                "a tile order goes with a production build (one schedule per feature, no timers, no frozen binding)"
            if tile_order == list(range(num_feats)):
                tile_order = None

        def placed(per_feature: list) -> list:
            return [per_feature[f] for f in tile_order] if tile_order is not None else list(per_feature)
        # the last passes of the tile walk drawn from ticket counters (rfx::TailTickets) instead
        # of dealt out: a production option, and the outlier tiles have their own drawn end
        assert not (drawn_tail and (outliers or timing or fixed_task_block_nums)), \
            "drawn_tail goes with neither outlier tiles nor timers nor a frozen binding"
        max_long_dim = max([(d + 3) // 4 * 4 for _, d in long_keys], default=4)
        fixed_arg = "c_fixed_task_block_nums" if fixed_task_block_nums else "nullptr"

        consts = f'''constexpr int NUM_FEATS = {num_feats};
constexpr int {vars_.EMBED_DIM_SUM} = {embed_dim_offsets[-1]};
constexpr int {vars_.BLOCK_THREADS} = {self.block_threads};
constexpr int {vars_.out_vec} = {self.out_vec()};
constexpr int OCCUPANCY = {occupancy if occupancy else 0};
constexpr int TILE_BYTES = {tile_bytes if tile_bytes else 0};     // 0: chosen per batch (rfx::kAutoTile*)
constexpr int NUM_BODIES = {len(body_ids)};
constexpr int NUM_CANDIDATES = {len(flat)};
constexpr int XCDS = {XCD_COUNT};
constexpr int XCD_SEGMENTS = {xcd_segments if xcd_aware else 0};
constexpr bool TIMING = {"true" if timing else "false"};
constexpr bool STATIC_BINDING = {"true" if fixed_task_block_nums else "false"};
#define RFX_BIND_ONCE {1 if bind_once else 0}
constexpr bool BIND_ONCE = RFX_BIND_ONCE;
static_assert(rfx::kBindKeepAddrs == 512, "the emitter decides by this where a tile finds its addresses");
// bytes of workspace the split-bag schedules need (0: no schedule splits bags)
constexpr long long SPLIT_BYTES = {workspace_floats * 4}LL;
#define RFX_HAS_SPLIT {1 if workspace_floats > 0 else 0}
constexpr bool HAS_SPLIT = SPLIT_BYTES > 0;
// outlier bags found ahead of the kernel and run as tiles of their own (rfx_outliers.hip.h)
#define RFX_OUTLIERS {1 if outliers else 0}
constexpr bool OUTLIERS = RFX_OUTLIERS;
constexpr int MAX_LONG_DIM = {max_long_dim};
// ... or, in their place in the workspace, the ticket counters of a drawn end of the tile walk
#define RFX_DRAWN_TAIL {int(drawn_tail)}
#define RFX_DRAWN_ALL {DRAWN_ALL}      // from this many passes on: every tile is drawn
constexpr int DRAWN_TAIL = RFX_DRAWN_TAIL;
static_assert(!(OUTLIERS && DRAWN_TAIL > 0), "one or the other");
using OutlierSpace = {"rfx::TailTickets" if drawn_tail else f"rfx::OutlierSpace<MAX_LONG_DIM, {outlier_capacity(num_feats)}>"};
constexpr long long OUTLIER_BYTES = OUTLIERS || DRAWN_TAIL > 0 ? (long long)sizeof(OutlierSpace) : 0LL;
#define RFX_TILE_ORDER {1 if tile_order is not None else 0}
// the binding table of a model that is bound once per launch (rfx::bind_once) comes last
constexpr long long BOUND_OFFSET = (SPLIT_BYTES + OUTLIER_BYTES + 255) / 256 * 256;
constexpr long long BOUND_BYTES = BIND_ONCE ? (long long)sizeof(rfx::BoundTables<NUM_FEATS>) : 0LL;
constexpr long long WORKSPACE_BYTES = BIND_ONCE ? BOUND_OFFSET + BOUND_BYTES : SPLIT_BYTES + OUTLIER_BYTES;
// recom_process_static_workspace: the same workspace as a file-scope device array of the library
constexpr long long STATIC_WORKSPACE_MAX = RECOM_STATIC_WORKSPACE_MAX_BYTES;
constexpr bool STATIC_WORKSPACE_FITS = WORKSPACE_BYTES <= STATIC_WORKSPACE_MAX;
constexpr long long STATIC_WORKSPACE_BYTES =
    STATIC_WORKSPACE_FITS && WORKSPACE_BYTES > 0 ? WORKSPACE_BYTES : 256;
static_assert(rfx::kBindMaxSplitTiles == {SPLIT_MAX_TILES} && rfx::kSplitGran == {SPLIT_GRANULARITY},
              "workspace regions were sized for this");

'''

        temp_storage_decl = "union KnlTempStorage {\n"
        functions = ""
        flat, cand_begin = self.flat_candidates()
        for feat_idx in body_ids:
            schedule, params = flat[feat_idx]
            temp_storage_decl += f"  {schedule.EmitShmemType(params)} f{feat_idx};\n"
            functions += f'''
__device__ {"__forceinline__" if inline else "__noinline__"} void ProcessFeat{feat_idx}(
    const char *__restrict__ {vars_.embed_table},
    const int *__restrict__ {vars_.indices},
    const int *__restrict__ {vars_.offsets},
    float *__restrict__ {vars_.output},
    const int {vars_.out_row_stride}, const int {vars_.embed_dim_offset},
    const int {vars_.bag_begin}, const int {vars_.bag_end},
    char *__restrict__ {vars_.shmem}, rfx::f32x4 *__restrict__ {vars_.stage},
    const int {vars_.split_part}, const int {vars_.split_parts},
    float *__restrict__ {vars_.split_region}, const int {vars_.skip_long},
    const int {vars_.one_per_bag}, rfx::MidBagQueue *{vars_.mid_queue}, const int {vars_.feat_id}) {{
  (void){vars_.mid_queue}; (void){vars_.feat_id};
  {schedule.EmitScheduleBody(params)}
}}
'''
        # one block-wide body per (element type, dim) that can have outliers
        long_cases, mid_cases = "", ""
        for k, (dtype_id, dim) in enumerate(long_keys):
            mid_cases += (f"        case {k}: rfx::wave_bag<{dtype_id}, {dim}, {self.out_vec()}>"
                          "(table, indices, beg, end, dst, lane); break;\n")
            meta = self._meta_of(dtype_id, dim)
            lanes = min(64, 1 << (meta.row_vectors - 1).bit_length())
            items = 4 if meta.elems_per_vector <= 4 else 2
            storage = (f"rfx::BlockBagStorage<{vars_.BLOCK_THREADS}, {dtype_id}, {dim}, {lanes}, "
                       f"{4 * self.block_threads}>")
            temp_storage_decl += f"  {storage} long{k};\n"
            long_cases += f'''        case {k}:
          rfx::split_part<{vars_.BLOCK_THREADS}, {dtype_id}, {dim}, {lanes}, {items}, {4 * self.block_threads}>(
              *reinterpret_cast<{storage} *>(&s), table, indices, offsets, d_output,
              {vars_.out_row_stride}, embed_dim_offset, e.bag, part, e.parts,
              &d_outliers->slots[e.first][0], MAX_LONG_DIM, &d_outliers->counters[entry]);
          break;
'''
        temp_storage_decl += "};\n\n"

        tables = _c_array("int", "c_cand_begin", cand_begin)
        if tile_order is not None:
            # one candidate per feature: a candidate's number is its feature's
            tables += _c_array("int", "c_cand_func_ids", placed([id_map[i] for i in range(len(flat))]))
            tables += _c_array("int", "c_cand_gran", placed([s.TileGranularity(p) for s, p in flat]))
            tables += _c_array("int", "c_ext_feat", tile_order)
        else:
            tables += _c_array("int", "c_cand_func_ids", [id_map[i] for i in range(len(flat))])
            tables += _c_array("int", "c_cand_gran", [s.TileGranularity(p) for s, p in flat])
        # first output column of every feature, and (last entry) the width of the output
        tables += _c_array("int", "c_embed_dim_offsets", placed(embed_dim_offsets[:-1]) + [embed_dim_offsets[-1]])
        tables += _c_array("int", "c_embed_dims", placed([s.meta.embed_dim for s, _ in self.feat_schedules]))
        tables += _c_array("int", "c_lookup_bytes",
                           placed([s.meta.row_bytes + INDEX_BYTES + lookup_overhead_bytes
                                   for s, _ in self.feat_schedules]))
        tables += _c_array("int", "c_bag_bytes",
                           placed([s.meta.embed_dim * 4 + BAG_FIXED_BYTES for s, _ in self.feat_schedules]))
        if has_split:
            # first float of each feature's region of the workspace (-1: the feature has none)
            tables += _c_array("long long", "c_split_region", placed(split_regions))
        if outliers:
            tables += _c_array("int", "c_long_thr", placed(long_thr))
            tables += _c_array("int", "c_long_body", placed(long_body_of))
        if fixed_task_block_nums:
            assert len(fixed_task_block_nums) == num_feats
            tables += _c_array("int", "c_fixed_task_block_nums",
                               [max(1, int(n)) for n in fixed_task_block_nums])

        # Timing builds: each workgroup adds the ticks of its tiles per feature in LDS and flushes
        # them to d_times once, when it has run out of tiles (an atomic per tile would sit in front
        # of the next tile's loads).  With d_times == nullptr a timing build runs untimed.
        timing_begin = '''
    unsigned long long t_begin = 0;
    if (d_times) {
      __syncthreads();
      t_begin = __builtin_amdgcn_s_memtime();
    }
''' if timing else ''
        timing_end = '''
    if (d_times) {
      __syncthreads();
      if (threadIdx.x == 0)
        s_ticks[feat_idx] += static_cast<unsigned int>(__builtin_amdgcn_s_memtime() - t_begin);
    }
''' if timing else ''
        timing_init = f'''
  __shared__ unsigned int s_ticks[NUM_FEATS];
  const unsigned long long t_kernel_begin = d_times ? wall_clock64() : 0;
  if (d_times)
    for (int f = threadIdx.x; f < NUM_FEATS; f += {vars_.BLOCK_THREADS}) s_ticks[f] = 0;
''' if timing else ''
        # ticks every workgroup spends before its first tile (the binding), entry NUM_FEATS
        timing_bound = '''
  const unsigned long long t_bound = d_times ? wall_clock64() : 0;
''' if timing else ''
        timing_flush = f'''
  if (d_times) {{
    __syncthreads();
    // the workgroup's end: before the counters are flushed, which is not part of its work
    const unsigned long long t_kernel_end = wall_clock64();
    for (int f = threadIdx.x; f < NUM_FEATS; f += {vars_.BLOCK_THREADS})
      if (s_ticks[f]) atomicAdd(&d_times[f], static_cast<unsigned long long>(s_ticks[f]));
    if (threadIdx.x == 0) {{
      // beyond the per-feature entries, on the constant 100 MHz clock (10 ns; the per-feature
      // ticks count shader cycles): the workgroup's time before its first tile, and all of it
      atomicAdd(&d_times[NUM_FEATS], t_bound - t_kernel_begin);
      atomicAdd(&d_times[NUM_FEATS + 1], t_kernel_end - t_kernel_begin);
    }}
  }}
''' if timing else ''

        need_stage = self.out_vec() == 4 and any(flat[i][0].NeedsOutputStage(flat[i][1]) for i in body_ids)
        stage_decl = (f"  __shared__ rfx::TeamStage<{vars_.BLOCK_THREADS}> s_stage;\n" if need_stage else "")
        call_args = (f"table, indices, offsets, d_output, {vars_.out_row_stride}, embed_dim_offset, "
                     f"{vars_.bag_begin}, {vars_.bag_end}, reinterpret_cast<char *>(&s), "
                     + ("&s_stage.seg[0][0]" if need_stage else "nullptr")
                     + f", {vars_.split_part}, {vars_.split_parts}, {vars_.split_region}, {vars_.skip_long}"
                     + f", {vars_.one_per_bag}, {vars_.mid_queue}, feat_idx")
        cases = "".join(
            f"      case {feat_idx}: ProcessFeat{feat_idx}({call_args}); break;\n"
            for feat_idx in body_ids)

        # the register budget that lets `occupancy` workgroups share a CU: hipcc reads the second
        # argument of __launch_bounds__ as wavefronts per SIMD, not workgroups per CU (the two are
        # the same number only for 256-thread workgroups on four SIMDs)
        launch_bounds = (f"__launch_bounds__({vars_.BLOCK_THREADS}, "
                         f"{waves_per_simd(occupancy, self.block_threads)})" if occupancy
                         else f"__launch_bounds__({vars_.BLOCK_THREADS})")
        if bind_once:
            bind_decl = "  __shared__ rfx::PrefixStorage<NUM_FEATS> s_bind;\n"
            bind_call = (f"  const int regular_tiles = rfx::load_prefix<NUM_FEATS, {vars_.BLOCK_THREADS}>"
                         "(s_bind, d_bound);\n  (void)tile_bytes;\n  (void)d_schedule_choice;")
            bound_src = "d_bound->"
        else:
            bind_decl = "  __shared__ rfx::BindingStorage<NUM_FEATS> s_bind;\n"
            bind_call = (f"  const int regular_tiles = rfx::bind_tiles<NUM_FEATS, {vars_.BLOCK_THREADS}, HAS_SPLIT,\n"
                         "                                            NUM_CANDIDATES == NUM_FEATS>(\n"
                         "      s_bind, io, tile_bytes, c_lookup_bytes, c_bag_bytes, c_cand_begin, c_cand_gran,\n"
                         f"      d_schedule_choice, {fixed_arg}, gridDim.x, d_embed_table_ptrs);\n  (void)d_bound;")
            bound_src = "s_bind."
        bind_kernel = f'''
// One workgroup binds the whole model for this launch (models of thousands of features).
extern "C" __global__ void __launch_bounds__(1024) BindKnl(
    const int64_t *__restrict__ d_io_ptrs, const char *__restrict__ d_arg_buffers,
    const int64_t *__restrict__ d_arg_buffer_offsets, const int batch, const int tile_bytes,
    const int *__restrict__ d_schedule_choice, const int grid_blocks,
    rfx::BoundTables<NUM_FEATS> *__restrict__ d_bound, const int *__restrict__ d_lookup_counts) {{
  __shared__ rfx::BindingStorage<NUM_FEATS> s_bind;
  const rfx::IoView io{{d_io_ptrs, d_arg_buffers, d_arg_buffer_offsets, batch, d_lookup_counts, {"c_ext_feat" if tile_order is not None else "nullptr"}}};
  rfx::bind_once<NUM_FEATS, 1024, HAS_SPLIT>(s_bind, d_bound, io, tile_bytes, c_lookup_bytes, c_bag_bytes,
                                  c_cand_begin, c_cand_gran, d_schedule_choice, {fixed_arg},
                                  grid_blocks);
}}
''' if bind_once else ''

        outlier_kernel = f'''
// Finds the bags that are too long for their feature's schedule (one thread per bag).
extern "C" __global__ void __launch_bounds__(256) OutlierKnl(
    const int64_t *__restrict__ d_io_ptrs, const char *__restrict__ d_arg_buffers,
    const int64_t *__restrict__ d_arg_buffer_offsets, const int batch,
    OutlierSpace *__restrict__ d_outliers) {{
  const rfx::IoView io{{d_io_ptrs, d_arg_buffers, d_arg_buffer_offsets, batch, nullptr,
                       {"c_ext_feat" if tile_order is not None else "nullptr"}}};
  rfx::find_outliers<NUM_FEATS>(d_outliers, io, c_long_thr, c_lookup_bytes);
}}
''' if outliers else ''
        outlier_begin = f'''
  // the parts of the outlier bags of this batch (0: none, or more than the list holds)
  const int outlier_tiles = rfx::outlier_parts(d_outliers);
  const int total_tiles = regular_tiles;
  // mid-size bags wait here for a wavefront of this workgroup
  __shared__ rfx::MidBagQueue s_mid_queue;
  rfx::mid_queue_init<{vars_.BLOCK_THREADS}>(&s_mid_queue);
  __syncthreads();
  rfx::MidBagQueue *const {vars_.mid_queue} = &s_mid_queue;
''' if outliers else f'''
  const int total_tiles = regular_tiles;
  (void)d_outliers;
  rfx::MidBagQueue *const {vars_.mid_queue} = nullptr;
'''
        drain_call = (f"if (rfx::mid_queue_pending({vars_.mid_queue})) DrainMidBags({vars_.mid_queue}, "
                      f"d_embed_table_ptrs, io, d_output, {vars_.out_row_stride});")
        # between its tiles a wavefront sums mid-size bags that wait in the workgroup's list
        loop_tail = f"    {drain_call}\n" if outliers else ""
        loop_head = '''  for (int walk = walk_first; walk < walk_last; walk += walk_step) {
    int tile = walk;
    if (by_xcd) {
      const int seg = walk / seg_len;
      tile = (seg * XCDS + xcd) * seg_len + (walk - seg * seg_len);
      if (tile >= total_tiles) continue;
    }
'''
        # Outlier parts are not dealt out with the regular tiles: a workgroup that has run its
        # regular tiles draws parts from a ticket counter until none is left.  The next ticket is
        # requested before the current part runs, so that its round trip is hidden behind the part.
        # (Regular tiles held back and drawn the same way after the parts, to even out the end,
        # were tried: a drawn tile needs the workgroup's wavefronts together, and with skewed bags
        # each such tile waits for its slowest wavefront -- 191-210 us against 171.)
        outlier_end = f'''
  // A wavefront without regular tiles left takes mid-size bags until the last wavefront of the
  // workgroup has finished its tiles and the list is empty.
  rfx::mid_queue_walk_done({vars_.mid_queue});
  for (;;) {{
    const bool open = rfx::mid_queue_open({vars_.mid_queue});
    if (rfx::mid_queue_pending({vars_.mid_queue}))
      DrainMidBags({vars_.mid_queue}, d_embed_table_ptrs, io, d_output, {vars_.out_row_stride});
    else if (!open)
      break;
    else
      __builtin_amdgcn_s_sleep(8);
  }}
  if (outlier_tiles > 0) {{
    __shared__ int s_ticket[2];
    int slot = 0;
    if (threadIdx.x == 0) s_ticket[0] = rfx::draw_outlier_part(d_outliers);
    for (;;) {{
      __syncthreads();
      const int tile = s_ticket[slot];
      if (tile >= outlier_tiles) break;
      int next = 0;
      if (threadIdx.x == 0) next = rfx::draw_outlier_part(d_outliers);
      const int entry = d_outliers->partmap[tile];
      const rfx::OutlierEntry e = d_outliers->entries[entry];
      const int part = tile - e.first;
      const char *table = rfx::global_ptr<char>(d_embed_table_ptrs[io.ext_of(e.feat)]);
      const int *indices = io.indices(e.feat);
      const int *offsets = io.offsets(e.feat);
      const int embed_dim_offset = c_embed_dim_offsets[e.feat];
      switch (c_long_body[e.feat]) {{
{long_cases.replace(chr(10) + "  ", chr(10))}        default: break;
      }}
      slot ^= 1;
      if (threadIdx.x == 0) s_ticket[slot] = next;
    }}
  }}
  __syncthreads();
  if (threadIdx.x == 0) rfx::outliers_done(d_outliers);
''' if outliers else ''
        drawn_begin = ''
        if drawn_tail:
            # every tile drawn: a workgroup's first ticket does not wait for the binding
            drawn_begin = '''
  int first_ticket = 0;
  if (DRAWN_TAIL >= RFX_DRAWN_ALL && threadIdx.x == 0)
    first_ticket = rfx::draw_tail_ticket(d_outliers, xcd_segments > 0 && gridDim.x % XCDS == 0 ? blockIdx.x % XCDS : 0);
'''
            loop_head = f'''  // The last DRAWN_TAIL passes of the walk are drawn: tickets of this workgroup's XCD (of the
  // whole device for a flat walk) count on from static_last.  A ticket is asked for one tile
  // ahead, so that its round trip hides behind a tile's work -- except the first one after the
  // dealt tiles, which a workgroup asks for only when those are done (asked for with its last
  // dealt tile, a workgroup that is late would be bound to one more tile before it knows: a
  // thousand features of five tiles per workgroup took 69.6 us that way, 68.6 us with the
  // round trip in the open).  When every tile is drawn, the first ticket is asked for ahead
  // of the binding.
  rfx::TailTickets *const d_tickets = d_outliers;
  __shared__ int s_ticket[2];
  const int static_last = DRAWN_TAIL >= RFX_DRAWN_ALL ? 0 :
      static_cast<int>(max(0ll, walk_last - static_cast<long long>(DRAWN_TAIL) * walk_step));
  int walk = walk_first, ticket_slot = 0, next_ticket = 0;
  bool drawing = false;
  for (;;) {{
    int at = 0;
    if (!drawing) {{
      if (walk < static_last) {{
        at = walk;
        walk += walk_step;
      }} else {{
        drawing = true;
        if (threadIdx.x == 0)
          s_ticket[0] = DRAWN_TAIL >= RFX_DRAWN_ALL ? first_ticket : rfx::draw_tail_ticket(d_tickets, xcd);
        continue;
      }}
    }} else {{
      __syncthreads();                         // the ticket is there, the previous tile is done
      at = static_last + s_ticket[ticket_slot];
      if (at >= walk_last) break;
      if (threadIdx.x == 0) next_ticket = rfx::draw_tail_ticket(d_tickets, xcd);
      ticket_slot ^= 1;
    }}
    int tile = at;
    if (by_xcd) {{
      const int seg = at / seg_len;
      tile = (seg * XCDS + xcd) * seg_len + (at - seg * seg_len);
    }}
    if (tile >= total_tiles) {{
      if (drawing && threadIdx.x == 0) s_ticket[ticket_slot] = next_ticket;
      continue;
    }}
'''
            loop_tail = '''    if (drawing && threadIdx.x == 0) s_ticket[ticket_slot] = next_ticket;
'''
            outlier_end = '''
  __syncthreads();
  if (threadIdx.x == 0) rfx::tail_tickets_done(d_tickets);
'''
        drain_func = f'''
// Sums mid-size bags from the workgroup's list for as long as the calling wavefront gets one.
__device__ __noinline__ void DrainMidBags(
    rfx::MidBagQueue *q, const int64_t *__restrict__ d_embed_table_ptrs, const rfx::IoView io,
    float *__restrict__ d_output, const int out_row_stride) {{
  const int lane = threadIdx.x & 63;
  int feat = 0, bag = 0;
  while (rfx::mid_queue_pop(q, &feat, &bag)) {{
    const char *table = rfx::global_ptr<char>(d_embed_table_ptrs[io.ext_of(feat)]);
    const int *indices = io.indices(feat);
    const int *offsets = io.offsets(feat);
    const int beg = __builtin_amdgcn_readfirstlane(offsets[bag]);
    const int end = __builtin_amdgcn_readfirstlane(offsets[bag + 1]);
    float *dst = d_output + static_cast<int64_t>(bag) * out_row_stride + c_embed_dim_offsets[feat];
    switch (c_long_body[feat]) {{
{mid_cases}      default: break;
    }}
  }}
}}
''' if outliers else ''
        # rfx::kBindKeepAddrs: the binding of a model of up to 512 features keeps every feature's
        # table / indices / offsets address in LDS, and whether the batch holds one lookup per bag
        keep_addrs = not bind_once and num_feats <= 512
        feature_addrs = f'''    // the feature's addresses, which the binding kept in LDS
    const char *table = rfx::global_ptr<char>(rfx::uniform64(s_bind.table_addr[feat_idx]));
    const int *indices = rfx::global_ptr<int>(rfx::uniform64(s_bind.indices_addr[feat_idx]));
    const int *offsets = rfx::global_ptr<int>(rfx::uniform64(s_bind.offsets_addr[feat_idx]));
    const int {vars_.one_per_bag} = __builtin_amdgcn_readfirstlane(s_bind.one_per_bag[feat_idx]);
''' if keep_addrs else f'''    const char *table = rfx::global_ptr<char>(d_embed_table_ptrs[io.ext_of(feat_idx)]);
    const int *indices = io.indices(feat_idx);
    const int *offsets = io.offsets(feat_idx);
    const int {vars_.one_per_bag} = 0;
'''
        kernel = bind_kernel + outlier_kernel + drain_func + f'''
extern "C" __global__ void {launch_bounds} FusedKnl(
    const int64_t *__restrict__ d_embed_table_ptrs,
    const int64_t *__restrict__ d_io_ptrs,
    const char *__restrict__ d_arg_buffers,
    const int64_t *__restrict__ d_arg_buffer_offsets,
    float *__restrict__ d_output,
    const int batch, const int tile_bytes, const int xcd_segments,
    const int *__restrict__ d_schedule_choice,
    unsigned long long *__restrict__ d_times, const int {vars_.out_row_stride},
    const rfx::BoundTables<NUM_FEATS> *__restrict__ d_bound, float *__restrict__ d_workspace,
    OutlierSpace *__restrict__ d_outliers, const int *__restrict__ d_lookup_counts) {{
{bind_decl}
  __shared__ KnlTempStorage s;
{stage_decl}{timing_init}{drawn_begin}
  const rfx::IoView io{{d_io_ptrs, d_arg_buffers, d_arg_buffer_offsets, batch, d_lookup_counts, {"c_ext_feat" if tile_order is not None else "nullptr"}}};
{bind_call}
{timing_bound}
{outlier_begin}
  // Tiles are ordered by feature.  Workgroup i runs on XCD i % XCDS.  With xcd_segments > 0 the
  // tile space is cut into XCDS * xcd_segments equal segments and segment s belongs to XCD
  // s % XCDS: a feature's tiles
  // -- and the table rows its bags share -- stay in the L2 of one or two XCDs instead of being
  // fetched into all of them, while every XCD still gets a sample of all kinds of features.
  int walk_first = blockIdx.x, walk_last = total_tiles, walk_step = gridDim.x;
  int xcd = 0, seg_len = 1;
  const bool by_xcd = xcd_segments > 0 && gridDim.x % XCDS == 0;
  if (by_xcd) {{
    seg_len = (total_tiles + XCDS * xcd_segments - 1) / (XCDS * xcd_segments);
    xcd = blockIdx.x % XCDS;
    walk_first = blockIdx.x / XCDS;
    walk_last = seg_len * xcd_segments;
    walk_step = gridDim.x / XCDS;
  }}
{loop_head}
{timing_begin if timing and timing_branch else ''}
    const int feat_idx = __builtin_amdgcn_readfirstlane(rfx::find_feature_wave<NUM_FEATS>(s_bind.prefix, tile));
    const int bags_per_tile = {bound_src}bags_per_tile[feat_idx];
    int {vars_.bag_begin} = (tile - s_bind.prefix[feat_idx]) * bags_per_tile;
    int {vars_.bag_end} = min(batch, {vars_.bag_begin} + bags_per_tile);
    // a feature whose bags are split over workgroups: bags_per_tile = -parts, the feature's tile
    // t is part t % parts of bag t / parts
    int {vars_.split_part} = 0, {vars_.split_parts} = 1;
    float *{vars_.split_region} = nullptr;
    if constexpr (HAS_SPLIT) {{
      if (bags_per_tile < 0) {{
        const int local = tile - s_bind.prefix[feat_idx];
        {vars_.split_parts} = -bags_per_tile;
        {vars_.bag_begin} = local / {vars_.split_parts};
        {vars_.split_part} = local - {vars_.bag_begin} * {vars_.split_parts};
        {vars_.bag_end} = {vars_.bag_begin} + 1;
      }}
      {vars_.split_region} = d_workspace + {"c_split_region[feat_idx]" if has_split else "0"};
    }}
{feature_addrs}    const int embed_dim_offset = c_embed_dim_offsets[feat_idx];
    const int {vars_.skip_long} = {"outlier_tiles > 0 && c_long_thr[feat_idx] > 0 ? c_long_thr[feat_idx] : 0x7fffffff" if outliers else "0x7fffffff"};
{timing_begin if timing and not timing_branch else ''}
    switch (c_cand_func_ids[{bound_src}cand[feat_idx]]) {{
{cases}      default: break;
    }}
{timing_end}
{loop_tail}  }}
{timing_flush}{outlier_end}}}

'''
        return consts + temp_storage_decl + functions + "\n" + tables + kernel

    def emit_process_func(self, timing: bool = False, occupancy: int = None) -> str:
        return '''
// Launches the kernels of one call on a->stream; `workspace` holds WORKSPACE_BYTES bytes (the
// caller's buffer or the library's static array) or is null when the library needs none.
static int launch_kernels(const recom_process_args *a, void *workspace) {
  const int64_t row_stride = a->output_row_stride ? a->output_row_stride : EMBED_DIM_SUM;
  const rfx::LaunchState *st = nullptr;
  hipError_t e = rfx::get_launch_state(FusedKnl, BLOCK_THREADS, OCCUPANCY, &st);
  if (e != hipSuccess) return static_cast<int>(e);
  const int grid = a->grid_blocks > 0 ? a->grid_blocks : st->cus * st->occupancy;
  if (grid <= 0) return static_cast<int>(hipErrorInvalidConfiguration);
  const int tile_bytes = a->tile_bytes > 0 ? a->tile_bytes : TILE_BYTES;
  const int xcd_segments = a->xcd_segments > 0 ? a->xcd_segments
                                               : (a->xcd_segments < 0 ? 0 : XCD_SEGMENTS);

  // hipLaunchKernel reports the error of this launch itself; the thread's last-error slot may
  // still hold the failure of an unrelated earlier call and is not consulted
  const char *arg_buffers = static_cast<const char *>(a->d_arg_buffers);
  int batch = a->batch, tile_arg = tile_bytes, xcd_arg = xcd_segments;
  int stride_arg = static_cast<int>(row_stride);
  void *outlier_space = OUTLIERS || DRAWN_TAIL > 0 ? static_cast<char *>(workspace) + SPLIT_BYTES : nullptr;
  void *bound = BIND_ONCE ? static_cast<char *>(workspace) + BOUND_OFFSET : nullptr;
  // The caller's events take the begin of the call's first kernel and the end of its last
  // (the fused kernel): a library that launches a kernel ahead of the fused one is timed whole.
  hipStream_t stream = static_cast<hipStream_t>(a->stream);
  hipEvent_t start_event = static_cast<hipEvent_t>(a->start_event);
  hipEvent_t stop_event = static_cast<hipEvent_t>(a->stop_event);
  auto launch = [&](const void *kernel, dim3 g, dim3 b, void **args, size_t lds, bool last) {
    hipEvent_t s0 = start_event, s1 = last ? stop_event : nullptr;
    start_event = nullptr;                                 // only the first kernel gets it
    if (s0 || s1) return hipExtLaunchKernel(kernel, g, b, args, lds, stream, s0, s1, 0);
    return hipLaunchKernel(kernel, g, b, args, lds, stream);
  };
#if RFX_OUTLIERS
  {
    void *outlier_args[] = {const_cast<int64_t **>(&a->d_io_ptrs), &arg_buffers,
                            const_cast<int64_t **>(&a->d_arg_buffer_offsets), &batch, &outlier_space};
    const unsigned gx = static_cast<unsigned>((batch + 255) / 256 > 64 ? 64 : (batch + 255) / 256);
    const unsigned gy = static_cast<unsigned>(NUM_FEATS > 1024 ? 1024 : NUM_FEATS);
    e = launch(reinterpret_cast<const void *>(OutlierKnl), dim3(gx, gy), dim3(256), outlier_args, 0, false);
    if (e != hipSuccess) return static_cast<int>(e);
  }
#endif
#if RFX_BIND_ONCE
  int grid_arg = grid;
  void *bind_args[] = {const_cast<int64_t **>(&a->d_io_ptrs), &arg_buffers,
                       const_cast<int64_t **>(&a->d_arg_buffer_offsets), &batch, &tile_arg,
                       const_cast<int32_t **>(&a->d_schedule_choice), &grid_arg, &bound,
                       const_cast<int32_t **>(&a->d_lookup_counts)};
  e = launch(reinterpret_cast<const void *>(BindKnl), dim3(1), dim3(1024), bind_args, 0, false);
  if (e != hipSuccess) return static_cast<int>(e);
#endif
  void *kernel_args[] = {
      const_cast<int64_t **>(&a->d_embed_table_ptrs), const_cast<int64_t **>(&a->d_io_ptrs),
      &arg_buffers, const_cast<int64_t **>(&a->d_arg_buffer_offsets),
      const_cast<float **>(&a->d_output), &batch, &tile_arg, &xcd_arg,
      const_cast<int32_t **>(&a->d_schedule_choice),
      const_cast<unsigned long long **>(&a->d_times), &stride_arg, &bound, &workspace,
      &outlier_space, const_cast<int32_t **>(&a->d_lookup_counts)};
  e = launch(reinterpret_cast<const void *>(FusedKnl), dim3(grid), dim3(BLOCK_THREADS), kernel_args,
             st->dyn_lds, true);
  return static_cast<int>(e);
}

// what both entry points check before any HIP call
static bool valid_process_args(const recom_process_args *a) {
  if (!a || !a->d_embed_table_ptrs || !a->d_output || a->batch < 0 ||
      (!a->d_io_ptrs && (!a->d_arg_buffers || !a->d_arg_buffer_offsets)))
    return false;
  if (!TIMING && a->d_times) return false;
  if (a->tile_bytes < 0 || a->grid_blocks < 0 || a->xcd_segments > 4096) return false;
  // the output: dense rows unless a stride is given; aligned for the widest store of the kernel
  const int64_t row_stride = a->output_row_stride ? a->output_row_stride : EMBED_DIM_SUM;
  return row_stride >= EMBED_DIM_SUM && row_stride <= 0x7fffffff && row_stride % OUT_VEC == 0 &&
         reinterpret_cast<uintptr_t>(a->d_output) % (OUT_VEC * sizeof(float)) == 0;
}

extern "C" int recom_process(const recom_process_args *a) {
  if (!valid_process_args(a)) return static_cast<int>(hipErrorInvalidValue);
  // split-bag schedules, outlier tiles and the once-per-launch binding keep their partial sums,
  // lists and tables in the caller's workspace
  if (WORKSPACE_BYTES > 0 && (!a->d_workspace || a->workspace_bytes < WORKSPACE_BYTES ||
                    reinterpret_cast<uintptr_t>(a->d_workspace) % 16 != 0))
    return static_cast<int>(hipErrorInvalidValue);
  if (a->batch == 0) return static_cast<int>(hipSuccess);
  return launch_kernels(a, WORKSPACE_BYTES > 0 ? a->d_workspace : nullptr);
}

// ---- the entry point that needs no caller workspace ----------------------------------------
// The workspace as a file-scope device array: every device the library runs on holds its own
// copy, at its own address, until the process ends.  In host code the name below is only a
// handle for hipGetSymbolAddress; kernels and fills get the address that call returns.
static __device__ __align__(256) char scratch[STATIC_WORKSPACE_BYTES];

// Puts back to zero what a launch expects to find at zero in the workspace: the arrival
// counters of every split-bag feature, and the header and the arrival counters of the outlier
// list.  A fill kernel, not hipMemsetAsync, so that a caller may capture the call in a graph.
extern "C" __global__ void __launch_bounds__(256) ScratchClearKnl(char *__restrict__ ws) {
  const int first = blockIdx.x * blockDim.x + threadIdx.x, step = gridDim.x * blockDim.x;
#if RFX_HAS_SPLIT
  for (int f = blockIdx.y; f < NUM_FEATS; f += gridDim.y) {
    if (c_split_region[f] < 0) continue;
    const int dim = c_embed_dims[f];
    int *counters = reinterpret_cast<int *>(ws) + c_split_region[f] +
                    static_cast<long long>(rfx::kSplitMaxTiles) * dim;
    for (int i = first; i < rfx::kSplitMaxTiles; i += step) counters[i] = 0;
  }
#endif
#if RFX_OUTLIERS
  if (blockIdx.y == 0) {
    OutlierSpace *sp = reinterpret_cast<OutlierSpace *>(ws + SPLIT_BYTES);
    int *hdr = reinterpret_cast<int *>(&sp->hdr);
    for (int i = first; i < static_cast<int>(sizeof(rfx::OutlierHeader) / 4); i += step) hdr[i] = 0;
    for (int i = first; i < OutlierSpace::kCap; i += step) sp->counters[i] = 0;
  }
#endif
#if RFX_DRAWN_TAIL
  if (blockIdx.y == 0) {
    int *tickets = reinterpret_cast<int *>(ws + SPLIT_BYTES);
    for (int i = first; i < static_cast<int>(sizeof(rfx::TailTickets) / 4); i += step) tickets[i] = 0;
  }
#endif
  (void)ws; (void)first; (void)step;
}

// device address of `scratch` on the current device, resolved once per device
static hipError_t static_workspace_address(char **out) {
  static char *addr[rfx::kMaxDevices];
  static std::mutex mu;
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (dev < 0 || dev >= rfx::kMaxDevices) return hipErrorInvalidDevice;
  std::lock_guard<std::mutex> lock(mu);
  if (!addr[dev]) {
    void *p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return e;
    if (!p) return hipErrorInvalidSymbol;
    addr[dev] = static_cast<char *>(p);
  }
  *out = addr[dev];
  return hipSuccess;
}

extern "C" int recom_process_static_workspace(const recom_process_args *a) {
  if (!valid_process_args(a)) return static_cast<int>(hipErrorInvalidValue);
  if (!STATIC_WORKSPACE_FITS) return RECOM_ESTATIC_WORKSPACE;
  if (a->batch == 0) return static_cast<int>(hipSuccess);
  if (WORKSPACE_BYTES == 0) return launch_kernels(a, nullptr);
  char *ws = nullptr;
  hipError_t e = static_workspace_address(&ws);
  if (e != hipSuccess) return static_cast<int>(e);
#if RFX_HAS_SPLIT || RFX_OUTLIERS
  // the array keeps what the last call left in it
  void *clear_args[] = {&ws};
  const unsigned gy = static_cast<unsigned>(NUM_FEATS > 64 ? 64 : NUM_FEATS);
  e = hipLaunchKernel(reinterpret_cast<const void *>(ScratchClearKnl), dim3(8, gy), dim3(256),
                      clear_args, 0, static_cast<hipStream_t>(a->stream));
  if (e != hipSuccess) return static_cast<int>(e);
#endif
  return launch_kernels(a, ws);
}
'''

    def emit_get_concurrent_blocks_func(self, occupancy: int = None) -> str:
        return '''
extern "C" int recom_get_launch_info(recom_launch_info *out) {
  if (!out) return static_cast<int>(hipErrorInvalidValue);
  const rfx::LaunchState *st = nullptr;
  hipError_t e = rfx::get_launch_state(FusedKnl, BLOCK_THREADS, OCCUPANCY, &st);
  if (e != hipSuccess) return static_cast<int>(e);
  *out = recom_launch_info{};
  out->compute_units = st->cus;
  out->occupancy = st->occupancy;
  out->dyn_lds_bytes = st->dyn_lds;
  out->natural_occupancy = st->natural_occupancy;
  out->api_occupancy = st->api_occupancy;
  out->num_vgprs = st->num_vgprs;
  out->static_lds_bytes = st->static_lds;
  out->lds_bytes_per_cu = st->lds_per_cu;
  out->padded_api_occupancy = st->padded_api_occupancy;
  return static_cast<int>(hipSuccess);
}

extern "C" int recom_get_workspace_bytes(int64_t *out) {
  if (!out) return static_cast<int>(hipErrorInvalidValue);
  *out = WORKSPACE_BYTES;
  return static_cast<int>(hipSuccess);
}

extern "C" int recom_get_max_concurrent_blocks(int32_t *out) {
  if (!out) return static_cast<int>(hipErrorInvalidValue);
  const rfx::LaunchState *st = nullptr;
  hipError_t e = rfx::get_launch_state(FusedKnl, BLOCK_THREADS, OCCUPANCY, &st);
  if (e != hipSuccess) return static_cast<int>(e);
  *out = st->cus * st->occupancy;
  return static_cast<int>(hipSuccess);
}
'''

    def emit_process_ops(self) -> str:
        return '''
extern "C" int recom_get_info(recom_info *out) {
  if (!out) return static_cast<int>(hipErrorInvalidValue);
  *out = recom_info{};
  out->abi_version = RECOM_ABI_VERSION;
  out->num_features = NUM_FEATS;
  out->embed_dim_sum = EMBED_DIM_SUM;
  out->block_threads = BLOCK_THREADS;
  out->occupancy = OCCUPANCY;
  out->num_bodies = NUM_BODIES;
  out->timing = TIMING ? 1 : 0;
  out->tile_bytes = TILE_BYTES;
  out->static_binding = STATIC_BINDING ? 1 : 0;
  out->num_candidates = NUM_CANDIDATES;
  out->xcd_segments = XCD_SEGMENTS;
  out->outliers = OUTLIERS ? 1 : 0;
  out->static_workspace = STATIC_WORKSPACE_FITS ? 1 : 0;
  return 0;
}

// host copies of the per-feature tables (the __constant__ arrays above are device symbols)
static const int h_embed_dims[] = {H_EMBED_DIMS};
static const int h_embed_dim_offsets[] = {H_EMBED_DIM_OFFSETS};
static const int h_dtypes[] = {H_DTYPES};
static const int h_row_strides[] = {H_ROW_STRIDES};
static const int h_cand_counts[] = {H_CAND_COUNTS};

extern "C" int recom_get_candidate_counts(int32_t *counts) {
  if (!counts) return static_cast<int>(hipErrorInvalidValue);
  for (int f = 0; f < NUM_FEATS; ++f) counts[f] = h_cand_counts[f];
  return 0;
}

extern "C" int recom_get_feature_tables(int32_t *embed_dims, int32_t *embed_dim_offsets,
                                        int32_t *dtypes, int32_t *row_strides) {
  for (int f = 0; f < NUM_FEATS; ++f) {
    if (embed_dims) embed_dims[f] = h_embed_dims[f];
    if (embed_dim_offsets) embed_dim_offsets[f] = h_embed_dim_offsets[f];
    if (dtypes) dtypes[f] = h_dtypes[f];
    if (row_strides) row_strides[f] = h_row_strides[f];
  }
  return 0;
}
'''.replace("H_EMBED_DIMS", ", ".join(map(str, self.embed_dims()))) \
   .replace("H_EMBED_DIM_OFFSETS", ", ".join(map(str, self.embed_dim_offsets()[:-1]))) \
   .replace("H_DTYPES", ", ".join(str(s.meta.dtype_id) for s, _ in self.feat_schedules)) \
   .replace("H_ROW_STRIDES", ", ".join(str(s.meta.row_stride) for s, _ in self.feat_schedules)) \
   .replace("H_CAND_COUNTS", ", ".join(str(len(c)) for c in self.feat_candidates))

    # ------------------------------------------------------------------ files

    def emit_if_updated(self, fname: str, code: str) -> bool:
        if os.path.exists(fname):
            with open(fname) as f:
                old = f.read()
                if old.strip() == code.strip():
                    return False

        with open(fname, "w") as f:
            f.write(code)
        return True

    def emit(self, ofname: str, occupancy: int = None, inline: bool = True,
             tune: bool = False, timing: bool = False, timing_branch: bool = False,
             fixed_task_block_nums: List[int] = None, tile_bytes: int = None,
             xcd_aware: bool = False, lookup_overhead_bytes: int = None,
             xcd_segments: int = 8, outliers: bool = False, bind_once: bool = None,
             tile_order: List[int] = None, drawn_tail: int = 0) -> None:
        """Write the device source.  ``occupancy`` = workgroups per CU the kernel is built and
        launched for (``__launch_bounds__`` budget, persistent grid size, and a dynamic-LDS pad
        that keeps further workgroups off the CU); ``tune`` is accepted for signature
        compatibility -- the pad is applied whenever an occupancy is given.  ``bind_once``: bind
        the model once per launch with a kernel of its own instead of in every workgroup of the
        fused kernel (None: ``binds_once_by_default``)."""
        code = "// generated by recflex_amd.code_emitter -- do not edit\n"
        code += self.emit_headers()
        code += self.emit_kernel(timing=timing, timing_branch=timing_branch,
                                 occupancy=occupancy, inline=inline,
                                 fixed_task_block_nums=fixed_task_block_nums,
                                 tile_bytes=tile_bytes, xcd_aware=xcd_aware,
                                 lookup_overhead_bytes=lookup_overhead_bytes,
                                 xcd_segments=xcd_segments, outliers=outliers, bind_once=bind_once,
                                 tile_order=tile_order, drawn_tail=drawn_tail)
        code += self.emit_process_func(timing=timing, occupancy=occupancy)
        code += self.emit_get_concurrent_blocks_func(occupancy=occupancy)
        code += self.emit_process_ops()

        self.emit_if_updated(ofname, code)

    def emit_host_op_headers(self) -> str:
        headers = {"<stdint.h>"}
        for schedule, params in self.feat_schedules:
            headers = headers.union(schedule.EmitPrepropHeaders())
        return ''.join(sorted(f"#include {header}\n" for header in headers)) + '\n'

    def emit_host_preprocess(self, fixed_task_block_nums: List[int] = None) -> str:
        num_feats = len(self.feat_schedules)
        v = PreprocessVars()
        seen: Dict[str, int] = {}
        id_map: Dict[int, int] = {}
        functions = ""
        for feat_idx, (schedule, params) in enumerate(self.feat_schedules):
            snippet = schedule.EmitHostPreprocess(params)
            if snippet not in seen:
                seen[snippet] = feat_idx
                functions += f'''
static int PreprocFeat{feat_idx}(
    const char *{v.raw_data}, const int64_t {v.raw_data_len}, const int32_t {v.num_lines},
    int32_t *{v.indices}, const int64_t {v.indices_capacity}, int32_t *{v.offsets},
    int64_t *{v.num_inputs_ref}) {{
{snippet}}}
'''
            id_map[feat_idx] = seen[snippet]

        table = ",\n".join(f"    PreprocFeat{id_map[f]}" for f in range(num_feats))
        dims = ", ".join(map(str, self.embed_dims()))
        return functions + f'''
typedef int (*PreprocFeatT)(const char *, const int64_t, const int32_t, int32_t *,
                            const int64_t, int32_t *, int64_t *);
static const PreprocFeatT preproc_feats[] = {{
{table}
}};
static const int32_t embed_dims[] = {{{dims}}};

extern "C" int32_t recom_host_num_features() {{ return {num_feats}; }}

// bytes of one pooled output row of feature `feat`
extern "C" int64_t recom_host_output_row_bytes(int32_t feat) {{
  return feat >= 0 && feat < {num_feats} ? int64_t(embed_dims[feat]) * 4 : -1;
}}

// parse the '\\n'-joined sample lines of feature `feat`
extern "C" int recom_host_preprocess_feat(
    int32_t feat, const char *{v.raw_data}, int64_t {v.raw_data_len}, int32_t {v.num_lines},
    int32_t *{v.indices}, int64_t {v.indices_capacity}, int32_t *{v.offsets},
    int64_t *{v.num_inputs_ref}) {{
  if (feat < 0 || feat >= {num_feats}) return RECOM_HOST_EINVAL;
  return preproc_feats[feat]({v.raw_data}, {v.raw_data_len}, {v.num_lines}, {v.indices},
                             {v.indices_capacity}, {v.offsets}, {v.num_inputs_ref});
}}
'''

    def emit_host(self, ofname: str, fixed_task_block_nums: List[int] = None) -> None:
        code = "// generated by recflex_amd.code_emitter -- do not edit\n"
        code += self.emit_host_op_headers()
        code += self.emit_host_preprocess(fixed_task_block_nums=fixed_task_block_nums)
        self.emit_if_updated(ofname, code)

    def emit_cmake_list(self, ofname: str, code_fname: str, host_fname: str,
                        subdirs: List[str] = [], includes: List[str] = [],
                        links: List[str] = [], host_links: List[str] = [],
                        extra: str = "", debug: bool = False) -> None:
        """CMake project (no compiled languages enabled) whose targets run hipcc for
        ``librecom.so`` and g++ for ``recom_host.so``; ``cmake .. && make`` in ``build/``
        produces both, as with the reference's generated CMakeLists.txt (codegen.py:489-568)."""
        basic = BasicBuilder()
        includes = list(includes) + [basic.include, basic.abi_include]
        inc_flags = " ".join(f"-I{inc}" for inc in includes)
        link_flags = " ".join(links)
        host_link_flags = " ".join(host_links)
        opt = "-g -O0" if debug else "-O3"
        add_subdirs = '\n'.join(f"add_subdirectory({subdir})" for subdir in subdirs)
        # the device side is header-only: a change of a schedule template rebuilds the library
        device_headers = " ".join(basic.device_headers())

        recom = f'''
add_custom_command(
  OUTPUT ${{CMAKE_BINARY_DIR}}/librecom.so
  COMMAND {basic.hipcc} {" ".join(basic.hip_flags)} {opt} {inc_flags}
          ${{CMAKE_SOURCE_DIR}}/{code_fname} {link_flags} -o ${{CMAKE_BINARY_DIR}}/librecom.so
  DEPENDS ${{CMAKE_SOURCE_DIR}}/{code_fname} {device_headers}
  VERBATIM)
add_custom_target(recom ALL DEPENDS ${{CMAKE_BINARY_DIR}}/librecom.so)
''' if code_fname else ''

        recom_host = f'''
add_custom_command(
  OUTPUT ${{CMAKE_BINARY_DIR}}/recom_host.so
  COMMAND {basic.cxx} {" ".join(basic.host_flags)} {opt} {inc_flags}
          ${{CMAKE_SOURCE_DIR}}/{host_fname} {basic.host_source} {host_link_flags}
          -o ${{CMAKE_BINARY_DIR}}/recom_host.so
  DEPENDS ${{CMAKE_SOURCE_DIR}}/{host_fname} {basic.host_source}
  VERBATIM)
add_custom_target(recom_host ALL DEPENDS ${{CMAKE_BINARY_DIR}}/recom_host.so)
''' if host_fname else ''

        code = f'''
cmake_minimum_required(VERSION 3.12 FATAL_ERROR)
project(recom_project LANGUAGES NONE)

# Add subdirectories
{add_subdirs}

# Add target recom_host
{recom_host}

# Add target recom
{recom}

# Extra area
{extra}
'''
        self.emit_if_updated(ofname, code)
