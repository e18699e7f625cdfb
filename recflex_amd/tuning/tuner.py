"""Two-stage, interference-aware schedule tuner for CDNA4.

Class, method and field names follow ``RecFlex/tuning/tuner.py:24-357`` (``BasicConfig``,
``TuneConfig``, ``Tuner.tune`` / ``solve`` / ``tune_occupancy`` / ``mutation_validation`` /
``tune_naive`` / ``tune_fixed_thread_binding`` / ``emit_codes``), and so does the output tree
under ``codegen_dir``: ``f{feat}/o{occ}/``, ``all/o{occ}/``, ``optimal/``, ``naive/``,
``mutation_f{id}/m{k}``, ``fixed_thread_binding_{mean,max}/``, with ``result.txt`` files and the
resume-by-files rule (an existing ``librecom.so`` / result is kept unless ``recompile`` /
``remeasure``).

Local stage: for every feature and occupancy, all candidate schedules of the feature are put
side by side as the "features" of one fused kernel, repeated until there are at least
``CUs * occupancy`` of them, over the same input data; the kernel is built for exactly
``occupancy`` workgroups per CU (``__launch_bounds__`` register budget + dynamic-LDS pad +
persistent grid of ``CUs * occupancy`` workgroups) with per-feature device timers; the candidate
with the smallest summed tile time wins.  Global stage: per occupancy, the whole model with the
winners is built and its ``FusedKnl`` time measured (rocprofv3 kernel statistics, or events);
the fastest occupancy is copied to ``optimal/`` together with ``optimal/schedule.json``.

CDNA4 specifics: occupancy is counted in 256-thread workgroups per CU (= wavefronts per SIMD),
1..8.  Kernels whose candidate lists are identical (features with the same dim and element type)
are compiled once and shared through ``.cache/``.
"""

import filecmp
import hashlib
import json
import os
import shutil
from typing import Dict, List, NamedTuple, Optional, Sequence, Tuple

import numpy as np

from recflex_amd.code_emitter import CodeEmitter, ScheduleBase, MetaData
from recflex_amd.code_emitter.codegen import (BAG_FIXED_BYTES, DEFAULT_TILE_BYTES, DRAWN_ALL, INDEX_BYTES,
                                               waves_per_simd)
from recflex_amd.model_build import DEFAULT_XCD_SEGMENTS
from recflex_amd.utils import compile_build, os_check
from recflex_amd.task_manager import TaskManager
from recflex_amd.parser import (parse_raw_data_batches, parse_table_shapes, parse_table_dtypes,
                                parse_schedule_types, parse_knl_total_time, parse_knl_batch_times)

from .measure import (measure_single_feat, rocprof_profile, measure_task_blocks, measure_feature_ticks,
                      tiles_per_feature,
                      measure_naive_candidate, measure_kernel_events, measure_tournament,
                      save_batches, KernelTimer, PROFILE_PASSES, PROFILE_WARMUP_PASSES)


class BasicConfig(NamedTuple):
    batch_sizes_fname: str
    data_fnames: List[str]
    schedule_config_fname: str
    table_config_fname: str
    codegen_dir: str
    subdirs: List[str] = []
    includes: List[str] = []
    links: List[str] = []
    host_links: List[str] = []
    block_threads: int = 256
    sample_batch_nums: int = 128


class TuneConfig(NamedTuple):
    occupancies: List[int]
    gpu_ids: List[int]
    sm_count: int
    num_processes: int = 8
    inline: bool = True
    recompile: bool = False
    remeasure: bool = False
    debug: bool = False
    # "rocprofv3": global-stage kernel time from rocprofv3 kernel statistics (spawned);
    # "events": events around each launch, in this process
    profiler: str = "rocprofv3"
    # run measurement workers in this process instead of one spawned process per measurement
    in_process: bool = True
    # traffic a tile carries in the tuning builds and contenders; 0 = sized by the device from
    # every batch (rfx::auto_tile_size), as untuned builds do
    tile_bytes: int = DEFAULT_TILE_BYTES
    # emit optimal/ with outlier tiles: bags far beyond their schedule's reach are found by a pass
    # over the offsets ahead of the fused kernel and summed by several workgroups (skewed data).
    # None: decided on the sampled batches -- if any of them holds such a bag, the mix is built
    # both ways and the faster call wins (Tuner.decide_outliers)
    outliers: Optional[bool] = None
    # undecided (None): kept only if the whole call is faster by this share on the samples
    outliers_min_gain: float = 0.02
    # the tile walk (Tuner.decide_walk): a drawn end, and the order of the features in the
    # kernel's tile space.  False: neither is tried; True: both; None: a drawn end on models
    # whose workgroups get a few tiles each at least, an order on models of at least
    # ``walk_stage_min_feats`` features whose workgroups get fewer than
    # ``walk_stage_max_tiles`` tiles each on the samples (with more, the deal evens out by itself)
    walk_stage: Optional[bool] = None
    walk_stage_min_feats: int = 64
    walk_stage_max_tiles: float = 16.0
    # passes drawn at the end of the walk that are tried (DRAWN_ALL: every tile), on models whose
    # workgroups get at least ``walk_drawn_min_tiles`` tiles each on the samples
    drawn_tail_candidates: Sequence[int] = (2, 4, 8, DRAWN_ALL)
    walk_drawn_min_tiles: float = 3.0
    # segments per XCD a drawn winner is also timed with (those finer than its own)
    walk_xcd_segments_candidates: Sequence[int] = (64, 128)
    walk_min_gain: float = 0.01
    # local-stage interference: "model" = every candidate of every feature is compiled into one
    # kernel of the whole model and timed while all other features run beside it;
    # "replicate" = per feature, the candidates side by side over the same data, replicated
    # until the GPU is full (the reference's scheme, RecFlex/tuning/tuner.py:112-141)
    interference: str = "model"
    rounds: int = 3
    refine_passes: int = 3
    top_k: int = 8
    # passes of the whole-kernel climb that follows the tile-time tournament (0 = none)
    climb_passes: int = 1
    # in-model local stage, second half: clusters of like features (same candidate list, same
    # class of bag length) decide one at a time.  Per cluster a production-shaped build holds the
    # cluster's ``cluster_top_k`` best-ranked candidates beside the pick of every other feature;
    # the whole kernel is timed with the cluster on each of them in turn and the cluster adopts
    # the fastest if it beats its current pick by ``cluster_min_gain``.  ``cluster_sweeps`` passes
    # over all clusters, heaviest first, ``num_processes`` builds at a time.
    # A scan over the options is followed by a head-to-head of the fastest against the current
    # pick (the fastest of nine noisy times looks better than it is), and the adoptions of one
    # group of builds -- all made against the same mix -- are then checked together in one more
    # build, old picks against new, and dropped if the new mix is not faster.
    cluster_stage: bool = True
    cluster_top_k: int = 8
    cluster_min_gain: float = 0.005
    cluster_sweeps: int = 1
    cluster_group: int = 8
    # a cluster build is trusted only if it runs the current mix within this share of the time of
    # the same mix built as it ships (heavy candidate bodies raise the registers and scratch of the
    # kernel they sit in: an int8 model's cluster builds ran its default mix 40 % slower than
    # its production build, and the options that won there lost 16 % in production)
    cluster_build_tolerance: float = 0.05
    # in-model local stage: compile every distinct candidate body alone for each occupancy and
    # keep out of that occupancy's tournament the ones that spill or come within
    # ``census_margin`` vector registers of the occupancy's budget (they cannot win, and their
    # scratch memory and registers slow every other candidate of the same kernel down)
    register_census: bool = True
    census_margin: int = 8
    # global stage, after the contenders are timed: hill climb on production builds.  The
    # winning mix is varied one feature at a time (heaviest first, that feature's
    # ``build_climb_top_k`` best tournament candidates), ``num_processes`` variants are compiled
    # side by side and timed as whole kernels, and the variants that are faster are adopted.
    # 0 trials = off; the budget bounds the compile time spent
    build_climb_trials: int = 0
    build_climb_top_k: int = 3
    build_climb_min_gain: float = 0.01
    # global stage: traffic-per-tile values of the run-time binding to try for every occupancy
    # (a launch parameter, no rebuild); empty = only tile_bytes
    tile_bytes_candidates: List[int] = []
    # global stage: L2-locality settings of the tile walk to try (launch parameter
    # xcd_segments; -1 = flat walk); empty = only the emitted default
    xcd_segments_candidates: List[int] = []
    # global stage: launch options whose time is within this share of a contender's fastest count
    # as equally fast, and of those the one with the fewest segments per XCD wins (fewer segments
    # = fewer L2s that fetch a feature's hot rows = less HBM traffic: C3 fetches 478 MB at 10
    # segments, 494 MB at 12, 512 MB at 16 and 541 MB at 24, in 119.7 / 119.9 / 118.2 / 118.2 us).
    # 0 = the fastest option wins; a deployment that shares the memory system with other kernels
    # may give away a per cent of time for the traffic
    launch_time_tolerance: float = 0.0
    # global stage: also time the untuned default schedules at every occupancy and keep them
    # if they win (tile times measured feature by feature do not always add up to kernel time)
    include_default: bool = True
    # global stage: a schedule file of an earlier tuning run of the same model (``schedule.json``
    # as ``solve`` writes it), timed as one more contender at every occupancy: a model that is
    # tuned again starts from what it has
    incumbent: Optional[str] = None
    # the incumbent is the only contender of the global stage (Tuner.solve_incumbent_only)
    only_incumbent: bool = False


def padded_sched_num(orig_num: int, max_concurrent_blocks: int) -> int:
    return (orig_num + max_concurrent_blocks - 1) // orig_num * orig_num


def pick_launch_option(launch_opts: List[Tuple[int, int]], times: List[float],
                       tolerance: float) -> int:
    """Index of the launch option (tile_bytes, xcd_segments) to keep: the fastest, unless options
    with fewer (positive) segments per XCD are within ``tolerance`` of it -- then the one with the
    fewest segments among those, the faster one on a tie.  The flat walk (segments <= 0) fetches
    the most and never wins a tie."""
    best = int(np.argmin(times))
    if launch_opts[best][1] <= 0:
        return best
    limit = times[best] * (1.0 + tolerance)
    near = [k for k, (_, xs) in enumerate(launch_opts) if xs > 0 and times[k] <= limit]
    return min(near, key=lambda k: (launch_opts[k][1], times[k]))



def release_device_memory() -> None:
    """Hands the device memory that this process's earlier measurements left in torch's caching
    allocator back to the driver.  The measurements that follow run in child processes, which
    build the model's tables again: for a model whose tables fill most of the device (C4) the
    child otherwise runs out of memory."""
    import gc
    import sys
    gc.collect()
    torch = sys.modules.get("torch")
    if torch is not None and torch.cuda.is_initialized():
        torch.cuda.synchronize()
        torch.cuda.empty_cache()


class Tuner:
    def __init__(self, basic_config: BasicConfig, schedule_mapping: Dict[str, type],
                 batches: List[List[Tuple[np.ndarray, np.ndarray]]] = None,
                 table_shapes: List[Tuple[int, int]] = None, data_types: List[str] = None,
                 schedule_types: List[List[type]] = None):
        """With only ``basic_config`` and ``schedule_mapping`` everything is read from the files
        the configuration names, as in the reference.  The keyword arguments supply the same
        information directly (synthetic workloads that have no dataset directory):
        ``batches[feat][k] = (indices, offsets)``."""
        self.basic = basic_config
        self.schedule_mapping = schedule_mapping
        self._given = (batches, table_shapes, data_types, schedule_types)
        self.get_raw_data_batches()
        self.get_metas()
        self.get_feat_schedules()
        self.num_feats: int = len(self.feat_schedules)
        self.gen_feat_sched_param_candidates()
        self.write_data_files()

    # ------------------------------------------------------------------ inputs

    def get_raw_data_batches(self):
        """``self.batches[feat]`` = list of ``(indices, offsets)`` int32 arrays, one per sampled
        batch; ``self.raw_data_batches`` keeps the text lines when they came from files."""
        given = self._given[0]
        if given is not None:
            self.raw_data_batches = None
            self.batches = given
            return self.batches
        from recflex_amd.host import RecomHost
        self.raw_data_batches = parse_raw_data_batches(self.basic.batch_sizes_fname,
                                                       self.basic.data_fnames,
                                                       self.basic.sample_batch_nums)
        host = RecomHost()
        self.batches = [[host.parse_lines(lines) for lines in feat] for feat in self.raw_data_batches]
        return self.raw_data_batches

    def get_metas(self):
        _, shapes, dtypes, _ = self._given
        self.table_shapes = shapes if shapes is not None else parse_table_shapes(self.basic.table_config_fname)
        if dtypes is not None:
            self.data_types = list(dtypes)
        elif shapes is None:
            self.data_types = parse_table_dtypes(self.basic.table_config_fname)
        else:
            self.data_types = ["float"] * len(self.table_shapes)
        self.metas: List[MetaData] = [MetaData(embed_dim=embed_dim, data_type=dt)
                                      for (nrows, embed_dim), dt in zip(self.table_shapes, self.data_types)]
        return self.metas

    def get_feat_schedules(self):
        feat_schedule_types = self._given[3]
        if feat_schedule_types is None:
            feat_schedule_types = parse_schedule_types(self.basic.schedule_config_fname, self.schedule_mapping)
        for f, types in enumerate(feat_schedule_types):
            if any(t is None for t in types):
                raise KeyError(f"feature {f}: unknown schedule class name in the schedule config")
        self.feat_schedules: List[List[ScheduleBase]] = [
            [schedule_type(meta, self.basic.block_threads) for schedule_type in schedule_types]
            for schedule_types, meta in zip(feat_schedule_types, self.metas)]
        return self.feat_schedules

    def gen_feat_sched_param_candidates(self):
        self.feat_sched_param_candidates: List[List[Tuple[ScheduleBase, NamedTuple]]] = [[] for _ in range(self.num_feats)]
        for feat_id in range(self.num_feats):
            for schedule in self.feat_schedules[feat_id]:
                for params in schedule.GenParamCandidates():
                    self.feat_sched_param_candidates[feat_id].append([schedule, params])
            if not self.feat_sched_param_candidates[feat_id]:
                # e.g. a template whose parameter space has no member for rows this wide: tune
                # nothing for this feature, run the default schedule
                from recflex_amd.schedules import default_schedule
                lens = [len(i) / max(1, len(o) - 1) for i, o in self.batches[feat_id]]
                sched, params = default_schedule(self.metas[feat_id], float(np.mean(lens)) if lens else 1.0,
                                                 self.basic.block_threads, one_hot=self.is_one_hot(feat_id))
                print(f"feature {feat_id}: its schedule classes "
                      f"({', '.join(type(s).__name__ for s in self.feat_schedules[feat_id])}) have no "
                      f"candidate for dim {self.metas[feat_id].embed_dim} {self.metas[feat_id].data_type}; "
                      f"using the default schedule {type(sched).__name__}{tuple(params)}", flush=True)
                self.feat_sched_param_candidates[feat_id].append([sched, params])

    def write_data_files(self):
        """Per-feature ``data/f{i}.npz`` under ``codegen_dir`` (what the workers read) and, for
        workloads given as arrays, a ``table_config.txt`` for the profiling driver."""
        self.data_dir = f"{self.basic.codegen_dir}/data"
        os.makedirs(self.data_dir, exist_ok=True)
        self.data_npzs = []
        for feat_id in range(self.num_feats):
            path = f"{self.data_dir}/f{feat_id}.npz"
            save_batches(path, self.batches[feat_id])
            self.data_npzs.append(path)
        self.table_config_fname = self.basic.table_config_fname
        if not self.table_config_fname or not os.path.exists(self.table_config_fname):
            self.table_config_fname = f"{self.data_dir}/table_config.txt"
            with open(self.table_config_fname, "w") as f:
                for (rows, dim), dt in zip(self.table_shapes, self.data_types):
                    f.write(f"{rows},{dim},{dt}\n")

    # ------------------------------------------------------------------ helpers

    def get_padded_sched_num(self, orig_num: int, max_concurrent_blocks: int) -> int:
        return padded_sched_num(orig_num, max_concurrent_blocks)

    def pad_sched_params(self, sched_params: List[Tuple[ScheduleBase, NamedTuple]], padded_num: int) -> List[Tuple[ScheduleBase, NamedTuple]]:
        padded_schedules = sched_params.copy()
        add_num = padded_num - len(sched_params)
        for i in range(add_num):
            padded_schedules.append(sched_params[i % len(sched_params)])
        return padded_schedules

    def get_output_build_dir(self, feat_id: int, occupancy: int) -> Tuple[str, str]:
        if feat_id >= 0:
            output_dir = f"{self.basic.codegen_dir}/f{feat_id}/o{occupancy}"
        else:
            output_dir = f"{self.basic.codegen_dir}/all/o{occupancy}"
        build_dir = f"{output_dir}/build"
        return output_dir, build_dir

    def emit_codes(self, output_dir: str, feat_schedules: List[Tuple[ScheduleBase, NamedTuple]],
                   occupancy: int, inline: bool = True, timing: bool = False, tune: bool = False,
                   fixed_task_block_nums: List[int] = None, debug: bool = False,
                   tile_bytes: int = None, host: bool = True, xcd_segments: int = 0,
                   outliers: bool = False, tile_order: List[int] = None, drawn_tail: int = 0) -> None:
        os.makedirs(output_dir, exist_ok=True)
        emitter = CodeEmitter(feat_schedules)
        if host:
            emitter.emit_host(f"{output_dir}/preprocess.cpp", fixed_task_block_nums=fixed_task_block_nums)
        emitter.emit(f"{output_dir}/process.hip", occupancy=occupancy, timing=timing, inline=inline, tune=tune,
                     fixed_task_block_nums=fixed_task_block_nums, tile_bytes=tile_bytes,
                     xcd_aware=xcd_segments > 0, xcd_segments=max(xcd_segments, 1), outliers=outliers,
                     tile_order=tile_order, drawn_tail=drawn_tail)
        emitter.emit_cmake_list(f"{output_dir}/CMakeLists.txt", code_fname="process.hip",
                                host_fname="preprocess.cpp" if host else None,
                                subdirs=self.basic.subdirs, includes=self.basic.includes, links=self.basic.links,
                                host_links=self.basic.host_links, debug=debug)
        if not tune:      # local-stage kernels are candidate lists, not a model's schedule
            emitter.dump_key(f"{output_dir}/schedule.json")

    # ---- compile cache: identical device sources are built once -----------------------------

    def _source_key(self, output_dir: str) -> str:
        """Key of everything a library is compiled from: the emitted source and the device
        headers it includes (a header edited between two runs must not find the old build)."""
        h = hashlib.sha256()
        with open(f"{output_dir}/process.hip", "rb") as f:
            h.update(f.read())
        h.update(self._headers_digest())
        return h.hexdigest()[:24]

    def _headers_digest(self) -> bytes:
        if not hasattr(self, "_headers_digest_cache"):
            from recflex_amd.code_emitter.build_basic import BasicBuilder
            h = hashlib.sha256()
            for path in BasicBuilder().device_headers():
                with open(path, "rb") as f:
                    h.update(f.read())
            self._headers_digest_cache = h.digest()
        return self._headers_digest_cache

    def _kept(self, output_dir: str, tune_config: TuneConfig) -> bool:
        """The resume-by-files rule (RecFlex/tuning/tuner.py:117): an existing library is kept --
        if it is what this directory's source gives under the device headers as they are now.  A
        library left by a run with older headers would load (or be refused for its ABI version)
        long after the compile step that should have replaced it."""
        lib = f"{output_dir}/build/librecom.so"
        if tune_config.recompile or not os.path.exists(lib):
            return False
        if not os.path.exists(f"{output_dir}/process.hip"):
            return True         # nothing to hold it against: the reference's rule as it is
        cached = self._cached_lib(self._source_key(output_dir))
        if not os.path.exists(cached):
            return False
        # the same file (a hard link), or a copy of it (where links are refused or were not kept)
        return os.path.samefile(lib, cached) or filecmp.cmp(lib, cached, shallow=False)

    def _cached_lib(self, key: str) -> str:
        return f"{self.basic.codegen_dir}/.cache/{key}/librecom.so"

    def _schedule_builds(self, jobs: List[Tuple[str, str]], tune_config: TuneConfig) -> None:
        """``jobs`` = (output_dir, build_dir) whose sources are emitted.  Builds each distinct
        source once (in parallel worker processes), then links every build dir to its library."""
        by_key: Dict[str, List[Tuple[str, str]]] = {}
        for output_dir, build_dir in jobs:
            by_key.setdefault(self._source_key(output_dir), []).append((output_dir, build_dir))
        to_publish = []
        for key, group in by_key.items():
            if os.path.exists(self._cached_lib(key)) and not tune_config.recompile:
                continue
            to_publish.append((key, group[0][1]))
        if to_publish:
            manager = TaskManager(list(range(max(1, tune_config.num_processes))))
            for key, build_dir in to_publish:
                os.makedirs(build_dir, exist_ok=True)
                stale = f"{build_dir}/librecom.so"      # a link to the cache from an earlier run:
                if os.path.exists(stale):               # make would call it up to date
                    os.remove(stale)
                manager.add_task(compile_build, (build_dir,))
            manager.join()
        for key, build_dir in to_publish:
            lib = f"{build_dir}/librecom.so"
            if not os.path.exists(lib):
                raise Exception(f"build failed: {lib} was not produced")
            os.makedirs(os.path.dirname(self._cached_lib(key)), exist_ok=True)
            cached = self._cached_lib(key)
            if not (os.path.exists(cached) and os.path.samefile(lib, cached)):
                shutil.copyfile(lib, cached)
        for key, group in by_key.items():
            for output_dir, build_dir in group:
                os.makedirs(build_dir, exist_ok=True)
                self._link_lib(self._cached_lib(key), f"{build_dir}/librecom.so")

    @staticmethod
    def _link_lib(src: str, dst: str) -> None:
        """Make ``dst`` the same file as ``src`` (hard link; a copy where links are refused)."""
        if os.path.exists(dst) and os.path.samefile(src, dst):
            return
        tmp = dst + ".tmp"
        if os.path.exists(tmp):
            os.remove(tmp)
        try:
            os.link(src, tmp)
        except OSError:
            shutil.copyfile(src, tmp)
        os.replace(tmp, dst)

    def _run_measure(self, manager: Optional[TaskManager], tune_config: TuneConfig, target, args,
                     gpu_id_default: int = 0) -> None:
        if tune_config.in_process:
            target(*args, gpu_id=tune_config.gpu_ids[0] if tune_config.gpu_ids else gpu_id_default)
        else:
            manager.add_task(target, args, ident_key="gpu_id")

    # ------------------------------------------------------------------ local stage

    def local_padded_num(self, feat_id: int, occupancy: int, tune_config: TuneConfig) -> int:
        return self.get_padded_sched_num(len(self.feat_sched_param_candidates[feat_id]),
                                         tune_config.sm_count * occupancy)

    def compile_local(self, tune_config: TuneConfig) -> None:
        jobs = []
        for feat_id in range(self.num_feats):
            for occupancy in tune_config.occupancies:
                output_dir, build_dir = self.get_output_build_dir(feat_id, occupancy)
                if not self._kept(output_dir, tune_config):
                    os.makedirs(build_dir, exist_ok=True)
                    padded = self.pad_sched_params(self.feat_sched_param_candidates[feat_id],
                                                   self.local_padded_num(feat_id, occupancy, tune_config))
                    self.emit_codes(output_dir=output_dir, feat_schedules=padded, occupancy=occupancy,
                                    inline=tune_config.inline, timing=True, tune=True,
                                    debug=tune_config.debug, tile_bytes=tune_config.tile_bytes, host=False)
                    jobs.append((output_dir, build_dir))
        self._schedule_builds(jobs, tune_config)

    def get_tournament_dir(self, occupancy: int) -> Tuple[str, str]:
        output_dir = f"{self.basic.codegen_dir}/tournament/o{occupancy}"
        return output_dir, f"{output_dir}/build"

    # ---- register census ----------------------------------------------------------------------

    @staticmethod
    def vgpr_budget(occupancy: int, block_threads: int = 256) -> int:
        """Vector registers per lane that ``occupancy`` workgroups of ``block_threads`` threads per
        CU leave a kernel on gfx950: 512 per SIMD in blocks of 8, shared by the wavefronts the
        SIMD then holds (one per 256-thread workgroup)."""
        return min(512, 512 // waves_per_simd(max(1, occupancy), block_threads) // 8 * 8)

    def _census_one(self, sched_param: Tuple[ScheduleBase, NamedTuple], occupancy: int,
                    tune_config: TuneConfig) -> Tuple[int, int]:
        """(vector registers, scratch bytes) of the fused kernel holding this one schedule."""
        import re
        import subprocess
        import tempfile
        from recflex_amd.code_emitter.build_basic import BasicBuilder
        basic = BasicBuilder()
        with tempfile.TemporaryDirectory(prefix="rfx_census_") as tmp:
            src = f"{tmp}/process.hip"
            CodeEmitter([sched_param]).emit(src, occupancy=occupancy, inline=tune_config.inline,
                                            tile_bytes=tune_config.tile_bytes)
            flags = [f for f in basic.hip_flags if f not in ("-shared", "-fPIC")]
            cmd = [basic.hipcc, *flags, "-O3", f"-I{basic.include}", f"-I{basic.abi_include}",
                   *(f"-I{inc}" for inc in self.basic.includes),
                   "--cuda-device-only", "-S", "-o", f"{tmp}/process.s", src]
            subprocess.run(cmd, check=True, stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
            with open(f"{tmp}/process.s") as f:
                text = f.read()
        vgprs = max(int(v) for v in re.findall(r"; NumVgprs: (\d+)", text))
        scratch = max(int(v) for v in re.findall(r"; ScratchSize: (\d+)", text))
        return vgprs, scratch

    def _body_key(self, sched: ScheduleBase, params: NamedTuple) -> str:
        """Key of a schedule body as it compiles: its emitted text and the device headers."""
        return hashlib.sha256(sched.EmitScheduleBody(params).encode() + self._headers_digest()).hexdigest()[:24]

    def register_census(self, occupancy: int, tune_config: TuneConfig) -> Dict[str, Tuple[int, int]]:
        """Registers and scratch of every distinct candidate body at this occupancy, keyed by the
        body text; compiled once (``.cache/census_o{occ}.json``), ``num_processes`` at a time."""
        from concurrent.futures import ThreadPoolExecutor
        cache_path = f"{self.basic.codegen_dir}/.cache/census_o{occupancy}.json"
        census: Dict[str, Tuple[int, int]] = {}
        if os.path.exists(cache_path) and not tune_config.recompile:
            with open(cache_path) as f:
                census = {k: tuple(v) for k, v in json.load(f).items()}
        todo: Dict[str, Tuple[ScheduleBase, NamedTuple]] = {}
        for cands in self.feat_sched_param_candidates:
            for sched, params in cands:
                key = self._body_key(sched, params)
                if key not in census:
                    todo.setdefault(key, (sched, params))
        if todo:
            print(f"register census, occupancy {occupancy}: {len(todo)} schedule bodies", flush=True)
            with ThreadPoolExecutor(max_workers=max(1, tune_config.num_processes)) as pool:
                done = pool.map(lambda sp: self._census_one(sp, occupancy, tune_config), todo.values())
                for key, res in zip(todo.keys(), done):
                    census[key] = res
            os.makedirs(os.path.dirname(cache_path), exist_ok=True)
            with open(cache_path, "w") as f:
                json.dump(census, f)
        return census

    def tournament_candidates(self, occupancy: int, tune_config: TuneConfig) -> List[List[int]]:
        """Per feature, the indices (into its candidate list) admitted to this occupancy's
        tournament: bodies that do not spill and stay ``census_margin`` registers under the
        occupancy's budget; the lightest body of the feature if none does."""
        if not tune_config.register_census:
            return [list(range(len(c))) for c in self.feat_sched_param_candidates]
        census = self.register_census(occupancy, tune_config)
        limit = self.vgpr_budget(occupancy, self.basic.block_threads) - tune_config.census_margin
        admitted = []
        for cands in self.feat_sched_param_candidates:
            stats = [census[self._body_key(s, p)] for s, p in cands]
            keep = [k for k, (vgprs, scratch) in enumerate(stats) if scratch == 0 and vgprs <= limit]
            if not keep:
                keep = [min(range(len(stats)), key=lambda k: (stats[k][1], stats[k][0]))]
            admitted.append(keep)
        return admitted

    def compile_tournament(self, tune_config: TuneConfig) -> None:
        """One timing build of the whole model per occupancy, holding the admitted candidates;
        ``admitted.json`` beside it maps its candidate numbers back to the full lists."""
        jobs = []
        for occupancy in tune_config.occupancies:
            output_dir, build_dir = self.get_tournament_dir(occupancy)
            if not self._kept(output_dir, tune_config):
                os.makedirs(build_dir, exist_ok=True)
                admitted = self.tournament_candidates(occupancy, tune_config)
                with open(f"{output_dir}/admitted.json", "w") as f:
                    json.dump(admitted, f)
                cands = [[self.feat_sched_param_candidates[feat][k] for k in keep]
                         for feat, keep in enumerate(admitted)]
                emitter = CodeEmitter(None, feat_candidates=cands)
                emitter.emit(f"{output_dir}/process.hip", occupancy=occupancy, timing=True,
                             inline=tune_config.inline, tune=True, tile_bytes=tune_config.tile_bytes)
                emitter.emit_cmake_list(f"{output_dir}/CMakeLists.txt", code_fname="process.hip",
                                        host_fname=None, subdirs=self.basic.subdirs,
                                        includes=self.basic.includes, links=self.basic.links,
                                        debug=tune_config.debug)
                jobs.append((output_dir, build_dir))
        self._schedule_builds(jobs, tune_config)

    def admitted_candidates(self, occupancy: int) -> List[List[int]]:
        output_dir, _ = self.get_tournament_dir(occupancy)
        path = f"{output_dir}/admitted.json"
        if not os.path.exists(path):
            return [list(range(len(c))) for c in self.feat_sched_param_candidates]
        with open(path) as f:
            return json.load(f)

    def is_one_hot(self, feat_id: int) -> bool:
        """No bag of the feature holds more than one lookup in any sampled batch (and there is
        at least one lookup)."""
        feat = self.batches[feat_id]
        longest = max((int(np.diff(off).max()) for _, off in feat if len(off) > 1), default=0)
        return longest == 1

    def default_choices(self) -> List[List[int]]:
        """Index, in every feature's candidate list, of the schedule ``default_schedule`` would
        pick from the mean bag length of the sampled batches (nearest candidate of the same
        template if the exact parameters are not in the list): a known-good mix the climb may
        start from."""
        from recflex_amd.schedules import default_schedule
        choice = []
        for feat_id, cands in enumerate(self.feat_sched_param_candidates):
            lens = [len(i) / max(1, len(o) - 1) for i, o in self.batches[feat_id]]
            sched, params = default_schedule(self.metas[feat_id], float(np.mean(lens)),
                                             self.basic.block_threads, one_hot=self.is_one_hot(feat_id))
            body = sched.EmitScheduleBody(params)
            pick, best_d = 0, None
            for k, (s, p) in enumerate(cands):
                if s.EmitScheduleBody(p) == body:
                    pick, best_d = k, -1
                    break
                if type(s) is type(sched):
                    d = sum(abs(a - b) for a, b in zip(p, params))
                    if best_d is None or d < best_d:
                        pick, best_d = k, d
            choice.append(pick)
        return [choice]

    def tune_in_model(self, tune_config: TuneConfig) -> Dict[int, Dict[int, List[float]]]:
        self.compile_tournament(tune_config)
        manager = None if tune_config.in_process else TaskManager(tune_config.gpu_ids)
        for occupancy in tune_config.occupancies:
            output_dir, build_dir = self.get_tournament_dir(occupancy)
            result_log = f"{output_dir}/result.json"
            if not os.path.exists(result_log) or tune_config.remeasure:
                admitted = self.admitted_candidates(occupancy)
                starts = [[self._nearest_admitted(feat, pick, admitted[feat])
                           for feat, pick in enumerate(choice)] for choice in self.default_choices()]
                args = (occupancy, f"{build_dir}/librecom.so", self.table_shapes, self.data_types,
                        self.data_npzs, result_log, tune_config.rounds, tune_config.refine_passes,
                        tune_config.top_k, 0.2, 3, 0, tune_config.climb_passes, starts)
                self._run_measure(manager, tune_config, measure_tournament, args)
        if manager:
            manager.join()
        results: Dict[int, Dict[int, List[float]]] = {feat_id: {} for feat_id in range(self.num_feats)}
        for occupancy in tune_config.occupancies:
            output_dir, _ = self.get_tournament_dir(occupancy)
            with open(f"{output_dir}/result.json") as f:        # absent if the worker failed
                times = json.load(f)["times"]
            admitted = self.admitted_candidates(occupancy)
            for feat_id in range(self.num_feats):
                # candidates kept out of this occupancy's tournament never win it
                full = [float("inf")] * len(self.feat_sched_param_candidates[feat_id])
                for k, t in zip(admitted[feat_id], times[feat_id]):
                    full[k] = t
                results[feat_id][occupancy] = full
        if tune_config.cluster_stage:
            for occupancy in tune_config.occupancies:
                picks = self.cluster_stage(occupancy, results, tune_config)
                for feat_id, k in enumerate(picks):
                    # an argmin over the scores reproduces the local stage's decision
                    scores = results[feat_id][occupancy]
                    finite = [t for t in scores if np.isfinite(t)]
                    scores[k] = (min(finite) if finite else 1.0) * 0.999
        return results

    # ---- local stage, by clusters of like features ----------------------------------------------

    BAG_LENGTH_CLASSES = (1.5, 4.0, 16.0, 64.0)      # mean lookups per bag: class boundaries

    def feature_clusters(self) -> List[List[int]]:
        """Features that share a candidate list (element type, dim, templates) and a class of mean
        bag length, heaviest cluster (by traffic in the sampled batches) first."""
        groups: Dict[tuple, List[int]] = {}
        for f in range(self.num_feats):
            lens = [len(i) / max(1, len(o) - 1) for i, o in self.batches[f]]
            mean = float(np.mean(lens)) if lens else 0.0
            cls = sum(mean > b for b in self.BAG_LENGTH_CLASSES)
            m = self.metas[f]
            key = (m.data_type, m.embed_dim, len(self.feat_sched_param_candidates[f]),
                   tuple(type(s).__name__ for s in self.feat_schedules[f]), self.is_one_hot(f), cls)
            groups.setdefault(key, []).append(f)
        weight = self.feature_traffic()
        return sorted(groups.values(), key=lambda g: -float(sum(weight[f] for f in g)))

    def feature_traffic(self) -> np.ndarray:
        """Bytes each feature moves in the sampled batches (rows + indices + output)."""
        return np.asarray([sum(len(i) for i, _ in self.batches[f]) * (self.metas[f].row_bytes + INDEX_BYTES)
                           + self.metas[f].embed_dim * 4 * sum(len(o) - 1 for _, o in self.batches[f])
                           for f in range(self.num_feats)], dtype=np.float64)

    def cluster_options(self, members: List[int], picks: List[int], occupancy: int,
                        measured_times: Dict[int, Dict[int, List[float]]], top_k: int) -> List[int]:
        """The candidates (indices into the members' common candidate list) a cluster tries: the
        ``top_k`` with the best summed rank scores of the local stage's first half, each
        member's score taken relative to its own best."""
        n = len(self.feat_sched_param_candidates[members[0]])
        total = np.zeros(n)
        for f in members:
            sc = np.asarray(measured_times[f][occupancy], dtype=np.float64)
            finite = sc[np.isfinite(sc)]
            total += np.where(np.isfinite(sc), sc / (finite.min() if finite.size else 1.0), np.inf)
        ranked = [int(k) for k in np.argsort(total, kind="stable") if np.isfinite(total[k])]
        return ranked[:top_k]

    def get_cluster_dir(self, occupancy: int, sweep: int, cluster: int) -> str:
        return f"{self.basic.codegen_dir}/clusters/o{occupancy}/s{sweep}_c{cluster}"

    def cluster_stage(self, occupancy: int, measured_times: Dict[int, Dict[int, List[float]]],
                      tune_config: TuneConfig) -> List[int]:
        """Second half of the in-model local stage (see ``TuneConfig.cluster_stage``).  Starts
        from the default-heuristic mix as it is -- also where the register census keeps a
        default pick out of this occupancy's tournament: the census judges a body alone, the
        default mix is what a production build at this occupancy runs, and moving such a pick to
        its nearest admitted neighbour made the start 20 % slower than the default on the int8
        model.  Returns the index of every feature's pick in its candidate list.
        ``clusters/o{occ}/result.json`` keeps what was measured."""
        result_log = f"{self.basic.codegen_dir}/clusters/o{occupancy}/result.json"
        if os.path.exists(result_log) and not tune_config.remeasure:
            with open(result_log) as f:
                return json.load(f)["picks"]
        picks = [int(k) for k in self.default_choices()[0]]
        start = list(picks)
        clusters = self.feature_clusters()
        timer = KernelTimer(self.table_shapes, self.data_types, self.data_npzs,
                            gpu_id=tune_config.gpu_ids[0])
        width = max(1, min(tune_config.num_processes, tune_config.cluster_group))
        log = []
        checks = []

        def emit_build(out: str, cands: list, note: dict) -> Optional[Tuple[str, str]]:
            """Emit a production-shaped build holding ``cands``; the job to schedule, if any."""
            if self._kept(out, tune_config) and os.path.exists(f"{out}/options.json"):
                return None
            os.makedirs(f"{out}/build", exist_ok=True)
            emitter = CodeEmitter(None, feat_candidates=cands)
            emitter.emit(f"{out}/process.hip", occupancy=occupancy, inline=tune_config.inline,
                         tune=True, tile_bytes=tune_config.tile_bytes)
            emitter.emit_cmake_list(f"{out}/CMakeLists.txt", code_fname="process.hip",
                                    host_fname=None, subdirs=self.basic.subdirs,
                                    includes=self.basic.includes, links=self.basic.links,
                                    debug=tune_config.debug)
            with open(f"{out}/options.json", "w") as f:
                json.dump(note, f)
            return out, f"{out}/build"

        for sweep in range(tune_config.cluster_sweeps):
            changed = False
            for lo in range(0, len(clusters), width):
                group = list(enumerate(clusters))[lo:lo + width]
                builds = []
                jobs = []
                for ci, members in group:
                    options = self.cluster_options(members, picks, occupancy, measured_times,
                                                   tune_config.cluster_top_k)
                    if not options:
                        continue
                    # option 0: every member keeps its pick; option j: all members run options[j-1]
                    cands = [[self.feat_sched_param_candidates[f][picks[f]]] for f in range(self.num_feats)]
                    for f in members:
                        cands[f] += [self.feat_sched_param_candidates[f][k] for k in options]
                    out = self.get_cluster_dir(occupancy, sweep, ci)
                    job = emit_build(out, cands, {"members": members, "options": options,
                                                  "picks": [picks[f] for f in members]})
                    if job:
                        jobs.append(job)
                    builds.append((ci, members, options, out))
                # the mix as it is now, built as it ships: what a cluster build's own time with
                # every cluster on its current pick has to come close to
                base_out = f"{self.get_cluster_dir(occupancy, sweep, lo)}_base"
                if self._build_full(base_out, [self.feat_sched_param_candidates[f][k]
                                               for f, k in enumerate(picks)], occupancy, tune_config):
                    jobs.append((base_out, f"{base_out}/build"))
                self._schedule_builds(jobs, tune_config)
                shipped_ns = timer.time_ns(f"{base_out}/build/librecom.so", xcd_segments=DEFAULT_XCD_SEGMENTS)
                wanted = []                                   # (members, new pick, log entry)
                for ci, members, options, out in builds:
                    lib = f"{out}/build/librecom.so"
                    times = timer.time_options(lib, members, len(options) + 1,
                                               xcd_segments=DEFAULT_XCD_SEGMENTS, seed=ci)
                    med = [float(np.median(t)) for t in times]
                    best = int(np.argmin(med))
                    entry = {"sweep": sweep, "cluster": ci, "members": members, "options": options,
                             "kept_picks": [picks[f] for f in members], "kernel_ns": med,
                             "shipped_ns": shipped_ns, "adopted": None, "head_to_head_ns": None}
                    log.append(entry)
                    gain = 1.0 - med[best] / med[0]
                    confirmed = 0.0
                    if med[0] > shipped_ns * (1.0 + tune_config.cluster_build_tolerance):
                        # the options' bodies change the kernel they sit in (registers, scratch):
                        # what this build measures says nothing about the kernel that ships
                        entry["unrepresentative"] = True
                        print(f"[clusters {occupancy}] sweep {sweep} cluster {ci}: its build runs the "
                              f"current mix in {med[0]:.0f} ns, the shipped build in {shipped_ns:.0f} ns: "
                              f"not used", flush=True)
                        continue
                    if best > 0 and gain >= tune_config.cluster_min_gain:
                        # the scan's winner against the current pick, taking turns
                        again = timer.time_options(lib, members, len(options) + 1, rounds=6, repeats=5,
                                                   xcd_segments=DEFAULT_XCD_SEGMENTS, only=[0, best],
                                                   seed=1000 + ci)
                        t_kept, t_best = float(np.median(again[0])), float(np.median(again[best]))
                        entry["head_to_head_ns"] = [t_kept, t_best]
                        confirmed = 1.0 - t_best / t_kept
                        if confirmed >= tune_config.cluster_min_gain:
                            wanted.append((members, options[best - 1], entry))
                    print(f"[clusters {occupancy}] sweep {sweep} cluster {ci} ({len(members)} features, "
                          f"dim {self.metas[members[0]].embed_dim}): kept {med[0]:.0f} ns, best option "
                          f"{med[best]:.0f} ns ({100 * gain:.2f} %)"
                          + (f", head to head {100 * confirmed:.2f} %" if entry["head_to_head_ns"] else ""),
                          flush=True)
                if len(wanted) > 1:
                    # the group's adoptions together, old picks against new, in one more build
                    switching = [f for members, _, _ in wanted for f in members]
                    cands = [[self.feat_sched_param_candidates[f][picks[f]]] for f in range(self.num_feats)]
                    for members, k, _ in wanted:
                        for f in members:
                            cands[f].append(self.feat_sched_param_candidates[f][k])
                    out = f"{self.get_cluster_dir(occupancy, sweep, lo)}_check"
                    job = emit_build(out, cands, {"members": switching})
                    self._schedule_builds([job] if job else [], tune_config)
                    # ... in which the adoptions join one by one, largest head-to-head gain first,
                    # each kept only if the kernel gets faster with it than without
                    lib = f"{out}/build/librecom.so"
                    wanted.sort(key=lambda w: w[2]["head_to_head_ns"][1] / w[2]["head_to_head_ns"][0])
                    current = np.zeros(self.num_feats, dtype=np.int32)
                    kept_now = []
                    for j, (members, k, entry) in enumerate(wanted):
                        trial = current.copy()
                        trial[members] = 1
                        both = timer.time_mixes(lib, [current, trial], rounds=6, repeats=5,
                                                xcd_segments=DEFAULT_XCD_SEGMENTS, seed=2000 + lo + j)
                        t_without, t_with = float(np.median(both[0])), float(np.median(both[1]))
                        if j == 0 and t_without > shipped_ns * (1.0 + tune_config.cluster_build_tolerance):
                            print(f"[clusters {occupancy}] sweep {sweep}: the check build runs the current "
                                  f"mix in {t_without:.0f} ns, the shipped build in {shipped_ns:.0f} ns: "
                                  f"nothing adopted", flush=True)
                            break
                        ok = t_with < t_without * (1.0 - tune_config.cluster_min_gain / 2)
                        checks.append({"sweep": sweep, "first_cluster": lo, "cluster": entry["cluster"],
                                       "joined_after": len(kept_now), "kernel_ns": [t_without, t_with],
                                       "kept": bool(ok)})
                        print(f"[clusters {occupancy}] sweep {sweep}: cluster {entry['cluster']} joining "
                              f"{len(kept_now)} adoptions: {t_without:.0f} -> {t_with:.0f} ns: "
                              f"{'kept' if ok else 'dropped'}", flush=True)
                        if ok:
                            current = trial
                            kept_now.append((members, k, entry))
                    wanted = kept_now
                for members, k, entry in wanted:
                    entry["adopted"] = k
                    for f in members:
                        picks[f] = k
                    changed = True
            if not changed:
                break
        os.makedirs(os.path.dirname(result_log), exist_ok=True)
        with open(result_log, "w") as f:
            json.dump({"picks": picks, "start": start, "clusters": log, "group_checks": checks}, f)
        return picks

    def _nearest_admitted(self, feat_id: int, pick: int, admitted: List[int]) -> int:
        """Position, in the admitted list, of candidate ``pick`` of the feature -- or of the
        admitted candidate of the same template closest to it in parameters."""
        if pick in admitted:
            return admitted.index(pick)
        cands = self.feat_sched_param_candidates[feat_id]
        sched, params = cands[pick]

        def distance(k: int) -> Tuple[int, int]:
            s, p = cands[k]
            if type(s) is not type(sched):
                return (1, 0)
            return (0, sum(abs(a - b) for a, b in zip(p, params)))
        return min(range(len(admitted)), key=lambda j: distance(admitted[j]))

    def tune(self, tune_config: TuneConfig) -> Dict[int, Dict[int, List[float]]]:
        if tune_config.interference == "model":
            return self.tune_in_model(tune_config)
        self.compile_local(tune_config)

        manager = None if tune_config.in_process else TaskManager(tune_config.gpu_ids)
        for feat_id in range(self.num_feats):
            for occupancy in tune_config.occupancies:
                output_dir, build_dir = self.get_output_build_dir(feat_id, occupancy)
                result_log = f"{output_dir}/result.txt"
                if not os.path.exists(result_log) or tune_config.remeasure:
                    args = ((feat_id, occupancy), self.data_npzs[feat_id], self.table_shapes[feat_id],
                            self.data_types[feat_id], len(self.feat_sched_param_candidates[feat_id]),
                            self.local_padded_num(feat_id, occupancy, tune_config),
                            f"{build_dir}/librecom.so", result_log)
                    self._run_measure(manager, tune_config, measure_single_feat, args)
        if manager:
            manager.join()

        results: Dict[int, Dict[int, List[float]]] = {feat_id: {} for feat_id in range(self.num_feats)}
        for feat_id in range(self.num_feats):
            for occupancy in tune_config.occupancies:
                output_dir, build_dir = self.get_output_build_dir(feat_id, occupancy)
                with open(f"{output_dir}/result.txt") as f:     # absent if the worker failed
                    results[feat_id][occupancy] = list(map(float, f.read().strip().split(' ')))
        return results

    def cluster_validation(self, occupancy: int, tune_config: TuneConfig) -> dict:
        """Do the cluster stage's whole-kernel times in its candidate-holding builds carry over to
        kernels built as they ship?  For every cluster of the first sweep (after
        ``cluster_stage``: reads ``clusters/o{occ}/result.json``) the production kernel of the
        mix the cluster was measured against is built with and without the cluster's fastest
        option, both are timed taking turns, and the change is set beside the one the cluster
        build showed.  Writes and returns ``clusters/o{occ}/validation.json``: per cluster the two
        relative changes, and their Spearman rank correlation.  (The cluster-wise counterpart of
        ``mutation_validation``.)"""
        root = f"{self.basic.codegen_dir}/clusters/o{occupancy}"
        with open(f"{root}/result.json") as f:
            doc = json.load(f)
        picks = list(doc["start"])
        rows, jobs, mixes = [], [], {}

        def production(name: str, mix_picks: List[int]) -> str:
            out = f"{root}/validation/{name}"
            mix = [self.feat_sched_param_candidates[f][k] for f, k in enumerate(mix_picks)]
            if self._build_full(out, mix, occupancy, tune_config):
                jobs.append((out, f"{out}/build"))
            return f"{out}/build/librecom.so"

        for entry in doc["clusters"]:
            if entry["sweep"] != 0:
                break
            ns = entry["kernel_ns"]
            best = int(np.argmin(ns[1:])) + 1 if len(ns) > 1 else 0
            if best > 0:
                swapped = list(picks)
                for f in entry["members"]:
                    swapped[f] = entry["options"][best - 1]
                key = hashlib.sha256(json.dumps(picks).encode()).hexdigest()[:10]
                mixes.setdefault(key, production(f"base_{key}", picks))
                rows.append({"cluster": entry["cluster"], "members": entry["members"],
                             "option": entry["options"][best - 1],
                             "cluster_build_change": ns[best] / ns[0] - 1.0,
                             "base": mixes[key], "swapped": production(f"c{entry['cluster']}", swapped)})
            if entry["adopted"] is not None:
                for f in entry["members"]:
                    picks[f] = entry["adopted"]
        self._schedule_builds(jobs, tune_config)
        timer = KernelTimer(self.table_shapes, self.data_types, self.data_npzs,
                            gpu_id=tune_config.gpu_ids[0])
        for row in rows:
            base, swapped = [], []
            for _ in range(5):                                  # taking turns
                base.append(timer.time_ns(row["base"], xcd_segments=DEFAULT_XCD_SEGMENTS, repeats=5))
                swapped.append(timer.time_ns(row["swapped"], xcd_segments=DEFAULT_XCD_SEGMENTS, repeats=5))
            row["production_ns"] = [float(np.median(base)), float(np.median(swapped))]
            row["production_change"] = row["production_ns"][1] / row["production_ns"][0] - 1.0
            del row["base"], row["swapped"]
            print(f"[cluster validation {occupancy}] cluster {row['cluster']}: cluster build "
                  f"{100 * row['cluster_build_change']:+.2f} %, production {100 * row['production_change']:+.2f} %",
                  flush=True)

        def ranks(v):
            order = np.argsort(v, kind="stable")
            r = np.empty(len(v))
            r[order] = np.arange(len(v))
            return r
        rho = None
        if len(rows) >= 3:
            a = ranks([r["cluster_build_change"] for r in rows])
            b = ranks([r["production_change"] for r in rows])
            rho = float(np.corrcoef(a, b)[0, 1])
        out = {"occupancy": occupancy, "rows": rows, "spearman": rho}
        with open(f"{root}/validation.json", "w") as f:
            json.dump(out, f, indent=1)
        print(f"[cluster validation {occupancy}] {len(rows)} clusters, Spearman rank correlation {rho}", flush=True)
        return out

    # ------------------------------------------------------------------ global stage

    def select_per_occupancy(self, measured_times: Dict[int, Dict[int, List[float]]],
                             occupancies: Sequence[int]) -> List[List[Tuple[ScheduleBase, NamedTuple]]]:
        occu_opt_sched_params: List[List[Tuple[ScheduleBase, NamedTuple]]] = [[] for _ in occupancies]
        for feat_id in range(self.num_feats):
            for i, occupancy in enumerate(occupancies):
                opt_idx = int(np.argmin(measured_times[feat_id][occupancy]))
                occu_opt_sched_params[i].append(self.feat_sched_param_candidates[feat_id][opt_idx])
        return occu_opt_sched_params

    def has_outlier_bags(self, sched_params: List[Tuple[ScheduleBase, NamedTuple]]) -> bool:
        """True if a sampled batch holds a bag that a library with outlier tiles would run as
        tiles of its own (beyond its feature's schedule and at least a tile's traffic)."""
        thresholds, _, _ = CodeEmitter(sched_params).long_bag_tables()
        batches = getattr(self, "batches", None)
        if not batches:
            return False
        for thr, feat in zip(thresholds, batches):
            if thr > 0 and any(len(off) > 1 and int(np.diff(off).max()) > thr for _, off in feat):
                return True
        return False

    def decide_outliers(self, sched_params: List[Tuple[ScheduleBase, NamedTuple]], occupancy: int,
                        tile_bytes: int, xcd_segments: int, tune_config: TuneConfig) -> bool:
        """Outlier tiles on or off for ``optimal/``, by measurement: if a sampled batch holds a
        bag that a library with outlier tiles would run as tiles of its own, the mix is built
        both ways and timed on the samples like a contender of the global stage; outlier tiles
        are kept if the whole call (the pass that finds the outliers included) is faster by
        ``TuneConfig.outliers_min_gain``.  Such a bag alone does not decide: the list and the
        arrival of the parts cost the fused kernel registers and LDS, and a model whose long bags
        are a small share of its traffic loses more to that than the outliers cost it (C4: 10 %).
        """
        if not self.has_outlier_bags(sched_params):
            print("outlier tiles: off (no sampled bag beyond its schedule's reach)", flush=True)
            return False
        dirs = {on: f"{self.basic.codegen_dir}/outliers_{'on' if on else 'off'}/o{occupancy}"
                for on in (False, True)}
        jobs = []
        for on, output_dir in dirs.items():
            self.emit_codes(output_dir=output_dir, feat_schedules=sched_params, occupancy=occupancy,
                            inline=tune_config.inline, debug=tune_config.debug, tile_bytes=tile_bytes,
                            xcd_segments=max(xcd_segments, 0), outliers=on)
            jobs.append((output_dir, f"{output_dir}/build"))
        self._schedule_builds(jobs, tune_config)
        manager = self._measure_manager(tune_config)
        if tune_config.profiler == "rocprofv3" or manager:
            release_device_memory()
        cfg = tune_config._replace(remeasure=True)
        for output_dir in dirs.values():
            self._kernel_time(output_dir, cfg, manager)
        if manager:
            manager.join()
        t_off, t_on = (self._read_kernel_time(dirs[on], tune_config) for on in (False, True))
        keep = t_on < t_off * (1.0 - tune_config.outliers_min_gain)
        print(f"outlier tiles: {'on' if keep else 'off'} (measured on the sampled batches: "
              f"{t_on:.0f} ns with, {t_off:.0f} ns without)", flush=True)
        return keep

    def sample_tiles(self, sched_params: List[Tuple[ScheduleBase, NamedTuple]], occupancy: int,
                     tile_bytes: int, tune_config: TuneConfig) -> np.ndarray:
        """Tiles the binding gives every feature of this mix, summed over the sampled batches."""
        metas = [s.meta for s, _ in sched_params]
        tiles = np.zeros(self.num_feats)
        batches = getattr(self, "batches", None) or []
        for k in range(len(batches[0]) if batches else 0):
            tiles += tiles_per_feature([feat[k][1] for feat in batches],
                                       [m.row_bytes + INDEX_BYTES for m in metas],
                                       [m.embed_dim * 4 + BAG_FIXED_BYTES for m in metas],
                                       [s.TileGranularity(p) for s, p in sched_params],
                                       tile_bytes or tune_config.tile_bytes,
                                       grid_blocks=tune_config.sm_count * occupancy)
        return tiles

    def _build_walk_timing(self, sched_params: List[Tuple[ScheduleBase, NamedTuple]], occupancy: int,
                           tile_bytes: int, xcd_segments: int, tune_config: TuneConfig) -> str:
        """Emit and build the mix with tick counters per feature; returns its directory."""
        output_dir = f"{self.basic.codegen_dir}/walk_timing/o{occupancy}"
        self.emit_codes(output_dir=output_dir, feat_schedules=sched_params, occupancy=occupancy,
                        inline=tune_config.inline, timing=True, debug=tune_config.debug,
                        tile_bytes=tile_bytes, xcd_segments=max(xcd_segments, 0))
        self._schedule_builds([(output_dir, f"{output_dir}/build")], tune_config)
        return output_dir

    def tile_time_order(self, sched_params: List[Tuple[ScheduleBase, NamedTuple]], occupancy: int,
                        tile_bytes: int, xcd_segments: int, tune_config: TuneConfig
                        ) -> Optional[List[int]]:
        """The features by the time one of their tiles takes, dearest first: a timing build of
        the mix as it ships (tick counters per feature) is run on the samples, and every
        feature's ticks are divided by the tiles the binding gives it.  (The tournament's tile
        times do not serve: its kernel holds every candidate, and an order by its figures was no
        better than the model's own.)  None if nothing can be told apart."""
        output_dir = self._build_walk_timing(sched_params, occupancy, tile_bytes, xcd_segments, tune_config)
        result = f"{output_dir}/feature_ticks.txt"
        if os.path.exists(result):
            os.remove(result)
        manager = None if tune_config.in_process else TaskManager(tune_config.gpu_ids[0:1])
        if manager:
            release_device_memory()
        args = (f"{output_dir}/build/librecom.so", self.table_shapes, self.data_types, self.data_npzs,
                result, tile_bytes, xcd_segments)
        self._run_measure(manager, tune_config, measure_feature_ticks, args)
        if manager:
            manager.join()
        if not os.path.exists(result):
            return None
        with open(result) as f:
            ticks = [float(line) for line in f if line.strip()]
        tiles = self.sample_tiles(sched_params, occupancy, tile_bytes, tune_config)
        if len(ticks) != self.num_feats:
            return None
        # features of one kind (schedule, parameters, row type and width) share one figure: a
        # single feature's few tiles are too few to tell its time from its neighbours'
        kinds: Dict[tuple, List[float]] = {}
        kind_of = [(type(s).__name__, tuple(p), s.meta.data_type, s.meta.embed_dim) for s, p in sched_params]
        for k, t, n in zip(kind_of, ticks, tiles):
            acc = kinds.setdefault(k, [0.0, 0.0])
            acc[0] += t
            acc[1] += n
        per_tile = [kinds[k][0] / kinds[k][1] if kinds[k][1] > 0 else 0.0 for k in kind_of]
        if len(set(round(v) for v in per_tile)) < 3:
            return None
        return sorted(range(self.num_feats), key=lambda f: (-per_tile[f], f))

    @staticmethod
    def _drawn_variants(tune_config: TuneConfig) -> Dict[str, Tuple[None, int]]:
        return {"drawn_all" if n >= DRAWN_ALL else f"drawn_{n}": (None, int(n))
                for n in tune_config.drawn_tail_candidates}

    def _build_walk_variants(self, variants: Dict[str, Tuple[Optional[List[int]], int]],
                             sched_params: List[Tuple[ScheduleBase, NamedTuple]], occupancy: int,
                             tile_bytes: int, xcd_segments: int, outliers: bool,
                             tune_config: TuneConfig) -> Dict[str, str]:
        """Emit and build ``walk_{name}/o{occ}`` for every variant (tile_order, drawn_tail);
        returns their directories."""
        dirs = {name: f"{self.basic.codegen_dir}/walk_{name}/o{occupancy}" for name in variants}
        jobs = []
        for name, (tile_order, drawn_tail) in variants.items():
            self.emit_codes(output_dir=dirs[name], feat_schedules=sched_params, occupancy=occupancy,
                            inline=tune_config.inline, debug=tune_config.debug, tile_bytes=tile_bytes,
                            xcd_segments=max(xcd_segments, 0), outliers=outliers,
                            tile_order=tile_order, drawn_tail=drawn_tail)
            jobs.append((dirs[name], f"{dirs[name]}/build"))
        self._schedule_builds(jobs, tune_config)
        return dirs

    def decide_walk(self, sched_params: List[Tuple[ScheduleBase, NamedTuple]], occupancy: int,
                    tile_bytes: int, xcd_segments: int, outliers: bool, tune_config: TuneConfig
                    ) -> Tuple[Optional[List[int]], int, int]:
        """(tile_order, drawn_tail, xcd_segments) for ``optimal/``, by measurement.

        A drawn end: the last passes of the tile walk -- or all of them -- are drawn from ticket
        counters instead of dealt out.  Workgroups whose tiles were cheap then take more of them,
        and the workgroups of an XCD stay together on neighbouring tiles, i.e. on the hot rows
        of one or two features at a time: 8-11 % on a model of 400 features and 80 tiles per
        workgroup, 3.5 % on one of 200 features with eight passes drawn (all of them: 2 %), a
        loss of 1-3 % on one of 100 features and 14 short tiles per workgroup.  Tried with
        ``TuneConfig.drawn_tail_candidates`` when the workgroups get at least
        ``walk_drawn_min_tiles`` tiles each and the library has no outlier tiles (which are
        drawn already).

        An order: with the features sorted by their time per tile, the strided deal hands every
        workgroup one tile of each kind, and a drawn end has cheap tiles to fill it with: 3 and
        7 % on a model of a thousand small features whose workgroups get five tiles each,
        1.6 % on one of a hundred features and 14 tiles per workgroup, nothing on one of 2 500
        features and 15.  Tried on models of ``walk_stage_min_feats`` features and more whose
        workgroups get fewer than ``walk_stage_max_tiles`` tiles.

        All variants are built, timed on the samples like contenders of the global stage, and
        the fastest is kept if it gains ``TuneConfig.walk_min_gain``.  A drawn winner is then
        timed with finer segments per XCD (``walk_xcd_segments_candidates``): drawing takes care
        of the balance inside an XCD, finer segments of the balance between them."""
        keep_as_is = (None, 0, xcd_segments)
        if tune_config.walk_stage is False:
            return keep_as_is
        batches = getattr(self, "batches", None) or [[]]
        per_workgroup = (self.sample_tiles(sched_params, occupancy, tile_bytes, tune_config).sum()
                         / max(1, len(batches[0])) / (tune_config.sm_count * occupancy))
        forced = tune_config.walk_stage is True
        variants = {"as_is": (None, 0)}
        if not outliers and (forced or per_workgroup >= tune_config.walk_drawn_min_tiles):
            variants.update(self._drawn_variants(tune_config))
        order = None
        if forced or (self.num_feats >= tune_config.walk_stage_min_feats
                      and per_workgroup < tune_config.walk_stage_max_tiles):
            order = self.tile_time_order(sched_params, occupancy, tile_bytes, xcd_segments, tune_config)
        if order is not None:
            variants["ordered"] = (order, 0)
            if not outliers:
                variants["ordered_drawn_2"] = (order, 2)
        if len(variants) == 1:
            return keep_as_is
        dirs = self._build_walk_variants(variants, sched_params, occupancy, tile_bytes, xcd_segments,
                                         outliers, tune_config)
        cfg = tune_config._replace(remeasure=True)

        def timed(runs: List[Tuple[str, int]]) -> List[float]:
            manager = self._measure_manager(tune_config)
            if tune_config.profiler == "rocprofv3" or manager:
                release_device_memory()
            for output_dir, xs in runs:
                self._kernel_time(output_dir, cfg, manager, 0, xs)
            if manager:
                manager.join()
            return [self._read_kernel_time(output_dir, tune_config, 0, xs) for output_dir, xs in runs]

        times = dict(zip(variants, timed([(dirs[name], 0) for name in variants])))
        best = min(times, key=times.get)
        keep = best if times[best] < times["as_is"] * (1.0 - tune_config.walk_min_gain) else "as_is"
        print("tile walk: " + ", ".join(f"{name} {t:.0f} ns" for name, t in times.items())
              + f": {keep.replace('_', ' ')}", flush=True)
        tile_order, drawn_tail = variants[keep]
        if drawn_tail and xcd_segments > 0:
            finer = [xs for xs in tune_config.walk_xcd_segments_candidates if xs > xcd_segments]
            if finer:
                finer_times = timed([(dirs[keep], xs) for xs in finer])
                k = int(np.argmin(finer_times))
                print(f"tile walk, segments per XCD: {xcd_segments}: {times[keep]:.0f} ns, "
                      + ", ".join(f"{xs}: {t:.0f} ns" for xs, t in zip(finer, finer_times)), flush=True)
                if finer_times[k] < times[keep] * (1.0 - tune_config.walk_min_gain):
                    xcd_segments = finer[k]
        return tile_order, drawn_tail, xcd_segments

    def solve(self, measured_times: Dict[int, Dict[int, List[float]]],
              tune_config: TuneConfig) -> Tuple[int, List[Tuple[ScheduleBase, NamedTuple]]]:
        occu_opt_sched_params = ([] if tune_config.only_incumbent else
                                 self.select_per_occupancy(measured_times, tune_config.occupancies))
        opt_occupancy, opt_sched_params = self.tune_occupancy(occu_opt_sched_params, tune_config)
        output_dir = self.opt_output_dir
        optimal = f"{self.basic.codegen_dir}/optimal"
        shutil.rmtree(optimal, ignore_errors=True)
        shutil.copytree(output_dir, optimal)
        tile_bytes = getattr(self, "opt_tile_bytes", tune_config.tile_bytes)
        xcd_segments = getattr(self, "opt_xcd_segments", 0)
        climbed = False
        if tune_config.build_climb_trials > 0:
            mix, t = self.build_climb(opt_sched_params, opt_occupancy, measured_times, tune_config,
                                      tile_bytes=tile_bytes, xcd_segments=xcd_segments)
            climbed = any(a[0].EmitScheduleBody(a[1]) != b[0].EmitScheduleBody(b[1])
                          for a, b in zip(mix, opt_sched_params))
            opt_sched_params = mix
            print(f"occupancy: {opt_occupancy} (after the build climb), t(ns): {t}", flush=True)
        outliers = tune_config.outliers
        if outliers is None:
            outliers = self.decide_outliers(opt_sched_params, opt_occupancy, tile_bytes, xcd_segments,
                                            tune_config)
        tile_order, drawn_tail, xcd_segments = self.decide_walk(
            opt_sched_params, opt_occupancy, tile_bytes, xcd_segments, bool(outliers), tune_config)
        # a contender whose library came out of the compile cache (the same source had been built
        # in another directory) has no host module of its own: optimal/ is then built in place
        import glob
        host_missing = not glob.glob(f"{optimal}/build/recom_host*.so")
        if climbed or tile_bytes != tune_config.tile_bytes or xcd_segments or outliers or host_missing \
                or tile_order is not None or drawn_tail:
            # make the winning launch parameters the defaults of the optimal library
            self.emit_codes(output_dir=optimal, feat_schedules=opt_sched_params, occupancy=opt_occupancy,
                            inline=tune_config.inline, debug=tune_config.debug, tile_bytes=tile_bytes,
                            xcd_segments=max(xcd_segments, 0), outliers=outliers,
                            tile_order=tile_order, drawn_tail=drawn_tail)
            shutil.rmtree(f"{optimal}/build", ignore_errors=True)   # the copied CMake cache names another dir
            compile_build(f"{optimal}/build")
        with open(f"{optimal}/schedule.json", "w") as f:
            json.dump({"occupancy": opt_occupancy, "tile_bytes": tile_bytes,
                       "xcd_segments": max(xcd_segments, 0), "outliers": bool(outliers),
                       "tile_order": tile_order, "drawn_tail": int(drawn_tail),
                       "schedules": CodeEmitter(opt_sched_params).serialize_config()}, f, indent=1)
        return opt_occupancy, opt_sched_params

    def solve_launch_only(self, tune_config: TuneConfig) -> Tuple[int, List[Tuple[ScheduleBase, NamedTuple]]]:
        """Global stage alone: the default schedule of every feature, swept over occupancy, traffic
        per tile and tile walk.  Needs no tuning build; ends like ``solve`` with ``optimal/``."""
        default_mix = [self.feat_sched_param_candidates[f][k]
                       for f, k in enumerate(self.default_choices()[0])]
        cfg = tune_config._replace(include_default=False)
        results = {f: {occ: [0.0 if c is default_mix[f] else 1.0
                             for c in self.feat_sched_param_candidates[f]]
                       for occ in cfg.occupancies} for f in range(self.num_feats)}
        return self.solve(results, cfg)

    def solve_incumbent_only(self, tune_config: TuneConfig) -> Tuple[int, List[Tuple[ScheduleBase, NamedTuple]]]:
        """Global stage for the mix of ``TuneConfig.incumbent`` alone: swept over occupancy,
        traffic per tile and tile walk, then the decisions on outlier tiles and on the walk.
        Needs no tuning build; ends like ``solve`` with ``optimal/``."""
        if not tune_config.incumbent:
            raise ValueError("no incumbent given")
        return self.solve({}, tune_config._replace(include_default=False, only_incumbent=True,
                                                   build_climb_trials=0))

    def _build_full(self, output_dir: str, sched_params, occupancy: Optional[int],
                    tune_config: TuneConfig, fixed_task_block_nums: List[int] = None,
                    timing: bool = False) -> bool:
        """Emit a whole-model kernel if its library is missing; True if a build is needed."""
        build_dir = f"{output_dir}/build"
        if self._kept(output_dir, tune_config):
            return False
        os.makedirs(build_dir, exist_ok=True)
        self.emit_codes(output_dir=output_dir, feat_schedules=sched_params, occupancy=occupancy,
                        inline=tune_config.inline, timing=timing, tune=False, debug=tune_config.debug,
                        fixed_task_block_nums=fixed_task_block_nums, tile_bytes=tune_config.tile_bytes)
        return True

    @staticmethod
    def _report_prefix(output_dir: str, tile_bytes: int, xcd_segments: int) -> str:
        return (f"{output_dir}/report" + (f".t{tile_bytes}" if tile_bytes else "")
                + (f".x{xcd_segments}" if xcd_segments else ""))

    def _kernel_time(self, output_dir: str, tune_config: TuneConfig, manager: Optional[TaskManager],
                     tile_bytes: int = 0, xcd_segments: int = 0) -> None:
        """Schedule the whole-kernel measurement of the model built in ``output_dir``
        (0 = the traffic per tile / tile walk the library was emitted with)."""
        build_dir = f"{output_dir}/build"
        report_prefix = self._report_prefix(output_dir, tile_bytes, xcd_segments)
        if tune_config.profiler == "rocprofv3":
            stats = f"{report_prefix}_kernel_stats.csv"
            if not os.path.exists(stats) or tune_config.remeasure:
                os_check(f"rm -f {report_prefix}_*.csv")
                args = (self.table_config_fname, build_dir, self.data_dir, self.basic.sample_batch_nums,
                        report_prefix, None, tile_bytes, xcd_segments)
                if manager:
                    manager.add_task(rocprof_profile, args, ident_key="gpu_id")
                else:
                    rocprof_profile(*args, gpu_id=tune_config.gpu_ids[0])
        else:
            result = f"{report_prefix}.events.txt"
            if not os.path.exists(result) or tune_config.remeasure:
                args = (f"{build_dir}/librecom.so", self.table_shapes, self.data_types, self.data_npzs,
                        result, tile_bytes, xcd_segments)
                self._run_measure(manager, tune_config, measure_kernel_events, args)

    def _read_kernel_time(self, output_dir: str, tune_config: TuneConfig, tile_bytes: int = 0,
                          xcd_segments: int = 0) -> float:
        report_prefix = self._report_prefix(output_dir, tile_bytes, xcd_segments)
        if tune_config.profiler == "rocprofv3":
            # per batch the median over the measured passes of the call's kernels (the fused
            # kernel and what the library launches ahead of it), summed over the batches: the
            # same quantity the events timer reports
            try:
                return float(sum(parse_knl_batch_times("FusedKnl", f"{report_prefix}_kernel_trace.csv",
                                                       PROFILE_PASSES, PROFILE_WARMUP_PASSES)))
            except (ValueError, OSError) as e:
                # say what the profiled child printed: the trace alone does not tell why it is short
                log = f"{report_prefix}.rocprofv3.log"
                tail = ""
                if os.path.exists(log):
                    with open(log, errors="replace") as f:
                        tail = "".join(f.readlines()[-15:])
                raise RuntimeError(f"no usable kernel trace for {output_dir} ({e}); the profiled "
                                   f"run printed:\n{tail}") from e
        with open(f"{report_prefix}.events.txt") as f:
            return float(f.read().strip())

    def _measure_manager(self, tune_config: TuneConfig) -> Optional[TaskManager]:
        if tune_config.in_process and tune_config.profiler != "rocprofv3":
            return None
        if tune_config.profiler == "rocprofv3" and tune_config.in_process:
            return None      # rocprof_profile spawns its own process; run them one after another
        return TaskManager(tune_config.gpu_ids[0:1])

    def default_contenders(self, tune_config: TuneConfig) -> list:
        """(directory, occupancy, schedules) of the default-heuristic mix at every occupancy: the
        contenders of the global stage that are known before anything is measured."""
        if not tune_config.include_default:
            return []
        default_mix = [self.feat_sched_param_candidates[f][k]
                       for f, k in enumerate(self.default_choices()[0])]
        return [(f"{self.basic.codegen_dir}/default/o{occupancy}", occupancy, default_mix)
                for occupancy in tune_config.occupancies]

    def incumbent_contenders(self, tune_config: TuneConfig) -> list:
        """(directory, occupancy, schedules) of the mix in ``TuneConfig.incumbent`` at every
        occupancy."""
        if not tune_config.incumbent:
            return []
        from recflex_amd.schedules import schedule_from_config
        with open(tune_config.incumbent) as f:
            doc = json.load(f)
        entries = doc["schedules"] if isinstance(doc, dict) else doc
        if len(entries) != self.num_feats:
            raise ValueError(f"{tune_config.incumbent} describes {len(entries)} features, the model has {self.num_feats}")
        mix = [schedule_from_config(e, meta, self.basic.block_threads) for e, meta in zip(entries, self.metas)]
        return [(f"{self.basic.codegen_dir}/incumbent/o{occupancy}", occupancy, mix)
                for occupancy in tune_config.occupancies]

    def compile_incumbent_contenders(self, tune_config: TuneConfig) -> None:
        """Emit and build ``incumbent/o{occ}`` (no GPU needed) and, where the launch options are
        given rather than swept (one candidate each), the drawn-end variants of the walk stage
        and its timing build, so that a run with ``only_incumbent`` finds them built."""
        contenders = self.incumbent_contenders(tune_config)
        jobs = []
        for output_dir, occupancy, sched_params in contenders:
            if self._build_full(output_dir, sched_params, occupancy, tune_config):
                jobs.append((output_dir, f"{output_dir}/build"))
        self._schedule_builds(jobs, tune_config)
        tile_opts = list(tune_config.tile_bytes_candidates) or [0]
        walk_opts = list(tune_config.xcd_segments_candidates) or [0]
        if tune_config.walk_stage is False or len(tile_opts) != 1 or len(walk_opts) != 1:
            return
        tile_bytes, xcd_segments = tile_opts[0] or tune_config.tile_bytes, walk_opts[0]
        for _, occupancy, sched_params in contenders:
            variants = dict({"as_is": (None, 0)}, **self._drawn_variants(tune_config))
            self._build_walk_variants(variants, sched_params, occupancy, tile_bytes, xcd_segments, False,
                                      tune_config)
            self._build_walk_timing(sched_params, occupancy, tile_bytes, xcd_segments, tune_config)

    def compile_default_contenders(self, tune_config: TuneConfig) -> None:
        """Emit and build ``default/o{occ}`` (no GPU needed)."""
        jobs = []
        for output_dir, occupancy, sched_params in self.default_contenders(tune_config):
            if self._build_full(output_dir, sched_params, occupancy, tune_config):
                jobs.append((output_dir, f"{output_dir}/build"))
        self._schedule_builds(jobs, tune_config)

    def tune_occupancy(self, occu_opt_sched_params: List[List[Tuple[ScheduleBase, NamedTuple]]],
                       tune_config: TuneConfig) -> Tuple[int, List[Tuple[ScheduleBase, NamedTuple]]]:
        # contenders: (directory, occupancy, schedules)
        contenders = []
        for occupancy, sched_params in zip(tune_config.occupancies, occu_opt_sched_params):
            contenders.append((self.get_output_build_dir(-1, occupancy)[0], occupancy, sched_params))
        contenders += self.default_contenders(tune_config)
        contenders += self.incumbent_contenders(tune_config)

        jobs = []
        for output_dir, occupancy, sched_params in contenders:
            if self._build_full(output_dir, sched_params, occupancy, tune_config):
                jobs.append((output_dir, f"{output_dir}/build"))
        self._schedule_builds(jobs, tune_config)

        launch_opts = [(tb, xs) for tb in (list(tune_config.tile_bytes_candidates) or [0])
                       for xs in (list(tune_config.xcd_segments_candidates) or [0])]
        manager = self._measure_manager(tune_config)
        if tune_config.profiler == "rocprofv3" or manager:
            release_device_memory()
        for output_dir, occupancy, _ in contenders:
            for tile_bytes, xcd_segments in launch_opts:
                self._kernel_time(output_dir, tune_config, manager, tile_bytes, xcd_segments)
        if manager:
            manager.join()

        times, best_opts = [], []
        for output_dir, occupancy, _ in contenders:
            per_opt = [self._read_kernel_time(output_dir, tune_config, tb, xs) for tb, xs in launch_opts]
            # contenders compete on their fastest option; the tolerance rule then settles the
            # launch option of the winner only (kept and fastest option differ by at most the
            # tolerance, which must not decide between contenders)
            times.append(float(np.min(per_opt)))
            k = pick_launch_option(launch_opts, per_opt, tune_config.launch_time_tolerance)
            best_opts.append(launch_opts[k])
            kind = "default" if "/default/o" in output_dir else ("incumbent" if "/incumbent/o" in output_dir else "tuned")
            print(f"occupancy: {occupancy} ({kind}), t(ns): {times[-1]}"
                  + (f", (tile_bytes, xcd_segments): {launch_opts[k]} (of "
                     f"{ {o: round(t) for o, t in zip(launch_opts, per_opt)} })" if len(launch_opts) > 1 else ""))

        opt_idx = int(np.argmin(times))
        self.opt_tile_bytes = best_opts[opt_idx][0] or tune_config.tile_bytes
        self.opt_xcd_segments = best_opts[opt_idx][1]
        self.opt_output_dir, opt_occupancy, opt_sched_params = contenders[opt_idx]
        return opt_occupancy, opt_sched_params

    def build_climb(self, start: List[Tuple[ScheduleBase, NamedTuple]], occupancy: int,
                    measured_times: Dict[int, Dict[int, List[float]]], tune_config: TuneConfig,
                    tile_bytes: int = 0, xcd_segments: int = 0
                    ) -> Tuple[List[Tuple[ScheduleBase, NamedTuple]], float]:
        """Hill climb on production builds (see ``TuneConfig.build_climb_trials``).  Tile times and
        even whole-kernel times taken inside the tournament build do not carry over exactly to a
        production build (other register allocation, other code size), so the last word goes to
        kernels built exactly as they ship.  Returns the improved mix and its time in ns."""
        climb_dir = f"{self.basic.codegen_dir}/climb/o{occupancy}"
        timer = KernelTimer(self.table_shapes, self.data_types, self.data_npzs,
                            gpu_id=tune_config.gpu_ids[0])
        cfg = tune_config._replace(tile_bytes=tile_bytes or tune_config.tile_bytes)

        def build_all(mixes: List[Tuple[str, list]]) -> None:
            jobs = []
            for name, mix in mixes:
                out = f"{climb_dir}/{name}"
                if not os.path.exists(f"{out}/build/librecom.so"):
                    os.makedirs(f"{out}/build", exist_ok=True)
                    self.emit_codes(output_dir=out, feat_schedules=mix, occupancy=occupancy,
                                    inline=cfg.inline, debug=cfg.debug, tile_bytes=cfg.tile_bytes,
                                    host=False, xcd_segments=max(xcd_segments, 0))
                    jobs.append((out, f"{out}/build"))
            self._schedule_builds(jobs, cfg)

        def time_of(name: str, repeats: int = 7) -> float:
            return timer.time_ns(f"{climb_dir}/{name}/build/librecom.so", repeats=repeats)

        best = list(start)
        build_all([("base0", best)])
        best_ns = time_of("base0", repeats=11)
        print(f"[build climb {occupancy}] start {best_ns:.0f} ns", flush=True)

        # Moves, heaviest first.  Group moves: all features that run the same body now (and have
        # the same candidate list) switch together to one of the candidates their summed
        # tournament scores rank best -- a change too small to measure on one light feature shows
        # when twenty features make it.  Then single-feature moves.
        lookups = [sum(len(i) for i, _ in self.batches[f]) for f in range(self.num_feats)]
        weight = np.asarray([lookups[f] * self.metas[f].row_bytes + self.metas[f].embed_dim * 4 *
                             sum(len(o) - 1 for _, o in self.batches[f])
                             for f in range(self.num_feats)], dtype=np.float64)
        top_k = tune_config.build_climb_top_k

        def scores_of(feat: int) -> np.ndarray:
            return np.asarray(measured_times[feat][occupancy], dtype=np.float64)

        groups: Dict[Tuple[str, int], List[int]] = {}
        for feat in range(self.num_feats):
            key = (best[feat][0].EmitScheduleBody(best[feat][1]), len(self.feat_sched_param_candidates[feat]))
            groups.setdefault(key, []).append(feat)
        moves: List[Tuple[List[int], int]] = []
        for feats in sorted(groups.values(), key=lambda g: -weight[g].sum()):
            if len(feats) < 2:
                continue
            ref = self.feat_sched_param_candidates[feats[0]]
            same = all(all(a[0].EmitScheduleBody(a[1]) == b[0].EmitScheduleBody(b[1])
                           for a, b in zip(ref, self.feat_sched_param_candidates[f])) for f in feats[1:])
            if not same:
                continue
            total = np.zeros(len(ref))
            for f in feats:
                sc = scores_of(f)
                finite = sc[np.isfinite(sc)]
                total += np.where(np.isfinite(sc), sc / (finite.min() if finite.size else 1.0), np.inf)
            ranked = [int(k) for k in np.argsort(total) if np.isfinite(total[k])]
            moves.extend((list(feats), k) for k in ranked[:top_k])
        for feat in np.argsort(-weight):
            sc = scores_of(int(feat))
            ranked = [int(k) for k in np.argsort(sc) if np.isfinite(sc[k])]
            moves.extend(([int(feat)], k) for k in ranked[:top_k])
        moves = moves[:tune_config.build_climb_trials]

        def body(cand) -> str:
            return cand[0].EmitScheduleBody(cand[1])

        width = max(1, tune_config.num_processes)
        generation = 0
        for lo in range(0, len(moves), width):
            batch = []
            for j, (feats, k) in enumerate(moves[lo:lo + width]):
                mix = list(best)
                for f in feats:
                    mix[f] = self.feat_sched_param_candidates[f][k]
                if all(body(mix[f]) == body(best[f]) for f in feats):
                    continue
                batch.append((f"g{generation}_m{lo + j}", feats, k, mix))
            if not batch:
                continue
            build_all([(name, mix) for name, _, _, mix in batch])
            gains = []
            for name, feats, k, _ in batch:
                t = time_of(name)
                if t < best_ns * (1.0 - tune_config.build_climb_min_gain):
                    gains.append((t, feats, k, name))
            if not gains:
                continue
            gains.sort(key=lambda g: g[0])
            # several moves may have helped: adopt those that touch different features together
            # if that is faster still
            merged = list(best)
            taken: set = set()
            adopted = 0
            for _, feats, k, _ in gains:
                if taken.isdisjoint(feats):
                    for f in feats:
                        merged[f] = self.feat_sched_param_candidates[f][k]
                    taken.update(feats)
                    adopted += 1
            generation += 1
            t_single = time_of(gains[0][3], repeats=11)
            t_merged = t_single
            if adopted > 1:
                build_all([(f"base{generation}", merged)])
                t_merged = time_of(f"base{generation}", repeats=11)
            if adopted > 1 and t_merged <= t_single and t_merged < best_ns:
                best, best_ns = merged, t_merged
            elif t_single < best_ns:
                best = list(best)
                for f in gains[0][1]:
                    best[f] = self.feat_sched_param_candidates[f][gains[0][2]]
                best_ns = t_single
            print(f"[build climb {occupancy}] after {lo + len(batch)} moves: {best_ns:.0f} ns", flush=True)
        return best, best_ns

    # ------------------------------------------------------------------ validation / ablations

    def compile_mutation(self, opt_sched_params: List[Tuple[ScheduleBase, NamedTuple]], opt_occupancy: int,
                         mut_feat_id: int, tune_config: TuneConfig) -> int:
        """Emit and build ``mutation_f{id}/m{k}``: the whole model with feature ``mut_feat_id``
        switched to its candidate ``k``, for every ``k`` (no GPU needed).  Returns the index of
        the candidate ``opt_sched_params`` holds for that feature (-1 if it is not in the list)."""
        mutation_dir = f"{self.basic.codegen_dir}/mutation_f{mut_feat_id}"
        candidates = self.feat_sched_param_candidates[mut_feat_id]
        opt_idx = -1
        jobs = []
        for candidate_id, mut_sched_param in enumerate(candidates):
            if tuple(mut_sched_param) == tuple(opt_sched_params[mut_feat_id]) or (
                    type(mut_sched_param[0]) is type(opt_sched_params[mut_feat_id][0])
                    and mut_sched_param[1] == opt_sched_params[mut_feat_id][1]):
                opt_idx = candidate_id
            mut_sched_params = list(opt_sched_params)
            mut_sched_params[mut_feat_id] = mut_sched_param
            output_dir = f"{mutation_dir}/m{candidate_id}"
            if self._build_full(output_dir, mut_sched_params, opt_occupancy, tune_config):
                jobs.append((output_dir, f"{output_dir}/build"))
        self._schedule_builds(jobs, tune_config)
        return opt_idx

    def mutation_validation(self, opt_sched_params: List[Tuple[ScheduleBase, NamedTuple]], opt_occupancy: int,
                            mut_feat_id: int, tune_config: TuneConfig) -> Tuple[List[float], int]:
        """Whole-kernel time with feature ``mut_feat_id`` switched to each of its candidates in
        turn; returns the times and the index of the tuner's own pick."""
        mutation_dir = f"{self.basic.codegen_dir}/mutation_f{mut_feat_id}"
        candidates = self.feat_sched_param_candidates[mut_feat_id]
        opt_idx = self.compile_mutation(opt_sched_params, opt_occupancy, mut_feat_id, tune_config)

        manager = self._measure_manager(tune_config)
        for candidate_id in range(len(candidates)):
            self._kernel_time(f"{mutation_dir}/m{candidate_id}", tune_config, manager)
        if manager:
            manager.join()
        times = [self._read_kernel_time(f"{mutation_dir}/m{candidate_id}", tune_config)
                 for candidate_id in range(len(candidates))]
        return times, opt_idx

    def _naive_dirs(self, feat_id: int, sched_param_id: int) -> Tuple[str, str]:
        output_dir = f"{self.basic.codegen_dir}/naive/f{feat_id}/s{sched_param_id}"
        return output_dir, f"{output_dir}/build"

    def compile_naive(self, tune_config: TuneConfig) -> None:
        """Emit and build ``naive/f{feat}/s{k}``: one single-feature kernel per candidate (no GPU
        needed; features with the same candidate list share their builds)."""
        get_output_build_dir = self._naive_dirs
        jobs = []
        for feat_id in range(self.num_feats):
            for sched_param_id, sched_param in enumerate(self.feat_sched_param_candidates[feat_id]):
                output_dir, build_dir = get_output_build_dir(feat_id, sched_param_id)
                if not self._kept(output_dir, tune_config):
                    os.makedirs(build_dir, exist_ok=True)
                    self.emit_codes(output_dir=output_dir, feat_schedules=[sched_param], occupancy=None,
                                    inline=tune_config.inline, timing=False, tune=False,
                                    debug=tune_config.debug, tile_bytes=tune_config.tile_bytes, host=False)
                    jobs.append((output_dir, build_dir))
        self._schedule_builds(jobs, tune_config)

    def tune_naive(self, tune_config: TuneConfig) -> Tuple[List[Tuple[ScheduleBase, NamedTuple]], float]:
        """Every candidate of every feature measured alone on the GPU (no interference, no
        occupancy control); the per-feature winners are fused and the whole kernel timed."""
        get_output_build_dir = self._naive_dirs
        self.compile_naive(tune_config)

        manager = None if tune_config.in_process else TaskManager(tune_config.gpu_ids)
        for feat_id in range(self.num_feats):
            for sched_param_id in range(len(self.feat_sched_param_candidates[feat_id])):
                output_dir, build_dir = get_output_build_dir(feat_id, sched_param_id)
                result_log = f"{output_dir}/result.txt"
                if not os.path.exists(result_log) or tune_config.remeasure:
                    args = ((feat_id, sched_param_id), self.data_npzs[feat_id], self.table_shapes[feat_id],
                            self.data_types[feat_id], f"{build_dir}/librecom.so", result_log)
                    self._run_measure(manager, tune_config, measure_naive_candidate, args)
        if manager:
            manager.join()

        opt_sched_params: List[Tuple[ScheduleBase, NamedTuple]] = []
        for feat_id in range(self.num_feats):
            times = []
            for sched_param_id in range(len(self.feat_sched_param_candidates[feat_id])):
                output_dir, build_dir = get_output_build_dir(feat_id, sched_param_id)
                with open(f"{output_dir}/result.txt") as f:
                    times.append(float(f.read().strip()))
            opt_sched_params.append(self.feat_sched_param_candidates[feat_id][int(np.argmin(times))])

        output_dir = f"{self.basic.codegen_dir}/naive/optimal"
        if self._build_full(output_dir, opt_sched_params, None, tune_config):
            self._schedule_builds([(output_dir, f"{output_dir}/build")], tune_config)
        manager = self._measure_manager(tune_config)
        self._kernel_time(output_dir, tune_config, manager)
        if manager:
            manager.join()
        return opt_sched_params, self._read_kernel_time(output_dir, tune_config)

    def compile_fixed_thread_binding(self, opt_sched_params: List[Tuple[ScheduleBase, NamedTuple]],
                                     choice: str, tune_config: TuneConfig,
                                     occupancy: int = None) -> List[int]:
        """Write ``fixed_thread_binding_{choice}/task_blocks.txt`` (the tiles per feature the
        run-time binding would choose for each sampled batch, computed on the CPU), freeze their
        mean / max into a kernel and build it (no GPU needed).  Returns the frozen counts."""
        assert choice in ["max", "mean"]
        output_dir = f"{self.basic.codegen_dir}/fixed_thread_binding_{choice}"
        fixed_blocks_path = f"{output_dir}/task_blocks.txt"
        if not os.path.exists(fixed_blocks_path) or tune_config.remeasure:
            os.makedirs(output_dir, exist_ok=True)
            metas = [s.meta for s, _ in opt_sched_params]
            measure_task_blocks(self.data_npzs,
                                [m.row_bytes + INDEX_BYTES for m in metas],
                                [m.embed_dim * 4 + BAG_FIXED_BYTES for m in metas],
                                [s.TileGranularity(p) for s, p in opt_sched_params],
                                tune_config.tile_bytes, fixed_blocks_path,
                                grid_blocks=tune_config.sm_count * (occupancy or self.natural_occupancy_guess()))

        task_block_batches: List[List[int]] = []
        with open(fixed_blocks_path) as f:
            for line in f.readlines():
                if line.strip():
                    task_block_batches.append(list(map(int, line.strip().split(','))))

        if choice == "max":
            fixed_task_blocks: List[int] = np.max(task_block_batches, axis=0).tolist()
        else:
            fixed_task_blocks: List[int] = np.mean(task_block_batches, axis=0, dtype=np.int32).tolist()
        fixed_task_blocks = [max(1, int(b)) for b in fixed_task_blocks]

        if self._build_full(output_dir, opt_sched_params, occupancy, tune_config,
                            fixed_task_block_nums=fixed_task_blocks):
            self._schedule_builds([(output_dir, f"{output_dir}/build")], tune_config)
        return fixed_task_blocks

    def natural_occupancy_guess(self) -> int:
        """Workgroups per CU of a library emitted without an occupancy (the frozen-binding
        ablation is): the grid the run-time binding of such a library sees is compute units x
        this.  The fused kernels here use 64 to 128 vector registers, which is 4 workgroups of
        256 threads per CU; other workgroup sizes scale."""
        return max(1, 4 * 256 // max(64, self.basic.block_threads))

    def tune_fixed_thread_binding(self, opt_sched_params: List[Tuple[ScheduleBase, NamedTuple]], choice: str,
                                  tune_config: TuneConfig, occupancy: int = None) -> Tuple[List[int], float]:
        """Ablation: the number of tiles per feature is frozen to the mean / max over the sampled
        batches of what the run-time binding chose, and baked into the kernel.  ``occupancy``:
        the workgroups per CU of the run-time-bound library it is compared with (its grid enters
        the binding's rules)."""
        fixed_task_blocks = self.compile_fixed_thread_binding(opt_sched_params, choice, tune_config,
                                                              occupancy)
        output_dir = f"{self.basic.codegen_dir}/fixed_thread_binding_{choice}"
        manager = self._measure_manager(tune_config)
        self._kernel_time(output_dir, tune_config, manager)
        if manager:
            manager.join()
        return fixed_task_blocks, self._read_kernel_time(output_dir, tune_config)
