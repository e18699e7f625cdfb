"""Tune the per-feature schedules and the occupancy of the fused embedding kernel of a model.

    python tune.py -m models/test [-o models/test/output] [-n 8] [-b 256]
                   [--local_only] [--naive] [--fixed_thread_binding] [--mutation_feat_id K]
                   [--recompile] [--remeasure] [--noinline] [--debug]

Flags as in the reference's ``examples/tune.py:35-51``.  ``-m`` names a model directory with
``table_config.txt``, ``schedule_config.txt`` and ``data/`` (``batch_sizes.txt`` + ``f{i}.txt``).
Additions: ``--workload c3`` tunes one of the built-in synthetic configurations instead of a
model directory; ``--compile_only`` stops after emitting and building the local-stage kernels
and the default-schedule contenders of the global stage (no GPU needed -- a later run finds
the libraries, measures, and builds only the mix it elects); ``--occupancies`` and
``--sample_batch_nums`` bound the search; ``--profiler events`` times the global stage with
events instead of spawning rocprofv3.  The result is ``<output>/optimal/`` (sources, library,
``schedule.json``).
"""

import argparse
import multiprocessing as mp
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

import numpy as np

from recflex_amd.tuning import Tuner, TuneConfig, BasicConfig
from recflex_amd.utils import get_data_fnames
from recflex_amd.code_emitter.build_basic import BasicBuilder

from schedules.reduce_by_key import ReduceByKeySchedule, ReduceByKeyParams
from schedules.multi_block_per_sample import MultiBlockPerSampleSchedule, MultiBlockPerSampleParams
from schedules.one_block_multi_sample import OneBlockMultiSampleSchedule, OneBlockMultiSampleParams
from schedules.warp_per_sample import WarpPerSampleSchedule, WarpPerSampleParams
from schedules.one_hot import OneHotSchedule, OneHotParams
from schedules.one_hot_multi_block import OneHotMultiBlockSchedule, OneHotMultiBlockParams
from recflex_amd.schedules import (ThreadPerBagSchedule, SubWavefrontPerBagSchedule,
                                   WavefrontPerBagSchedule, BlockPerBagSchedule, OneHotBagSchedule)

# number of compute units and resident threads per CU of an MI355X, used when a run only
# compiles and no device can be queried
MI355X_CUS = 256
MI355X_THREADS_PER_CU = 2048


def parse_args() -> argparse.Namespace:
    parser = argparse.ArgumentParser()
    parser.add_argument("-m", "--model_dir", type=str)
    parser.add_argument("-o", "--output_dir", type=str)
    parser.add_argument("-n", "--num_processes", type=int, default=8)
    parser.add_argument("-b", "--block_threads", type=int, default=256)
    parser.add_argument("--mutation_feat_id", type=int)
    parser.add_argument("--naive", action="store_true", default=False)
    parser.add_argument("--fixed_thread_binding", action="store_true", default=False)
    parser.add_argument("--thread_binding_choice", type=str, default="mean", choices=["mean", "max"])
    parser.add_argument("--local_only", action="store_true", default=False)
    parser.add_argument("--recompile", action="store_true", default=False)
    parser.add_argument("--remeasure", action="store_true", default=False)
    parser.add_argument("--noinline", action="store_true", default=False)
    parser.add_argument("--debug", action="store_true", default=False)
    parser.add_argument("--workload", type=str, help="built-in synthetic configuration (c1..c5)")
    parser.add_argument("--workload_batches", type=int, default=2)
    parser.add_argument("--compile_only", action="store_true", default=False)
    parser.add_argument("--launch_only", action="store_true", default=False,
                        help="skip the local stage: default schedules, swept over occupancy and the "
                             "launch parameters of the run-time binding")
    parser.add_argument("--occupancies", type=str, help="comma-separated workgroups per CU to try")
    parser.add_argument("--sample_batch_nums", type=int, default=128)
    parser.add_argument("--profiler", type=str, default="rocprofv3", choices=["rocprofv3", "events"])
    parser.add_argument("--tile_bytes", type=str, default="",
                        help="traffic per tile of the tuning builds and contenders (bytes; default 65536); "
                             "auto = sized by the device from every batch, as untuned builds do")
    parser.add_argument("--tile_bytes_candidates", type=str,
                        help="comma-separated traffic-per-tile values swept in the global stage")
    parser.add_argument("--xcd_segments_candidates", type=str,
                        help="comma-separated tile-walk settings swept in the global stage "
                             "(-1 = flat, n > 0 = n segments per XCD)")
    parser.add_argument("--launch_time_tolerance", type=float, default=0.0,
                        help="global stage: launch options within this share of the fastest count "
                             "as equally fast and the one with the fewest segments per XCD (the "
                             "least HBM traffic) is kept; 0 = the fastest")
    parser.add_argument("--outliers", choices=["auto", "on", "off"], default="auto",
                        help="emit the optimal library with outlier tiles: bags far longer than "
                             "their feature's schedule suits are found ahead of the fused kernel "
                             "and summed by several workgroups (for data with skewed bag lengths); "
                             "auto = if the sampled batches hold such a bag, the optimal mix is "
                             "built both ways and timed on them, and the faster call is kept")
    parser.add_argument("--walk_stage", choices=["auto", "on", "off"], default="auto",
                        help="after the global stage, try the winning mix with its features laid out in "
                             "the tile space by their time per tile, and with the last passes of the "
                             "tile walk (2, 8, all) drawn from ticket counters, and keep what is faster on the "
                             "samples; auto = a drawn end for models whose workgroups get three tiles each "
                             "or more, an order for models of 64 features and more whose workgroups "
                             "get fewer than sixteen")
    parser.add_argument("--build_climb_trials", type=int, default=0,
                        help="global stage: that many single-feature variants of the winning mix are "
                             "built as production kernels and timed; the faster ones are adopted")
    parser.add_argument("--climb_passes", type=int, default=1,
                        help="in-model local stage: passes of the whole-kernel climb inside the "
                             "tournament build (0 = rank by tile time only)")
    parser.add_argument("--build_climb_top_k", type=int, default=3,
                        help="build climb: tournament candidates tried per feature")
    parser.add_argument("--no_cluster_stage", action="store_true", default=False,
                        help="in-model local stage: stop after the tournament (rank by tile time and "
                             "its own climb) instead of letting clusters of like features decide on "
                             "whole-kernel time in production-shaped builds")
    parser.add_argument("--incumbent", type=str,
                        help="schedule.json of an earlier tuning run of this model: one more contender of "
                             "the global stage (and the start of the build climb if it wins)")
    parser.add_argument("--incumbent_only", action="store_true", default=False,
                        help="global stage for the --incumbent mix alone (occupancy, traffic per tile, "
                             "tile walk, outlier tiles): no tuning build, no other contender")
    parser.add_argument("--validate_clusters", action="store_true", default=False,
                        help="after tuning: build, for every cluster, the production kernel with and "
                             "without the cluster's fastest option and set the change beside the one "
                             "the cluster stage measured (clusters/o<occ>/validation.json)")
    parser.add_argument("--cluster_top_k", type=int, default=8,
                        help="cluster stage: candidates a cluster tries")
    parser.add_argument("--cluster_sweeps", type=int, default=1)
    parser.add_argument("--no_register_census", action="store_true", default=False,
                        help="in-model local stage: admit every candidate to every occupancy's "
                             "tournament, also those that spill registers there")
    parser.add_argument("--interference", type=str, default="model", choices=["model", "replicate"],
                        help="local stage: candidates timed inside the whole model, or per feature "
                             "against copies of themselves (the reference's scheme)")
    args = parser.parse_args()
    if not args.model_dir and not args.workload:
        parser.error("one of -m/--model_dir and --workload is required")
    return args


def all_templates():
    return [ThreadPerBagSchedule, SubWavefrontPerBagSchedule, WavefrontPerBagSchedule, BlockPerBagSchedule]


def create_tuner(args: argparse.Namespace) -> Tuner:
    BasicBuilder().build()          # the CPU text front end, once
    if getattr(args, "workload", None):
        from recflex_amd.workloads import make_workload, gen_inputs
        wl = make_workload(args.workload)
        output_dir = args.output_dir or os.path.join(ROOT, "recflex_amd", "_models", f"tune_{args.workload}")
        batches = [[] for _ in range(wl.num_features)]
        for k in range(args.workload_batches):
            # batches of the same distribution as the benchmark's, never the benchmark's own
            indices, offsets = gen_inputs(wl._replace(seed=wl.seed + 7919 * (k + 1)))
            for f in range(wl.num_features):
                batches[f].append((indices[f], offsets[f]))
        basic_config = BasicConfig(batch_sizes_fname="", data_fnames=[], schedule_config_fname="",
                                   table_config_fname="", codegen_dir=output_dir,
                                   block_threads=args.block_threads,
                                   sample_batch_nums=args.workload_batches)
        return Tuner(basic_config, schedule_mapping=globals(), batches=batches,
                     table_shapes=[(f.rows, f.dim) for f in wl.features],
                     data_types=[f.data_type for f in wl.features],
                     # the row-copy template only where no sampled bag holds more than one lookup
                     schedule_types=[all_templates() + ([OneHotBagSchedule] if
                                                        max(int(np.diff(o).max()) for _, o in batches[f]) <= 1
                                                        else [])
                                     for f in range(wl.num_features)])

    model_dir = args.model_dir
    data_dir = os.path.join(model_dir, "data")
    data_fnames = get_data_fnames(data_dir)
    output_dir = args.output_dir if args.output_dir else os.path.join(model_dir, "output")
    basic_config = BasicConfig(batch_sizes_fname=os.path.join(data_dir, "batch_sizes.txt"),
                               data_fnames=data_fnames,
                               schedule_config_fname=os.path.join(model_dir, "schedule_config.txt"),
                               table_config_fname=os.path.join(model_dir, "table_config.txt"),
                               codegen_dir=output_dir,
                               block_threads=args.block_threads,
                               sample_batch_nums=getattr(args, "sample_batch_nums", 128))
    return Tuner(basic_config=basic_config, schedule_mapping=globals())


def create_tune_config(args: argparse.Namespace) -> TuneConfig:
    try:
        from recflex_amd.hip_helper import HipInfoQuerier
        querier = HipInfoQuerier()
        gpu_ids = querier.gpu_ids
        sm_count, max_threads_per_sm = querier.get_sm_thread_count()
    except Exception as exc:
        if not args.compile_only:
            raise
        print(f"no device to query ({exc}); assuming an MI355X for the compile-only run")
        gpu_ids, sm_count, max_threads_per_sm = [0], MI355X_CUS, MI355X_THREADS_PER_CU
    if args.occupancies:
        occupancies = [int(v) for v in args.occupancies.split(",")]
    else:
        occupancies = list(range(1, max_threads_per_sm // args.block_threads + 1))
    kwargs = {"register_census": not args.no_register_census,
              "cluster_stage": not args.no_cluster_stage, "cluster_top_k": args.cluster_top_k,
              "cluster_sweeps": args.cluster_sweeps, "incumbent": args.incumbent,
              "build_climb_trials": args.build_climb_trials,
              "build_climb_top_k": args.build_climb_top_k,
              "climb_passes": args.climb_passes, "outliers": {"auto": None, "on": True, "off": False}[args.outliers],
              "walk_stage": {"auto": None, "on": True, "off": False}[args.walk_stage]}
    if args.tile_bytes:
        kwargs["tile_bytes"] = 0 if args.tile_bytes == "auto" else int(args.tile_bytes)
    if args.xcd_segments_candidates:
        kwargs["xcd_segments_candidates"] = [int(v) for v in args.xcd_segments_candidates.split(",")]
    if args.launch_time_tolerance:
        kwargs["launch_time_tolerance"] = args.launch_time_tolerance
    if args.tile_bytes_candidates:
        kwargs["tile_bytes_candidates"] = [int(v) for v in args.tile_bytes_candidates.split(",")]
    return TuneConfig(occupancies=occupancies, gpu_ids=gpu_ids, sm_count=sm_count,
                      num_processes=args.num_processes, recompile=args.recompile,
                      remeasure=args.remeasure, inline=not args.noinline, debug=args.debug,
                      profiler=args.profiler, interference=args.interference, **kwargs)


def main():
    args = parse_args()
    tuner = create_tuner(args)
    tune_config = create_tune_config(args)

    if args.compile_only:
        if not args.incumbent_only:
            if args.launch_only:
                pass                    # the global stage alone needs no tuning build
            elif tune_config.interference == "model":
                tuner.compile_tournament(tune_config)
            else:
                tuner.compile_local(tune_config)
            # ... and the contenders of the global stage that are known without a measurement
            tuner.compile_default_contenders(tune_config)
        tuner.compile_incumbent_contenders(tune_config)
        print(f"kernels built under {tuner.basic.codegen_dir}")
        return

    if args.launch_only:
        occupancy, sched_params = tuner.solve_launch_only(tune_config)
        print(occupancy, tuner.opt_tile_bytes, tuner.opt_xcd_segments)
        return

    if args.incumbent_only:
        if not args.incumbent:
            raise SystemExit("--incumbent_only needs --incumbent <schedule.json>")
        occupancy, sched_params = tuner.solve_incumbent_only(tune_config)
        print(occupancy, tuner.opt_tile_bytes, tuner.opt_xcd_segments)
        return

    if not args.naive:
        tune_results = tuner.tune(tune_config)
        print(tune_results)
        if not args.local_only:
            occupancy, sched_params = tuner.solve(tune_results, tune_config)
            print(occupancy, sched_params)
            if args.validate_clusters and tune_config.interference == "model" and tune_config.cluster_stage:
                tuner.cluster_validation(occupancy, tune_config)

            if args.fixed_thread_binding:
                fixed_task_blocks, t = tuner.tune_fixed_thread_binding(opt_sched_params=sched_params,
                                                                       choice=args.thread_binding_choice,
                                                                       tune_config=tune_config,
                                                                       occupancy=occupancy)
                print(fixed_task_blocks)
                print(f"Fixed thread binding result: {t/1e6} ms")

            if args.mutation_feat_id is not None and args.mutation_feat_id >= 0:
                mut_times, opt_idx = tuner.mutation_validation(opt_sched_params=sched_params, opt_occupancy=occupancy,
                                                               mut_feat_id=args.mutation_feat_id, tune_config=tune_config)
                print(mut_times, np.argmin(mut_times), opt_idx)
    else:
        tune_results, t = tuner.tune_naive(tune_config)
        print(tune_results)
        print(f"Naive-tuning result: {t/1e6} ms")


if __name__ == "__main__":
    mp.set_start_method("spawn")
    main()
