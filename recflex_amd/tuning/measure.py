"""Measurement workers of the tuner.

Function names and roles follow ``RecFlex/tuning/measure.py:20-122``:

* ``measure_single_feat``   local stage: every candidate schedule of one feature runs as its own
  "feature" of one fused kernel over the same data (replicated until the GPU is full, which is
  the simulated interference); the kernel is a timing build, and the time of a candidate is the
  sum of the device ticks of its tiles.  Writes ``result.txt`` (space separated floats)
  atomically.
* ``measure_naive_candidate``  one candidate alone on the GPU, timed with events.
* ``rocprof_profile``       global stage: run ``run_script.py`` under
  ``rocprofv3 --kernel-trace --stats`` (the reference uses ``nsys profile``) and leave the
  kernel statistics next to the build.
* ``measure_kernel_events`` the same quantity without an external profiler (events around each
  launch), for machines where spawning the profiler is not wanted.
* ``measure_task_blocks``   tiles per feature and batch under the run-time binding (input of
  the fixed-thread-binding ablation).

A worker may run in a spawned process pinned to one GPU (``gpu_id`` keyword, set through
``HIP_VISIBLE_DEVICES``) or be called directly: emitted libraries are plain ``dlopen`` handles,
so one process can measure any number of them -- the reference needs a process per library
because ``TORCH_LIBRARY(recom)`` can be registered once (``measure.py:23-24``).
"""

import json
import time
import os
import shutil
import subprocess
import sys
from typing import List, Optional, Sequence, Tuple

import numpy as np


def _pin_gpu(gpu_id: Optional[int]) -> None:
    if gpu_id is None:
        raise Exception("No valid GPU provided!")
    # only effective before the HIP runtime starts, i.e. in a freshly spawned worker
    if "torch" not in sys.modules:
        os.environ["HIP_VISIBLE_DEVICES"] = str(gpu_id)


def load_batches(data_npz: str) -> List[Tuple[np.ndarray, np.ndarray]]:
    """``[(indices, offsets)]`` of one feature, as written by ``save_batches``."""
    z = np.load(data_npz)
    n = int(z["num_batches"])
    return [(z[f"indices{k}"], z[f"offsets{k}"]) for k in range(n)]


def save_batches(data_npz: str, batches: Sequence[Tuple[np.ndarray, np.ndarray]]) -> None:
    arrays = {"num_batches": np.int64(len(batches))}
    for k, (idx, off) in enumerate(batches):
        arrays[f"indices{k}"] = np.asarray(idx, dtype=np.int32)
        arrays[f"offsets{k}"] = np.asarray(off, dtype=np.int32)
    tmp = data_npz + ".tmp.npz"
    np.savez(tmp, **arrays)
    os.replace(tmp, data_npz)


def make_table(table_shape: Tuple[int, int], data_type: str, device, ones: bool = True):
    """Table of the right storage type; ``ones`` as in the reference's tuning runs
    (``measure.py:41``), else N(0, 0.01)."""
    import torch
    from recflex_amd.quant import quantize_rowwise_int8
    from recflex_amd.workloads import FeatureSpec, gen_table
    rows, dim = table_shape
    if not ones:       # built chunk by chunk: no fp32 copy of a large fp16 / int8 table
        return gen_table(FeatureSpec(rows, dim, data_type, 1.0, True, 0.0, 0.0), seed=rows + dim,
                         device=device)
    w = torch.ones(rows, dim, dtype=torch.float32, device=device)
    if data_type == "half":
        return w.half()
    if data_type == "int8":
        return quantize_rowwise_int8(w)
    return w


def _write_atomically(path: str, text: str) -> None:
    tmp = path + ".tmp"
    with open(tmp, "w") as f:
        f.write(text)
    os.replace(tmp, path)


def _timed_launches(launch, reps: int, burst: int = 4) -> float:
    """Median over ``reps`` of the time per launch in ns.  Each sample brackets ``burst``
    back-to-back launches with one event pair, after one launch that keeps the GPU busy while the
    host queues them, so that the host's launch overhead is not part of the measurement."""
    import torch
    samples = []
    for _ in range(reps):
        start = torch.cuda.Event(enable_timing=True)
        end = torch.cuda.Event(enable_timing=True)
        launch()
        start.record()
        for _ in range(burst):
            launch()
        end.record()
        end.synchronize()
        samples.append(start.elapsed_time(end) * 1e6 / burst)
    return sorted(samples)[len(samples) // 2]


def measure_single_feat(ident: Tuple[int, int], data_npz: str, table_shape: Tuple[int, int],
                        data_type: str, num_schedules: int, num_padded_schedules: int,
                        librecom_path: str, output_path: str, gpu_id: int = None) -> Optional[List[float]]:
    feat_id, occupancy = ident
    print(f"Feat {feat_id}, Occ {occupancy}, GPU {gpu_id}", flush=True)
    try:
        _pin_gpu(gpu_id)
        import torch
        assert torch.cuda.is_available()
        from recflex_amd.rec_modules import FeatEmbed

        dev = torch.device("cuda", torch.cuda.current_device())
        table = make_table(table_shape, data_type, dev)
        layer = FeatEmbed(dev, embed_tables=[table for _ in range(num_padded_schedules)],
                          librecom=librecom_path)
        accum = torch.zeros([num_schedules], dtype=torch.float64)
        for idx, off in load_batches(data_npz):
            d_idx = torch.from_numpy(idx).to(dev)
            d_off = torch.from_numpy(off).to(dev)
            _, task_times = layer.forward_indices([d_idx] * num_padded_schedules,
                                                  [d_off] * num_padded_schedules,
                                                  timing=True, timing_schedules=num_schedules)
            accum += task_times
        torch.cuda.synchronize()
        result = [t.item() for t in accum]
        _write_atomically(output_path, ' '.join(str(t) for t in result))
        return result
    except Exception as e:  # a failed worker leaves no result file; the tuner notices that
        print(f"[{ident}] Exception {type(e).__name__}: {e}", flush=True)
        return None


def measure_tournament(ident: int, librecom_path: str, table_shapes: Sequence[Tuple[int, int]],
                       data_types: Sequence[str], data_npzs: Sequence[str], output_path: str,
                       rounds: int = 3, refine_passes: int = 3, top_k: int = 8,
                       probe_fraction: float = 0.2, probes_per_candidate: int = 3, seed: int = 0,
                       climb_passes: int = 1, start_choices: Sequence[Sequence[int]] = (),
                       gpu_id: int = None) -> Optional[List[List[float]]]:
    """Local stage inside the real model: the library holds every candidate of every feature
    and each launch runs one candidate per feature (``d_schedule_choice``), so a candidate is
    timed against the memory traffic of all the other features, not against copies of itself.

    Exploration: ``rounds`` times, every feature walks a random permutation of its candidates
    (one launch per step, all features step together); a candidate's score is its mean summed
    tile time.  Refinement, ``refine_passes`` times: every feature runs its current best except a
    random ``probe_fraction`` of the features, each of which tries one of its ``top_k``
    candidates; the scores measured against this near-final background replace the exploration
    scores of those candidates and the best is re-elected.

    Whole-kernel climb, ``climb_passes`` times: tile times are a zero-sum measure once the kernel
    is bound by memory bandwidth (a schedule that keeps more loads in flight finishes its own
    tiles sooner by slowing the others down), so the elected mix -- or any of ``start_choices``
    (e.g. the untuned default) that runs faster -- is then improved against the kernel's own
    duration: feature by feature, heaviest first, each of the feature's ``top_k`` candidates is
    swapped in and kept if the whole launch gets faster.  The kept candidates get the lowest
    score of their feature, so that an argmin over the scores reproduces the final mix.

    Writes ``{"times": [[score per candidate] per feature], "best": [...], "kernel_ns": t}``."""
    print(f"Tournament, Occ {ident}, GPU {gpu_id}", flush=True)
    try:
        _pin_gpu(gpu_id)
        import torch
        assert torch.cuda.is_available()
        from recflex_amd.rec_modules import FeatEmbed

        dev = torch.device("cuda", torch.cuda.current_device())
        tables = [make_table(s, t, dev, ones=False) for s, t in zip(table_shapes, data_types)]
        layer = FeatEmbed(dev, embed_tables=tables, librecom=librecom_path)
        counts = layer.lib.candidate_counts
        num_feats = len(counts)
        per_feat = [load_batches(p) for p in data_npzs]
        device_batches = []
        for k in range(len(per_feat[0])):
            device_batches.append(([torch.from_numpy(b[k][0]).to(dev) for b in per_feat],
                                   [torch.from_numpy(b[k][1]).to(dev) for b in per_feat]))
        rng = np.random.default_rng(seed)
        last_beat = [time.monotonic()]

        def beat(what: str) -> None:
            """A progress line every 20 s or so: long phases of a large model are otherwise silent."""
            if time.monotonic() - last_beat[0] > 20.0:
                last_beat[0] = time.monotonic()
                print(f"[tournament {ident}] {what}", flush=True)

        def launch(choice: np.ndarray) -> np.ndarray:
            d_choice = torch.from_numpy(choice.astype(np.int32)).to(dev)
            total = np.zeros(num_feats, dtype=np.float64)
            for d_idx, d_off in device_batches:
                _, t = layer.forward_indices(d_idx, d_off, timing=True, schedule_choice=d_choice)
                total += t.numpy()
            return total

        launch(np.zeros(num_feats, dtype=np.int32))      # warm-up
        # ---- exploration
        sums = [np.zeros(c) for c in counts]
        hits = [np.zeros(c) for c in counts]
        steps = max(counts)
        for _ in range(rounds):
            perms = [rng.permutation(c) for c in counts]
            for j in range(steps):
                choice = np.array([perms[f][j % counts[f]] for f in range(num_feats)])
                t = launch(choice)
                beat(f"exploration, step {j + 1} of {steps}")
                for f in range(num_feats):
                    sums[f][choice[f]] += t[f]
                    hits[f][choice[f]] += 1
        score = [s / np.maximum(h, 1) for s, h in zip(sums, hits)]
        best = np.array([int(np.argmin(sc)) for sc in score])

        # ---- refinement against the incumbent mix
        for _ in range(refine_passes):
            tops = [np.argsort(sc)[:min(top_k, len(sc))] for sc in score]
            rsum = [np.zeros(c) for c in counts]
            rhit = [np.zeros(c) for c in counts]
            launches = int(np.ceil(max(len(t) for t in tops) * probes_per_candidate / probe_fraction))
            for _ in range(launches):
                choice = best.copy()
                probing = rng.random(num_feats) < probe_fraction
                for f in np.nonzero(probing)[0]:
                    choice[f] = rng.choice(tops[f])
                t = launch(choice)
                beat("refinement")
                for f in range(num_feats):
                    rsum[f][choice[f]] += t[f]
                    rhit[f][choice[f]] += 1
            for f in range(num_feats):
                seen = rhit[f] > 0
                refined = np.where(seen, rsum[f] / np.maximum(rhit[f], 1), np.inf)
                worst_seen = refined[seen].max() if seen.any() else 0.0
                # candidates not re-measured keep their exploration score, but never beat a
                # candidate that was measured against the incumbent mix
                score[f] = np.where(seen, refined, np.maximum(score[f], worst_seen))
                best[f] = int(np.argmin(score[f]))
        # ---- whole-kernel climb
        outs = [layer.forward_indices(d_idx, d_off) for d_idx, d_off in device_batches]
        # address tables uploaded once: no per-feature host work inside the timed launches
        bound_batches = [layer.bind_inputs(d_idx, d_off) for d_idx, d_off in device_batches]

        def kernel_ns(choice: np.ndarray, reps: int = 3) -> float:
            d_choice = torch.from_numpy(choice.astype(np.int32)).to(dev)
            total = 0.0
            for bound, out in zip(bound_batches, outs):
                total += _timed_launches(
                    lambda: layer.forward_indices(bound, out=out, schedule_choice=d_choice), reps)
            return total

        best_ns = None
        if climb_passes > 0:
            for _ in range(10):
                kernel_ns(best, reps=1)                      # clocks up
            best_ns = kernel_ns(best, reps=5)
            for start in start_choices:
                cand = np.array([min(max(int(c), 0), n - 1) for c, n in zip(start, counts)])
                t = kernel_ns(cand, reps=5)
                print(f"[tournament {ident}] start mix {t:.0f} ns vs elected {best_ns:.0f} ns", flush=True)
                if t < best_ns:
                    best, best_ns = cand, t
            share = launch(best)
            order = np.argsort(-share)
            for _ in range(climb_passes):
                for f in order:
                    for c in np.argsort(score[f])[:min(top_k, counts[f])]:
                        if c == best[f]:
                            continue
                        trial = best.copy()
                        trial[f] = c
                        t = kernel_ns(trial)
                        beat(f"climb, best {best_ns:.0f} ns")
                        if t < best_ns * 0.995:
                            t = kernel_ns(trial, reps=5)     # confirm before keeping
                            if t < best_ns * 0.995:
                                best, best_ns = trial, t
            for f in range(num_feats):
                score[f][best[f]] = min(score[f].min(), score[f][best[f]]) * 0.999
            print(f"[tournament {ident}] kernel after climb {best_ns:.0f} ns", flush=True)
        torch.cuda.synchronize()
        result = [sc.tolist() for sc in score]
        _write_atomically(output_path, json.dumps({"times": result, "best": [int(b) for b in best],
                                                   "kernel_ns": best_ns}))
        return result
    except Exception as e:
        print(f"[tournament {ident}] Exception {type(e).__name__}: {e}", flush=True)
        return None


def measure_naive_candidate(ident: Tuple[int, int], data_npz: str, table_shape: Tuple[int, int],
                            data_type: str, librecom_path: str, output_path: str,
                            gpu_id: int = None) -> Optional[float]:
    feat_id, sched_param_id = ident
    print(f"Feat {feat_id}, Schedule {sched_param_id}, GPU {gpu_id}", flush=True)
    try:
        _pin_gpu(gpu_id)
        import torch
        assert torch.cuda.is_available()
        from recflex_amd.rec_modules import FeatEmbed

        dev = torch.device("cuda", torch.cuda.current_device())
        layer = FeatEmbed(dev, embed_tables=[make_table(table_shape, data_type, dev)],
                          librecom=librecom_path)
        accum_ms = 0.0
        for idx, off in load_batches(data_npz):
            d_idx = [torch.from_numpy(idx).to(dev)]
            d_off = [torch.from_numpy(off).to(dev)]
            out = layer.forward_indices(d_idx, d_off)    # warm-up (first launch sets the grid up)
            accum_ms += _timed_launches(lambda: layer.forward_indices(d_idx, d_off, out=out), 3) / 1e6
        _write_atomically(output_path, str(accum_ms))
        return accum_ms
    except Exception as e:
        print(f"[{ident}] Exception {type(e).__name__}: {e}", flush=True)
        return None


def _run_script_args(table_config_fname: str, build_dir: str, data_dir: str,
                     sample_batch_nums: int, spec_feat_id: Optional[int]) -> List[str]:
    script_path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "run_script.py")
    # absolute paths: the profiler is started from /tmp, where it writes its scratch files
    args = [sys.executable, script_path, "--table_config_fname", os.path.abspath(table_config_fname),
            "--build_dir", os.path.abspath(build_dir), "--data_dir", os.path.abspath(data_dir),
            "--sample_batch_nums", str(sample_batch_nums)]
    if spec_feat_id is not None:
        args += ["--spec_feat_id", str(spec_feat_id)]
    return args


# the profiled program runs the sampled batches this many times; the first pass is warm-up and
# the global stage takes each batch's median over the others (parser.parse_knl_batch_times)
PROFILE_PASSES = 4
PROFILE_WARMUP_PASSES = 1


def rocprof_profile(table_config_fname: str, build_dir: str, data_dir: str, sample_batch_nums: int,
                    report_prefix: str, spec_feat_id: int = None, tile_bytes: int = 0,
                    xcd_segments: int = 0, passes: int = PROFILE_PASSES, gpu_id: int = None) -> None:
    """Runs ``run_script.py`` on the built model as a child process under rocprofv3
    (``--kernel-trace --stats``; the program itself stands right after ``--``) and leaves
    ``{report_prefix}_kernel_stats.csv`` and ``{report_prefix}_kernel_trace.csv``."""
    if gpu_id is None:
        raise Exception("No valid GPU provided!")
    rocprof = shutil.which("rocprofv3") or "/opt/rocm/bin/rocprofv3"
    out_dir = os.path.dirname(os.path.abspath(report_prefix))
    name = os.path.basename(report_prefix)
    cmd = [rocprof, "--kernel-trace", "--stats", "--output-format", "csv", "-d", out_dir, "-o", name,
           "--"] + _run_script_args(table_config_fname, build_dir, data_dir, sample_batch_nums,
                                    spec_feat_id) + ["--tile_bytes", str(tile_bytes),
                                                    "--xcd_segments", str(xcd_segments),
                                                    "--repeats", str(passes)]
    env = dict(os.environ)
    env["HIP_VISIBLE_DEVICES"] = str(gpu_id)
    env.setdefault("TMPDIR", "/tmp")
    # like nsys in the reference, the profiler's own exit status is not trusted; the stats file
    # is.  What the run printed is kept beside the report for the case that no file appears.
    with open(f"{os.path.abspath(report_prefix)}.rocprofv3.log", "w") as log:
        subprocess.run(cmd, env=env, cwd="/tmp", stdout=log, stderr=subprocess.STDOUT)


# the reference's name for the global-stage worker
nsys_profile = rocprof_profile


def measure_kernel_events(librecom_path: str, table_shapes: Sequence[Tuple[int, int]],
                          data_types: Sequence[str], data_npzs: Sequence[str], output_path: str,
                          tile_bytes: int = 0, xcd_segments: int = 0, repeats: int = 7, warmup: int = 10,
                          gpu_id: int = None) -> Optional[float]:
    """Total FusedKnl time in ns over all batches (median of ``repeats`` launches per batch),
    measured with events on the launch stream; written to ``output_path``."""
    try:
        _pin_gpu(gpu_id)
        import torch
        from recflex_amd.rec_modules import FeatEmbed

        dev = torch.device("cuda", torch.cuda.current_device())
        tables = [make_table(s, t, dev, ones=False) for s, t in zip(table_shapes, data_types)]
        layer = FeatEmbed(dev, embed_tables=tables, librecom=librecom_path)
        per_feat = [load_batches(p) for p in data_npzs]
        total_ns = 0.0
        for k in range(len(per_feat[0])):
            d_idx = [torch.from_numpy(b[k][0]).to(dev) for b in per_feat]
            d_off = [torch.from_numpy(b[k][1]).to(dev) for b in per_feat]
            out = layer.forward_indices(d_idx, d_off)       # its buffer is reused below
            bound = layer.bind_inputs(d_idx, d_off)         # no per-feature host work when timed
            for _ in range(warmup):                         # let the clocks settle
                layer.forward_indices(bound, out=out, tile_bytes=tile_bytes,
                                      xcd_segments=xcd_segments)
            total_ns += _timed_launches(
                lambda: layer.forward_indices(bound, out=out, tile_bytes=tile_bytes,
                                              xcd_segments=xcd_segments), repeats)
        _write_atomically(output_path, str(total_ns))
        return total_ns
    except Exception as e:
        print(f"[{librecom_path}] Exception {type(e).__name__}: {e}", flush=True)
        return None


def measure_feature_ticks(librecom_path: str, table_shapes: Sequence[Tuple[int, int]],
                          data_types: Sequence[str], data_npzs: Sequence[str], output_path: str,
                          tile_bytes: int = 0, xcd_segments: int = 0, repeats: int = 3,
                          gpu_id: int = None) -> Optional[np.ndarray]:
    """Workgroup ticks per feature of a timing build of the whole model, summed over the
    batches (mean of ``repeats`` launches each); one number per line of ``output_path``."""
    try:
        _pin_gpu(gpu_id)
        import torch
        from recflex_amd.rec_modules import FeatEmbed

        dev = torch.device("cuda", torch.cuda.current_device())
        tables = [make_table(s, t, dev, ones=False) for s, t in zip(table_shapes, data_types)]
        layer = FeatEmbed(dev, embed_tables=tables, librecom=librecom_path)
        per_feat = [load_batches(p) for p in data_npzs]
        total = np.zeros(len(per_feat), dtype=np.float64)
        for k in range(len(per_feat[0])):
            bound = layer.bind_inputs([torch.from_numpy(b[k][0]).to(dev) for b in per_feat],
                                      [torch.from_numpy(b[k][1]).to(dev) for b in per_feat])
            out = layer.forward_indices(bound, tile_bytes=tile_bytes, xcd_segments=xcd_segments)
            acc = np.zeros(len(per_feat), dtype=np.float64)
            for _ in range(repeats):
                _, ticks = layer.forward_indices(bound, timing=True, out=out, tile_bytes=tile_bytes,
                                                 xcd_segments=xcd_segments)
                acc += ticks.numpy()
            total += acc / repeats
        _write_atomically(output_path, "".join(f"{v:.1f}\n" for v in total))
        return total
    except Exception as e:
        print(f"[{librecom_path}] Exception {type(e).__name__}: {e}", flush=True)
        return None


class KernelTimer:
    """Times the FusedKnl of several libraries of one model over the same tables and batches,
    which stay on the device between calls (the production-build climb times hundreds of
    libraries; building the tables anew for each would cost more than the measurements)."""

    def __init__(self, table_shapes: Sequence[Tuple[int, int]], data_types: Sequence[str],
                 data_npzs: Sequence[str], gpu_id: int = None):
        _pin_gpu(gpu_id)
        import torch
        self.dev = torch.device("cuda", torch.cuda.current_device())
        self.tables = [make_table(s, t, self.dev, ones=False) for s, t in zip(table_shapes, data_types)]
        per_feat = [load_batches(p) for p in data_npzs]
        self.batches = []
        for k in range(len(per_feat[0])):
            self.batches.append(([torch.from_numpy(b[k][0]).to(self.dev) for b in per_feat],
                                 [torch.from_numpy(b[k][1]).to(self.dev) for b in per_feat]))
        self.outs = None

    def time_ns(self, librecom_path: str, tile_bytes: int = 0, xcd_segments: int = 0,
                repeats: int = 7, warmup: int = 4) -> float:
        """Sum over the batches of the median time per launch, in ns."""
        from recflex_amd.rec_modules import FeatEmbed
        layer = FeatEmbed(self.dev, embed_tables=self.tables, librecom=librecom_path)
        if self.outs is None:
            self.outs = [layer.forward_indices(d_idx, d_off).clone() for d_idx, d_off in self.batches]
        total = 0.0
        for (d_idx, d_off), out in zip(self.batches, self.outs):
            bound = layer.bind_inputs(d_idx, d_off)         # no per-feature host work when timed
            run = lambda: layer.forward_indices(bound, out=out, tile_bytes=tile_bytes,
                                                xcd_segments=xcd_segments)
            for _ in range(warmup):
                run()
            total += _timed_launches(run, repeats)
        return total


    def time_options(self, librecom_path: str, members: Sequence[int], num_options: int,
                     rounds: int = 3, repeats: int = 3, warmup: int = 4, tile_bytes: int = 0,
                     xcd_segments: int = 0, only: Sequence[int] = None, seed: int = 0) -> List[List[float]]:
        """A library that holds ``num_options`` candidates for each feature in ``members`` (and one
        for every other feature): the whole kernel's time, summed over the batches, with all
        members on option 0, all on option 1, ...  The options take turns ``rounds`` times in an
        order drawn anew for every round, so that neither a drift of the clocks nor a place in
        the order favours one of them; returns the ``rounds`` times (ns) of each option (``only``:
        of these options, the others get an empty list)."""
        from recflex_amd.librecom import RecomLib
        counts = RecomLib(librecom_path).candidate_counts
        for f in members:
            if counts[f] != num_options:
                raise ValueError(f"feature {f} holds {counts[f]} candidates, expected {num_options}")
        todo = list(range(num_options)) if only is None else list(only)
        mixes = []
        for k in todo:
            c = np.zeros(len(counts), dtype=np.int32)
            c[list(members)] = k
            mixes.append(c)
        measured = self.time_mixes(librecom_path, mixes, rounds=rounds, repeats=repeats, warmup=warmup,
                                   tile_bytes=tile_bytes, xcd_segments=xcd_segments, seed=seed)
        times: List[List[float]] = [[] for _ in range(num_options)]
        for k, t in zip(todo, measured):
            times[k] = t
        return times

    def time_mixes(self, librecom_path: str, mixes: Sequence[np.ndarray], rounds: int = 3,
                   repeats: int = 3, warmup: int = 4, tile_bytes: int = 0, xcd_segments: int = 0,
                   seed: int = 0) -> List[List[float]]:
        """The whole kernel's time (ns, summed over the batches) of a library that holds several
        candidates per feature, for each of ``mixes`` (one candidate number per feature).  The
        mixes take turns ``rounds`` times, in an order drawn anew for every round."""
        import torch
        from recflex_amd.rec_modules import FeatEmbed
        layer = FeatEmbed(self.dev, embed_tables=self.tables, librecom=librecom_path)
        if self.outs is None:
            self.outs = [layer.forward_indices(d_idx, d_off).clone() for d_idx, d_off in self.batches]
        bound = [layer.bind_inputs(d_idx, d_off) for d_idx, d_off in self.batches]
        choices = [torch.from_numpy(np.asarray(c, dtype=np.int32)).to(self.dev) for c in mixes]
        rng = np.random.default_rng(seed)
        times: List[List[float]] = [[] for _ in mixes]
        for choice in choices:                             # every mix warmed up once
            for b, out in zip(bound, self.outs):
                for _ in range(warmup):
                    layer.forward_indices(b, out=out, tile_bytes=tile_bytes, xcd_segments=xcd_segments,
                                          schedule_choice=choice)
        for _ in range(rounds):
            for k in rng.permutation(len(choices)):
                total = 0.0
                for b, out in zip(bound, self.outs):
                    run = lambda: layer.forward_indices(b, out=out, tile_bytes=tile_bytes,
                                                        xcd_segments=xcd_segments,
                                                        schedule_choice=choices[int(k)])
                    run()
                    total += _timed_launches(run, repeats)
                times[int(k)].append(total)
        return times


MAX_TILE_FACTOR = 8      # rfx::kMaxTileFactor
PLENTY_TILES_PER_WORKGROUP = 2                      # rfx::kPlentyTilesPerWorkgroup
AUTO_TILES_PER_WORKGROUP = 64                       # rfx::kAutoTilesPerWorkgroup
AUTO_TILE_MIN, AUTO_TILE_MAX = 64 * 1024, 256 * 1024    # rfx::kAutoTileMin / kAutoTileMax
AUTO_TILE_FLOOR = 4 * 1024                              # rfx::kAutoTileFloor


def auto_tile_bytes(offsets: Sequence[np.ndarray], lookup_bytes: Sequence[int],
                    bag_bytes: Sequence[int], grid_blocks: int) -> int:
    """Host restatement of the tile size the device picks when none is given
    (``rfx::auto_tile_size``): the batch's traffic over 64 tiles per workgroup of the grid, within
    64..256 KiB, in steps of 4 KiB; a batch of less than 64 KiB per workgroup gets about two tiles
    per workgroup, at least 4 KiB, in steps of 1 KiB."""
    total = 0
    for off, lb, bb in zip(offsets, lookup_bytes, bag_bytes):
        batch = len(off) - 1
        if batch > 0:
            total += int(off[-1] - off[0]) * lb + batch * bb
    grid = max(1, grid_blocks)
    t = total // (grid * AUTO_TILES_PER_WORKGROUP)
    if t >= AUTO_TILE_MIN:
        return min(t, AUTO_TILE_MAX) & ~4095
    t = total // (2 * grid)
    return min(max(t, AUTO_TILE_FLOOR), AUTO_TILE_MIN) & ~1023


def tiles_per_feature(offsets: Sequence[np.ndarray], lookup_bytes: Sequence[int],
                      bag_bytes: Sequence[int], gran: Sequence[int], tile_bytes: int,
                      grid_blocks: int = 0) -> List[int]:
    """Host restatement of the device binding (``rfx::bind_tiles``): tiles each feature gets
    for this batch on a grid of ``grid_blocks`` workgroups (0: unknown, taken as too large for
    the whole-pass rule of plentiful tiles to apply).  A schedule that can split bags over
    workgroups (granularity -1) counts as one bag per workgroup pass: a binding frozen at emit
    time never splits.  ``tile_bytes`` <= 0: the size the device picks for this batch."""
    out = []
    num_feats = len(offsets)
    if tile_bytes <= 0:
        tile_bytes = auto_tile_bytes(offsets, lookup_bytes, bag_bytes, grid_blocks)
    for off, lb, bb, g in zip(offsets, lookup_bytes, bag_bytes, gran):
        g = 1 if g < 0 else g
        batch = len(off) - 1
        if batch <= 0:
            out.append(0)
            continue
        cost = int(off[-1] - off[0]) * lb + batch * bb
        tiles = min(max(-(-cost // tile_bytes), 1), batch)
        bpt = -(-batch // tiles)
        whole = -(-bpt // g) * g
        plenty = grid_blocks > 0 and (batch // g) * num_feats >= PLENTY_TILES_PER_WORKGROUP * grid_blocks
        if bpt >= g or plenty or whole * (cost // batch) <= MAX_TILE_FACTOR * tile_bytes:
            bpt = whole
        out.append(-(-batch // bpt))
    return out


def measure_task_blocks(data_npzs: Sequence[str], lookup_bytes: Sequence[int],
                        bag_bytes: Sequence[int], gran: Sequence[int], tile_bytes: int,
                        output_path: str, grid_blocks: int = 0) -> None:
    """One line per batch: comma separated tile counts per feature (CPU only).  ``grid_blocks``:
    the workgroups of the grid the counts are for (compute units x occupancy), which the
    binding's whole-pass rule looks at."""
    per_feat = [load_batches(p) for p in data_npzs]
    lines = []
    for k in range(len(per_feat[0])):
        tiles = tiles_per_feature([b[k][1] for b in per_feat], lookup_bytes, bag_bytes, gran, tile_bytes,
                                  grid_blocks=grid_blocks)
        lines.append(','.join(str(t) for t in tiles))
    _write_atomically(output_path, '\n'.join(lines) + '\n')
