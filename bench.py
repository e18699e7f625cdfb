"""Benchmark of the fused-embedding hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c3] [--also c1,c2,c4,c5]
                    [--batches 8] [--live-traffic headline|all|off]

A step is one launch of the fused kernel over one batch of the synthetic workload; tables,
indices, offsets and the output buffer are resident in HBM before the timed region starts.
The timed loops rotate through ``--batches`` different batches of the workload (same
distributions, other seeds; batch 0 is the configuration's own seeded batch), all resident, so
that no launch finds the lines of the launch before it in the 256 MB Infinity Cache beyond the
rows the batches really share.  Prints ONE JSON line.

Byte counts per launch (Zipf-hot rows are served from the caches, so they differ):

* ``algorithmic_bytes``: rows + int32 indices + int32 offsets + fp32 output, a row counted as
  often as it is looked up -- what the path delivers; its rate can exceed the HBM peak and is
  not a fraction of it (``algorithmic_gbps``, ``roofline.algorithmic_frac``);
* ``compulsory_bytes``: every distinct 128-byte line of the touched rows once, plus indices,
  offsets and output -- what must come from memory even with perfect caches (batch 0);
* ``memory_traffic_bytes``: what the L2 caches exchanged with the memory side (rocprofv3
  ``FETCH_SIZE`` + ``WRITE_SIZE``, each scaled by its reading for a plain copy of known size in
  the same run), averaged over the rotated batches.  For the headline workload the two counter
  runs are made by this very run (``bench.py`` starts ``rocprofv3 --pmc ... -- python3 bench.py
  --pmc-child`` twice before it touches the GPU itself); the other workloads take the figure
  recorded in ``benchaid/hbm_traffic.json`` for the library as built now, or ``null``.  The
  device offers no counter that tells an Infinity-Cache hit from a DRAM access, so this is L2-miss
  traffic: an upper bound of what crossed the HBM pins.

``value`` = ``memory_traffic_bytes`` / wall time per step (GB/s, at most the 8 TB/s of the pins);
``roofline.achieved`` = the same bytes / the fused kernel's own duration, ``roofline.frac`` that
over 8 TB/s.  Where no traffic figure exists both fall back to the compulsory bytes, a lower
bound (``roofline.basis`` says which).
"""

import argparse
import json
import os
import shutil
import subprocess
import sys
import tempfile
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0   # MI355X, HBM3E, published
METRIC = "fused-kernel µs + achieved HBM GB/s (% of MI355X peak) per model config"
BATCH_SEED_STRIDE = 104729          # batch k of a rotation is drawn with seed + k * this
CALIBRATION_COPY_BYTES = 768 << 20
TRAFFIC_KIND = ("L2-miss traffic: rocprofv3 FETCH_SIZE + WRITE_SIZE, what the L2 caches exchange with the "
                "memory side; no counter of this device separates Infinity-Cache hits from DRAM accesses")


TOL = {"float": (1e-5, 1e-6), "half": (1e-3, 1e-6), "int8": (1e-3, 1e-6)}


def parse_args():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=48)
    p.add_argument("--warmup", type=int, default=8)
    p.add_argument("--workload", type=str, default="c3",
                   help="headline configuration (prebuilt model name: c1..c5, refa, reff4, fewbags, c3_skew)")
    p.add_argument("--also", type=str, default="c1,c2,c4,c5",
                   help="comma-separated further configurations reported under 'configs'")
    p.add_argument("--batches", type=int, default=8,
                   help="distinct resident batches the timed loops rotate through")
    p.add_argument("--live-traffic", choices=["headline", "all", "off"], default="headline",
                   help="which workloads get their memory traffic from rocprofv3 counter runs made "
                        "by this run (child processes); the others use the recorded figures")
    p.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline / check leg")
    p.add_argument("--tile-bytes", type=int, default=0)
    p.add_argument("--grid-blocks", type=int, default=0)
    p.add_argument("--xcd-segments", type=int, default=0,
                   help="tile walk: 0 = as emitted, -1 = flat, n = n segments per XCD")
    p.add_argument("--copy-calibration", type=int, default=0,
                   help="also launch one plain device-to-device copy of this many bytes (for "
                        "scaling rocprofv3 FETCH_SIZE / WRITE_SIZE readings)")
    p.add_argument("--no-gather-probe", action="store_true",
                   help="skip the gather probe (bare fetch of the same rows, no sums, no output)")
    p.add_argument("--no-torch-gpu", action="store_true",
                   help="skip the unfused leg (one torch embedding_bag launch per feature on the GPU)")
    p.add_argument("--cpu-features", type=int, default=0,
                   help="bound the CPU leg to this many features (0 = choose from the size)")
    p.add_argument("--pmc-child", action="store_true",
                   help="internal: only the calibration copy and the rotated launches of --workload "
                        "(the program a counter run profiles)")
    return p.parse_args()


def pick_model(name: str) -> str:
    """Prefer the tuned build of a configuration when its schedule file exists."""
    from recflex_amd import prebuilt
    tuned = f"{name}_tuned"
    if tuned in prebuilt.model_names() and \
            os.path.exists(os.path.join(prebuilt.TUNED_DIR, f"{name}_schedule.json")):
        return tuned
    return name


def rotation_size(wl, lookups0: int, wanted: int, free_bytes: int) -> int:
    """Batches that fit beside the tables: each holds its indices and offsets; a few GB are left
    for the output, the probe and the allocator."""
    per_batch = lookups0 * 4 + wl.num_features * (wl.batch + 1) * 4
    room = free_bytes - 2 * wl.batch * wl.embed_dim_sum * 4 - (6 << 30)
    return max(1, min(wanted, int(room // max(1, per_batch))))


def cpu_leg(wl, tables, indices, offsets, gpu_out, max_features: int):
    """Times the oracle on the host cores over a bounded sample (the first ``n`` features that
    keep the work near 10-30 s) and checks the GPU output of those features against it."""
    import torch
    from oracle import oracle
    from recflex_amd.workloads import row_bytes

    torch.set_num_threads(os.cpu_count() or 1)
    cores = torch.get_num_threads()
    lookups = [len(i) for i in indices]
    # bound the sample: at most ~60 M lookups (a few seconds per pass on a server CPU)
    budget, n, acc = 60_000_000, 0, 0
    while n < wl.num_features and (n == 0 or acc + lookups[n] <= budget):
        acc += lookups[n]
        n += 1
    if max_features:
        n = min(n, max_features)
    feats = list(range(n))
    host_tables = []
    for f in feats:
        spec = wl.features[f]
        host_tables.append(oracle.decode_table(tables[f].cpu().numpy(), spec.dim, spec.data_type))
    idx = [indices[f] for f in feats]
    off = [offsets[f] for f in feats]

    want = oracle.pooled_sum_torch(host_tables, idx, off)            # warm-up + the check values
    times = []
    t_start = time.perf_counter()
    while len(times) < 3 or (time.perf_counter() - t_start < 5.0 and len(times) < 200):
        t0 = time.perf_counter()
        oracle.pooled_sum_torch(host_tables, idx, off)
        times.append(time.perf_counter() - t0)
    t = sorted(times)[len(times) // 2]
    sample_bytes = sum(lookups[f] * (row_bytes(wl.features[f].dim, wl.features[f].data_type) + 4)
                       + (wl.batch + 1) * 4 + wl.batch * wl.features[f].dim * 4 for f in feats)

    ok, worst = True, 0.0
    col = 0
    got = gpu_out[:, :sum(wl.features[f].dim for f in feats)].cpu().numpy()
    for f in feats:
        spec = wl.features[f]
        rtol, atol = TOL[spec.data_type]
        good, max_abs, max_rel = oracle.within_tolerance(got[:, col:col + spec.dim],
                                                         want[:, col:col + spec.dim], rtol, atol)
        ok = ok and good
        worst = max(worst, max_rel)
        col += spec.dim
    return {
        "value": sample_bytes / t / 1e9, "unit": "GB/s (algorithmic bytes)", "cores": cores, "kind": "port",
        "sample": f"features 0..{n - 1} of {wl.num_features} at full batch {wl.batch} "
                  f"({sum(lookups[f] for f in feats)} lookups), median of {len(times)} passes of per-feature "
                  f"torch embedding_bag(sum)+cat on fp32 host tables"
                  + (" (fp16/int8 tables dequantised to fp32 beforehand, untimed)"
                     if wl.features[0].data_type != "float" else ""),
        "seconds": t, "lookups_per_s": sum(lookups[f] for f in feats) / t,
    }, {"checked_features": n, "pass": bool(ok), "max_rel_err_beyond_atol": worst}


def torch_gpu_leg(wl, tables, d_idx, d_off, steps: int, out) -> dict:
    """The unfused way on the same GPU, for scale: one torch ``embedding_bag(sum)`` launch per
    feature and a concatenation, timed with events over ``steps`` passes.  fp32 and fp16 tables
    only (torch has no kernel for the int8 row format); its output is checked against the fused
    kernel's."""
    import torch
    import torch.nn.functional as F

    if any(f.data_type == "int8" for f in wl.features):
        return {"skipped": "int8 rows have no torch embedding_bag"}

    def one_pass():
        cols = [F.embedding_bag(d_idx[f], tables[f], d_off[f], mode="sum", include_last_offset=True)
                for f in range(wl.num_features)]
        return torch.cat([c.float() for c in cols], dim=1)

    got = one_pass()
    torch.cuda.synchronize()
    ref = out.view(wl.batch, wl.embed_dim_sum)
    rtol = 1e-5 if wl.features[0].data_type == "float" else 2e-3     # torch accumulates fp16 in fp16
    close = bool(torch.allclose(got, ref, rtol=rtol, atol=1e-5))
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(steps):
        one_pass()
    end.record()
    torch.cuda.synchronize()
    return {"us_per_pass": start.elapsed_time(end) * 1e3 / steps, "launches_per_pass": wl.num_features + 1,
            "agrees_with_fused": close}


class Rotation:
    """The workload's tables, ``K`` resident batches of it, the library and one output buffer."""

    def __init__(self, name: str, wanted_batches: int):
        import torch
        from recflex_amd import prebuilt
        from recflex_amd.rec_modules import FeatEmbed
        from recflex_amd.workloads import gen_inputs, gen_tables

        self.name = name
        self.model = pick_model(name)
        self.wl = prebuilt.model_spec(self.model).workload
        lib_path = prebuilt.ensure_built(self.model)
        self.dev = torch.device("cuda", 0)
        wl = self.wl
        free, _ = torch.cuda.mem_get_info(self.dev)
        if wl.table_bytes() > free * 0.95:
            raise RuntimeError(f"{name}: tables need {wl.table_bytes() / 1e9:.1f} GB, {free / 1e9:.1f} GB free")
        t0 = time.perf_counter()
        self.tables = gen_tables(wl, self.dev)
        workers = min(16, os.cpu_count() or 1)
        self.indices, self.offsets = gen_inputs(wl, workers=workers)         # batch 0: the seeded batch
        free, _ = torch.cuda.mem_get_info(self.dev)
        self.batches = rotation_size(wl, sum(len(i) for i in self.indices), wanted_batches, free)
        self.layer = FeatEmbed(self.dev, embed_tables=self.tables, librecom=lib_path)
        self.lookups = []            # per batch: lookups per feature
        self.d_inputs = []           # per batch: device tensors, kept alive
        self.bound = []              # per batch: validated inputs with their address table uploaded
        for k in range(self.batches):
            idx, off = (self.indices, self.offsets) if k == 0 else \
                gen_inputs(wl._replace(seed=wl.seed + BATCH_SEED_STRIDE * k), workers=workers)
            d_idx = [torch.from_numpy(i).to(self.dev) for i in idx]
            d_off = [torch.from_numpy(o).to(self.dev) for o in off]
            self.lookups.append([len(i) for i in idx])
            self.d_inputs.append((d_idx, d_off))
            self.bound.append(self.layer.bind_inputs(d_idx, d_off))
        self.out = torch.empty(wl.batch * wl.embed_dim_sum, dtype=torch.float32, device=self.dev)
        self.setup_s = time.perf_counter() - t0

    def launch(self, k: int, tile_bytes=0, grid_blocks=0, xcd_segments=0, **kwargs):
        return self.layer.forward_indices(self.bound[k % self.batches], tile_bytes=tile_bytes,
                                          grid_blocks=grid_blocks, xcd_segments=xcd_segments,
                                          out=self.out, **kwargs)


def run_config(name: str, steps: int, warmup: int, with_cpu: bool, tile_bytes: int,
               grid_blocks: int, cpu_features: int, xcd_segments: int = 0,
               gather_probe: bool = True, torch_gpu: bool = False, batches: int = 8,
               live_traffic: dict = None) -> dict:
    import torch
    from recflex_amd import prebuilt
    from benchaid.hbm_traffic import recorded_traffic
    from recflex_amd.hip_helper import HipEvent
    from recflex_amd.workloads import algorithmic_bytes, compulsory_bytes

    rot = Rotation(name, batches)
    wl, dev, K = rot.wl, rot.dev, rot.batches
    opts = dict(tile_bytes=tile_bytes, grid_blocks=grid_blocks, xcd_segments=xcd_segments)

    alg_per_batch = [algorithmic_bytes(wl, lk) for lk in rot.lookups]
    alg_bytes = sum(alg_per_batch) / K                     # mean over the rotation
    comp_bytes = compulsory_bytes(wl, rot.indices, rot.offsets)     # batch 0
    lookups_mean = sum(sum(lk) for lk in rot.lookups) / K
    # memory traffic per launch as the counters gave it: measured by this run, or recorded for
    # this very library
    traffic = live_traffic if live_traffic else recorded_traffic(rot.model)

    for i in range(warmup):
        rot.launch(i, **opts)
    torch.cuda.synchronize()

    # K steps bracketed by synchronisation, rotating through the batches: whole-job rate
    t0 = time.perf_counter()
    for i in range(steps):
        rot.launch(i, **opts)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0

    # per-launch kernel duration with HIP events on the launch stream.  The events are handed to
    # the launch itself (hipExtLaunchKernel) and take the begin and end of the kernel's dispatch:
    # what a kernel trace shows for the same launch.
    def attached(ks):
        pairs = [(HipEvent(), HipEvent()) for _ in ks]
        for k, pair in zip(ks, pairs):
            rot.launch(k, kernel_events=pair, **opts)
        torch.cuda.synchronize()
        return [s.elapsed_us(e) for s, e in pairs]

    durs = attached(range(steps))                           # rotated
    per_batch_us = [sum(durs[k::K]) / len(durs[k::K]) for k in range(K)]
    kernel_us_avg = sum(durs) / len(durs)
    kernel_us_med = sorted(durs)[len(durs) // 2]
    single = attached([0] * steps)                          # batch 0 launched again and again
    kernel_us_single = sum(single) / len(single)

    # the same with a pair of event records around every launch: this also spans the dispatch of
    # the kernel and the events' own packets, about two microseconds
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    stream = torch.cuda.current_stream(dev)
    for i, (s, e) in enumerate(zip(starts, ends)):
        s.record(stream)
        rot.launch(i, **opts)
        e.record(stream)
    torch.cuda.synchronize()
    around = [s.elapsed_time(e) * 1e3 for s, e in zip(starts, ends)]
    kernel_us_event_pairs = sum(around) / len(around)

    kernel_us_dense = dense_launch_us(dev, lambda i: rot.launch(i, **opts))

    kernel_s = kernel_us_avg * 1e-6
    step_s = wall / steps
    mem_bytes = traffic["bytes"] if traffic else comp_bytes
    res = {
        "workload": name, "model": rot.model, "features": wl.num_features, "batch": wl.batch,
        "embed_dim_sum": wl.embed_dim_sum, "lookups": int(sum(rot.lookups[0])),
        "rotated_batches": K, "lookups_mean_over_rotation": lookups_mean,
        "table_gb": round(wl.table_bytes() / 1e9, 2),
        "algorithmic_bytes": int(alg_per_batch[0]), "algorithmic_bytes_mean_over_rotation": alg_bytes,
        "compulsory_bytes": int(comp_bytes),
        "memory_traffic_bytes": traffic["bytes"] if traffic else None,
        "memory_traffic_read_bytes": traffic["read_bytes"] if traffic else None,
        "memory_traffic_written_bytes": traffic["written_bytes"] if traffic else None,
        "memory_traffic_source": traffic["source"] if traffic else None,
        "traffic_over_compulsory": (traffic["bytes"] / comp_bytes) if traffic else None,
        "ms_per_step": step_s * 1e3,
        # the fused kernel's own duration per launch (events attached to the dispatch), mean over
        # the rotation; per batch of the rotation; and batch 0 launched again and again
        "kernel_us_avg": kernel_us_avg, "kernel_us_median": kernel_us_med,
        "kernel_us_per_batch": per_batch_us, "kernel_us_single_batch_replayed": kernel_us_single,
        # an event record before and one after every launch
        "kernel_us_event_pairs": kernel_us_event_pairs,
        # launch-to-launch period of a captured graph of launches: no event packets and no host
        # between the kernels (null if the capture failed)
        "kernel_us_dense": kernel_us_dense,
        "lookups_per_s": lookups_mean / kernel_s,
        # whole-job rates: the K timed steps by the wall clock
        "job_memory_gbps": mem_bytes / step_s / 1e9,
        "job_algorithmic_gbps": alg_bytes / step_s / 1e9,
        # by the kernel's own duration
        "algorithmic_gbps": alg_bytes / kernel_s / 1e9,
        "compulsory_gbps": comp_bytes / kernel_s / 1e9,
        "memory_gbps": mem_bytes / kernel_s / 1e9,
        "memory_basis": "counters" if traffic else "compulsory_bytes",
        "frac_of_hbm_peak": mem_bytes / kernel_s / 1e9 / HBM_PEAK_GBPS,
        "bodies": rot.layer.lib.info.num_bodies, "occupancy": rot.layer.lib.info.occupancy,
        "grid_blocks": grid_blocks or rot.layer.max_concurrent_blocks,
        "setup_s": round(rot.setup_s, 2),
    }
    d_idx, d_off = rot.d_inputs[0]
    ticks_model = rot.model + "_ticks"
    if ticks_model in prebuilt.model_names() and os.path.exists(prebuilt.lib_path(ticks_model)):
        res["binding"] = binding_share(dev, rot.tables, prebuilt.lib_path(ticks_model), d_idx, d_off)
    if gather_probe:
        # another kernel that fetches the same rows and does nothing else: an empirical
        # reference for this batch, not a bound
        from benchaid import gather_probe as gp
        from recflex_amd.workloads import row_stride
        gp.build()                      # compiles only if the library was not built ahead
        probe = gp.GatherProbe(dev, rot.tables, d_idx, [row_stride(f.dim, f.data_type) for f in wl.features])
        best = probe.best_time_us(steps=min(steps, 10))
        res["gather_probe_us"] = best["us"]
        res["gather_probe_setting"] = {k: v for k, v in best.items() if k != "us"}
        # batch 0 replayed, both by event records around the launch
        single_pairs = event_pairs_us(dev, lambda: rot.launch(0, **opts), min(steps, 20))
        res["kernel_over_gather_probe"] = single_pairs / best["us"]
        # ... and the same rows fetched plus an output of this size written as whole cache lines
        with_output = probe.time_with_output_us(best, rot.out, steps=min(steps, 10))
        res["gather_write_probe_us"] = with_output
        res["kernel_over_gather_write_probe"] = single_pairs / with_output
        del probe
    out = rot.launch(0, **opts)          # batch 0's output: what the checks look at
    torch.cuda.synchronize()
    out = out.view(wl.batch, wl.embed_dim_sum)
    if torch_gpu:
        res["torch_gpu_unfused"] = torch_gpu_leg(wl, rot.tables, d_idx, d_off, min(steps, 20), out)
    if with_cpu:
        res["cpu_baseline"], res["check"] = cpu_leg(wl, rot.tables, rot.indices, rot.offsets,
                                                    out, cpu_features)
    del rot, out, d_idx, d_off
    torch.cuda.empty_cache()
    return res


def event_pairs_us(dev, launch, steps: int) -> float:
    import torch
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
             for _ in range(steps)]
    for s, e in pairs:
        s.record()
        launch()
        e.record()
    torch.cuda.synchronize()
    d = sorted(s.elapsed_time(e) * 1e3 for s, e in pairs)
    return d[len(d) // 2]


TICK_NS = 10.0      # the workgroup-level entries of a timing build count the constant 100 MHz clock


def binding_share(dev, tables, ticks_lib: str, d_idx, d_off, launches: int = 5) -> dict:
    """The share of a workgroup's time that passes before its first tile, read from the tick
    counters of the model's timing build (the same schedules and launch parameters with
    clock stamps at kernel entry, after the binding and at the end of the workgroup)."""
    import torch
    from recflex_amd.rec_modules import FeatEmbed
    layer = FeatEmbed(dev, embed_tables=tables, librecom=ticks_lib)
    bound = layer.bind_inputs(d_idx, d_off)
    for _ in range(3):
        layer.forward_indices(bound)
    torch.cuda.synchronize()
    before, total = [], []
    for _ in range(launches):
        layer.forward_indices(bound, timing=True)
        b, t = layer.last_workgroup_ticks
        before.append(b)
        total.append(t)
    grid = layer.max_concurrent_blocks
    res = {"model": os.path.basename(os.path.dirname(os.path.dirname(ticks_lib))),
           "workgroups": grid,
           "binding_ns_per_workgroup": sum(before) / len(before) / grid * TICK_NS,
           "total_ns_per_workgroup": sum(total) / len(total) / grid * TICK_NS,
           "binding_share": sum(before) / sum(total)}
    del layer
    return res


RANDOM_LINE_ROWS = 1 << 25          # x 128 bytes = 4 GiB


def random_line_gbps(dev, steps: int) -> dict:
    """GB/s at which this device fetches 128-byte lines at uniformly random addresses of a 4 GiB
    table (every lookup one whole line, 16 Mi lookups), by the gather probe at its fastest
    setting and by a stock ``torch.index_select`` of the same index stream on the same table:
    what the memory system gives a gather without any reuse, measured live, to be read beside
    the 8 TB/s that sequential traffic reaches at the pins."""
    import torch
    from benchaid.gather_probe import GatherProbe
    lookups = 1 << 24
    table = torch.zeros((RANDOM_LINE_ROWS, 32), dtype=torch.float32, device=dev)
    gen = torch.Generator(device=dev)
    gen.manual_seed(4711)
    idx = torch.randint(0, RANDOM_LINE_ROWS, (lookups,), dtype=torch.int32, device=dev, generator=gen)
    probe = GatherProbe(dev, [table], [idx], [128])
    best = probe.best_time_us(steps=min(steps, 10))
    del probe
    res = {"probe_gbps": lookups * 128 / (best["us"] * 1e-6) / 1e9}
    try:
        # stock torch: reads the same lines, and writes them out as well (a gather with output)
        dst = torch.empty((lookups, 32), dtype=torch.float32, device=dev)
        us = event_pairs_us(dev, lambda: torch.index_select(table, 0, idx, out=dst), 5)
        res["torch_index_select_gbps_read"] = lookups * 128 / (us * 1e-6) / 1e9
        res["torch_index_select_gbps_read_and_written"] = 2 * lookups * 128 / (us * 1e-6) / 1e9
        del dst
    except Exception as exc:      # an extra figure: never lose the run over it
        res["torch_index_select_error"] = f"{type(exc).__name__}: {exc}"
    del table, idx
    torch.cuda.empty_cache()
    return res


DENSE_LAUNCHES = 24


def dense_launch_us(dev, launch):
    """Microseconds per launch when DENSE_LAUNCHES launches (``launch(i)``, rotating through the
    resident batches) run back to back from one captured graph, two events around each replay
    (median of five replays).  An event pair around a single launch also spans the dispatch of
    the kernel and the event's own packets, about two microseconds that matter for a kernel of
    ten; this figure leaves them out."""
    import torch
    try:
        graph = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream(dev)
        side.wait_stream(torch.cuda.current_stream(dev))
        with torch.cuda.stream(side):
            launch(0)
            torch.cuda.synchronize()
            with torch.cuda.graph(graph, stream=side):
                for i in range(DENSE_LAUNCHES):
                    launch(i)
        torch.cuda.synchronize()
        times = []
        for _ in range(5):
            s = torch.cuda.Event(enable_timing=True)
            e = torch.cuda.Event(enable_timing=True)
            s.record()
            graph.replay()
            e.record()
            e.synchronize()
            times.append(s.elapsed_time(e) * 1e3 / DENSE_LAUNCHES)
        del graph
        return sorted(times)[len(times) // 2]
    except Exception as exc:      # the figure is an extra: never lose the run over it
        print(f"bench.py: dense launch timing skipped ({type(exc).__name__}: {exc})", file=sys.stderr)
        return None


# ------------------------------------------------------------------------------------------------
# memory traffic from counter runs made by this run
# ------------------------------------------------------------------------------------------------

def pmc_child(args) -> None:
    """What a counter run profiles: one calibration copy, then the workload's rotated launches."""
    import torch
    from benchaid.gather_probe import calibration_copy
    calibration_copy(args.copy_calibration or CALIBRATION_COPY_BYTES)
    rot = Rotation(args.workload, args.batches)
    opts = dict(tile_bytes=args.tile_bytes, grid_blocks=args.grid_blocks, xcd_segments=args.xcd_segments)
    for i in range(args.warmup + args.steps):
        rot.launch(i, **opts)
    torch.cuda.synchronize()
    print(json.dumps({"pmc_child": args.workload, "model": rot.model, "rotated_batches": rot.batches,
                      "launches": args.warmup + args.steps}))


def measure_traffic_live(workload: str, args, keep_dir: str = None) -> dict:
    """Starts ``rocprofv3 --pmc FETCH_SIZE`` and ``--pmc WRITE_SIZE`` as child processes, each
    profiling ``python3 bench.py --pmc-child`` (the program stands right after ``--``; this
    process is not replaced and has not touched the GPU yet), and turns the two counter files
    into bytes per launch of FusedKnl, scaled by the calibration copy of the same run."""
    from benchaid import hbm_traffic
    rocprof = shutil.which("rocprofv3") or "/opt/rocm/bin/rocprofv3"
    if not os.path.exists(rocprof):
        raise FileNotFoundError("rocprofv3 not found")
    tmp = keep_dir or tempfile.mkdtemp(prefix="bench_pmc_")
    launches, warm = 2 * args.batches, 2
    env = dict(os.environ)
    env.setdefault("TMPDIR", "/tmp")
    dirs = {}
    try:
        for counter in ("FETCH_SIZE", "WRITE_SIZE"):
            out_dir = os.path.join(tmp, f"{workload}_{counter}")
            dirs[counter] = out_dir
            cmd = [rocprof, "--pmc", counter, "--output-format", "csv", "-d", out_dir, "-o", "x", "--",
                   shutil.which("python3") or sys.executable, os.path.join(ROOT, "bench.py"),
                   "--pmc-child", "--workload", workload, "--batches", str(args.batches),
                   "--steps", str(launches), "--warmup", str(warm),
                   "--copy-calibration", str(CALIBRATION_COPY_BYTES),
                   "--tile-bytes", str(args.tile_bytes), "--grid-blocks", str(args.grid_blocks),
                   "--xcd-segments", str(args.xcd_segments)]
            os.makedirs(out_dir, exist_ok=True)
            with open(os.path.join(out_dir, "run.log"), "w") as log:
                subprocess.run(cmd, env=env, cwd="/tmp", stdout=log, stderr=subprocess.STDOUT,
                               timeout=420)
        rec = hbm_traffic.traffic_from_counter_files(dirs["FETCH_SIZE"], dirs["WRITE_SIZE"],
                                                     CALIBRATION_COPY_BYTES, skip_first=warm)
        rec["source"] = (f"rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE child runs of this bench.py run: "
                         f"{rec['dispatches']} FusedKnl dispatches over {args.batches} rotated batches "
                         f"after {warm} warm-up launches, calibrated by one copy of {CALIBRATION_COPY_BYTES} B "
                         f"({rec['fetch_bytes_per_unit']:.1f} / {rec['write_bytes_per_unit']:.1f} B per unit)")
        return rec
    finally:
        if not keep_dir:
            shutil.rmtree(tmp, ignore_errors=True)


def leftover_children() -> list:
    """Processes this run started that are still alive (there should be none at the end)."""
    try:
        import psutil
        return [f"{p.pid}:{' '.join(p.cmdline()[:4])}" for p in psutil.Process().children(recursive=True)]
    except Exception:
        return []


def main():
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py: this path runs on one GPU; --gpus {args.gpus} is not supported "
              "(the value reported is one GPU's throughput)", file=sys.stderr)
        sys.exit(2)

    # counter runs first: child processes, before this process initialises the GPU
    live = {}
    if not args.pmc_child and args.live_traffic != "off":
        names = [args.workload] + ([n for n in args.also.split(",") if n and n != args.workload]
                                   if args.live_traffic == "all" else [])
        for name in names:
            try:
                live[name] = measure_traffic_live(name, args)
            except Exception as exc:      # fall back to the recorded figure, and say so
                print(f"bench.py: live counter runs for {name} failed ({type(exc).__name__}: {exc}); "
                      "using the recorded traffic", file=sys.stderr)

    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the fused kernel has no CPU fallback", file=sys.stderr)
        sys.exit(3)

    if args.pmc_child:
        pmc_child(args)
        return

    if args.copy_calibration > 0:
        from benchaid.gather_probe import calibration_copy
        calibration_copy(args.copy_calibration)     # reads that many bytes, writes as many

    probe = not args.no_gather_probe
    head = run_config(args.workload, args.steps, args.warmup, not args.no_cpu, args.tile_bytes,
                      args.grid_blocks, args.cpu_features, args.xcd_segments, probe,
                      torch_gpu=not args.no_torch_gpu, batches=args.batches,
                      live_traffic=live.get(args.workload))
    others = {}
    for name in [n for n in args.also.split(",") if n and n != args.workload]:
        try:
            others[name] = run_config(name, args.steps, args.warmup, not args.no_cpu,
                                      args.tile_bytes, args.grid_blocks, args.cpu_features,
                                      args.xcd_segments, probe, batches=args.batches,
                                      live_traffic=live.get(name))
        except Exception as exc:  # a configuration that does not fit must not hide the headline
            others[name] = {"error": f"{type(exc).__name__}: {exc}"}

    line = {
        "metric": METRIC,
        "value": head["job_memory_gbps"],
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": head["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": f"synthetic (seeded; tables N(0,0.01) generated on device; {head['rotated_batches']} "
                "resident batches rotated through every timed loop)",
        "config": {"workload": f"{head['workload'].upper()}: {head['features']} features, batch "
                               f"{head['batch']}, sum(dim) {head['embed_dim_sum']}, "
                               f"{head['lookups']} lookups, {head['table_gb']} GB of tables",
                   "build": head["model"], "bodies": head["bodies"],
                   "occupancy": head["occupancy"], "grid_blocks": head["grid_blocks"],
                   "rotated_batches": head["rotated_batches"]},
        "value_definition": ("bytes the L2 caches exchanged with the memory side per launch (counters; "
                             "compulsory bytes if roofline.basis says so) / wall time per step"),
        "fused_kernel_us": head["kernel_us_avg"],
        "kernel_us": head["kernel_us_avg"],
        "kernel_us_median": head["kernel_us_median"],
        "kernel_us_per_batch": head["kernel_us_per_batch"],
        "kernel_us_single_batch_replayed": head["kernel_us_single_batch_replayed"],
        "kernel_us_dense": head["kernel_us_dense"],
        "kernel_us_event_pairs": head["kernel_us_event_pairs"],
        "binding": head.get("binding"),
        "lookups_per_s": head["lookups_per_s"],
        # the rate of what the path delivers (a row counted once per lookup): above the pins'
        # peak where hot rows come from the caches, and no fraction of it
        "algorithmic_gbps": head["algorithmic_gbps"],
        "job_algorithmic_gbps": head["job_algorithmic_gbps"],
        # achieved = bytes the L2s exchanged with the memory side per launch / FusedKnl's duration
        "roofline": {"bound": "hbm", "achieved": head["memory_gbps"], "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": head["frac_of_hbm_peak"], "basis": head["memory_basis"],
                     "traffic": head["memory_traffic_bytes"], "traffic_kind": TRAFFIC_KIND,
                     "traffic_read_bytes": head["memory_traffic_read_bytes"],
                     "traffic_written_bytes": head["memory_traffic_written_bytes"],
                     "traffic_source": head["memory_traffic_source"], "kernel": "FusedKnl",
                     "kernel_us": head["kernel_us_avg"],
                     "compulsory_bytes_per_launch": head["compulsory_bytes"],
                     "compulsory_frac": head["compulsory_gbps"] / HBM_PEAK_GBPS,
                     "traffic_over_compulsory": head["traffic_over_compulsory"],
                     "algorithmic_bytes_per_launch": head["algorithmic_bytes_mean_over_rotation"],
                     "algorithmic_achieved": head["algorithmic_gbps"],
                     "algorithmic_frac": head["algorithmic_gbps"] / HBM_PEAK_GBPS},
    }
    if probe:
        # what a gather without reuse reaches on this device, and the kernel's memory-side rate
        # against it
        rl = random_line_gbps(torch.device("cuda", 0), args.steps)
        line["roofline"]["random_line_gbps"] = rl["probe_gbps"]
        line["roofline"]["random_line"] = rl
        line["roofline"]["frac_of_random_line_rate"] = head["memory_gbps"] / rl["probe_gbps"]
    for key in ("gather_probe_us", "kernel_over_gather_probe", "gather_write_probe_us",
                "kernel_over_gather_write_probe"):
        if key in head:
            line["roofline"][key] = head[key]
    if "torch_gpu_unfused" in head:
        line["torch_gpu_unfused"] = head["torch_gpu_unfused"]
    if "cpu_baseline" in head:
        line["cpu_baseline"] = head["cpu_baseline"]
        line["check"] = head["check"]
    if others:
        line["configs"] = others
    left = leftover_children()
    if left:
        print(f"bench.py: child processes still alive at the end: {left}", file=sys.stderr)
    line["child_processes_left"] = len(left)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
