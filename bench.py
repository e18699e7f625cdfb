"""Benchmark of the fused-embedding hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c3] [--also c1,c2,c5]

A step is one launch of the fused kernel over one batch of the synthetic workload whose inputs
(tables, indices, offsets) and output buffer are already resident in HBM.  Prints ONE JSON line:
``value`` is the whole-job rate of the headline workload (C3, the heterogeneous 100-feature
configuration) in algorithmic GB/s -- the bytes the path delivers (rows + indices + offsets +
output, a row counted as often as it is looked up) over the wall time of the K timed steps --
next to kernel microseconds, pooled lookups per second, the roofline object for ``FusedKnl``
and the CPU baseline (the oracle: per-feature torch ``embedding_bag(mode="sum")`` + concat on
the host cores) timed in the same run, which is also the correctness check of the GPU result.
``--also`` adds the same figures for further configurations under ``"configs"``.

Three byte counts per launch, because Zipf-hot rows are served from the caches:

* ``algorithmic_bytes``: every lookup's row counted (what a cache-less device would move); the
  rate it gives (``algorithmic_gbps``) can exceed the HBM peak and is not a roofline fraction;
* ``compulsory_bytes``: every distinct 128-byte line of the touched rows once, plus indices,
  offsets and output -- what must cross the HBM pins even with perfect caches, computed live;
* ``hbm_traffic_bytes``: what did cross them (rocprofv3 FETCH_SIZE / WRITE_SIZE, recorded in
  ``recflex_amd/tuned/hbm_traffic.json`` for the library it was measured on; ``null`` when the
  library in use is not that one).

``roofline.frac`` = HBM bytes per launch / kernel time / 8 TB/s, with the measured traffic where
it is known and the compulsory bytes (a lower bound of the traffic) otherwise; it cannot exceed 1.
``roofline.random_line_gbps`` is the rate at which the same device fetches 128-byte lines at
uniformly random addresses (measured in the same run): the ceiling for a gather without reuse.
"""

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0   # MI355X, HBM3E, published
METRIC = "fused-kernel \u00b5s + achieved HBM GB/s (% of MI355X peak) per model config"


TOL = {"float": (1e-5, 1e-6), "half": (1e-3, 1e-6), "int8": (1e-3, 1e-6)}


def parse_args():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=50)
    p.add_argument("--warmup", type=int, default=10)
    p.add_argument("--workload", type=str, default="c3",
                   help="headline configuration (prebuilt model name: c1..c5, c3_tuned)")
    p.add_argument("--also", type=str, default="c1,c2,c4,c5",
                   help="comma-separated further configurations reported under 'configs'")
    p.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline / check leg")
    p.add_argument("--tile-bytes", type=int, default=0)
    p.add_argument("--grid-blocks", type=int, default=0)
    p.add_argument("--xcd-segments", type=int, default=0,
                   help="tile walk: 0 = as emitted, -1 = flat, n = n segments per XCD")
    p.add_argument("--copy-calibration", type=int, default=0,
                   help="also launch one plain device-to-device copy of this many bytes (for "
                        "scaling rocprofv3 FETCH_SIZE / WRITE_SIZE readings)")
    p.add_argument("--no-gather-floor", action="store_true",
                   help="skip the gather probe (bare fetch of the same rows, no sums, no output)")
    p.add_argument("--no-torch-gpu", action="store_true",
                   help="skip the unfused leg (one torch embedding_bag launch per feature on the GPU)")
    p.add_argument("--cpu-features", type=int, default=0,
                   help="bound the CPU leg to this many features (0 = choose from the size)")
    return p.parse_args()


def pick_model(name: str) -> str:
    """Prefer the tuned build of a configuration when its schedule file exists."""
    from recflex_amd import prebuilt
    tuned = f"{name}_tuned"
    if tuned in prebuilt.model_names() and \
            os.path.exists(os.path.join(prebuilt.TUNED_DIR, f"{name}_schedule.json")):
        return tuned
    return name


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
        "value": sample_bytes / t / 1e9, "unit": "GB/s", "cores": cores, "kind": "port",
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


def run_config(name: str, steps: int, warmup: int, with_cpu: bool, tile_bytes: int,
               grid_blocks: int, cpu_features: int, xcd_segments: int = 0,
               gather_floor: bool = True, torch_gpu: bool = False) -> dict:
    import torch
    from recflex_amd import prebuilt
    from recflex_amd.rec_modules import FeatEmbed
    from recflex_amd.hbm_traffic import recorded_traffic_bytes
    from recflex_amd.workloads import algorithmic_bytes, compulsory_bytes, gen_inputs, gen_tables

    model = pick_model(name)
    spec = prebuilt.model_spec(model)
    wl = spec.workload
    lib_path = prebuilt.ensure_built(model)
    dev = torch.device("cuda", 0)

    free, total = torch.cuda.mem_get_info(dev)
    need = wl.table_bytes()
    if need > free * 0.95:
        raise RuntimeError(f"{name}: tables need {need / 1e9:.1f} GB, {free / 1e9:.1f} GB free")

    t0 = time.perf_counter()
    tables = gen_tables(wl, dev)
    indices, offsets = gen_inputs(wl)
    d_idx = [torch.from_numpy(i).to(dev) for i in indices]
    d_off = [torch.from_numpy(o).to(dev) for o in offsets]
    layer = FeatEmbed(dev, embed_tables=tables, librecom=lib_path)
    setup_s = time.perf_counter() - t0

    lookups = [len(i) for i in indices]
    alg_bytes = algorithmic_bytes(wl, lookups)
    comp_bytes = compulsory_bytes(wl, indices, offsets)
    # HBM bytes per launch as the counters gave them, if they were taken on this very library
    traffic = recorded_traffic_bytes(model)

    bound = layer.bind_inputs(d_idx, d_off)      # inputs validated, address table uploaded: once
    run = lambda: layer.forward_indices(bound, tile_bytes=tile_bytes, grid_blocks=grid_blocks,
                                        xcd_segments=xcd_segments)
    for _ in range(warmup):
        out = run()
    torch.cuda.synchronize()

    # K steps bracketed by synchronisation: whole-job rate
    t0 = time.perf_counter()
    for _ in range(steps):
        out = run()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0

    # per-launch kernel duration with HIP events on the launch stream.  The events are handed to
    # the launch itself (hipExtLaunchKernel) and take the begin and end of the kernel's dispatch:
    # what a kernel trace shows for the same launch.
    from recflex_amd.hip_helper import HipEvent
    outbuf = torch.empty(wl.batch * wl.embed_dim_sum, dtype=torch.float32, device=dev)
    pairs = [(HipEvent(), HipEvent()) for _ in range(steps)]
    for pair in pairs:
        layer.forward_indices(bound, tile_bytes=tile_bytes, grid_blocks=grid_blocks,
                              xcd_segments=xcd_segments, out=outbuf, kernel_events=pair)
    torch.cuda.synchronize()
    durs = sorted(s.elapsed_us(e) for s, e in pairs)   # us
    kernel_us_avg = sum(durs) / len(durs)
    kernel_us_med = durs[len(durs) // 2]
    del pairs

    # the same with a pair of event records around every launch: this also spans the dispatch of
    # the kernel and the events' own packets, about two microseconds
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    stream = torch.cuda.current_stream(dev)
    for s, e in zip(starts, ends):
        s.record(stream)
        layer.forward_indices(bound, tile_bytes=tile_bytes, grid_blocks=grid_blocks,
                              xcd_segments=xcd_segments, out=outbuf)
        e.record(stream)
    torch.cuda.synchronize()
    around = sorted(s.elapsed_time(e) * 1e3 for s, e in zip(starts, ends))
    kernel_us_event_pairs = sum(around) / len(around)

    kernel_us_dense = dense_launch_us(dev, lambda: layer.forward_indices(
        bound, tile_bytes=tile_bytes, grid_blocks=grid_blocks, xcd_segments=xcd_segments, out=outbuf))

    kernel_s = kernel_us_avg * 1e-6
    hbm_bytes = traffic if traffic is not None else comp_bytes
    res = {
        "workload": name, "model": model, "features": wl.num_features, "batch": wl.batch,
        "embed_dim_sum": wl.embed_dim_sum, "lookups": int(sum(lookups)),
        "table_gb": round(wl.table_bytes() / 1e9, 2),
        "algorithmic_bytes": int(alg_bytes), "compulsory_bytes": int(comp_bytes),
        "hbm_traffic_bytes": traffic,
        "traffic_over_compulsory": (traffic / comp_bytes) if traffic is not None else None,
        "ms_per_step": wall / steps * 1e3,
        # the fused kernel's own duration per launch (events attached to the dispatch)
        "kernel_us_avg": kernel_us_avg, "kernel_us_median": kernel_us_med,
        # an event record before and one after every launch
        "kernel_us_event_pairs": kernel_us_event_pairs,
        # launch-to-launch period of a captured graph of launches: no event packets and no host
        # between the kernels (null if the capture failed)
        "kernel_us_dense": kernel_us_dense,
        "lookups_per_s": sum(lookups) / kernel_s,
        # whole-job rate: the K timed steps by the wall clock
        "job_algorithmic_gbps": alg_bytes / (wall / steps) / 1e9,
        # by the kernel's own duration
        "algorithmic_gbps": alg_bytes / kernel_s / 1e9,
        "compulsory_gbps": comp_bytes / kernel_s / 1e9,
        "hbm_gbps": hbm_bytes / kernel_s / 1e9,
        "hbm_basis": "hbm_counters" if traffic is not None else "compulsory_bytes",
        "frac_of_hbm_peak": hbm_bytes / kernel_s / 1e9 / HBM_PEAK_GBPS,
        "bodies": layer.lib.info.num_bodies, "occupancy": layer.lib.info.occupancy,
        "grid_blocks": grid_blocks or layer.max_concurrent_blocks,
        "setup_s": round(setup_s, 2),
    }
    ticks_model = model + "_ticks"
    if ticks_model in prebuilt.model_names() and os.path.exists(prebuilt.lib_path(ticks_model)):
        res["binding"] = binding_share(dev, tables, prebuilt.lib_path(ticks_model), d_idx, d_off)
    if gather_floor:
        # the memory system's floor for this batch: the same rows fetched and dropped
        from recflex_amd import gather_probe
        from recflex_amd.gather_probe import GatherProbe
        from recflex_amd.workloads import row_stride
        gather_probe.build()            # compiles only if the library was not built ahead
        probe = GatherProbe(dev, tables, d_idx, [row_stride(f.dim, f.data_type) for f in wl.features])
        floor = probe.best_time_us(steps=min(steps, 10))
        res["gather_floor_us"] = floor["us"]
        res["gather_floor_setting"] = {k: v for k, v in floor.items() if k != "us"}
        res["kernel_over_gather_floor"] = kernel_us_event_pairs / floor["us"]   # both by event records
        # ... and the same rows fetched plus an output of this size written as whole cache lines
        with_output = probe.time_with_output_us(floor, outbuf, steps=min(steps, 10))
        res["gather_write_floor_us"] = with_output
        res["kernel_over_gather_write_floor"] = kernel_us_event_pairs / with_output
        del probe
    if torch_gpu:
        res["torch_gpu_unfused"] = torch_gpu_leg(wl, tables, d_idx, d_off, min(steps, 20), out)
    if with_cpu:
        res["cpu_baseline"], res["check"] = cpu_leg(wl, tables, indices, offsets,
                                                    out, cpu_features)
    del layer, tables, d_idx, d_off, out, outbuf
    torch.cuda.empty_cache()
    return res


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


RANDOM_LINE_ROWS = 1 << 24          # x 128 bytes = 2 GiB


def random_line_gbps(dev, steps: int) -> float:
    """GB/s at which this device fetches 128-byte lines at uniformly random addresses of a 2 GiB
    table (every lookup one whole line, 16 Mi lookups, the gather probe at its fastest setting):
    the ceiling of the memory system for a gather without any reuse, measured live, to be read
    beside the 8 TB/s that sequential traffic reaches at the pins."""
    import torch
    from recflex_amd.gather_probe import GatherProbe
    table = torch.zeros((RANDOM_LINE_ROWS, 32), dtype=torch.float32, device=dev)
    gen = torch.Generator(device=dev)
    gen.manual_seed(4711)
    idx = torch.randint(0, RANDOM_LINE_ROWS, (RANDOM_LINE_ROWS,), dtype=torch.int32, device=dev,
                        generator=gen)
    probe = GatherProbe(dev, [table], [idx], [128])
    best = probe.best_time_us(steps=min(steps, 10))
    del probe, table, idx
    torch.cuda.empty_cache()
    return RANDOM_LINE_ROWS * 128 / (best["us"] * 1e-6) / 1e9


DENSE_LAUNCHES = 20


def dense_launch_us(dev, launch):
    """Microseconds per launch when DENSE_LAUNCHES launches run back to back from one captured
    graph, two events around each replay (median of five replays).  An event pair around a
    single launch also spans the dispatch of the kernel and the event's own packets, about two
    microseconds that matter for a kernel of ten; this figure leaves them out."""
    import torch
    try:
        graph = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream(dev)
        side.wait_stream(torch.cuda.current_stream(dev))
        with torch.cuda.stream(side):
            launch()
            torch.cuda.synchronize()
            with torch.cuda.graph(graph, stream=side):
                for _ in range(DENSE_LAUNCHES):
                    launch()
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


def main():
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py: this path runs on one GPU; --gpus {args.gpus} is not supported "
              "(the value reported is one GPU's throughput)", file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the fused kernel has no CPU fallback", file=sys.stderr)
        sys.exit(3)

    if args.copy_calibration > 0:
        from recflex_amd.gather_probe import calibration_copy
        calibration_copy(args.copy_calibration)     # reads that many bytes, writes as many

    floor = not args.no_gather_floor
    head = run_config(args.workload, args.steps, args.warmup, not args.no_cpu, args.tile_bytes,
                      args.grid_blocks, args.cpu_features, args.xcd_segments, floor,
                      torch_gpu=not args.no_torch_gpu)
    others = {}
    for name in [n for n in args.also.split(",") if n and n != args.workload]:
        try:
            others[name] = run_config(name, args.steps, args.warmup, not args.no_cpu,
                                      args.tile_bytes, args.grid_blocks, args.cpu_features,
                                      args.xcd_segments, floor)
        except Exception as exc:  # a configuration that does not fit must not hide the headline
            others[name] = {"error": f"{type(exc).__name__}: {exc}"}

    line = {
        "metric": METRIC,
        "value": head["job_algorithmic_gbps"],
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": head["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic (seeded; tables N(0,0.01) generated on device)",
        "config": {"workload": f"{head['workload'].upper()}: {head['features']} features, batch "
                               f"{head['batch']}, sum(dim) {head['embed_dim_sum']}, "
                               f"{head['lookups']} lookups, {head['table_gb']} GB of tables",
                   "build": head["model"], "bodies": head["bodies"],
                   "occupancy": head["occupancy"], "grid_blocks": head["grid_blocks"]},
        "value_definition": "algorithmic bytes per launch (rows + int32 indices + int32 offsets + fp32 "
                            "output, a row counted once per lookup) / wall time per step",
        "kernel_us": head["kernel_us_avg"],
        "kernel_us_median": head["kernel_us_median"],
        "kernel_us_dense": head["kernel_us_dense"],
        "kernel_us_event_pairs": head["kernel_us_event_pairs"],
        "binding": head.get("binding"),
        "lookups_per_s": head["lookups_per_s"],
        # achieved = bytes that crossed the HBM pins per launch / FusedKnl's duration: the
        # counters' figure where it was taken on this library, else the compulsory bytes (every
        # distinct memory line once), which the traffic cannot be below; never above the peak
        "roofline": {"bound": "hbm", "achieved": head["hbm_gbps"], "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": head["frac_of_hbm_peak"], "basis": head["hbm_basis"],
                     "traffic": head["hbm_traffic_bytes"], "kernel": "FusedKnl",
                     "compulsory_bytes_per_launch": head["compulsory_bytes"],
                     "traffic_over_compulsory": head["traffic_over_compulsory"],
                     "algorithmic_bytes_per_launch": head["algorithmic_bytes"],
                     "algorithmic_gbps": head["algorithmic_gbps"]},
    }
    if floor:
        # what a gather without reuse reaches on this device, and the kernel's HBM rate against it
        line["roofline"]["random_line_gbps"] = random_line_gbps(torch.device("cuda", 0), args.steps)
        line["roofline"]["frac_of_random_line_rate"] = head["hbm_gbps"] / line["roofline"]["random_line_gbps"]
    if "gather_floor_us" in head:
        # time of the bare fetch of the same rows (gather probe): what the memory system allows
        line["roofline"]["gather_floor_us"] = head["gather_floor_us"]
        line["roofline"]["kernel_over_gather_floor"] = head["kernel_over_gather_floor"]
        # the gather plus the writing of an output of this size (whole lines, once)
        line["roofline"]["gather_write_floor_us"] = head["gather_write_floor_us"]
        line["roofline"]["kernel_over_gather_write_floor"] = head["kernel_over_gather_write_floor"]
    if "torch_gpu_unfused" in head:
        line["torch_gpu_unfused"] = head["torch_gpu_unfused"]
    if "cpu_baseline" in head:
        line["cpu_baseline"] = head["cpu_baseline"]
        line["check"] = head["check"]
    if others:
        line["configs"] = others
    print(json.dumps(line))


if __name__ == "__main__":
    main()
