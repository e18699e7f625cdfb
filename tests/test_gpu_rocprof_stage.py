"""GPU: the global stage timed by rocprofv3 (reference: ``RecFlex/tuning/measure.py:98-122`` runs
``run_script.py`` under ``nsys profile``, ``RecFlex/parser.py:71-85`` reads the kernel's total
back).  The profiler is started as a child process with the profiled program right after
``--``; the calling process is never replaced.  Model: C3 at half its batch with capped tables
(kernels of tens of microseconds), default schedules, built ahead of time for two occupancies."""

import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def test_tune_occupancy_under_rocprofv3_agrees_with_the_events_timer():
    from recflex_amd import prebuilt
    from recflex_amd.parser import parse_knl_batch_times, parse_knl_calls_and_average, parse_knl_total_time
    from recflex_amd.tuning.measure import PROFILE_PASSES, PROFILE_WARMUP_PASSES
    d = prebuilt.rocprof_fixture_dir()
    occupancies = prebuilt.ROCPROF_FIXTURE_OCCUPANCIES
    for occ in occupancies:
        lib = os.path.join(d, "all", f"o{occ}", "build", "librecom.so")
        if not os.path.exists(lib):
            raise RuntimeError(f"{lib} is not built: run __graft_entry__.build() first")
    tuner = prebuilt.make_rocprof_tuner()
    mix = prebuilt.fixture_default_mix(tuner)
    batches = len(tuner.batches[0])

    print(f"[case] tune_occupancy with profiler=rocprofv3, occupancies {occupancies}", flush=True)
    cfg = prebuilt.rocprof_tune_config(profiler="rocprofv3", remeasure=True)
    best_occ, sched = tuner.tune_occupancy([mix] * len(occupancies), cfg)
    assert best_occ in occupancies and len(sched) == tuner.num_feats
    by_profiler = {}
    for occ in occupancies:
        out = os.path.join(d, "all", f"o{occ}")
        stats, trace = f"{out}/report_kernel_stats.csv", f"{out}/report_kernel_trace.csv"
        assert os.path.exists(stats) and os.path.exists(trace), open(f"{out}/report.rocprofv3.log").read()[-2000:]
        calls, avg_ns = parse_knl_calls_and_average("FusedKnl", stats)
        assert calls == batches * PROFILE_PASSES and avg_ns > 0
        assert parse_knl_total_time("FusedKnl", stats) == pytest.approx(calls * avg_ns, rel=1e-6)
        per_batch = parse_knl_batch_times("FusedKnl", trace, PROFILE_PASSES, PROFILE_WARMUP_PASSES)
        assert len(per_batch) == batches and min(per_batch) > 0
        by_profiler[occ] = tuner._read_kernel_time(out, cfg)
        assert by_profiler[occ] == pytest.approx(sum(per_batch))
    assert best_occ == min(by_profiler, key=by_profiler.get)

    print("[case] the same libraries under the events timer", flush=True)
    ev = prebuilt.rocprof_tune_config(profiler="events", remeasure=True)
    by_events = {}
    for occ in occupancies:
        out = os.path.join(d, "all", f"o{occ}")
        tuner._kernel_time(out, ev, None)
        by_events[occ] = tuner._read_kernel_time(out, ev)
    print("ns per pass over the batches: rocprofv3", by_profiler, "events", by_events, flush=True)
    for occ in occupancies:
        # the two clocks see the same kernel: the events figure also holds the gap between two
        # launches of a burst, so it may be a little larger, never half or double
        assert 0.5 < by_profiler[occ] / by_events[occ] < 2.0, (occ, by_profiler, by_events)
    # both rank the occupancies alike, unless the two are within 10 % of each other
    ratio_p = by_profiler[occupancies[0]] / by_profiler[occupancies[1]]
    ratio_e = by_events[occupancies[0]] / by_events[occupancies[1]]
    assert (ratio_p > 1) == (ratio_e > 1) or abs(ratio_p - 1) < 0.1 or abs(ratio_e - 1) < 0.1
    assert abs(np.log(ratio_p / ratio_e)) < np.log(1.25), (by_profiler, by_events)


def test_walk_stage_times_the_drawn_ends_and_every_walk_computes_the_same():
    """``Tuner.decide_walk`` on the same model (its variants built ahead of time): the mix as it
    is and with 2 / 4 / 8 / all passes drawn are timed, a drawn winner also with finer segments;
    whatever it keeps is one of what it tried, and the library whose tiles are all drawn gives
    the bits of the one whose tiles are dealt out."""
    import torch
    from recflex_amd import prebuilt
    from recflex_amd.code_emitter.codegen import DRAWN_ALL
    from recflex_amd.rec_modules import FeatEmbed
    from recflex_amd.tuning.measure import make_table
    d = prebuilt.rocprof_fixture_dir()
    occupancy, tile_bytes, xcd_segments = prebuilt.ROCPROF_FIXTURE_WALK
    libs = {name: os.path.join(d, f"walk_{name}", f"o{occupancy}", "build", "librecom.so")
            for name in ("as_is", "drawn_2", "drawn_4", "drawn_8", "drawn_all")}
    for lib in libs.values():
        if not os.path.exists(lib):
            raise RuntimeError(f"{lib} is not built: run __graft_entry__.build() first")
    stamps = {name: os.path.getmtime(lib) for name, lib in libs.items()}
    tuner = prebuilt.make_rocprof_tuner()
    mix = prebuilt.fixture_default_mix(tuner)
    print("[case] walk stage on the 100-feature fixture, events timer", flush=True)
    # (no order is tried here: its variants depend on a measurement and cannot be built ahead)
    cfg = prebuilt.rocprof_tune_config(profiler="events", remeasure=True, walk_drawn_min_tiles=0.0,
                                       walk_stage_min_feats=10 ** 6)
    order, drawn, segments = tuner.decide_walk(mix, occupancy, tile_bytes, xcd_segments, False, cfg)
    assert order is None
    assert drawn in (0, 2, 4, 8, DRAWN_ALL)
    assert segments == xcd_segments or (drawn and segments in cfg.walk_xcd_segments_candidates)
    assert stamps == {name: os.path.getmtime(lib) for name, lib in libs.items()}, "a variant was built again"
    for name in libs:
        t = tuner._read_kernel_time(os.path.dirname(os.path.dirname(libs[name])), cfg)
        assert t > 0
    dev = torch.device("cuda", 0)
    torch.manual_seed(3)
    tables = [make_table(shape, dtype, dev, ones=False) for shape, dtype in zip(tuner.table_shapes, tuner.data_types)]
    idx = [torch.from_numpy(feat[0][0]).to(dev) for feat in tuner.batches]
    off = [torch.from_numpy(feat[0][1]).to(dev) for feat in tuner.batches]
    outs = {}
    for name in ("as_is", "drawn_all", "drawn_2"):
        layer = FeatEmbed(dev, embed_tables=tables, librecom=libs[name])
        outs[name] = layer.forward_indices(idx, off).clone()
    torch.cuda.synchronize()
    assert not torch.isnan(outs["as_is"]).any()
    for name in ("drawn_all", "drawn_2"):
        assert torch.equal(outs[name].view(torch.int32), outs["as_is"].view(torch.int32)), name

