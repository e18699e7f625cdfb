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
