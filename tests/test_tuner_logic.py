"""Tuner host logic on the CPU: candidate padding, selection arithmetic against the oracle's
restatement of tuner.py, resume-by-files, failure of a measurement worker, the compile cache,
the host restatement of the device binding, and the TaskManager."""

import json
import multiprocessing as mp
import os

import numpy as np
import pytest

from helpers import oracle
from recflex_amd.code_emitter import MetaData
from recflex_amd.schedules import SCHEDULE_MAPPING, WarpPerSampleSchedule, OneHotSchedule
from recflex_amd.tuning import BasicConfig, TuneConfig, Tuner
from recflex_amd.tuning.tuner import padded_sched_num
from recflex_amd.tuning.measure import load_batches, tiles_per_feature


def _tiny_tuner(tmp_path, feats=2, batches=2):
    rng = np.random.default_rng(5)
    data = []
    for f in range(feats):
        bl = []
        for _ in range(batches):
            lens = rng.integers(0, 5, 16)
            off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
            bl.append((rng.integers(0, 100, off[-1]).astype(np.int32), off))
        data.append(bl)
    cfg = BasicConfig("", [], "", "", str(tmp_path / "out"), block_threads=256, sample_batch_nums=batches)
    return Tuner(cfg, SCHEDULE_MAPPING, batches=data, table_shapes=[(100, 16)] * feats,
                 data_types=["float"] * feats,
                 schedule_types=[[OneHotSchedule], [WarpPerSampleSchedule]][:feats])


def test_padding_matches_reference_rule(tmp_path):
    t = _tiny_tuner(tmp_path)
    for n in (1, 5, 24, 152):
        for m in (1, 108, 256 * 8):
            assert padded_sched_num(n, m) == oracle.padded_sched_num(n, m)
            assert t.get_padded_sched_num(n, m) == oracle.padded_sched_num(n, m)
    cands = t.feat_sched_param_candidates[0]
    padded = t.pad_sched_params(cands, 2 * len(cands) + 3)
    assert padded == oracle.pad_sched_params(cands, 2 * len(cands) + 3)


def test_selection_is_argmin_per_occupancy(tmp_path):
    t = _tiny_tuner(tmp_path)
    n0, n1 = (len(c) for c in t.feat_sched_param_candidates)
    rng = np.random.default_rng(1)
    times = {0: {2: rng.random(n0).tolist(), 4: rng.random(n0).tolist()},
             1: {2: rng.random(n1).tolist(), 4: rng.random(n1).tolist()}}
    picked = t.select_per_occupancy(times, [2, 4])
    want = oracle.solve_local(times, [2, 4])
    for i in range(2):
        for f in range(2):
            assert picked[i][f] is t.feat_sched_param_candidates[f][want[i][f]]


def test_data_files_round_trip(tmp_path):
    t = _tiny_tuner(tmp_path)
    for f in range(2):
        back = load_batches(t.data_npzs[f])
        assert len(back) == 2
        for (i0, o0), (i1, o1) in zip(back, t.batches[f]):
            assert np.array_equal(i0, i1) and np.array_equal(o0, o1)
    lines = open(t.table_config_fname).read().split()
    assert lines == ["100,16,float", "100,16,float"]


def test_missing_result_file_raises_like_the_reference(tmp_path):
    """A measuring worker that fails leaves no result.txt; tune() then raises
    FileNotFoundError when it collects the results (tuner.py:143-150)."""
    t = _tiny_tuner(tmp_path)
    cfg = TuneConfig(occupancies=[4], gpu_ids=[0], sm_count=4, num_processes=1, in_process=True,
                     interference="replicate")
    # pretend the libraries exist so that nothing is compiled; the measurement then fails
    # (no GPU / not a real library) and is swallowed by the worker
    for f in range(2):
        _, build_dir = t.get_output_build_dir(f, 4)
        os.makedirs(build_dir, exist_ok=True)
        open(f"{build_dir}/librecom.so", "wb").close()
    with pytest.raises(FileNotFoundError):
        t.tune(cfg)


def test_resume_uses_existing_results(tmp_path):
    t = _tiny_tuner(tmp_path)
    cfg = TuneConfig(occupancies=[2], gpu_ids=[0], sm_count=4, num_processes=1, in_process=True,
                     interference="replicate")
    for f in range(2):
        out, build_dir = t.get_output_build_dir(f, 2)
        os.makedirs(build_dir, exist_ok=True)
        open(f"{build_dir}/librecom.so", "wb").close()
        n = len(t.feat_sched_param_candidates[f])
        with open(f"{out}/result.txt", "w") as fh:
            fh.write(" ".join(str(float((k * 7 + f) % n)) for k in range(n)))
    res = t.tune(cfg)          # neither compiles nor measures
    assert set(res) == {0, 1} and len(res[0][2]) == len(t.feat_sched_param_candidates[0])
    assert int(np.argmin(res[0][2])) == 0


def test_tournament_results_are_read_back(tmp_path):
    """Default local stage: one result.json per occupancy under tournament/o{occ}."""
    t = _tiny_tuner(tmp_path)
    cfg = TuneConfig(occupancies=[2, 4], gpu_ids=[0], sm_count=4, num_processes=1, in_process=True,
                     cluster_stage=False)      # the tournament alone: the cluster stage measures on a GPU
    counts = [len(c) for c in t.feat_sched_param_candidates]
    for occ in (2, 4):
        out, build_dir = t.get_tournament_dir(occ)
        os.makedirs(build_dir, exist_ok=True)
        open(f"{build_dir}/librecom.so", "wb").close()
        times = [[float((k * 3 + occ + f) % n) + 1 for k in range(n)] for f, n in enumerate(counts)]
        with open(f"{out}/result.json", "w") as fh:
            json.dump({"times": times, "best": [0, 0]}, fh)
    res = t.tune(cfg)
    assert [len(res[f][4]) for f in range(2)] == counts
    picked = t.select_per_occupancy(res, [2, 4])
    want = oracle.solve_local(res, [2, 4])
    assert picked[1][1] is t.feat_sched_param_candidates[1][want[1][1]]
    os.remove(f"{t.get_tournament_dir(4)[0]}/result.json")
    with pytest.raises(FileNotFoundError):
        t.tune(cfg)


def test_local_kernel_emission_and_cache_key(tmp_path):
    t = _tiny_tuner(tmp_path, feats=2)
    cfg = TuneConfig(occupancies=[4], gpu_ids=[0], sm_count=8, num_processes=1)
    n = len(t.feat_sched_param_candidates[0])
    assert t.local_padded_num(0, 4, cfg) == oracle.padded_sched_num(n, 32)
    out, _ = t.get_output_build_dir(0, 4)
    padded = t.pad_sched_params(t.feat_sched_param_candidates[0], t.local_padded_num(0, 4, cfg))
    t.emit_codes(out, padded, 4, timing=True, tune=True, host=False)
    src = open(f"{out}/process.hip").read()
    assert f"constexpr int NUM_FEATS = {len(padded)};" in src and "TIMING = true" in src
    assert f"constexpr int NUM_BODIES = {n};" in src
    key = t._source_key(out)
    t.emit_codes(out, padded, 4, timing=True, tune=True, host=False)
    assert t._source_key(out) == key
    assert not os.path.exists(f"{out}/schedule.json")      # only whole models record theirs
    t.emit_codes(str(tmp_path / "m"), padded[:3], 4, host=False)
    cfgs = json.load(open(tmp_path / "m" / "schedule.json"))
    assert len(cfgs) == 3 and cfgs[0]["schedule"] == "OneHotSchedule"


def test_host_binding_restatement():
    """tiles_per_feature mirrors rfx::bind_tiles: cost / tile_bytes tiles, at least one, at most
    one per bag; a tile that holds a whole workgroup pass is rounded up to whole passes."""
    off = np.arange(0, 2049 * 10, 10, dtype=np.int32)          # 2048 bags of 10 lookups
    # 20480 lookups * 132 B + 2048 * 132 B = 2973696 B -> 46 tiles of 64 KiB wanted
    tiles = tiles_per_feature([off], [132], [132], [16], 65536)
    # bags per tile = round_up(ceil(2048 / 46), 16) = 48 -> ceil(2048 / 48) = 43 tiles
    assert tiles == [43]
    # a pass of 1024 bags = 1.49 MB > 8 tiles' worth: the tile is not grown to a pass
    assert tiles_per_feature([off], [132], [132], [1024], 65536) == [46]   # ceil(2048/45)
    # a pass of 256 bags = 372 KB <= 8 x 64 KiB: whole passes
    assert tiles_per_feature([off], [132], [132], [256], 65536) == [8]
    # no tile size given: the one the device would pick for this batch and grid
    from recflex_amd.tuning.measure import auto_tile_bytes
    auto = auto_tile_bytes([off], [132], [132], 16)
    assert tiles_per_feature([off], [132], [132], [16], 0, grid_blocks=16) == \
        tiles_per_feature([off], [132], [132], [16], auto, grid_blocks=16)
    assert tiles_per_feature([off], [132], [132], [1024], 1024) == [2048]  # never more than bags
    assert tiles_per_feature([off], [132], [132], [16], 1 << 30) == [1]
    empty = np.zeros(1, dtype=np.int32)
    assert tiles_per_feature([empty], [132], [132], [16], 65536) == [0]


def _sleep_and_record(path, ident=None):
    import time
    time.sleep(0.05)
    with open(path, "a") as f:
        f.write(f"{ident}\n")


def _boom(ident=None):
    raise RuntimeError("worker failed")


def test_task_manager_returns_resources_and_survives_failures(tmp_path):
    """task_manager.py:27-39: one resource per running task, handed back in `finally`."""
    from recflex_amd.task_manager import TaskManager
    if mp.get_start_method(allow_none=True) != "spawn":
        mp.set_start_method("spawn", force=True)
    log = str(tmp_path / "log.txt")
    tm = TaskManager(["gpu0", "gpu1"])
    for _ in range(5):
        tm.add_task(_sleep_and_record, (log,), ident_key="ident")
    tm.add_task(_boom, (), ident_key="ident")
    tm.join()
    lines = open(log).read().split()
    assert len(lines) == 5 and set(lines) <= {"gpu0", "gpu1"}
    assert tm.resource_queue.qsize() == 2          # both resources are back
    assert sorted(tm.exit_codes) == [0, 0, 0, 0, 0, 1]


def test_task_manager_outlives_a_task_it_cannot_start(tmp_path):
    """An argument that cannot be pickled (spawn) loses that one task: the single resource keeps
    serving, join() returns, and a second round of tasks runs too."""
    import threading
    from recflex_amd.task_manager import TaskManager
    if mp.get_start_method(allow_none=True) != "spawn":
        mp.set_start_method("spawn", force=True)
    log = str(tmp_path / "log.txt")
    tm = TaskManager(["only"])
    tm.add_task(_sleep_and_record, (log,), ident_key="ident")
    tm.add_task(_sleep_and_record, (threading.Lock(),), ident_key="ident")      # not picklable
    tm.add_task(_sleep_and_record, (log,), ident_key="ident")
    done = threading.Thread(target=tm.join, daemon=True)
    done.start()
    done.join(60)
    assert not done.is_alive(), "join() hangs after a task that could not be started"
    assert open(log).read().split() == ["only", "only"]
    assert sorted(tm.exit_codes, key=str) == [0, 0, None]
    tm.add_task(_sleep_and_record, (log,), ident_key="ident")                   # the next round
    tm.join()
    assert len(open(log).read().split()) == 3 and tm.resource_queue.qsize() == 1


def test_register_census_filters_the_tournament(tmp_path, monkeypatch):
    """Candidates that spill, or come within the margin of the occupancy's register budget, stay
    out of that occupancy's tournament; results are mapped back to the full candidate lists."""
    t = _tiny_tuner(tmp_path)
    assert [Tuner.vgpr_budget(o) for o in (1, 2, 3, 4, 5, 6, 8)] == [512, 256, 168, 128, 96, 80, 64]
    cfg = TuneConfig(occupancies=[4], gpu_ids=[0], sm_count=4, num_processes=2, in_process=True)

    def fake_census(sched_param, occupancy, tune_config):      # no compiler in this test
        params = sched_param[1]
        heavy = sum(params) % 3 == 0
        return (124 if heavy else 60 + sum(params) % 40, 64 if sum(params) % 5 == 0 else 0)

    monkeypatch.setattr(t, "_census_one", fake_census)
    admitted = t.tournament_candidates(4, cfg)
    for feat, keep in enumerate(admitted):
        cands = t.feat_sched_param_candidates[feat]
        assert keep and keep == sorted(keep)
        for k, cand in enumerate(cands):
            vgprs, scratch = fake_census(cand, 4, cfg)
            assert (k in keep) == (scratch == 0 and vgprs <= 128 - cfg.census_margin)
    assert os.path.exists(f"{t.basic.codegen_dir}/.cache/census_o4.json")
    # a second call reads the cache
    monkeypatch.setattr(t, "_census_one", lambda *a: (_ for _ in ()).throw(AssertionError("recompiled")))
    assert t.tournament_candidates(4, cfg) == admitted
    # nothing fits: the lightest body is admitted anyway
    assert all(len(k) == 1 for k in t.tournament_candidates(4, cfg._replace(census_margin=128)))

    out, build_dir = t.get_tournament_dir(4)
    os.makedirs(build_dir, exist_ok=True)
    open(f"{build_dir}/librecom.so", "wb").close()
    with open(f"{out}/admitted.json", "w") as fh:
        json.dump(admitted, fh)
    with open(f"{out}/result.json", "w") as fh:
        json.dump({"times": [[float(j + 1) for j in range(len(k))] for k in admitted]}, fh)
    res = t.tune(cfg._replace(cluster_stage=False))      # the tournament's scores as they are
    for feat, keep in enumerate(admitted):
        full = res[feat][4]
        assert len(full) == len(t.feat_sched_param_candidates[feat])
        assert [full[k] for k in keep] == [float(j + 1) for j in range(len(keep))]
        assert all(np.isinf(full[k]) for k in range(len(full)) if k not in keep)
        assert t._nearest_admitted(feat, keep[-1], keep) == len(keep) - 1
        assert 0 <= t._nearest_admitted(feat, 0, keep) < len(keep)


def test_build_climb_adopts_faster_production_builds(tmp_path, monkeypatch):
    """The climb on production builds, with the compiler and the GPU replaced: a kernel's time is
    the sum of a fixed cost per schedule body, so the optimum over the tried candidates is known."""
    import recflex_amd.tuning.tuner as tuner_mod
    t = _tiny_tuner(tmp_path)
    occ = 4

    def body_cost(cand) -> float:
        text = cand[0].EmitScheduleBody(cand[1])
        return 1000.0 + (sum(map(ord, text)) * 7919) % 500

    def fake_builds(jobs, tune_config):
        for out, build_dir in jobs:
            os.makedirs(build_dir, exist_ok=True)
            open(f"{build_dir}/librecom.so", "wb").close()

    class FakeTimer:
        def __init__(self, *a, **k):
            pass

        def time_ns(self, lib, repeats=7, **k):
            entries = json.load(open(os.path.join(os.path.dirname(os.path.dirname(lib)), "schedule.json")))
            from recflex_amd.schedules import schedule_from_config
            return sum(body_cost(schedule_from_config(e, MetaData(e["embed_dim"], e.get("data_type", "float"))))
                       for e in entries)

    monkeypatch.setattr(t, "_schedule_builds", fake_builds)
    monkeypatch.setattr(tuner_mod, "KernelTimer", FakeTimer)
    cands = t.feat_sched_param_candidates
    # tournament scores rank the candidates in list order; the start is each feature's last one
    scores = {f: {occ: [float(k) for k in range(len(c))]} for f, c in enumerate(cands)}
    start = [c[-1] for c in cands]
    cfg = TuneConfig(occupancies=[occ], gpu_ids=[0], sm_count=4, num_processes=3, in_process=True,
                     build_climb_trials=100, build_climb_top_k=4, build_climb_min_gain=0.001)
    mix, t_ns = t.build_climb(start, occ, scores, cfg)
    want = 0.0
    for f, c in enumerate(cands):
        tried = [c[-1]] + c[:4]
        want += min(body_cost(x) for x in tried)
        assert body_cost(mix[f]) == min(body_cost(x) for x in tried)
    assert t_ns == pytest.approx(want)
    assert t_ns <= sum(body_cost(x) for x in start)
    # no trials: the start mix comes back with its own time
    mix0, t0 = t.build_climb(start, occ, scores, cfg._replace(build_climb_trials=0))
    assert mix0 == start and t0 == pytest.approx(sum(body_cost(x) for x in start))


def test_profiler_command_uses_absolute_paths(tmp_path, monkeypatch):
    """The global stage starts rocprofv3 from /tmp; a model directory given relative to the
    caller's directory must still be found."""
    from recflex_amd.tuning.measure import _run_script_args
    monkeypatch.chdir(tmp_path)
    args = _run_script_args("models/t/table_config.txt", "models/t/out/build", "models/t/data", 4, None)
    for flag in ("--table_config_fname", "--build_dir", "--data_dir"):
        value = args[args.index(flag) + 1]
        assert os.path.isabs(value) and value.startswith(str(tmp_path))
    assert os.path.isabs(args[1]) and args[1].endswith("run_script.py")


def test_automatic_tile_size_rule():
    """The tile size the device chooses when none is given, restated on the host: 64 tiles per
    workgroup of the grid, clamped to 64..256 KiB, multiples of 4 KiB; a batch of less than
    64 KiB per workgroup: two tiles per workgroup, 4..64 KiB, multiples of 1 KiB."""
    from recflex_amd.tuning.measure import auto_tile_bytes
    off = lambda n_bags, per_bag: np.arange(n_bags + 1, dtype=np.int64) * per_bag
    # tiny batch (1.35 MB over 1024 workgroups): the floor
    assert auto_tile_bytes([off(512, 4)] * 4, [132] * 4, [132] * 4, 1024) == 4 * 1024
    # 55 MB over 1024 workgroups: half a workgroup's share, 26 KiB
    total = 26 * (4096 * 260 + 4096 * 260)
    got = auto_tile_bytes([off(4096, 1)] * 26, [260] * 26, [260] * 26, 1024)
    assert got == (total // 2048) & ~1023 == 26 * 1024
    # 3.4 GB over 1024 workgroups: less than 64 KiB per tile at 64 tiles per workgroup, far more
    # at two -- the lower bound of large batches
    assert auto_tile_bytes([off(8192, 30)] * 100, [132] * 100, [132] * 100, 1024) == 64 * 1024
    # 10.5 GB over 1280 workgroups: 128 KiB after rounding down to 4 KiB
    got = auto_tile_bytes([off(16384, 20)] * 200, [148] * 200, [516] * 200, 1280)
    total = 200 * (16384 * 20 * 148 + 16384 * 516)
    assert got == (total // (1280 * 64)) & ~4095 and 64 * 1024 < got < 256 * 1024 and got % 4096 == 0
    # tens of GB: the upper bound
    assert auto_tile_bytes([off(8192, 300)] * 400, [516] * 400, [516] * 400, 1024) == 256 * 1024
    # a grid of one workgroup and an empty batch do not divide by zero
    assert auto_tile_bytes([np.zeros(1, dtype=np.int64)], [36], [36], 0) == 4 * 1024


def test_outlier_tiles_are_switched_on_by_the_sampled_data():
    """tune.py --outliers auto: the optimal library gets outlier tiles if a sampled batch holds
    a bag beyond its feature's schedule that carries at least 128 KiB of traffic."""
    from recflex_amd.code_emitter import MetaData
    from recflex_amd.schedules import default_schedule
    from recflex_amd.tuning.tuner import Tuner
    fs = [default_schedule(MetaData(32), 4), default_schedule(MetaData(128), 1)]
    # 132-byte lookups: 993 of them make 128 KiB; 516-byte lookups: 255
    tuner = Tuner.__new__(Tuner)
    short = np.array([0, 3, 3, 900], dtype=np.int32)
    tuner.batches = [[(None, short)], [(None, np.array([0, 1, 2, 250], dtype=np.int32))]]
    assert not tuner.has_outlier_bags(fs)
    tuner.batches = [[(None, short), (None, np.array([0, 5, 1200, 1201], dtype=np.int32))],
                     [(None, np.array([0, 1, 2, 3], dtype=np.int32))]]
    assert tuner.has_outlier_bags(fs)
    tuner.batches = [[(None, short)], [(None, np.array([0, 1, 300, 301], dtype=np.int32))]]
    assert tuner.has_outlier_bags(fs)
    del tuner.batches
    assert not tuner.has_outlier_bags(fs)


def test_outlier_tiles_are_kept_only_if_the_call_is_faster(tmp_path, monkeypatch):
    """An outlier bag in the samples makes the tuner build the mix with and without outlier tiles
    and time both; the tiles stay only if the whole call gains ``outliers_min_gain``.  Without
    such a bag nothing is built."""
    tuner = _tiny_tuner(tmp_path)
    mix = [c[0] for c in tuner.feat_sched_param_candidates]
    built, times = [], {}
    monkeypatch.setattr(Tuner, "_schedule_builds", lambda self, jobs, cfg: built.extend(j[0] for j in jobs))
    monkeypatch.setattr(Tuner, "_kernel_time", lambda self, d, cfg, mgr, tb=0, xs=0: None)
    monkeypatch.setattr(Tuner, "_read_kernel_time",
                        lambda self, d, cfg, tb=0, xs=0: times["on" if "outliers_on" in d else "off"])
    cfg = TuneConfig(occupancies=[4], gpu_ids=[0], sm_count=4, num_processes=1, in_process=True,
                     cluster_stage=False)
    monkeypatch.setattr(Tuner, "has_outlier_bags", lambda self, sp: False)
    assert tuner.decide_outliers(mix, 4, 65536, 16, cfg) is False and not built
    monkeypatch.setattr(Tuner, "has_outlier_bags", lambda self, sp: True)
    times.update(on=900.0, off=1000.0)
    assert tuner.decide_outliers(mix, 4, 65536, 16, cfg) is True
    assert len(built) == 2 and any("outliers_on" in d for d in built)
    on_src = open([d for d in built if "outliers_on" in d][0] + "/process.hip").read()
    off_src = open([d for d in built if "outliers_off" in d][0] + "/process.hip").read()
    assert "find_outliers" in on_src and "find_outliers" not in off_src
    times.update(on=990.0, off=1000.0)            # within the margin: not worth a second kernel
    assert tuner.decide_outliers(mix, 4, 65536, 16, cfg) is False
    times.update(on=1100.0, off=1000.0)           # C4's case
    assert tuner.decide_outliers(mix, 4, 65536, 16, cfg) is False


def test_tile_walk_is_decided_by_measurement(tmp_path, monkeypatch):
    """The walk stage builds the mix as it is, with 2 / 8 / all passes of the tile walk drawn,
    ordered by time per tile and ordered with a drawn end, times them all and keeps the fastest
    only if it gains ``walk_min_gain``; a drawn winner is timed with finer segments per XCD as
    well; with outlier tiles nothing is drawn; left to itself the stage tries a drawn end where
    workgroups get a few tiles each and an order on wide models of few tiles per workgroup."""
    tuner = _tiny_tuner(tmp_path)
    mix = [c[0] for c in tuner.feat_sched_param_candidates]
    built, times, asked = [], {}, []
    monkeypatch.setattr(Tuner, "_schedule_builds", lambda self, jobs, cfg: built.extend(j[0] for j in jobs))
    monkeypatch.setattr(Tuner, "_kernel_time", lambda self, d, cfg, mgr, tb=0, xs=0: asked.append((d, xs)))
    monkeypatch.setattr(Tuner, "_read_kernel_time",
                        lambda self, d, cfg, tb=0, xs=0:
                        times[(d.split("/walk_")[1].split("/")[0], xs) if xs else d.split("/walk_")[1].split("/")[0]])
    monkeypatch.setattr(Tuner, "tile_time_order", lambda self, sp, occ, tb, xs, cfg: [1, 0])
    cfg = TuneConfig(occupancies=[4], gpu_ids=[0], sm_count=4, num_processes=1, in_process=True,
                     cluster_stage=False)
    assert tuner.decide_walk(mix, 4, 65536, 16, False, cfg._replace(walk_stage=False)) == (None, 0, 16)
    assert not built
    on = cfg._replace(walk_stage=True)
    names = ["as_is", "drawn_2", "drawn_4", "drawn_8", "drawn_all", "ordered", "ordered_drawn_2"]
    times.update(dict.fromkeys(names, 1000.0))
    times.update(ordered=940.0, ordered_drawn_2=900.0)
    times.update({("ordered_drawn_2", 64): 905.0, ("ordered_drawn_2", 128): 895.0})   # within the margin
    assert tuner.decide_walk(mix, 4, 65536, 16, False, on) == ([1, 0], 2, 16)
    assert [d.split("/walk_")[1].split("/")[0] for d in built] == names
    drawn = open([d for d in built if "ordered_drawn_2" in d][0] + "/process.hip").read()
    assert "#define RFX_DRAWN_TAIL 2" in drawn and "c_ext_feat" in drawn
    every = open([d for d in built if "drawn_all" in d][0] + "/process.hip").read()
    assert "#define RFX_DRAWN_TAIL 100000" in every and "c_ext_feat" not in every
    times.update(drawn_all=800.0)
    times.update({("drawn_all", 64): 790.0, ("drawn_all", 128): 700.0})
    assert tuner.decide_walk(mix, 4, 65536, 16, False, on) == (None, 100000, 128)
    assert tuner.decide_walk(mix, 4, 65536, 64, False, on) == (None, 100000, 128)
    assert tuner.decide_walk(mix, 4, 65536, 0, False, on) == (None, 100000, 0)    # a flat walk stays flat
    times.update(dict.fromkeys(names, 1000.0))
    times.update(ordered=995.0, drawn_8=996.0)      # within the margin
    del asked[:]
    assert tuner.decide_walk(mix, 4, 65536, 16, False, on) == (None, 0, 16)
    assert all(xs == 0 for _, xs in asked)            # no drawn winner, no finer segments timed
    del built[:]
    times.update(ordered=900.0)
    assert tuner.decide_walk(mix, 4, 65536, 16, True, on) == ([1, 0], 0, 16)
    assert len(built) == 2 and not any("drawn" in d for d in built)
    # left to itself: 2 features x 16 bags on 16 workgroups are less than a tile each -- nothing
    # is drawn, and the model is not wide
    del built[:]
    assert tuner.decide_walk(mix, 4, 65536, 16, False, cfg) == (None, 0, 16) and not built
    few = cfg._replace(walk_drawn_min_tiles=0.01)
    times.update(dict.fromkeys(names, 1000.0))
    times.update(drawn_8=900.0)
    times.update({("drawn_8", 64): 950.0, ("drawn_8", 128): 960.0})
    assert tuner.decide_walk(mix, 4, 65536, 16, False, few) == (None, 8, 16)
    assert [d.split("/walk_")[1].split("/")[0] for d in built] == ["as_is", "drawn_2", "drawn_4", "drawn_8", "drawn_all"]
    del built[:]
    assert tuner.decide_walk(mix, 4, 65536, 16, True, few) == (None, 0, 16) and not built
    wide = cfg._replace(walk_stage_min_feats=2, walk_stage_max_tiles=1e9)
    times.update(ordered=900.0)
    assert tuner.decide_walk(mix, 4, 65536, 16, True, wide) == ([1, 0], 0, 16)
    assert tuner.decide_walk(mix, 4, 65536, 16, True, wide._replace(walk_stage_max_tiles=0.01)) == (None, 0, 16)
    assert tuner.decide_walk(mix, 4, 65536, 16, True, wide._replace(walk_stage_min_feats=3)) == (None, 0, 16)


def test_incumbent_alone_goes_through_the_global_stage(tmp_path, monkeypatch):
    """``solve_incumbent_only``: the mix of a schedule file is the only contender; no tuning
    results are needed, and ``optimal/schedule.json`` records what the stage decided."""
    import recflex_amd.tuning.tuner as tuner_mod
    from recflex_amd.code_emitter import CodeEmitter
    tuner = _tiny_tuner(tmp_path)
    mix = [c[-1] for c in tuner.feat_sched_param_candidates]
    inc = tmp_path / "inc.json"
    inc.write_text(json.dumps({"occupancy": 4, "schedules": CodeEmitter(mix).serialize_config()}))
    timed = []
    monkeypatch.setattr(Tuner, "_schedule_builds", lambda self, jobs, cfg: None)
    monkeypatch.setattr(Tuner, "_kernel_time", lambda self, d, cfg, mgr, tb=0, xs=0: timed.append(d))
    monkeypatch.setattr(Tuner, "_read_kernel_time", lambda self, d, cfg, tb=0, xs=0: 1000.0)
    monkeypatch.setattr(Tuner, "decide_outliers", lambda self, *a: False)
    monkeypatch.setattr(Tuner, "decide_walk", lambda self, sp, occ, tb, xs, outl, cfg: (None, 8, 64))
    monkeypatch.setattr(tuner_mod, "compile_build", lambda d: None)
    cfg = TuneConfig(occupancies=[4], gpu_ids=[0], sm_count=4, num_processes=1, in_process=True,
                     incumbent=str(inc), profiler="events")
    occ, picked = tuner.solve_incumbent_only(cfg)
    assert occ == 4 and all("/incumbent/o4" in d for d in timed) and timed
    assert [s.EmitScheduleBody(p) for s, p in picked] == [s.EmitScheduleBody(p) for s, p in mix]
    doc = json.load(open(f"{tuner.basic.codegen_dir}/optimal/schedule.json"))
    assert doc["drawn_tail"] == 8 and doc["xcd_segments"] == 64 and doc["tile_order"] is None
    assert doc["schedules"] == CodeEmitter(mix).serialize_config()
    src = open(f"{tuner.basic.codegen_dir}/optimal/process.hip").read()
    assert "#define RFX_DRAWN_TAIL 8" in src and "XCD_SEGMENTS = 64" in src
    with pytest.raises(ValueError):
        tuner.solve_incumbent_only(cfg._replace(incumbent=None))


def test_schedule_transfer_adopts_unanimous_picks_by_kind():
    """``transfer_schedule``: a kind of feature (width, type, bag-length class, default schedule)
    takes the source's tuned pick where the source's features of that kind agree; a split vote
    or an unknown kind keeps the default."""
    from recflex_amd.tuning.transfer import feature_kind, transfer_schedule
    d = lambda lanes: {"schedule": "SubWavefrontPerBagSchedule", "params": {"lanes_x": lanes}, "embed_dim": 0}
    src_feats = [(16, "float", 8.2)] * 5 + [(32, "float", 1.0)] * 4 + [(64, "float", 40.0)] * 2
    src_default = [d(4)] * 5 + [d(8)] * 4 + [d(16)] * 2
    src_tuned = [d(2)] * 4 + [d(4)] + [d(8)] * 2 + [d(1)] * 2 + [d(16)] * 2     # 80 %; split; unchanged
    dst_feats = [(16, "float", 9.9), (16, "float", 16.0), (32, "float", 1.2), (64, "float", 44.0), (16, "half", 8.0)]
    dst_default = [d(4), d(4), d(8), d(16), d(4)]
    out, counts = transfer_schedule(src_feats, src_default, src_tuned, dst_feats, dst_default)
    assert [e["params"]["lanes_x"] for e in out] == [2, 4, 8, 16, 4]
    assert counts == {"changed": 1, "kept": 1, "unknown_kind": 3}
    assert out[0] is not dst_default[0] and dst_default[0]["params"]["lanes_x"] == 4
    assert feature_kind(16, "float", 8.2, d(4)) == feature_kind(16, "float", 15.9, d(4))
    assert feature_kind(16, "float", 3.4, d(4)) != feature_kind(16, "float", 3.6, d(4))
    out, counts = transfer_schedule(src_feats, src_default, src_tuned, dst_feats, dst_default, agree=0.5)
    assert counts == {"changed": 1, "kept": 2, "unknown_kind": 2}     # at 50 % the split vote's first pick counts
    with pytest.raises(ValueError):
        transfer_schedule(src_feats, src_default[:-1], src_tuned, dst_feats, dst_default)


def test_tile_order_comes_from_the_ticks_of_the_mix_as_it_ships(tmp_path, monkeypatch):
    """The order key is ticks per tile of a timing build of the chosen mix, pooled over the
    features of one kind (schedule, parameters, row type, width): dearest kind first, features
    of a kind in their own order; fewer than three distinct figures order nothing."""
    import recflex_amd.tuning.tuner as tuner_mod
    rng = np.random.default_rng(9)
    dims, data = [16, 16, 64, 64, 32], []
    for f in range(5):
        lens = rng.integers(1, 6, 64)
        off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        data.append([(rng.integers(0, 100, off[-1]).astype(np.int32), off)])
    cfg = BasicConfig("", [], "", "", str(tmp_path / "out"), block_threads=256, sample_batch_nums=1)
    tuner = Tuner(cfg, SCHEDULE_MAPPING, batches=data, table_shapes=[(100, d) for d in dims],
                  data_types=["float"] * 5, schedule_types=[[WarpPerSampleSchedule]] * 5)
    mix = [c[0] for c in tuner.feat_sched_param_candidates]
    emitted = {}
    monkeypatch.setattr(Tuner, "emit_codes", lambda self, **kw: emitted.update(kw))
    monkeypatch.setattr(Tuner, "_schedule_builds", lambda self, jobs, cfg: None)
    ticks = [100.0, 300.0, 50.0, 70.0, 5000.0]      # kind (dim 16): 400, (dim 64): 120, (dim 32): 5000

    def fake_ticks(lib, shapes, types, npzs, out, tb, xs, gpu_id=None):
        os.makedirs(os.path.dirname(out), exist_ok=True)
        with open(out, "w") as f:
            f.write("".join(f"{t}\n" for t in ticks))
    monkeypatch.setattr(tuner_mod, "measure_feature_ticks", fake_ticks)
    tcfg = TuneConfig(occupancies=[4], gpu_ids=[0], sm_count=4, num_processes=1, in_process=True)
    # tile_bytes tiny enough that every feature gets one tile per bag-granule: equal tile counts
    order = tuner.tile_time_order(mix, 4, 64, 16, tcfg)
    assert emitted["timing"] is True and emitted["feat_schedules"] is mix
    tiles = tiles_per_feature([d[0][1] for d in data], [d * 4 + 4 for d in dims], [d * 4 + 4 for d in dims],
                              [s.TileGranularity(p) for s, p in mix], 64, grid_blocks=16)
    per_kind = {16: (ticks[0] + ticks[1]) / (tiles[0] + tiles[1]), 64: (ticks[2] + ticks[3]) / (tiles[2] + tiles[3]),
                32: ticks[4] / tiles[4]}
    want = sorted(range(5), key=lambda f: (-per_kind[dims[f]], f))
    assert order == want and order[0] == 4 and order.index(0) < order.index(1)
    ticks[:] = [100.0, 100.0, 100.0, 100.0, 100.0]
    tuner2 = Tuner(cfg, SCHEDULE_MAPPING, batches=data[:2] * 2 + data[:1], table_shapes=[(100, 16)] * 5,
                   data_types=["float"] * 5, schedule_types=[[WarpPerSampleSchedule]] * 5)
    assert tuner2.tile_time_order([c[0] for c in tuner2.feat_sched_param_candidates], 4, 64, 16, tcfg) is None


def test_kernel_trace_parser_groups_calls_and_takes_medians(tmp_path):
    """rocprofv3 ``*_kernel_trace.csv``: a call is a FusedKnl dispatch plus the library's own
    kernels launched ahead of it; per batch the median over the passes after the warm-up pass."""
    from recflex_amd.parser import parse_knl_batch_times, parse_knl_call_durations
    header = ('"Kind","Agent_Id","Queue_Id","Stream_Id","Thread_Id","Dispatch_Id","Kernel_Id","Kernel_Name",'
              '"Correlation_Id","Start_Timestamp","End_Timestamp","LDS_Block_Size","Scratch_Size","VGPR_Count",'
              '"Accum_VGPR_Count","SGPR_Count","Workgroup_Size_X","Workgroup_Size_Y","Workgroup_Size_Z",'
              '"Grid_Size_X","Grid_Size_Y","Grid_Size_Z"')
    rows, t = [], 1000
    # 3 passes over 2 batches; pass 0 is slow (warm-up); an unrelated kernel in between
    fused = [[900, 500], [100, 300], [120, 340]]
    aux = [[50, 0], [10, 0], [30, 0]]             # OutlierKnl ahead of batch 0 only
    for p in range(3):
        for b in range(2):
            if aux[p][b]:
                rows.append(("OutlierKnl", t, t + aux[p][b])); t += aux[p][b] + 7
            rows.append(("__amd_rocclr_copyBuffer", t, t + 40)); t += 47
            rows.append(("FusedKnl", t, t + fused[p][b])); t += fused[p][b] + 7
    body = "\n".join(f'"KERNEL_DISPATCH","Agent 1",1,0,8,{i},2,"{n}",{i},{s},{e},512,0,52,0,80,256,1,1,262144,1,1'
                     for i, (n, s, e) in enumerate(reversed(rows)))      # file order is not time order
    path = tmp_path / "report_kernel_trace.csv"
    path.write_text(header + "\n" + body + "\n")
    assert parse_knl_call_durations("FusedKnl", str(path)) == [950, 500, 110, 300, 150, 340]
    assert parse_knl_call_durations("FusedKnl", str(tmp_path / "report")) == [950, 500, 110, 300, 150, 340]
    assert parse_knl_batch_times("FusedKnl", str(path), passes=3, skip_passes=1) == [130.0, 320.0]
    with pytest.raises(ValueError):
        parse_knl_batch_times("FusedKnl", str(path), passes=4)
    with pytest.raises(FileNotFoundError):
        parse_knl_call_durations("FusedKnl", str(tmp_path / "nothing"))


def test_launch_option_ties_go_to_the_fewest_segments():
    from recflex_amd.tuning.tuner import pick_launch_option
    opts = [(65536, -1), (65536, 1), (65536, 8), (65536, 10), (65536, 12), (65536, 16), (65536, 24)]
    times = [120.0, 131.7, 125.6, 119.7, 119.9, 118.2, 118.2]
    assert opts[pick_launch_option(opts, times, 0.015)] == (65536, 10)     # within 1.5 % of 118.2
    assert opts[pick_launch_option(opts, times, 0.0)] == (65536, 16)       # no tolerance: the fastest
    assert opts[pick_launch_option(opts, times, 0.2)] == (65536, 1)
    # the flat walk wins only by being the fastest, and is never preferred on a tie
    assert opts[pick_launch_option(opts, [100.0] + times[1:], 0.015)] == (65536, -1)
    assert opts[pick_launch_option(opts, [118.3] + times[1:], 0.015)] == (65536, 10)
    # two tile sizes at the same segment count: the faster of the two
    opts2 = [(32768, 8), (65536, 8), (65536, 16)]
    assert opts2[pick_launch_option(opts2, [101.0, 100.5, 100.0], 0.015)] == (65536, 8)


def test_whole_passes_when_tiles_are_plentiful():
    """A pass of 4 bags of 160 KB each is more than 8 tiles of 64 KiB: on a small batch the tile
    stays below a pass (more workgroups get work), on a batch whose whole passes already give
    every workgroup of the grid two tiles it is a whole pass (no idle teams)."""
    off = np.arange(0, 2049 * 320, 320, dtype=np.int64)          # 2 048 bags of 320 lookups
    args = ([off] * 100, [516] * 100, [516] * 100, [4] * 100, 65536)
    assert tiles_per_feature(*args)[0] == 2048                   # grid unknown: one bag per tile
    assert tiles_per_feature(*args, grid_blocks=1280)[0] == 512  # 512 * 100 >= 2 * 1280
    few = ([off[:33]] * 4, [516] * 4, [516] * 4, [4] * 4, 65536)
    assert tiles_per_feature(*few, grid_blocks=1280)[0] == 32    # 8 * 4 < 2 * 1280: spread out


def test_cluster_stage_adopts_by_whole_kernel_time(tmp_path, monkeypatch):
    """Local stage by clusters: like features form one cluster, a cluster tries its best-ranked
    candidates and adopts the one that makes the whole kernel faster by the minimum gain -- and
    keeps its picks otherwise; an argmin over the returned scores reproduces the decision.
    (No compiler and no GPU: builds and kernel times are stand-ins.)"""
    import recflex_amd.tuning.tuner as tuner_mod
    rng = np.random.default_rng(3)
    data = []
    for f in range(5):
        mean = [1, 1, 30, 30, 300][f]
        bl = []
        for _ in range(2):
            lens = np.full(16, mean) if mean == 1 else rng.poisson(mean, 16)
            off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
            bl.append((rng.integers(0, 100, off[-1]).astype(np.int32), off))
        data.append(bl)
    cfg = BasicConfig("", [], "", "", str(tmp_path / "out"), block_threads=256, sample_batch_nums=2)
    t = Tuner(cfg, SCHEDULE_MAPPING, batches=data, table_shapes=[(100, 16)] * 5, data_types=["float"] * 5,
              schedule_types=[[WarpPerSampleSchedule]] * 5)
    clusters = t.feature_clusters()
    assert sorted(map(sorted, clusters)) == [[0, 1], [2, 3], [4]]
    assert clusters[0] == [4]                                  # the heaviest cluster first
    n = len(t.feat_sched_param_candidates[0])
    tc = TuneConfig(occupancies=[4], gpu_ids=[0], sm_count=4, num_processes=2, in_process=True,
                    register_census=False, cluster_top_k=3, cluster_min_gain=0.01)
    # rank scores of the first half: candidate 5 best for every feature, then 2, then 7
    scores = np.full(n, 10.0)
    scores[[5, 2, 7]] = [1.0, 2.0, 3.0]
    measured = {f: {4: scores.tolist()} for f in range(5)}
    assert t.cluster_options([2, 3], [0] * 5, 4, measured, 3) == [5, 2, 7]

    monkeypatch.setattr(Tuner, "_schedule_builds", lambda self, jobs, cfg_: None)
    monkeypatch.setattr(Tuner, "_kept", lambda self, out, cfg_: False)
    asked = []

    class FakeTimer:
        """Feature 4's option 2 (candidate 2) is 10 % faster in the scan and head to head; features
        2 and 3 see 0.2 %, below the minimum gain; features 0 and 1 see an option win the scan
        by 3 % that loses head to head (the fastest of several noisy times)."""
        def __init__(self, *a, **k):
            pass

        def time_ns(self, lib, **kw):                          # the mix built as it ships
            return 100.0

        def time_options(self, lib, members, num_options, only=None, **kw):
            asked.append((tuple(members), num_options, tuple(only) if only else None))
            base = [[100.0] * 3 for _ in range(num_options)]
            if tuple(members) == (4,):
                base[2] = [90.0, 91.0, 89.0]
            if tuple(members) == (2, 3):
                base[1] = [99.8, 99.9, 99.7]
            if tuple(members) == (0, 1):
                base[3] = [97.0] * 3 if only is None else [100.2] * 3
            return base

    monkeypatch.setattr(tuner_mod, "KernelTimer", FakeTimer)
    start = [t._nearest_admitted(f, k, list(range(n))) for f, k in enumerate(t.default_choices()[0])]
    picks = t.cluster_stage(4, measured, tc)
    assert asked == [((4,), 4, None), ((4,), 4, (0, 2)), ((2, 3), 4, None), ((0, 1), 4, None),
                     ((0, 1), 4, (0, 3))]
    assert picks[4] == 2 and picks[:4] == start[:4]
    doc = json.load(open(tmp_path / "out" / "clusters" / "o4" / "result.json"))
    assert doc["picks"] == picks and [c["adopted"] for c in doc["clusters"]] == [2, None, None]
    assert doc["clusters"][2]["head_to_head_ns"] == [100.0, 100.2] and doc["group_checks"] == []
    # a second call reads the result file
    monkeypatch.setattr(tuner_mod, "KernelTimer", None)
    assert t.cluster_stage(4, measured, tc) == picks


def test_cluster_adoptions_of_one_group_are_checked_together(tmp_path, monkeypatch):
    """Two clusters of one group each win their head-to-head against the same old mix; in one
    more build, old picks against new, they join one by one, the larger gain first -- and the
    second, which makes the kernel slower once the first is in, is dropped."""
    import recflex_amd.tuning.tuner as tuner_mod
    rng = np.random.default_rng(4)
    data = []
    for f in range(3):
        mean = [30, 30, 300][f]
        bl = []
        for _ in range(2):
            lens = rng.poisson(mean, 16)
            off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
            bl.append((rng.integers(0, 100, off[-1]).astype(np.int32), off))
        data.append(bl)
    cfg = BasicConfig("", [], "", "", str(tmp_path / "out"), block_threads=256, sample_batch_nums=2)
    t = Tuner(cfg, SCHEDULE_MAPPING, batches=data, table_shapes=[(100, 16)] * 3, data_types=["float"] * 3,
              schedule_types=[[WarpPerSampleSchedule]] * 3)
    n = len(t.feat_sched_param_candidates[0])
    tc = TuneConfig(occupancies=[4], gpu_ids=[0], sm_count=4, num_processes=4, in_process=True,
                    register_census=False, cluster_top_k=2, cluster_min_gain=0.01)
    scores = np.full(n, 10.0)
    scores[[5, 2]] = [1.0, 2.0]
    measured = {f: {4: scores.tolist()} for f in range(3)}
    monkeypatch.setattr(Tuner, "_schedule_builds", lambda self, jobs, cfg_: None)
    monkeypatch.setattr(Tuner, "_kept", lambda self, out, cfg_: False)

    class FakeTimer:
        def __init__(self, *a, **k):
            pass

        def time_ns(self, lib, **kw):
            return 100.0

        def time_options(self, lib, members, num_options, only=None, **kw):
            base = [[100.0] * 3 for _ in range(num_options)]
            base[1] = [95.0] * 3 if tuple(members) == (2,) else [97.0] * 3
            return base

        def time_mixes(self, lib, mixes, **kw):                # the group check: old against new
            def t(mix):
                mix = list(mix)
                return {(0, 0, 0): 100.0, (0, 0, 1): 95.0, (1, 1, 1): 96.0}[tuple(mix)]
            return [[t(m)] * 3 for m in mixes]

    monkeypatch.setattr(tuner_mod, "KernelTimer", FakeTimer)
    start = [t._nearest_admitted(f, k, list(range(n))) for f, k in enumerate(t.default_choices()[0])]
    picks = t.cluster_stage(4, measured, tc)
    doc = json.load(open(tmp_path / "out" / "clusters" / "o4" / "result.json"))
    assert [(c["cluster"], c["joined_after"], c["kept"]) for c in doc["group_checks"]] == \
        [(0, 0, True), (1, 1, False)]
    assert picks[2] == 5 and picks[:2] == start[:2]            # the 5 % gain stays, the 3 % one goes
    assert [c["adopted"] for c in doc["clusters"]] == [5, None]


def test_cluster_build_that_is_not_like_the_shipped_build_is_not_used(tmp_path, monkeypatch):
    """A cluster build that runs the current mix 40 % slower than the production build of that
    mix (its candidates' bodies cost everybody registers) decides nothing, however good its
    options look in it."""
    import recflex_amd.tuning.tuner as tuner_mod
    t = _tiny_tuner(tmp_path)
    n0, n1 = (len(c) for c in t.feat_sched_param_candidates)
    tc = TuneConfig(occupancies=[4], gpu_ids=[0], sm_count=4, num_processes=2, in_process=True,
                    register_census=False, cluster_top_k=2)
    measured = {0: {4: list(np.arange(n0, 0, -1.0))}, 1: {4: list(np.arange(n1, 0, -1.0))}}
    monkeypatch.setattr(Tuner, "_schedule_builds", lambda self, jobs, cfg_: None)
    monkeypatch.setattr(Tuner, "_kept", lambda self, out, cfg_: False)

    class FakeTimer:
        def __init__(self, *a, **k):
            pass

        def time_ns(self, lib, **kw):
            return 100.0

        def time_options(self, lib, members, num_options, only=None, **kw):
            return [[140.0] * 3] + [[110.0] * 3 for _ in range(num_options - 1)]

    monkeypatch.setattr(tuner_mod, "KernelTimer", FakeTimer)
    start = [t._nearest_admitted(f, k, list(range(len(t.feat_sched_param_candidates[f]))))
             for f, k in enumerate(t.default_choices()[0])]
    assert t.cluster_stage(4, measured, tc) == start
    doc = json.load(open(tmp_path / "out" / "clusters" / "o4" / "result.json"))
    assert all(c.get("unrepresentative") and c["adopted"] is None for c in doc["clusters"])


def test_task_blocks_of_the_frozen_binding_see_the_grid(tmp_path):
    """measure_task_blocks hands the grid (compute units x occupancy) to the host restatement of
    the binding, so the frozen counts are the ones the run-time binding chooses on that grid."""
    from recflex_amd.tuning.measure import measure_task_blocks, save_batches
    off = np.arange(0, 2049 * 320, 320, dtype=np.int32)
    idx = np.zeros(int(off[-1]), dtype=np.int32)
    paths = []
    for f in range(100):
        paths.append(str(tmp_path / f"f{f}.npz"))
        save_batches(paths[-1], [(idx, off)])
    args = (paths, [516] * 100, [516] * 100, [4] * 100, 65536)
    measure_task_blocks(*args, str(tmp_path / "unknown.txt"))
    measure_task_blocks(*args, str(tmp_path / "grid.txt"), grid_blocks=256 * 5)
    assert open(tmp_path / "unknown.txt").read().split(",")[0] == "2048"
    assert open(tmp_path / "grid.txt").read().split(",")[0] == "512"


def test_an_existing_library_is_kept_only_if_it_is_the_build_of_todays_sources(tmp_path, monkeypatch):
    """The resume-by-files rule keeps ``build/librecom.so`` when it is the cache entry of the
    directory's ``process.hip`` under the current device headers -- and rebuilds otherwise."""
    t = _tiny_tuner(tmp_path)
    cfg = TuneConfig(occupancies=[4], gpu_ids=[0], sm_count=4, num_processes=2, in_process=True)
    out = str(tmp_path / "some" / "o4")
    os.makedirs(f"{out}/build")
    assert not t._kept(out, cfg)                                 # nothing there
    with open(f"{out}/build/librecom.so", "wb") as f:
        f.write(b"library bytes")
    assert t._kept(out, cfg)                                     # no source to hold it against
    with open(f"{out}/process.hip", "w") as f:
        f.write("// source\n")
    assert not t._kept(out, cfg)                                 # a library nobody vouches for
    cached = t._cached_lib(t._source_key(out))
    os.makedirs(os.path.dirname(cached))
    with open(cached, "wb") as f:
        f.write(b"library bytes")
    assert t._kept(out, cfg)                                     # a copy of the cache entry
    assert not t._kept(out, cfg._replace(recompile=True))
    with open(f"{out}/build/librecom.so", "wb") as f:
        f.write(b"other bytes..")                                # same size, other content
    assert not t._kept(out, cfg)
    os.remove(f"{out}/build/librecom.so")
    os.link(cached, f"{out}/build/librecom.so")
    assert t._kept(out, cfg)                                     # the cache entry itself
    monkeypatch.setattr(t, "_headers_digest", lambda: b"headers edited since")
    assert not t._kept(out, cfg)                                 # built under other headers
