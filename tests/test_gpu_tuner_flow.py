"""GPU: the text entry point (dataset lines -> fused kernel) and the tuner's measuring stages on
the small model directory tests/golden/model_test, whose kernels are built ahead of time."""

import json
import os
import shutil

import numpy as np
import pytest

from helpers import ROOT, oracle

pytestmark = pytest.mark.gpu

MODEL_DIR = os.path.join(ROOT, "tests", "golden", "model_test")


def _fixture():
    from recflex_amd import prebuilt
    d = prebuilt.tune_fixture_dir()
    if not os.path.exists(os.path.join(d, "default", "build", "librecom.so")):
        raise RuntimeError(f"{d} is not built: run __graft_entry__.build() first")
    return d, prebuilt.make_fixture_tuner(MODEL_DIR)


def _check_text_model(model, tuner, raw_batches, rtol=1e-4, atol=1e-4):
    import torch
    dims = [d for _, d in tuner.table_shapes]
    host_tables = [t.cpu().numpy() for t in model.embed_layer.embed_tables]
    for raw in raw_batches:
        out = model(raw)
        torch.cuda.synchronize()
        got = out.view(-1, sum(dims)).cpu().numpy()
        parsed = [oracle.parse_lines_python(lines) for lines in raw]
        want = oracle.pooled_sum_c(host_tables, dims, tuner.data_types,
                                   [p[0] for p in parsed], [p[1] for p in parsed])
        assert got.shape == want.shape == (len(raw[0]), sum(dims))
        # default: N(0,1) tables and bags of up to 500 lookups, as in the reference's own run,
        # at its tolerance (examples/test.py:85, atol = rtol = 1e-4)
        ok, max_abs, max_rel = oracle.within_tolerance(got, want, rtol, atol)
        assert ok, (max_abs, max_rel)


def test_text_entry_point_matches_oracle():
    """FeatProcessEmbed(raw lines) with the generated host front end, as examples/test.py --check."""
    import torch
    from recflex_amd.parser import parse_raw_data_batches
    from recflex_amd.rec_modules import FeatProcessEmbed
    from recflex_amd.utils import find_file, import_from_path
    d, tuner = _fixture()
    build_dir = os.path.join(d, "default", "build")
    recom_host = import_from_path("recom_host", find_file(build_dir, "recom_host*.so"))
    assert recom_host.num_features == 6
    raw_batches = parse_raw_data_batches(tuner.basic.batch_sizes_fname, tuner.basic.data_fnames, 3,
                                         seed=0, feat_major=False)
    print(f"[case] text path, {len(raw_batches)} batches of sizes {[len(b[0]) for b in raw_batches]}", flush=True)
    model = FeatProcessEmbed(recom_host, torch.device("cuda", 0), table_shapes=tuner.table_shapes,
                             librecom_path=f"{build_dir}/librecom.so")
    _check_text_model(model, tuner, raw_batches)
    # event-timed variant of the same call
    res, ms = model(raw_batches[0], timing_kernel=True)
    assert ms > 0 and res.numel() == len(raw_batches[0][0]) * 96
    # the path's own gate for fp32 tables -- 1e-5 relative or 1e-6 absolute -- on N(0, 0.01) tables
    print("[case] text path on N(0, 0.01) tables at 1e-5 / 1e-6", flush=True)
    g = torch.Generator(device="cuda:0")
    g.manual_seed(2024)
    tables = [torch.randn(shape, generator=g, device="cuda:0") * 0.01 for shape in tuner.table_shapes]
    model = FeatProcessEmbed(recom_host, torch.device("cuda", 0), embed_tables=tables,
                             librecom_path=f"{build_dir}/librecom.so")
    _check_text_model(model, tuner, raw_batches, rtol=1e-5, atol=1e-6)


def test_local_stage_replicated_candidates():
    """Reference-style local stage: all candidates of a feature side by side, padded to fill
    the GPU, per-candidate device timers."""
    from recflex_amd import prebuilt
    d, tuner = _fixture()
    cfg = prebuilt.fixture_tune_config(interference="replicate", occupancies=[4], remeasure=True)
    print("[case] local stage, replicate", flush=True)
    res = tuner.tune(cfg)
    assert set(res) == set(range(6))
    for f in range(6):
        t = res[f][4]
        assert len(t) == len(tuner.feat_sched_param_candidates[f])
        assert all(np.isfinite(t)) and min(t) > 0


def test_tournament_then_global_stage():
    """Default local stage (candidates timed inside the whole model), selection, global
    occupancy sweep; the winning library must still compute the right thing."""
    import torch
    from recflex_amd import prebuilt
    from recflex_amd.parser import parse_raw_data_batches
    from recflex_amd.rec_modules import FeatProcessEmbed
    from recflex_amd.host import RecomHost
    d, tuner = _fixture()
    cfg = prebuilt.fixture_tune_config(interference="model", remeasure=True, rounds=1, refine_passes=1)
    print("[case] tournament local stage", flush=True)
    res = tuner.tune(cfg)
    for occ in cfg.occupancies:
        admitted = tuner.admitted_candidates(occ)      # what the register census let in
        for f in range(6):
            t = np.asarray(res[f][occ])
            assert len(t) == len(tuner.feat_sched_param_candidates[f]) and admitted[f]
            assert np.isfinite(t[admitted[f]]).all() and t.min() > 0
            assert np.isinf(np.delete(t, admitted[f])).all()
    picked = tuner.select_per_occupancy(res, cfg.occupancies)
    for i, occ in enumerate(cfg.occupancies):
        for f in range(6):
            assert picked[i][f] is tuner.feat_sched_param_candidates[f][int(np.argmin(res[f][occ]))]
    if shutil.which("hipcc") is None and not os.path.exists("/opt/rocm/bin/hipcc"):
        pytest.skip("global stage builds one kernel per occupancy and needs hipcc")
    print("[case] global stage (builds 2 small kernels)", flush=True)
    occ, sched = tuner.solve(res, cfg)
    assert occ in cfg.occupancies and len(sched) == 6
    doc = json.load(open(os.path.join(d, "optimal", "schedule.json")))
    assert doc["occupancy"] == occ and len(doc["schedules"]) == 6
    raw_batches = parse_raw_data_batches(tuner.basic.batch_sizes_fname, tuner.basic.data_fnames, 2,
                                         seed=1, feat_major=False)
    model = FeatProcessEmbed(RecomHost(), torch.device("cuda", 0), table_shapes=tuner.table_shapes,
                             librecom_path=os.path.join(d, "optimal", "build", "librecom.so"))
    _check_text_model(model, tuner, raw_batches)


def test_cluster_stage_decides_the_local_stage():
    """The local stage's second half: clusters of like features try their best-ranked candidates
    in production-shaped builds (compiled here: one small kernel per cluster) and decide on
    whole-kernel time; the scores ``tune`` returns elect exactly that mix, and the library the
    global stage builds from it computes the right thing."""
    import torch
    from recflex_amd import prebuilt
    from recflex_amd.parser import parse_raw_data_batches
    from recflex_amd.rec_modules import FeatProcessEmbed
    from recflex_amd.host import RecomHost
    if shutil.which("hipcc") is None and not os.path.exists("/opt/rocm/bin/hipcc"):
        pytest.skip("the cluster stage builds one kernel per cluster and needs hipcc")
    d, tuner = _fixture()
    shutil.rmtree(os.path.join(d, "clusters"), ignore_errors=True)
    cfg = prebuilt.fixture_tune_config(interference="model", occupancies=[4], remeasure=True, rounds=1,
                                       refine_passes=1, climb_passes=0, cluster_stage=True,
                                       cluster_top_k=3, cluster_min_gain=0.0, include_default=False)
    print("[case] tournament + cluster stage at 4 workgroups per CU", flush=True)
    res = tuner.tune(cfg)
    doc = json.load(open(os.path.join(d, "clusters", "o4", "result.json")))
    clusters = tuner.feature_clusters()
    assert sorted(f for c in clusters for f in c) == list(range(6))
    assert len(doc["clusters"]) == len(clusters) and len(doc["picks"]) == 6
    admitted = tuner.admitted_candidates(4)
    for entry in doc["clusters"]:
        assert len(entry["kernel_ns"]) == len(entry["options"]) + 1 and min(entry["kernel_ns"]) > 0
        assert all(k in admitted[f] for f in entry["members"] for k in entry["options"])
        if entry["adopted"] is not None:           # with no minimum gain: the fastest option
            assert entry["adopted"] == entry["options"][int(np.argmin(entry["kernel_ns"])) - 1]
            assert all(doc["picks"][f] == entry["adopted"] for f in entry["members"])
    for f in range(6):
        assert int(np.argmin(res[f][4])) == doc["picks"][f]
    print("[case] global stage on the elected mix (builds 1 small kernel)", flush=True)
    occ, sched = tuner.solve(res, cfg)
    assert occ == 4
    for f in range(6):
        assert sched[f] is tuner.feat_sched_param_candidates[f][doc["picks"][f]]
    raw_batches = parse_raw_data_batches(tuner.basic.batch_sizes_fname, tuner.basic.data_fnames, 2,
                                         seed=2, feat_major=False)
    model = FeatProcessEmbed(RecomHost(), torch.device("cuda", 0), table_shapes=tuner.table_shapes,
                             librecom_path=os.path.join(d, "optimal", "build", "librecom.so"))
    _check_text_model(model, tuner, raw_batches)


def test_compressed_model_flow():
    """``examples/run_model.sh``: the model is compressed to one representative per cluster of
    like features (``compress.py``), the representatives' candidates are measured (``tune.py
    --local_only``), ``decompress.py`` spreads libraries and results back over the full model,
    whose tuner then finds them (nothing to compile or measure in its local stage) and goes on
    to the global stage."""
    import subprocess
    import sys
    import torch
    from recflex_amd import prebuilt
    from recflex_amd.parser import parse_raw_data_batches
    from recflex_amd.rec_modules import FeatProcessEmbed
    from recflex_amd.host import RecomHost
    root = prebuilt.compress_fixture_dir()
    small = os.path.join(root, "model")
    if not os.path.exists(os.path.join(small, "output", "f0", "o4", "build", "librecom.so")):
        raise RuntimeError(f"{root} is not built: run __graft_entry__.build() first")
    clusters = [[int(t) for t in line.split(",")] for line in open(os.path.join(small, "feat_map.txt"))]
    assert clusters == [[0, 1, 2, 3], [4], [5]]

    print("[case] local stage of the compressed model (3 representatives)", flush=True)
    cfg = prebuilt.fixture_tune_config(interference="replicate", occupancies=[4], remeasure=True)
    small_tuner = prebuilt.make_fixture_tuner(small, codegen_dir=os.path.join(small, "output"))
    small_res = small_tuner.tune(cfg)
    assert set(small_res) == {0, 1, 2}

    full = os.path.join(root, "full")
    shutil.rmtree(full, ignore_errors=True)
    shutil.copytree(os.path.join(root, "src"), full)
    subprocess.run([sys.executable, os.path.join(ROOT, "examples", "decompress.py"), "-i", small, "-o", full],
                   check=True)

    print("[case] the full model finds the spread results; global stage (builds 1 small kernel)", flush=True)
    tuner = prebuilt.make_fixture_tuner(full, codegen_dir=os.path.join(full, "output"))
    before = {f: os.path.getmtime(os.path.join(full, "output", f"f{f}", "o4", "result.txt")) for f in range(6)}
    keep = prebuilt.fixture_tune_config(interference="replicate", occupancies=[4], include_default=False)
    res = tuner.tune(keep)
    for rep, members in enumerate(clusters):
        for f in members:
            assert res[f][4] == small_res[rep][4]
            assert os.path.getmtime(os.path.join(full, "output", f"f{f}", "o4", "result.txt")) == before[f]
    if shutil.which("hipcc") is None and not os.path.exists("/opt/rocm/bin/hipcc"):
        pytest.skip("the global stage builds the selected mix and needs hipcc")
    occ, sched = tuner.solve(res, keep)
    assert occ == 4 and len(sched) == 6
    # like features were given the same schedule
    assert all(sched[f][1] == sched[0][1] and type(sched[f][0]) is type(sched[0][0]) for f in (1, 2, 3))
    raw_batches = parse_raw_data_batches(tuner.basic.batch_sizes_fname, tuner.basic.data_fnames, 2,
                                         seed=3, feat_major=False)
    model = FeatProcessEmbed(RecomHost(), torch.device("cuda", 0), table_shapes=tuner.table_shapes,
                             librecom_path=os.path.join(full, "output", "optimal", "build", "librecom.so"))
    _check_text_model(model, tuner, raw_batches)
