"""GPU: the tuner's ablation modes (``tune_fixed_thread_binding``, ``mutation_validation``,
``tune_naive``; reference ``RecFlex/tuning/tuner.py:207-357``) and the fused embedding + MLP
model (``RecomModel``, ``examples/end_to_end.py``; reference ``RecFlex/rec_modules.py:143-179``,
``examples/end_to_end.py:43-51``) on the small model directory tests/golden/model_test, whose
kernels are built ahead of time."""

import importlib.util
import os

import numpy as np
import pytest

from helpers import ROOT, oracle

pytestmark = pytest.mark.gpu

MODEL_DIR = os.path.join(ROOT, "tests", "golden", "model_test")


def _fixture():
    from recflex_amd import prebuilt
    d = prebuilt.tune_fixture_dir()
    need = [os.path.join(d, "default", "build", "librecom.so"),
            os.path.join(d, "fixed_thread_binding_mean", "build", "librecom.so"),
            os.path.join(d, "naive", "f0", "s0", "build", "librecom.so"),
            os.path.join(d, f"mutation_f{prebuilt.ABLATION_MUTATED_FEATURE}", "m0", "build", "librecom.so")]
    for path in need:
        if not os.path.exists(path):
            raise RuntimeError(f"{path} is not built: run __graft_entry__.build() first")
    return d, prebuilt.make_fixture_tuner(MODEL_DIR)


def _integer_tables(tuner, dev):
    import torch
    g = torch.Generator(device=dev)
    g.manual_seed(4711)
    return [torch.randint(-8, 9, shape, generator=g, device=dev, dtype=torch.int32).float()
            for shape in tuner.table_shapes]


def _run_batches(lib_path, tuner, tables, dev, **launch):
    """Outputs of the library on every sampled batch of the fixture, as numpy arrays."""
    import torch
    from recflex_amd.rec_modules import FeatEmbed
    layer = FeatEmbed(dev, embed_tables=tables, librecom=lib_path)
    outs = []
    for k in range(len(tuner.batches[0])):
        d_idx = [torch.from_numpy(tuner.batches[f][k][0]).to(dev) for f in range(tuner.num_feats)]
        d_off = [torch.from_numpy(tuner.batches[f][k][1]).to(dev) for f in range(tuner.num_feats)]
        outs.append(layer.forward_indices(d_idx, d_off, **launch).cpu().numpy())
    return outs, layer


def _oracle_batches(tuner, tables):
    dims = [d for _, d in tuner.table_shapes]
    host_tables = [t.cpu().numpy() for t in tables]
    return [oracle.pooled_sum_c(host_tables, dims, tuner.data_types,
                                [tuner.batches[f][k][0] for f in range(tuner.num_feats)],
                                [tuner.batches[f][k][1] for f in range(tuner.num_feats)])
            for k in range(len(tuner.batches[0]))]


@pytest.mark.parametrize("choice", ["mean", "max"])
def test_fixed_thread_binding(choice):
    """The tile count per feature frozen at emit time (mean / max over the sampled batches of
    what the run-time binding chooses): a STATIC_BINDING library whose output has the bits of the
    run-time-bound one and of the oracle on integer-valued tables, a ``task_blocks.txt`` with one
    line per batch, and a positive kernel time."""
    import torch
    from recflex_amd import prebuilt
    from recflex_amd.librecom import RecomLib
    d, tuner = _fixture()
    dev = torch.device("cuda", 0)
    cfg = prebuilt.fixture_tune_config(tile_bytes=prebuilt.ABLATION_TILE_BYTES, remeasure=False)
    mix = prebuilt.fixture_default_mix(tuner)
    print(f"[case] fixed thread binding, choice={choice}", flush=True)
    fixed, t_ns = tuner.tune_fixed_thread_binding(mix, choice, cfg, occupancy=prebuilt.ABLATION_OCCUPANCY)
    assert len(fixed) == tuner.num_feats and all(b >= 1 for b in fixed) and t_ns > 0
    # the frozen counts are the mean / max of the per-batch lines (which the CPU wrote)
    lines = [list(map(int, ln.split(","))) for ln in
             open(os.path.join(d, f"fixed_thread_binding_{choice}", "task_blocks.txt")).read().split()]
    assert len(lines) == len(tuner.batches[0]) and all(len(ln) == tuner.num_feats for ln in lines)
    want_fixed = np.max(lines, axis=0) if choice == "max" else np.mean(lines, axis=0, dtype=np.int32)
    assert fixed == [max(1, int(b)) for b in want_fixed]
    assert max(fixed) > 1, "2 KiB tiles must give the multi-hot features several tiles"

    lib_path = os.path.join(d, f"fixed_thread_binding_{choice}", "build", "librecom.so")
    assert RecomLib(lib_path).info.static_binding == 1
    tables = _integer_tables(tuner, dev)
    frozen, _ = _run_batches(lib_path, tuner, tables, dev)
    bound, layer = _run_batches(os.path.join(d, "default", "build", "librecom.so"), tuner, tables, dev,
                                tile_bytes=prebuilt.ABLATION_TILE_BYTES)
    assert layer.lib.info.static_binding == 0
    for k, (a, b, w) in enumerate(zip(frozen, bound, _oracle_batches(tuner, tables))):
        assert a.shape == b.shape == w.shape
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), f"batch {k}: frozen != run-time bound"
        assert np.array_equal(a.view(np.uint32), w.view(np.uint32)), f"batch {k}: frozen != oracle"


def test_mutation_validation():
    """One whole-model kernel per candidate of the mutated feature: a finite, positive time for
    each, the index of the tuner's own pick among them, and every mutated library still computes
    the oracle's bits."""
    import torch
    from recflex_amd import prebuilt
    d, tuner = _fixture()
    dev = torch.device("cuda", 0)
    feat = prebuilt.ABLATION_MUTATED_FEATURE
    cfg = prebuilt.fixture_tune_config(tile_bytes=prebuilt.ABLATION_TILE_BYTES, remeasure=True)
    mix = prebuilt.fixture_default_mix(tuner)
    print(f"[case] mutation validation of feature {feat}", flush=True)
    times, opt_idx = tuner.mutation_validation(mix, prebuilt.ABLATION_OCCUPANCY, feat, cfg)
    n = len(tuner.feat_sched_param_candidates[feat])
    assert len(times) == n and all(np.isfinite(t) and t > 0 for t in times)
    assert 0 <= opt_idx < n and tuner.feat_sched_param_candidates[feat][opt_idx] is mix[feat]
    tables = _integer_tables(tuner, dev)
    want = _oracle_batches(tuner, tables)
    for k in range(n):
        got, _ = _run_batches(os.path.join(d, f"mutation_f{feat}", f"m{k}", "build", "librecom.so"),
                              tuner, tables, dev)
        for g, w in zip(got, want):
            assert np.array_equal(g.view(np.uint32), w.view(np.uint32)), f"mutation {k}"


def test_tune_naive():
    """Every candidate measured alone, the per-feature winners fused: one schedule per feature,
    each the argmin of that feature's ``result.txt`` files, and a library that passes parity."""
    import shutil
    import torch
    from recflex_amd import prebuilt
    d, tuner = _fixture()
    if shutil.which("hipcc") is None and not os.path.exists("/opt/rocm/bin/hipcc"):
        pytest.skip("the fused kernel of the winners is built after the measurements: needs hipcc")
    dev = torch.device("cuda", 0)
    cfg = prebuilt.fixture_tune_config(tile_bytes=prebuilt.ABLATION_TILE_BYTES, remeasure=True)
    print("[case] naive tuning (measures 192 single-feature kernels, builds 1 small kernel)", flush=True)
    sched, t_ns = tuner.tune_naive(cfg)
    assert len(sched) == tuner.num_feats and t_ns > 0
    for f in range(tuner.num_feats):
        times = [float(open(os.path.join(d, "naive", f"f{f}", f"s{k}", "result.txt")).read())
                 for k in range(len(tuner.feat_sched_param_candidates[f]))]
        assert all(np.isfinite(t) and t > 0 for t in times)
        assert sched[f] is tuner.feat_sched_param_candidates[f][int(np.argmin(times))]
    tables = _integer_tables(tuner, dev)
    got, _ = _run_batches(os.path.join(d, "naive", "optimal", "build", "librecom.so"), tuner, tables, dev)
    for g, w in zip(got, _oracle_batches(tuner, tables)):
        assert np.array_equal(g.view(np.uint32), w.view(np.uint32))


def test_recom_model_matches_torch_mlp_on_oracle_embedding():
    """``RecomModel`` = fused embedding, reshape to ``[-1, output_units]``, Linear + ReLU ...,
    Linear + Sigmoid.  With fixed weights its output equals the same MLP applied in fp32 on the
    CPU to the oracle's pooled output (1e-5); the layer list has the reference's shape."""
    import torch
    import torch.nn as nn
    from recflex_amd.parser import parse_raw_data_batches
    from recflex_amd.rec_modules import FeatPreprocess, RecomModel
    from recflex_amd.utils import find_file, import_from_path
    d, tuner = _fixture()
    dev = torch.device("cuda", 0)
    build_dir = os.path.join(d, "default", "build")
    recom_host = import_from_path("recom_host", find_file(build_dir, "recom_host*.so"))
    torch.manual_seed(99)
    tables = [torch.randn(shape, device=dev) * 0.01 for shape in tuner.table_shapes]
    mlp_units = [64, 16]
    print("[case] RecomModel with MLP", mlp_units, flush=True)
    model = RecomModel(mlp_units, dev, embed_tables=tables, librecom=f"{build_dir}/librecom.so")
    units = [model.embed_layer.output_units] + mlp_units + [1]
    kinds = [type(m) for m in model.mlp]
    assert kinds == [nn.Linear, nn.ReLU, nn.Linear, nn.ReLU, nn.Linear, nn.Sigmoid]
    linears = [m for m in model.mlp if isinstance(m, nn.Linear)]
    assert [(m.in_features, m.out_features) for m in linears] == list(zip(units[:-1], units[1:]))
    assert all(m.bias is not None and m.weight.device.type == "cuda" for m in linears)
    cpu_mlp = nn.Sequential(*[nn.Linear(i, o) for i, o in zip(units[:-1], units[1:])])
    for src, dst in zip(linears, cpu_mlp):
        dst.load_state_dict({k: v.detach().cpu() for k, v in src.state_dict().items()})

    preprocess = FeatPreprocess(recom_host, dev, output_units=model.embed_layer.output_units)
    raw_batches = parse_raw_data_batches(tuner.basic.batch_sizes_fname, tuner.basic.data_fnames, 3,
                                         seed=2, feat_major=False)
    dims = [dim for _, dim in tuner.table_shapes]
    host_tables = [t.cpu().numpy() for t in tables]
    for raw in raw_batches:
        with torch.no_grad():
            got = model(*preprocess(raw, model.embed_layer.max_concurrent_blocks))
        torch.cuda.synchronize()
        parsed = [oracle.parse_lines_python(lines) for lines in raw]
        pooled = oracle.pooled_sum_c(host_tables, dims, tuner.data_types,
                                     [p[0] for p in parsed], [p[1] for p in parsed])
        with torch.no_grad():
            x = torch.from_numpy(pooled)
            for i, lin in enumerate(cpu_mlp):
                x = lin(x)
                x = torch.sigmoid(x) if i + 1 == len(cpu_mlp) else torch.relu(x)
        assert got.shape == (len(raw[0]), 1) and got.dtype == torch.float32
        assert torch.allclose(got.cpu(), x, rtol=1e-5, atol=1e-6), float((got.cpu() - x).abs().max())
        assert float(got.min()) > 0.0 and float(got.max()) < 1.0


def test_end_to_end_measure_returns_a_positive_time():
    """``examples/end_to_end.py``'s ``measure``: host preprocess outside the timed region, the
    model per batch, accumulated milliseconds."""
    import torch
    from recflex_amd.parser import parse_raw_data_batches
    from recflex_amd.rec_modules import FeatPreprocess, RecomModel
    from recflex_amd.utils import find_file, import_from_path
    spec = importlib.util.spec_from_file_location("end_to_end_example",
                                                  os.path.join(ROOT, "examples", "end_to_end.py"))
    e2e = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(e2e)
    d, tuner = _fixture()
    dev = torch.device("cuda", 0)
    build_dir = os.path.join(d, "default", "build")
    recom_host = import_from_path("recom_host", find_file(build_dir, "recom_host*.so"))
    model = RecomModel([32], dev, table_shapes=tuner.table_shapes, librecom=f"{build_dir}/librecom.so")
    preprocess = FeatPreprocess(recom_host, dev, output_units=model.embed_layer.output_units)
    raw_batches = parse_raw_data_batches(tuner.basic.batch_sizes_fname, tuner.basic.data_fnames, 4,
                                         seed=0, feat_major=False)
    print("[case] end_to_end.measure over", len(raw_batches), "batches", flush=True)
    t_ms = e2e.measure(preprocess, model, model.embed_layer.max_concurrent_blocks, raw_batches)
    assert np.isfinite(t_ms) and t_ms > 0


def test_frozen_binding_example_gives_the_bits_of_the_run_time_binding(capsys):
    """``examples/ablation_fixed_binding.py`` on C3 at full size: the library whose tile counts
    were frozen for the benchmark batch and the run-time-bound one give identical bits on that
    batch, on shorter batches and on batches with longer bags; every time is positive."""
    import json
    import sys
    from recflex_amd import prebuilt
    for name in ("c3_tuned", "c3_tuned_static"):
        if not os.path.exists(prebuilt.lib_path(name)):
            raise RuntimeError(f"{name} is not built: run __graft_entry__.build() first")
    spec = importlib.util.spec_from_file_location(
        "ablation_fixed_binding", os.path.join(ROOT, "examples", "ablation_fixed_binding.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    print("[case] examples/ablation_fixed_binding.py --workload c3 --steps 3", flush=True)
    argv = sys.argv
    sys.argv = ["ablation_fixed_binding.py", "--workload", "c3", "--steps", "3"]
    try:
        mod.main()
    finally:
        sys.argv = argv
    summary = json.loads(capsys.readouterr().out.strip().splitlines()[-1])
    assert len(summary["cases"]) >= 8
    for case in summary["cases"]:
        assert case["identical_bits"], case["batch"]
        assert case["run_time_binding_us"] > 0 and case["frozen_binding_us"] > 0
