"""Named, reproducible models (workload + per-feature schedules) whose fused-kernel libraries
are built ahead of time, in-tree, under ``recflex_amd/_models/<name>/build/``.

GPU machines only load what is already built here; ``ensure_built`` compiles a model only if
its library is missing.  Names:

``c1`` .. ``c5``     the five benchmark configurations at full size, default (untuned) schedules
``cN_tuned``       CN with the schedules, occupancy and launch parameters recorded in
                   ``recflex_amd/tuned/cN_schedule.json`` (written by ``examples/tune.py``); the
                   default build if that file is absent
``cN_tuned_ticks`` c2_tuned / c3_tuned as timing builds (tick counters at kernel entry, after the
                   binding and at the end of each workgroup): ``bench.py`` reads the binding's
                   share of a workgroup's time from them
``c3_tuned_static`` c3_tuned with the tiles per feature frozen at emit time to what the run-time
                   binding chooses for the benchmark batch (the reference's fixed-thread-binding
                   ablation, ``examples/ablation_fixed_binding.py``)
``c1_o2``, ``c1_o5`` C1 built for 2 and 5 workgroups per CU (its light kernel reaches 8 by
                   itself, so the dynamic-LDS pad has to hold the others off)
``c3_flat``        C3 with the flat tile walk instead of the XCD-segmented one (for comparison)
``c2s`` .. ``c5s``   shrunken C2..C5 (fewer rows / features / samples) that a CPU checker can follow
``variants``       one feature per (element type, dim, schedule candidate) over a spread of the
                   candidate space of all four templates, with ragged bags (up to ~1500 lookups)
                   and integer-valued tables, so that sums are exact in any order
``edge``           dims that force 8- and 4-byte row vectors and unaligned output columns
``onehots``        the row-copy template at a spread of its candidates for fp32, fp16 and int8
                   rows, integer-valued tables
``longbags``       a dozen samples with bags of thousands of lookups (and some short and empty
                   ones) under the split-bag schedule: several workgroups per bag
``c3s_bind_once``  c3s bound once per launch by the binding kernel (``bind_once=True``), although
                   small enough for the per-workgroup binding
``c3s_outliers``   c3s with integer-valued tables, emitted with ``outliers=True``: bags beyond a
                   schedule's threshold are found ahead of the kernel and run as tiles of their
                   own; every tenth feature under the split-bag schedule
``c4s_outliers``, ``c5s_outliers``  c4s (fp16) and c5s (int8) with integer-valued tables and
                   outlier tiles
``c3_skew``        C3 with bag lengths from a lognormal (sigma 1.5) of the same means and
                   integer-valued tables, default schedules, emitted with outlier tiles;
                   ``c3_skew_plain``: the same without them
``fewbags``        8 fp32 features x 16 samples x 20 000 lookups, default schedules (split-bag);
                   ``fewbags_unsplit``: the same with one workgroup per bag, for comparison;
                   ``fewbags64`` / ``fewbags128`` / ``fewbags512``: the same lookups as 64 x 4 000,
                   128 x 2 500 and 512 x 1 000
``manysplit``      17 fp16 features of dim 256 under the split-bag schedule: 36 MB of workspace,
                   more than the static array of ``recom_process_static_workspace`` may hold
``refa``, ``reff4`` models shaped like the reference's example models A and a quarter of F (1 000 and
                   2 500 small features, batch 256; ``workloads.REF_SHAPED``), default schedules;
                   ``refa_tuned`` / ``reff4_tuned``: with ``tuned/refa_schedule.json`` /
                   ``tuned/reff4_schedule.json`` if that file exists
``wide``           1 500 small features (several binding rounds per thread)
``wider``          2 500 small features (bound once per launch by the binding kernel)
``widest``         4 500 small features (more than 64 chunks of 64 features: the prefix sum's second
                   level and the feature search walk their first level in two rounds)
"""

import json
import os
from typing import Callable, Dict, List, NamedTuple, Optional

import numpy as np

from .code_emitter import MetaData
from .model_build import FeatSchedules, build_model, default_feat_schedules, feat_schedules_from_entries
from .schedules import (BlockPerBagSchedule, SplitBagSchedule, SubWavefrontPerBagSchedule,
                        ThreadPerBagSchedule, WavefrontPerBagSchedule)
from .workloads import FeatureSpec, Workload, make_workload

PACKAGE_DIR = os.path.dirname(os.path.abspath(__file__))
MODELS_DIR = os.path.join(PACKAGE_DIR, "_models")
TUNED_DIR = os.path.join(PACKAGE_DIR, "tuned")
BLOCK_THREADS = 256


class ModelSpec(NamedTuple):
    workload: Workload
    feat_schedules: FeatSchedules
    occupancy: Optional[int]
    emit_kwargs: dict = {}


def metas_of(wl: Workload) -> List[MetaData]:
    return [MetaData(f.dim, f.data_type) for f in wl.features]


def expected_bag_len(f: FeatureSpec) -> float:
    return f.mean_bag * (1.0 - f.empty_frac)


# workgroups per CU the untuned models are built for (128 vector registers per lane)
DEFAULT_OCCUPANCY = 4


def is_one_hot(f: FeatureSpec) -> bool:
    return f.fixed_len and round(f.mean_bag) <= 1


def _default(wl: Workload, occupancy: Optional[int] = DEFAULT_OCCUPANCY, **emit_kwargs) -> ModelSpec:
    fs = default_feat_schedules(metas_of(wl), [expected_bag_len(f) for f in wl.features], BLOCK_THREADS,
                                one_hot=[is_one_hot(f) for f in wl.features])
    return ModelSpec(wl, fs, occupancy, emit_kwargs)


def _tuned(wl: Workload, fname: str) -> ModelSpec:
    path = os.path.join(TUNED_DIR, fname)
    if not os.path.exists(path):
        return _default(wl)
    with open(path) as f:
        doc = json.load(f)
    entries = doc["schedules"] if isinstance(doc, dict) else doc
    occupancy = doc.get("occupancy") if isinstance(doc, dict) else None
    fs = feat_schedules_from_entries(entries, BLOCK_THREADS)
    assert len(fs) == wl.num_features
    kwargs = {}
    if isinstance(doc, dict) and doc.get("tile_bytes"):
        kwargs["tile_bytes"] = doc["tile_bytes"]
    if isinstance(doc, dict) and doc.get("xcd_segments", 0) > 0:
        kwargs.update(xcd_aware=True, xcd_segments=doc["xcd_segments"])
    else:
        kwargs.update(xcd_aware=False)      # the tuned walk is the flat one
    if isinstance(doc, dict) and doc.get("tile_order"):
        kwargs["tile_order"] = [int(f) for f in doc["tile_order"]]
    if isinstance(doc, dict) and doc.get("drawn_tail"):
        kwargs["drawn_tail"] = int(doc["drawn_tail"])
    if isinstance(doc, dict) and doc.get("outliers"):
        kwargs["outliers"] = True
    return ModelSpec(wl, fs, occupancy, kwargs)


def _frozen_binding(spec: ModelSpec) -> ModelSpec:
    """The model with the tiles per feature frozen at emit time to what the run-time binding
    chooses for the workload's own (seeded) batch: the fixed-thread-binding ablation."""
    from .code_emitter.codegen import BAG_FIXED_BYTES, DEFAULT_TILE_BYTES, INDEX_BYTES
    from .tuning.measure import tiles_per_feature
    from .workloads import gen_inputs
    _, offsets = gen_inputs(spec.workload)
    metas = [s.meta for s, _ in spec.feat_schedules]
    counts = tiles_per_feature(offsets, [m.row_bytes + INDEX_BYTES for m in metas],
                               [m.embed_dim * 4 + BAG_FIXED_BYTES for m in metas],
                               [s.TileGranularity(p) for s, p in spec.feat_schedules],
                               spec.emit_kwargs.get("tile_bytes") or DEFAULT_TILE_BYTES,
                               grid_blocks=TUNE_FIXTURE_SM_COUNT * (spec.occupancy or DEFAULT_OCCUPANCY))
    return spec._replace(emit_kwargs=dict(_plain_walk(spec.emit_kwargs),
                                          fixed_task_block_nums=[max(1, c) for c in counts]))


def _plain_walk(emit_kwargs: dict) -> dict:
    """The emit options without a tile order and a drawn end, which go with neither tick
    counters nor a frozen binding nor outlier tiles."""
    return {k: v for k, v in emit_kwargs.items() if k not in ("tile_order", "drawn_tail")}


def _with_ticks(spec: ModelSpec) -> ModelSpec:
    return spec._replace(emit_kwargs=dict(_plain_walk(spec.emit_kwargs), timing=True))


def _variants() -> ModelSpec:
    """A spread of every template's candidate list for each (element type, dim)."""
    rng = np.random.default_rng(77)
    feats: List[FeatureSpec] = []
    scheds: FeatSchedules = []
    combos = [("float", 8), ("float", 32), ("float", 128), ("float", 256),
              ("half", 16), ("half", 64), ("half", 256),
              ("int8", 16), ("int8", 64), ("int8", 128)]
    for data_type, dim in combos:
        meta = MetaData(dim, data_type)
        for cls, take in ((ThreadPerBagSchedule, 3), (SubWavefrontPerBagSchedule, 8),
                          (WavefrontPerBagSchedule, 4), (BlockPerBagSchedule, 2)):
            sched = cls(meta, BLOCK_THREADS)
            cands = sched.GenParamCandidates()
            if not cands:
                continue
            picks = sorted(set(int(i) for i in np.linspace(0, len(cands) - 1, min(take, len(cands)))))
            for i in picks:
                mean = float(rng.choice([0.7, 3.0, 17.0, 90.0]))
                if cls is BlockPerBagSchedule:
                    mean = float(rng.choice([40.0, 1500.0]))     # > one LDS chunk of indices
                feats.append(FeatureSpec(int(rng.integers(50, 5000)), dim, data_type, mean, False,
                                         0.1, 1.0))
                scheds.append((sched, cands[i]))
    return ModelSpec(Workload("variants", 96, 4242, tuple(feats), "integer"), scheds, DEFAULT_OCCUPANCY)


def _edge() -> ModelSpec:
    dims = [("float", 1), ("float", 2), ("float", 6), ("float", 12), ("float", 20), ("half", 2),
            ("half", 4), ("half", 12), ("int8", 4), ("int8", 8), ("int8", 24), ("float", 3)]
    feats = [FeatureSpec(300 + 7 * i, d, t, 5.0, False, 0.2, 0.9) for i, (t, d) in enumerate(dims)]
    wl = Workload("edge", 70, 99, tuple(feats), "integer")
    fs = default_feat_schedules(metas_of(wl), [4.0] * len(feats), BLOCK_THREADS)
    return ModelSpec(wl, fs, None)      # no occupancy: natural register use, no LDS pad


def _other_block_size(block_threads: int) -> ModelSpec:
    """Every element type and template at a workgroup size other than 256 (``tune.py -b``)."""
    combos = [("float", 8, 3.0), ("float", 32, 40.0), ("float", 128, 1.0), ("half", 64, 25.0),
              ("half", 256, 2.0), ("int8", 32, 9.0), ("int8", 128, 60.0), ("float", 64, 900.0)]
    feats = [FeatureSpec(400 + 31 * i, d, t, m, False, 0.1, 1.0) for i, (t, d, m) in enumerate(combos)]
    wl = Workload(f"b{block_threads}", 150, 515 + block_threads, tuple(feats), "integer")
    fs = default_feat_schedules(metas_of(wl), [expected_bag_len(f) for f in feats], block_threads)
    # the default rules pick sub-wavefront teams throughout: put the other templates in by hand
    for f, cls in ((0, ThreadPerBagSchedule), (1, WavefrontPerBagSchedule), (3, WavefrontPerBagSchedule),
                   (len(feats) - 1, BlockPerBagSchedule)):
        sched = cls(MetaData(feats[f].dim, feats[f].data_type), block_threads)
        fs[f] = (sched, sched.GenParamCandidates()[0])
    return ModelSpec(wl, fs, None)


def _onehots() -> ModelSpec:
    """The row-copy template (``OneHotBagSchedule``) for every element type at a spread of its
    (column lanes, bags per team) candidates.  The workload itself holds exactly one lookup per
    bag; the tests also feed the library empty bags, bags of many lookups and batches that have
    as many lookups as bags without having one per bag."""
    from .schedules import OneHotBagSchedule
    feats: List[FeatureSpec] = []
    scheds: FeatSchedules = []
    for i, (data_type, dim) in enumerate([("float", 64), ("float", 8), ("float", 128), ("half", 32),
                                          ("half", 128), ("int8", 64), ("int8", 128)]):
        sched = OneHotBagSchedule(MetaData(dim, data_type), BLOCK_THREADS)
        cands = sched.GenParamCandidates()
        for k in sorted(set(int(j) for j in np.linspace(0, len(cands) - 1, min(4, len(cands))))):
            feats.append(FeatureSpec(700 + 53 * len(feats), dim, data_type, 1.0, True, 0.0, 1.0))
            scheds.append((sched, cands[k]))
    return ModelSpec(Workload("onehots", 333, 909, tuple(feats), "integer"), scheds, DEFAULT_OCCUPANCY)


def _long_bags() -> ModelSpec:
    """Few, very long bags: every bag of the long features is summed by several workgroups
    (``SplitBagSchedule``); the last two features have short bags and stay unsplit."""
    combos = [("float", 128, 6000.0), ("float", 64, 2500.0), ("half", 256, 4000.0),
              ("int8", 128, 5000.0), ("float", 16, 3000.0), ("half", 32, 9000.0),
              ("int8", 64, 1200.0), ("float", 32, 5.0), ("half", 64, 40.0)]
    feats = [FeatureSpec(2000 + 97 * i, d, t, m, False, 0.15, 1.0) for i, (t, d, m) in enumerate(combos)]
    wl = Workload("longbags", 12, 31337, tuple(feats), "integer")
    scheds: FeatSchedules = []
    for i, f in enumerate(feats):
        sched = SplitBagSchedule(MetaData(f.dim, f.data_type), BLOCK_THREADS)
        cands = sched.GenParamCandidates()
        scheds.append((sched, cands[(3 * i) % len(cands)]))
    return ModelSpec(wl, scheds, DEFAULT_OCCUPANCY)


def _c3s_outliers() -> ModelSpec:
    """c3s with integer-valued tables and outlier tiles; every tenth feature runs the split-bag
    schedule, so that the library's workspace holds split regions and the outlier list."""
    wl = make_workload("C3", batch=192, max_rows=60_000)._replace(name="c3s_outliers",
                                                                   table_values="integer")
    spec = _default(wl, outliers=True)
    fs = list(spec.feat_schedules)
    for f in range(0, len(fs), 10):
        sched = SplitBagSchedule(fs[f][0].meta, BLOCK_THREADS)
        fs[f] = (sched, sched.GenParamCandidates()[0])
    return spec._replace(feat_schedules=fs)


def _c3_skew(outliers: bool) -> ModelSpec:
    """Heavy-tailed bag lengths: some thousand bags per batch far beyond their schedule."""
    wl = make_workload("C3")
    wl = wl._replace(name="c3_skew", table_values="integer",
                     features=tuple(f._replace(len_sigma=1.5) for f in wl.features))
    # the schedules and launch parameters tuned for C3 (the same features; only the bag lengths
    # differ): 167 against 171 us for the default mix at five workgroups per CU, 181 at four
    spec = _tuned(wl, "c3_schedule.json")
    return spec._replace(emit_kwargs=dict(_plain_walk(spec.emit_kwargs), outliers=outliers))


def _few_bags(split: bool, bags: int = 16, lookups: float = 20000.0) -> ModelSpec:
    """Fewer bags than the device has workgroups, each of ``lookups`` lookups (16 x 20 000 by
    default; 64 x 4 000, 128 x 2 500 and 512 x 1 000 are the same eight features with the same
    2.5 M lookups cut into more, shorter bags)."""
    feats = tuple(FeatureSpec(2_000_000, d, "float", lookups, False, 0.0, 1.0)
                  for d in (32, 64, 128, 64, 32, 128, 64, 64))
    wl = Workload("fewbags", bags, 77, feats, "integer")
    fs = default_feat_schedules(metas_of(wl), [f.mean_bag for f in feats], BLOCK_THREADS)
    assert all(isinstance(s, SplitBagSchedule) for s, _ in fs)
    if not split:
        fs = [(BlockPerBagSchedule(s.meta, BLOCK_THREADS), p) for s, p in fs]
    # 20 vector registers and 6.5 KB of LDS: eight workgroups per CU cover each other's waits
    # for index chunks, partial sums and arrival counters (177 -> 156 us at four)
    return ModelSpec(wl, fs, 8)


def _many_split() -> ModelSpec:
    """More split-bag workspace than a library's static device array may hold (32 MiB)."""
    feats = tuple(FeatureSpec(5000 + f, 256, "half", 3000.0, False, 0.0, 1.0) for f in range(17))
    wl = Workload("manysplit", 8, 1717, feats, "integer")
    sched = SplitBagSchedule(MetaData(256, "half"), BLOCK_THREADS)
    params = sched.GenParamCandidates()[0]
    return ModelSpec(wl, [(sched, params)] * len(feats), DEFAULT_OCCUPANCY)


def _wide(num_features: int = 1500, name: str = "wide") -> ModelSpec:
    """Many small features: several rounds of the binding loop per thread and a prefix array
    longer than a wavefront scan covers at once, as in the reference's own models.  Above
    ``codegen.BIND_ONCE_MIN_FEATS`` features the binding is computed once per launch by a kernel
    of its own (``wider``)."""
    rng = np.random.default_rng(num_features)
    feats = []
    for i in range(num_features):
        dim = int(rng.choice([4, 8, 16, 32, 64]))
        mean = float(rng.choice([1.0, 1.0, 3.0, 12.0, 40.0]))
        feats.append(FeatureSpec(int(rng.integers(64, 512)), dim, "float", mean, mean == 1.0,
                                 0.0 if mean == 1.0 else 0.3, 1.05))
    wl = Workload(name, 40, num_features, tuple(feats), "integer")
    # (2 500 features would fit the per-workgroup binding; ``wider`` is there for the other one)
    return _default(wl, bind_once=True) if num_features > 2048 else _default(wl)


def _ordered(spec: ModelSpec, name: str, seed: int, drawn_tail: int = 0, **emit_kwargs) -> ModelSpec:
    """The same model and schedules with the features laid out in the kernel's tile space in a
    random order (``tile_order``) and, if asked for, the last passes of the tile walk drawn."""
    order = [int(f) for f in np.random.default_rng(seed).permutation(len(spec.feat_schedules))]
    kwargs = dict(spec.emit_kwargs, tile_order=order, **emit_kwargs)
    if drawn_tail:
        kwargs["drawn_tail"] = drawn_tail
    return spec._replace(workload=spec.workload._replace(name=name), emit_kwargs=kwargs)


def _c3s_ordered() -> ModelSpec:
    """c3s_outliers' model (integer tables, every tenth feature split) without outlier tiles, in
    a random tile order with the last two passes drawn."""
    spec = _c3s_outliers()
    spec = spec._replace(emit_kwargs={k: v for k, v in spec.emit_kwargs.items() if k != "outliers"})
    return _ordered(spec, "c3s_ordered", 11, drawn_tail=2)


def _drawn_all(spec: ModelSpec, name: str, **emit_kwargs) -> ModelSpec:
    """The same model and schedules with every tile of the walk drawn from the ticket counters."""
    from .code_emitter.codegen import DRAWN_ALL
    kwargs = {k: v for k, v in spec.emit_kwargs.items() if k != "outliers"}
    kwargs.update(drawn_tail=DRAWN_ALL, **emit_kwargs)
    return spec._replace(workload=spec.workload._replace(name=name), emit_kwargs=kwargs)


_SPECS: Dict[str, Callable[[], ModelSpec]] = {
    "c1": lambda: _default(make_workload("C1")),
    "c2": lambda: _default(make_workload("C2")),
    "c3": lambda: _default(make_workload("C3")),
    "c4": lambda: _default(make_workload("C4")),
    "c5": lambda: _default(make_workload("C5")),
    "c2_tuned": lambda: _tuned(make_workload("C2"), "c2_schedule.json"),
    "c3_tuned": lambda: _tuned(make_workload("C3"), "c3_schedule.json"),
    "c4_tuned": lambda: _tuned(make_workload("C4"), "c4_schedule.json"),
    "c5_tuned": lambda: _tuned(make_workload("C5"), "c5_schedule.json"),
    # c2_tuned / c3_tuned with the tick counters of a timing build: the share of a workgroup's
    # time that passes before its first tile (the binding), reported by bench.py
    "c2_tuned_ticks": lambda: _with_ticks(_tuned(make_workload("C2"), "c2_schedule.json")),
    "c3_tuned_ticks": lambda: _with_ticks(_tuned(make_workload("C3"), "c3_schedule.json")),
    # c3_tuned with its binding frozen for the benchmark batch (examples/ablation_fixed_binding.py)
    "c3_tuned_static": lambda: _frozen_binding(_tuned(make_workload("C3"), "c3_schedule.json")),
    "c1_o2": lambda: _default(make_workload("C1"), occupancy=2),
    "c1_o5": lambda: _default(make_workload("C1"), occupancy=5),
    "c3_flat": lambda: _default(make_workload("C3"), xcd_aware=False),
    "c2s": lambda: _default(make_workload("C2", batch=512, max_rows=200_000)),
    "c3s": lambda: _default(make_workload("C3", batch=192, max_rows=60_000)),
    "c4s": lambda: _default(make_workload("C4", batch=128, num_features=48, max_rows=30_000)),
    "c5s": lambda: _default(make_workload("C5", batch=256, num_features=24, max_rows=50_000)),
    # a model of fewer features than the binding keeps addresses for in LDS, bound once per launch
    # by the binding kernel all the same (an emit option)
    "c3s_bind_once": lambda: _default(make_workload("C3", batch=192, max_rows=60_000), bind_once=True),
    "c3s_outliers": _c3s_outliers,
    # tile orders: features in a random order in the tile space (addresses kept in LDS / read per
    # tile / bound once per launch; with split regions, with outlier tiles), drawn ends
    "c3s_ordered": _c3s_ordered,
    "c3s_outliers_ordered": lambda: _ordered(_c3s_outliers(), "c3s_outliers_ordered", 12),
    "wide_ordered": lambda: _ordered(_wide(), "wide_ordered", 13, drawn_tail=1),
    "wider_ordered": lambda: _ordered(_wide(2500, "wider"), "wider_ordered", 14, drawn_tail=3),
    "onehots_ordered": lambda: _ordered(_onehots(), "onehots_ordered", 15, drawn_tail=8),
    "c3s_drawn_all": lambda: _drawn_all(_c3s_outliers(), "c3s_drawn_all"),
    "wide_drawn_all_flat": lambda: _drawn_all(_wide(), "wide_drawn_all_flat", xcd_aware=False),
    # fp16 and int8 tables with outlier tiles (integer-valued: sums exact)
    "c4s_outliers": lambda: _default(make_workload("C4", batch=128, num_features=48, max_rows=30_000)
                                     ._replace(name="c4s_outliers", table_values="integer"), outliers=True),
    "c5s_outliers": lambda: _default(make_workload("C5", batch=256, num_features=24, max_rows=50_000)
                                     ._replace(name="c5s_outliers", table_values="integer"), outliers=True),
    "variants": _variants,
    "edge": _edge,
    "onehots": _onehots,
    "longbags": _long_bags,
    "c3_skew": lambda: _c3_skew(True),
    "c3_skew_plain": lambda: _c3_skew(False),
    "fewbags": lambda: _few_bags(True),
    "fewbags_unsplit": lambda: _few_bags(False),
    "fewbags64": lambda: _few_bags(True, 64, 4000.0),
    "fewbags128": lambda: _few_bags(True, 128, 2500.0),
    "fewbags512": lambda: _few_bags(True, 512, 1000.0),
    "manysplit": _many_split,
    "wide": _wide,
    "wider": lambda: _wide(2500, "wider"),
    "widest": lambda: _wide(4500, "widest"),
    # models shaped like the reference's own examples (workloads.REF_SHAPED), default schedules
    "refa": lambda: _default(make_workload("REFA")),
    "reff4": lambda: _default(make_workload("REFF4")),
    "refa_tuned": lambda: _tuned(make_workload("REFA"), "refa_schedule.json"),
    "reff4_tuned": lambda: _tuned(make_workload("REFF4"), "reff4_schedule.json"),
    "b128": lambda: _other_block_size(128),
    "b512": lambda: _other_block_size(512),
}


def model_names() -> List[str]:
    return list(_SPECS)


def model_spec(name: str) -> ModelSpec:
    if name not in _SPECS:
        raise KeyError(f"unknown prebuilt model {name!r}; known: {model_names()}")
    return _SPECS[name]()


def model_dir(name: str) -> str:
    return os.path.join(MODELS_DIR, name)


def lib_path(name: str) -> str:
    return os.path.join(model_dir(name), "build", "librecom.so")


def build(name: str) -> str:
    spec = model_spec(name)
    return build_model(model_dir(name), spec.feat_schedules, rebuild=True, occupancy=spec.occupancy,
                       **spec.emit_kwargs)


def ensure_built(name: str) -> str:
    path = lib_path(name)
    return path if os.path.exists(path) else build(name)


def build_all(names: Optional[List[str]] = None) -> Dict[str, str]:
    return {name: build(name) for name in (names or model_names())}


# ------------------------------------------------------------------------------------------------
# a model directory in the text formats (table_config / schedule_config / data/), built ahead of
# time the way tune.py and test.py would: local-stage tuning kernels and a default-schedule model
# ------------------------------------------------------------------------------------------------

TUNE_FIXTURE_OCCUPANCIES = [2, 4]
TUNE_FIXTURE_SM_COUNT = 256          # compute units of an MI355X


def tune_fixture_dir() -> str:
    return os.path.join(MODELS_DIR, "tune_fixture")


def make_fixture_tuner(model_dir: str, sample_batch_nums: int = 4, codegen_dir: str = None):
    from .schedules import SCHEDULE_MAPPING
    from .tuning import BasicConfig, Tuner
    from .utils import get_data_fnames
    data_dir = os.path.join(model_dir, "data")
    cfg = BasicConfig(batch_sizes_fname=os.path.join(data_dir, "batch_sizes.txt"),
                      data_fnames=get_data_fnames(data_dir),
                      schedule_config_fname=os.path.join(model_dir, "schedule_config.txt"),
                      table_config_fname=os.path.join(model_dir, "table_config.txt"),
                      codegen_dir=codegen_dir or tune_fixture_dir(), block_threads=BLOCK_THREADS,
                      sample_batch_nums=sample_batch_nums)
    return Tuner(cfg, SCHEDULE_MAPPING)


def fixture_tune_config(**overrides):
    from .tuning import TuneConfig
    kwargs = dict(occupancies=TUNE_FIXTURE_OCCUPANCIES, gpu_ids=[0], sm_count=TUNE_FIXTURE_SM_COUNT,
                  num_processes=4, profiler="events", in_process=True, cluster_stage=False)
    kwargs.update(overrides)
    return TuneConfig(**kwargs)


# the ablation modes of the fixture: tiles of 2 KiB, so that its small features still get several
# tiles each and a frozen binding differs from one tile per feature
ABLATION_TILE_BYTES = 2048
ABLATION_OCCUPANCY = 4
ABLATION_MUTATED_FEATURE = 0


def fixture_default_mix(tuner) -> list:
    """The default schedule of every feature, as entries of the tuner's candidate lists."""
    return [tuner.feat_sched_param_candidates[f][k] for f, k in enumerate(tuner.default_choices()[0])]


def build_tune_fixture(model_dir: str) -> str:
    """Local-stage kernels of the fixture model, ``default/`` (default schedules, with the
    generated host front end) and the kernels of the tuner's ablation modes (one per candidate
    of ``tune_naive``, the mutations of one feature, the two frozen bindings), all under
    ``_models/tune_fixture``: a GPU machine then only measures."""
    import multiprocessing as mp
    if mp.get_start_method(allow_none=True) != "spawn":
        mp.set_start_method("spawn", force=True)
    tuner = make_fixture_tuner(model_dir)
    tuner.compile_local(fixture_tune_config(recompile=True, interference="replicate", occupancies=[4]))
    tuner.compile_tournament(fixture_tune_config(recompile=True, interference="model"))
    mean_lens = [float(np.mean([len(i) / max(1, len(o) - 1) for i, o in feat])) for feat in tuner.batches]
    fs = default_feat_schedules(tuner.metas, mean_lens, BLOCK_THREADS)
    build_model(os.path.join(tune_fixture_dir(), "default"), fs, rebuild=True, occupancy=None)
    ablation = fixture_tune_config(recompile=True, tile_bytes=ABLATION_TILE_BYTES)
    tuner.compile_naive(ablation)
    mix = fixture_default_mix(tuner)
    tuner.compile_mutation(mix, ABLATION_OCCUPANCY, ABLATION_MUTATED_FEATURE, ablation)
    for choice in ("mean", "max"):
        tuner.compile_fixed_thread_binding(mix, choice, ablation._replace(remeasure=True),
                                           occupancy=ABLATION_OCCUPANCY)
    return tune_fixture_dir()


# ------------------------------------------------------------------------------------------------
# the global stage under rocprofv3: a 100-feature model whose fused kernel runs tens of
# microseconds (C3 at half its batch, tables capped at 200 000 rows), default schedules, built
# for two occupancies
# ------------------------------------------------------------------------------------------------

ROCPROF_FIXTURE_OCCUPANCIES = [2, 5]


def rocprof_fixture_dir() -> str:
    return os.path.join(MODELS_DIR, "tune_rocprof")


def make_rocprof_tuner():
    """Tuner over one seeded batch of the shrunken C3 (the arrays are regenerated from the seed
    wherever this runs, and written to ``tune_rocprof/data`` for the profiled program)."""
    from .schedules import SCHEDULE_MAPPING
    from .tuning import BasicConfig, Tuner
    from .workloads import gen_inputs
    wl = make_workload("C3", batch=1024, max_rows=200_000)
    indices, offsets = gen_inputs(wl._replace(seed=wl.seed + 7919))
    cfg = BasicConfig(batch_sizes_fname="", data_fnames=[], schedule_config_fname="",
                      table_config_fname="", codegen_dir=rocprof_fixture_dir(),
                      block_threads=BLOCK_THREADS, sample_batch_nums=1)
    templates = [ThreadPerBagSchedule, SubWavefrontPerBagSchedule, WavefrontPerBagSchedule,
                 BlockPerBagSchedule]
    return Tuner(cfg, SCHEDULE_MAPPING, batches=[[(i, o)] for i, o in zip(indices, offsets)],
                 table_shapes=[(f.rows, f.dim) for f in wl.features],
                 data_types=[f.data_type for f in wl.features],
                 schedule_types=[templates for _ in wl.features])


def rocprof_tune_config(**overrides):
    return fixture_tune_config(occupancies=ROCPROF_FIXTURE_OCCUPANCIES, include_default=False,
                               tile_bytes=0, **overrides)


# what the walk stage is run with on this fixture: (occupancy, tile_bytes, xcd_segments)
ROCPROF_FIXTURE_WALK = (5, 0, 16)


def build_rocprof_fixture() -> str:
    """``tune_rocprof/all/o{2,5}``: the default mix as whole-model kernels, what
    ``Tuner.tune_occupancy`` measures; ``tune_rocprof/walk_*/o5``: the same mix as it is and
    with 2 / 4 / 8 / all passes of its tile walk drawn, what ``Tuner.decide_walk`` times."""
    import multiprocessing as mp
    if mp.get_start_method(allow_none=True) != "spawn":
        mp.set_start_method("spawn", force=True)
    tuner = make_rocprof_tuner()
    cfg = rocprof_tune_config(recompile=True)
    mix = fixture_default_mix(tuner)
    jobs = []
    for occupancy in cfg.occupancies:
        output_dir, build_dir = tuner.get_output_build_dir(-1, occupancy)
        if tuner._build_full(output_dir, mix, occupancy, cfg):
            jobs.append((output_dir, build_dir))
    tuner._schedule_builds(jobs, cfg)
    occupancy, tile_bytes, xcd_segments = ROCPROF_FIXTURE_WALK
    variants = dict({"as_is": (None, 0)}, **tuner._drawn_variants(cfg))
    tuner._build_walk_variants(variants, mix, occupancy, tile_bytes, xcd_segments, False, cfg)
    return rocprof_fixture_dir()


# ------------------------------------------------------------------------------------------------
# the compressed-model flow (examples/run_model.sh): one representative per cluster of like
# features is tuned, the results are spread back over the full model
# ------------------------------------------------------------------------------------------------

def compress_fixture_dir() -> str:
    return os.path.join(MODELS_DIR, "tune_compress")


def build_compress_fixture(model_dir: str) -> str:
    """``tune_compress/src``: the fixture model; ``tune_compress/model``: the same compressed by
    ``examples/compress.py`` (its four like one-hot features become one), with the
    reference-style local-stage kernels of its representatives built under
    ``tune_compress/model/output``."""
    import multiprocessing as mp
    import shutil
    import subprocess
    import sys
    if mp.get_start_method(allow_none=True) != "spawn":
        mp.set_start_method("spawn", force=True)
    root = compress_fixture_dir()
    shutil.rmtree(root, ignore_errors=True)
    # the fixture model with its like features described by one data_config line (features are
    # clustered within a line): ``one-hot,1,c`` four times becomes ``one-hot,4,c``
    src = os.path.join(root, "src")
    shutil.copytree(model_dir, src)
    merged: List[List[str]] = []
    with open(os.path.join(model_dir, "data_config.txt")) as f:
        for line in f:
            fields = line.strip().split(",")
            if len(fields) < 3:
                continue
            if merged and merged[-1][0] == fields[0] and merged[-1][2:] == fields[2:]:
                merged[-1][1] = str(int(merged[-1][1]) + int(fields[1]))
            else:
                merged.append(fields)
    with open(os.path.join(src, "data_config.txt"), "w") as f:
        f.writelines(",".join(fields) + "\n" for fields in merged)
    small = os.path.join(root, "model")
    script = os.path.join(os.path.dirname(PACKAGE_DIR), "examples", "compress.py")
    subprocess.run([sys.executable, script, "-m", src, "-o", small], check=True,
                   stdout=subprocess.DEVNULL)
    tuner = make_fixture_tuner(small, codegen_dir=os.path.join(small, "output"))
    tuner.compile_local(fixture_tune_config(recompile=True, interference="replicate", occupancies=[4]))
    return root


# ------------------------------------------------------------------------------------------------
# the two command-line entry points run end to end (examples/tune.py -m ..., then
# examples/test.py -m ... -o .../optimal --check): everything tune.py can compile before it has
# measured anything is built ahead, so a GPU machine only measures and builds the mix it elects
# ------------------------------------------------------------------------------------------------

ENTRY_TUNE_FLAGS = ["--occupancies", "4", "--sample_batch_nums", "2", "-n", "4"]


def entry_fixture_dir() -> str:
    return os.path.join(MODELS_DIR, "tune_entry")


def build_entry_point_fixture(model_dir: str) -> str:
    """``tune_entry/model``: a copy of the fixture model directory with ``output/`` as
    ``examples/tune.py -m tune_entry/model --compile_only`` leaves it (tournament kernel and
    default-schedule contender at the occupancy of ``ENTRY_TUNE_FLAGS``)."""
    import shutil
    import subprocess
    import sys
    root = entry_fixture_dir()
    shutil.rmtree(root, ignore_errors=True)
    model = os.path.join(root, "model")
    shutil.copytree(model_dir, model)
    script = os.path.join(os.path.dirname(PACKAGE_DIR), "examples", "tune.py")
    subprocess.run([sys.executable, script, "-m", model, "--compile_only", "--recompile", *ENTRY_TUNE_FLAGS],
                   check=True, stdout=subprocess.DEVNULL)
    return root
