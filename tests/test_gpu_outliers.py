"""GPU parity of a library emitted with outlier tiles (bags found ahead of the kernel and summed
by several workgroups)."""

import numpy as np
import pytest

from helpers import oracle_output, require_lib

pytestmark = pytest.mark.gpu

CAP, PARTS = 4096, 16384      # rfx::kOutlierCap, rfx::kOutlierPartCap


def _inject(rng, wl, indices, offsets, plan):
    """plan: {feature: [extra lookups, ...]} -- each entry lengthens one random bag; an int
    instead of a list lengthens every bag of the feature."""
    indices, offsets = list(indices), list(offsets)
    for f, extras in plan.items():
        lens = np.diff(offsets[f]).astype(np.int64)
        if isinstance(extras, int):
            lens += extras
            extras = []
        for extra in extras:
            lens[rng.integers(0, wl.batch)] += extra
        off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        indices[f] = rng.integers(0, wl.features[f].rows, int(off[-1])).astype(np.int32)
        offsets[f] = off
    return indices, offsets


@pytest.mark.parametrize("case", ["none", "few", "many", "overflow", "mid", "mid_overflow"])
def test_outlier_tiles_are_bit_exact(case):
    """No outlier at all; a few bags of 300 to 20 000 lookups in features of every kind of
    schedule; some hundred outliers; more than the list holds (4 096), where the launch falls back
    to a wavefront per outlier; some hundred mid-size bags (beyond their schedule's reach, below
    the outlier threshold: they go through the workgroup's list in LDS to whichever wavefront
    has time); every bag of twenty features mid-size, more than that list holds (192 per
    workgroup), where a bag is summed by the wavefront that met it.  Three launches each on one
    workspace, whose list header and arrival counters must be back at zero afterwards.
    Integer-valued tables: bit for bit."""
    import torch
    from recflex_amd import prebuilt
    from recflex_amd.rec_modules import FeatEmbed
    from recflex_amd.workloads import gen_inputs, gen_tables

    spec = prebuilt.model_spec("c3s_outliers")
    wl = spec.workload
    assert wl.table_values == "integer"
    assert sum(type(s).__name__ == "SplitBagSchedule" for s, _ in spec.feat_schedules) == 10
    dev = torch.device("cuda", 0)
    print(f"[case] c3s_outliers {case}: F={wl.num_features} B={wl.batch}", flush=True)
    tables = gen_tables(wl, dev)
    host_tables = [t.cpu().numpy() for t in tables]
    layer = FeatEmbed(dev, embed_tables=tables, librecom=require_lib("c3s_outliers"))
    assert layer.workspace is not None
    rng = np.random.default_rng(len(case))
    base_idx, base_off = gen_inputs(wl)
    for launch in range(3):
        feats = rng.permutation(wl.num_features)
        if case == "none":
            plan = {}
        elif case == "few":
            plan = {int(f): [int(x)] for f, x in zip(feats[:6], (300, 2000, 20000, 4200, 5000, 9000))}
        elif case == "many":
            plan = {int(f): [2000 + 371 * k for k in range(12)] for f in feats[:10]}
        elif case == "overflow":
            plan = {int(f): 2500 for f in feats[:60]}
        elif case == "mid":
            plan = {int(f): [70 + 13 * k for k in range(40)] for f in feats[:12]}
        else:
            plan = {int(f): 90 + 7 * int(f) % 60 for f in feats[:20]}
        indices, offsets = _inject(rng, wl, base_idx, base_off, plan)
        d_idx = [torch.from_numpy(i).to(dev) for i in indices]
        d_off = [torch.from_numpy(o).to(dev) for o in offsets]
        got = layer.forward_indices(d_idx, d_off).cpu().numpy()
        want = oracle_output(wl, host_tables, indices, offsets)
        bad = np.argwhere(got.view(np.uint32) != want.view(np.uint32))
        assert bad.size == 0, f"launch {launch}: {len(bad)} elements differ, first at {bad[:5].tolist()}"
        # the outlier space follows the split regions of every tenth feature: header (32 ints),
        # CAP entries of 4 ints, CAP counters, PARTS part -> entry, PARTS slots of 128 floats
        ws = layer.workspace.cpu().numpy()
        ws = ws[len(ws) - (32 + 4 * CAP + CAP + PARTS + PARTS * 128):]
        assert not ws[:3].any() and not ws[5], f"launch {launch}: list header not cleared: {ws[:6].tolist()}"
        assert not ws[32 + 4 * CAP:32 + 5 * CAP].any(), f"launch {launch}: arrival counters not reset"
        # what the launch found: bags beyond their schedule's threshold and 128 KiB of traffic
        # (split-bag features take bags of any length themselves)
        expect = 0
        for (sched, params), feat, off in zip(spec.feat_schedules, wl.features, offsets):
            if sched.LongBagThreshold(params) > 0:
                thr = max(sched.LongBagThreshold(params), -(-131072 // (4 * feat.dim + 4)))
                expect += int((np.diff(off) > thr).sum())
        assert int(ws[3]) == expect, (int(ws[3]), expect)
        if case == "overflow":
            assert expect > CAP
        elif case in ("few", "many"):
            assert 0 < expect <= CAP and int(ws[4]) >= expect


@pytest.mark.parametrize("name", ["c4s_outliers", "c5s_outliers"])
@pytest.mark.parametrize("case", ["few", "mid"])
def test_outlier_tiles_on_fp16_and_int8_rows(name, case):
    """The block-wide parts, the workgroup's list of mid-size bags and the wavefront that sums
    them, on fp16 and int8 rows (scale and bias, staged output): a few bags of 300 to 20 000
    lookups, and some hundred bags between their schedule's reach and the outlier threshold.
    Two launches on one workspace; integer-valued tables, bit for bit."""
    import torch
    from recflex_amd import prebuilt
    from recflex_amd.rec_modules import FeatEmbed
    from recflex_amd.workloads import gen_inputs, gen_tables

    spec = prebuilt.model_spec(name)
    wl = spec.workload
    assert wl.table_values == "integer"
    dev = torch.device("cuda", 0)
    print(f"[case] {name} {case}: F={wl.num_features} B={wl.batch}", flush=True)
    tables = gen_tables(wl, dev)
    host_tables = [t.cpu().numpy() for t in tables]
    layer = FeatEmbed(dev, embed_tables=tables, librecom=require_lib(name))
    assert layer.lib.info.outliers == 1 and layer.workspace is not None
    rng = np.random.default_rng(len(name) + len(case))
    base_idx, base_off = gen_inputs(wl)
    for launch in range(2):
        feats = rng.permutation(wl.num_features)
        if case == "few":
            plan = {int(f): [int(x)] for f, x in zip(feats[:6], (300, 2000, 20000, 4200, 5000, 9000))}
        else:
            plan = {int(f): [70 + 13 * k for k in range(30)] for f in feats[:8]}
        indices, offsets = _inject(rng, wl, base_idx, base_off, plan)
        got = layer.forward_indices([torch.from_numpy(i).to(dev) for i in indices],
                                    [torch.from_numpy(o).to(dev) for o in offsets]).cpu().numpy()
        want = oracle_output(wl, host_tables, indices, offsets)
        bad = np.argwhere(got.view(np.uint32) != want.view(np.uint32))
        assert bad.size == 0, f"launch {launch}: {len(bad)} elements differ, first at {bad[:5].tolist()}"
