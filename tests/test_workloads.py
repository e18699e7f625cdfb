"""Synthetic configurations C1..C5: shapes named by the benchmark definition, determinism,
distribution sanity and the algorithmic byte formula."""

import numpy as np
import pytest

from recflex_amd.workloads import (algorithmic_bytes, bounded_zipf, gen_feature_inputs, gen_inputs,
                                   make_workload, row_bytes, row_stride, FeatureSpec)


def test_shapes_of_the_five_configs():
    c1, c2, c3, c4, c5 = (make_workload(n) for n in ("C1", "C2", "C3", "C4", "C5"))
    assert (c1.num_features, c1.batch, c1.embed_dim_sum) == (4, 512, 128)
    assert all(f.rows == 100_000 and f.dim == 32 and f.fixed_len and f.mean_bag == 4 for f in c1.features)
    assert (c2.num_features, c2.batch, c2.embed_dim_sum) == (26, 4096, 1664)
    assert all(1_000 <= f.rows <= 10_000_000 and f.zipf_alpha == 1.05 and f.mean_bag == 1 for f in c2.features)
    assert (c3.num_features, c3.batch) == (100, 2048)
    assert {f.dim for f in c3.features} <= {8, 16, 32, 64, 128}
    assert all(1 <= f.mean_bag <= 200 and 0.8 <= f.zipf_alpha <= 1.2 and f.empty_frac == 0.05 for f in c3.features)
    assert (c4.num_features, c4.batch) == (400, 8192) and {f.data_type for f in c4.features} == {"half"}
    assert {f.dim for f in c4.features} <= {16, 32, 64, 128, 256}
    assert (c5.num_features, c5.batch, c5.embed_dim_sum) == (200, 16384, 25600)
    assert {f.data_type for f in c5.features} == {"int8"} and all(f.dim == 128 for f in c5.features)
    assert c4.table_bytes() < 288 * 2 ** 30          # fits the HBM of one MI355X


def test_inputs_are_deterministic_and_well_formed():
    wl = make_workload("C3", batch=64, max_rows=5000)
    a_idx, a_off = gen_inputs(wl)
    b_idx, b_off = gen_inputs(wl)
    for f, spec in enumerate(wl.features):
        assert np.array_equal(a_idx[f], b_idx[f]) and np.array_equal(a_off[f], b_off[f])
        assert a_off[f].dtype == np.int32 and a_idx[f].dtype == np.int32
        assert a_off[f][0] == 0 and len(a_off[f]) == 65 and a_off[f][-1] == len(a_idx[f])
        assert np.all(np.diff(a_off[f]) >= 0)
        if len(a_idx[f]):
            assert 0 <= a_idx[f].min() and a_idx[f].max() < spec.rows


def test_c1_and_c2_bag_lengths():
    i, o = gen_inputs(make_workload("C1"))
    assert all(np.all(np.diff(x) == 4) for x in o)
    i, o = gen_inputs(make_workload("C2", batch=128))
    assert all(np.all(np.diff(x) == 1) for x in o)


def test_zipf_is_heavy_headed_and_bounded():
    rng = np.random.default_rng(0)
    for alpha in (0.8, 1.0, 1.2):
        r = bounded_zipf(rng, alpha, 1_000_000, 200_000)
        assert r.min() >= 1 and r.max() <= 1_000_000
        # rank 1..100 of a million carries a large share of the mass
        assert (r <= 100).mean() > 0.05
        # and the share falls with the rank: first decade > second decade of ranks
        assert (r <= 10).mean() > ((r > 10) & (r <= 20)).mean()


def test_empty_fraction_and_poisson_mean():
    spec = FeatureSpec(1000, 8, "float", 20.0, False, 0.05, 1.0)
    idx, off = gen_feature_inputs(spec, 20000, np.random.SeedSequence(1))
    lens = np.diff(off)
    assert 0.035 < (lens == 0).mean() < 0.065
    assert 19.0 < lens[lens > 0].mean() < 21.0


def test_algorithmic_bytes_formula():
    assert (row_bytes(64, "float"), row_bytes(64, "half"), row_bytes(128, "int8")) == (256, 128, 132)
    assert (row_stride(64, "float"), row_stride(128, "int8")) == (256, 144)
    wl = make_workload("C1")
    idx, off = gen_inputs(wl)
    # rows 1.05 MB + indices 32 KB + offsets 8 KB + output 262 KB
    want = 4 * (2048 * 128 + 2048 * 4 + 513 * 4 + 512 * 32 * 4)
    assert algorithmic_bytes(wl, [len(i) for i in idx]) == want == 1351696
    wl2 = make_workload("C2")
    idx, _ = gen_inputs(wl2)
    assert algorithmic_bytes(wl2, [len(i) for i in idx]) == 26 * (4096 * 260 + 4097 * 4 + 4096 * 256)


def test_compulsory_bytes_counts_each_memory_line_once():
    """Against a brute-force set of touched line numbers, for rows narrower than a line (several
    rows per line), rows of whole lines, and the 144-byte int8 rows that straddle lines."""
    from recflex_amd.workloads import (FeatureSpec, Workload, algorithmic_bytes, compulsory_bytes,
                                       distinct_row_lines, row_bytes, row_stride)
    rng = np.random.default_rng(5)
    for dim, dt in ((8, "float"), (32, "float"), (128, "float"), (16, "half"), (128, "int8"), (24, "int8")):
        stride, payload = row_stride(dim, dt), row_bytes(dim, dt)
        idx = rng.integers(0, 500, 3000)
        want = set()
        for r in idx.tolist():
            want.update(range(r * stride // 128, (r * stride + payload - 1) // 128 + 1))
        assert distinct_row_lines(idx, stride, payload) == len(want), (dim, dt)
    assert distinct_row_lines(np.zeros(0, np.int32), 64, 64) == 0
    # one row looked up a thousand times is one row's lines
    assert distinct_row_lines(np.full(1000, 7), 512, 512) == 4
    feats = (FeatureSpec(1000, 32, "float", 3.0, False, 0.0, 1.05), FeatureSpec(50, 128, "int8", 9.0, False, 0.1, 0.0))
    wl = Workload("t", 64, 3, feats)
    indices, offsets = gen_inputs(wl)
    comp = compulsory_bytes(wl, indices, offsets)
    alg = algorithmic_bytes(wl, [len(i) for i in indices])
    out_lines = -(-64 * 160 * 4 // 128)
    expect = out_lines * 128
    for spec, i, o in zip(feats, indices, offsets):
        expect += distinct_row_lines(i, row_stride(spec.dim, spec.data_type), row_bytes(spec.dim, spec.data_type)) * 128
        expect += -(-len(i) * 4 // 128) * 128 + -(-len(o) * 4 // 128) * 128
    assert comp == expect and comp % 128 == 0
    # hot rows are counted once: far fewer bytes than the algorithmic count for the 50-row table
    assert comp < alg + 4 * 128
