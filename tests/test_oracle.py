"""Pins the CPU oracle before anything is compared with it.

The reference holds no golden vectors for this path (its only check is examples/test.py:68-86
on random data), so the oracle is pinned by what the mathematics fixes: a brute-force loop on
tiny inputs, closed forms that a dropped term / wrong index / transposed operand would break,
the library routine the reference's check is built on (torch embedding / embedding_bag), and
agreement between the independent C and numpy/torch restatements.
"""

import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from helpers import oracle, ROOT

GOLDEN = os.path.join(ROOT, "tests", "golden")


def _ragged(rng, batch, max_len, rows, empty_every=4):
    lens = rng.integers(0, max_len + 1, batch)
    lens[::empty_every] = 0
    offsets = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    indices = rng.integers(0, rows, offsets[-1]).astype(np.int32)
    return indices, offsets


def test_brute_force_tiny():
    rng = np.random.default_rng(0)
    tables = [rng.standard_normal((11, 3)).astype(np.float32), rng.standard_normal((5, 4)).astype(np.float32)]
    ins = [_ragged(rng, 9, 6, t.shape[0]) for t in tables]
    idx, off = [i for i, _ in ins], [o for _, o in ins]
    want = oracle.pooled_sum_python(tables, idx, off)
    got_t = oracle.pooled_sum_torch(tables, idx, off)
    got_c = oracle.pooled_sum_c(tables, [3, 4], ["float", "float"], idx, off)
    assert np.array_equal(want.view(np.uint32), got_c.view(np.uint32))
    assert np.array_equal(want.view(np.uint32), got_t.view(np.uint32))


def test_reference_check_definition():
    """examples/test.py:68-86: F.embedding(LongTensor(indices), table).sum(0) per sample."""
    rng = np.random.default_rng(1)
    table = rng.standard_normal((40, 8)).astype(np.float32)
    idx, off = _ragged(rng, 17, 9, 40)
    got = oracle.pooled_sum_c([table], [8], ["float"], [idx], [off])
    t = torch.from_numpy(table)
    for b in range(17):
        ind = torch.from_numpy(idx[off[b]:off[b + 1]].astype(np.int64))
        pooled = F.embedding(ind, t).sum(0)
        assert torch.allclose(pooled, torch.from_numpy(got[b]), atol=1e-6, rtol=1e-6)
        if len(ind) == 0:
            assert not got[b].any()


def test_closed_form_ones_table_gives_bag_length():
    rng = np.random.default_rng(2)
    idx, off = _ragged(rng, 50, 300, 1000)
    table = np.ones((1000, 5), dtype=np.float32)
    lens = np.diff(off).astype(np.float32)
    for fn in (lambda: oracle.pooled_sum_c([table], [5], ["float"], [idx], [off]),
               lambda: oracle.pooled_sum_torch([table], [idx], [off])):
        out = fn()
        assert np.array_equal(out, np.repeat(lens[:, None], 5, axis=1))


def test_closed_form_row_id_table_gives_index_sum_and_column_identity():
    """table[r, d] = r * 8 + d: a wrong row, a wrong column or a transposed table all show."""
    rng = np.random.default_rng(3)
    rows, dim = 200, 8
    table = (np.arange(rows)[:, None] * 8 + np.arange(dim)[None, :]).astype(np.float32)
    idx, off = _ragged(rng, 30, 20, rows)
    out = oracle.pooled_sum_c([table], [dim], ["float"], [idx], [off])
    for b in range(30):
        seg = idx[off[b]:off[b + 1]].astype(np.int64)
        want = seg.sum() * 8 + np.arange(dim) * len(seg)
        assert np.array_equal(out[b], want.astype(np.float32))   # exact: small integers


def test_concat_layout_offsets():
    """Feature f occupies columns [sum of earlier dims, +dim_f) (codegen.py:227-231)."""
    rng = np.random.default_rng(4)
    dims = [3, 1, 6]
    tables = [np.full((7, d), float(k + 1), dtype=np.float32) for k, d in enumerate(dims)]
    ins = [_ragged(rng, 5, 4, 7, empty_every=5) for _ in dims]
    idx, off = [i for i, _ in ins], [o for _, o in ins]
    out = oracle.pooled_sum_c(tables, dims, ["float"] * 3, idx, off)
    assert out.shape == (5, 10)
    col = 0
    for k, d in enumerate(dims):
        lens = np.diff(off[k]).astype(np.float32)
        assert np.array_equal(out[:, col:col + d], np.repeat(lens[:, None] * (k + 1), d, axis=1))
        col += d


def test_c_oracle_matches_torch_bitwise_on_random_fp32():
    rng = np.random.default_rng(5)
    tables = [(rng.standard_normal((3000, d)) * 0.01).astype(np.float32) for d in (8, 32, 100)]
    ins = [_ragged(rng, 64, 150, 3000) for _ in tables]
    idx, off = [i for i, _ in ins], [o for _, o in ins]
    a = oracle.pooled_sum_c(tables, [8, 32, 100], ["float"] * 3, idx, off)
    b = oracle.pooled_sum_torch(tables, idx, off)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


def test_half_decode_every_bit_pattern():
    lib = oracle._load()
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([lib.oracle_half_to_float(int(b)) for b in bits], dtype=np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_half_tables_are_widened_exactly():
    rng = np.random.default_rng(6)
    t16 = (rng.standard_normal((500, 16)) * 0.01).astype(np.float16)
    idx, off = _ragged(rng, 40, 30, 500)
    a = oracle.pooled_sum_c([t16], [16], ["half"], [idx], [off])
    b = oracle.pooled_sum_torch([oracle.decode_table(t16, 16, "half")], [idx], [off])
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


def _int8_table(rng, rows, dim, scale, bias):
    stride = oracle.int8_row_stride(dim)
    t = np.zeros((rows, stride), dtype=np.uint8)
    t[:, :dim] = rng.integers(0, 256, (rows, dim), dtype=np.uint8)
    sb = np.stack([np.full(rows, scale, np.float16), np.full(rows, bias, np.float16)], axis=1)
    t[:, dim:dim + 4] = sb.view(np.uint8)
    return t


def test_int8_closed_forms():
    rng = np.random.default_rng(7)
    dim = 16
    # scale 1, bias 0: value == code
    t = _int8_table(rng, 50, dim, 1.0, 0.0)
    assert np.array_equal(oracle.decode_table(t, dim, "int8"), t[:, :dim].astype(np.float32))
    # scale 0.5, bias -3: exact in fp32
    t = _int8_table(rng, 50, dim, 0.5, -3.0)
    assert np.array_equal(oracle.decode_table(t, dim, "int8"), t[:, :dim].astype(np.float32) * 0.5 - 3.0)
    # stride / position of scale and bias: dim 20 -> stride 32, scale at byte 20
    assert oracle.int8_row_stride(20) == 32 and oracle.int8_row_stride(128) == 144
    idx, off = _ragged(rng, 20, 12, 50)
    a = oracle.pooled_sum_c([t], [dim], ["int8"], [idx], [off])
    b = oracle.pooled_sum_torch([oracle.decode_table(t, dim, "int8")], [idx], [off])
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


def test_int8_random_scales_c_vs_numpy():
    rng = np.random.default_rng(8)
    dim, rows = 24, 300
    t = _int8_table(rng, rows, dim, 1.0, 0.0)
    sb = (rng.standard_normal((rows, 2)) * 0.01).astype(np.float16)
    t[:, dim:dim + 4] = sb.view(np.uint8)
    idx, off = _ragged(rng, 33, 40, rows)
    a = oracle.pooled_sum_c([t], [dim], ["int8"], [idx], [off])
    b = oracle.pooled_sum_torch([oracle.decode_table(t, dim, "int8")], [idx], [off])
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


def test_out_of_range_index_is_an_error():
    table = np.zeros((4, 2), dtype=np.float32)
    with pytest.raises(RuntimeError):
        oracle.pooled_sum_c([table], [2], ["float"], [np.array([4], np.int32)], [np.array([0, 1], np.int32)])


# ---------------------------------------------------------------------------------- text front end

LINES = ["3,5,7", "", "12", "0", "1,,2", "9,", ",4", "007", "1 2;3"]


def test_line_parser_semantics():
    """warp_per_sample_preprocess.cu:14-32: every non-digit ends an index, a non-empty line
    always ends one, an empty line is an empty bag."""
    idx, off = oracle.parse_lines_python(LINES)
    assert idx.tolist() == [3, 5, 7, 12, 0, 1, 0, 2, 9, 0, 0, 4, 7, 1, 2, 3]
    assert off.tolist() == [0, 3, 3, 4, 5, 8, 10, 12, 13, 16]
    idx_c, off_c = oracle.parse_lines_c(LINES)
    assert np.array_equal(idx, idx_c) and np.array_equal(off, off_c)


def test_line_parser_offsets_are_exclusive_prefix_sums():
    rng = np.random.default_rng(9)
    lines = [",".join(str(int(v)) for v in rng.integers(0, 10 ** 6, rng.integers(0, 12))) for _ in range(200)]
    idx, off = oracle.parse_lines_c(lines)
    lens = [len(l.split(",")) if l else 0 for l in lines]
    assert off.tolist() == np.concatenate([[0], np.cumsum(lens)]).tolist()
    assert idx.tolist() == [int(v) for l in lines if l for v in l.split(",")]


def test_batch_sampling_is_legacy_numpy_stream():
    """parser.py:34-40 with the frozen legacy RandomState stream; values below are what
    numpy's MT19937-based ``choice`` yields for these seeds (checked against two call styles)."""
    from recflex_amd.parser import sample_batch_ids
    for n, k, seed in [(32, 8, 0), (128, 128, 0), (1000, 128, 3), (5, 128, 1)]:
        want = oracle.sample_batch_ids_legacy(n, k, seed)
        rs = np.sort(np.random.RandomState(seed).choice(n, min(k, n), replace=False))
        assert np.array_equal(want, rs)
        assert np.array_equal(sample_batch_ids(n, k, seed), want)
    assert oracle.sample_batch_ids_legacy(32, 8, 0).tolist() == sorted(
        np.random.RandomState(0).permutation(32)[:8].tolist())


# ---------------------------------------------------------------------------------- tuner arithmetic

def test_padding_rule():
    """tuner.py:83-91: smallest multiple of n that is >= n + max_concurrent_blocks - 1, filled
    by cycling through the candidates."""
    assert oracle.padded_sched_num(5, 12) == 15
    assert oracle.padded_sched_num(24, 108) == 120
    assert oracle.padded_sched_num(152, 108) == 152
    assert oracle.padded_sched_num(7, 1) == 7
    for n in range(1, 40):
        for m in range(1, 300, 7):
            p = oracle.padded_sched_num(n, m)
            assert p % n == 0 and p >= m and p - n < m + n - 1
    assert oracle.pad_sched_params(list("abc"), 8) == list("abcabcab")


def test_solve_and_block_time_reduction():
    times = {0: {1: [3.0, 1.0, 2.0], 2: [0.5, 0.7, 0.9]}, 1: {1: [5.0, 6.0], 2: [9.0, 8.0]}}
    assert oracle.solve_local(times, [1, 2]) == [[1, 0], [0, 1]]
    assert oracle.solve_global([30.0, 10.0, 20.0], [1, 2, 4]) == 2
    mapping = [(0, 0), (0, 1), (1, 0), (2, 0), (2, 1), (2, 2)]
    assert oracle.reduce_block_times(mapping, [1, 2, 4, 8, 16, 32], 3) == [3.0, 4.0, 56.0]
    assert oracle.reduce_block_times(mapping, [1, 2, 4, 8, 16, 32], 2) == [3.0, 4.0]


# ---------------------------------------------------------------------------------- golden fixtures

def test_golden_fixtures():
    """Small committed input/output vectors (written by tests/golden/make_golden.py from the
    pinned oracle): a change of the oracle's results shows up here."""
    path = os.path.join(GOLDEN, "pooled_small.npz")
    z = np.load(path)
    n = int(z["num_features"])
    dims = z["dims"].tolist()
    dts = [str(s) for s in z["data_types"]]
    tables = [z[f"table{f}"] for f in range(n)]
    idx = [z[f"indices{f}"] for f in range(n)]
    off = [z[f"offsets{f}"] for f in range(n)]
    got = oracle.pooled_sum_c(tables, dims, dts, idx, off)
    assert np.array_equal(got.view(np.uint32), z["expected"].view(np.uint32))
    decoded = [oracle.decode_table(t, d, dt) for t, d, dt in zip(tables, dims, dts)]
    got_t = oracle.pooled_sum_torch(decoded, idx, off)
    assert np.array_equal(got_t.view(np.uint32), z["expected"].view(np.uint32))
