"""CPU text front end (librecflex_host.so, recom_host_* in include/recflex_hip.h) against the
oracle's restatement of the reference's line splitter, plus the packed-buffer layout."""

import numpy as np
import pytest

from helpers import oracle
from recflex_amd.code_emitter.build_basic import BasicBuilder
from recflex_amd.host import RecomHost, RecomHostError


@pytest.fixture(scope="module")
def host():
    return RecomHost(BasicBuilder().build())


CASES = [
    ["3,5,7", "", "12", "0", "1,,2", "9,", ",4", "007", "1 2;3"],
    [""],
    ["", "", ""],
    ["5"],
    ["1,2", ""],
    ["", "1,2"],
    [],
    ["2147483647", "0"],
]


@pytest.mark.parametrize("lines", CASES)
def test_parse_matches_oracle(host, lines):
    idx, off = host.parse_lines(lines)
    want_idx, want_off = oracle.parse_lines_python(lines)
    assert idx.dtype == np.int32 and off.dtype == np.int32
    assert np.array_equal(idx, want_idx)
    assert np.array_equal(off, want_off)


def test_parse_random_against_both_oracles(host):
    rng = np.random.default_rng(10)
    seps = [",", " ", ";", ",,"]
    lines = []
    for _ in range(500):
        n = int(rng.integers(0, 15))
        sep = seps[int(rng.integers(0, len(seps)))]
        lines.append(sep.join(str(int(v)) for v in rng.integers(0, 2 ** 31 - 1, n)))
    idx, off = host.parse_lines(lines)
    for want_idx, want_off in (oracle.parse_lines_python(lines), oracle.parse_lines_c(lines)):
        assert np.array_equal(idx, want_idx) and np.array_equal(off, want_off)


def test_parse_rejects_values_beyond_int32(host):
    with pytest.raises(RecomHostError):
        host.parse_lines(["2147483648"])


def test_raw_entry_point_error_codes(host):
    import ctypes
    lib = host.lib
    off = (ctypes.c_int32 * 3)()
    idx = (ctypes.c_int32 * 8)()
    n = ctypes.c_int64()
    # capacity too small
    assert lib.recom_host_parse_lines(b"1,2", 3, 1, idx, 1, off, ctypes.byref(n)) == -2
    # more lines than announced / fewer lines than announced
    assert lib.recom_host_parse_lines(b"1\n2\n3", 5, 2, idx, 8, off, ctypes.byref(n)) == -3
    assert lib.recom_host_parse_lines(b"1", 1, 2, idx, 8, off, ctypes.byref(n)) == -3
    # NULL outputs
    assert lib.recom_host_parse_lines(b"1", 1, 1, idx, 1, None, ctypes.byref(n)) == -1
    # one trailing newline after the last line is fine
    assert lib.recom_host_parse_lines(b"7\n", 2, 1, idx, 1, off, ctypes.byref(n)) == 0
    assert (n.value, idx[0], off[0], off[1]) == (1, 7, 0, 1)


def test_alignment_helpers(host):
    """128-byte alignment of utils.cuh:60-68."""
    assert [host.alignmem(x) for x in (0, 1, 127, 128, 129, 4 * 513)] == [0, 128, 128, 128, 256, 2176]


def test_pack_layout(host):
    rng = np.random.default_rng(11)
    batch = 37
    offsets, indices = [], []
    for f in range(5):
        lens = rng.integers(0, 6, batch)
        if f == 3:
            lens[:] = 0          # a feature without any lookup
        off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        offsets.append(off)
        indices.append(rng.integers(0, 1000, off[-1]).astype(np.int32))
    packed, byte_offsets = host.pack(offsets, indices)
    assert packed.dtype == np.int32 and byte_offsets.dtype == np.int64
    assert byte_offsets[0] == 0 and len(byte_offsets) == 6
    raw = packed.view(np.uint8)
    for f in range(5):
        start = int(byte_offsets[f])
        assert start % 128 == 0
        off_bytes = (batch + 1) * 4
        got_off = raw[start:start + off_bytes].view(np.int32)
        assert np.array_equal(got_off, offsets[f])
        idx_start = start + host.alignmem(off_bytes)
        got_idx = raw[idx_start:idx_start + 4 * len(indices[f])].view(np.int32)
        assert np.array_equal(got_idx, indices[f])
        # padding is zero
        assert not raw[start + off_bytes:idx_start].any()
        end = int(byte_offsets[f + 1])
        assert end == idx_start + host.alignmem(4 * len(indices[f]))
        assert not raw[idx_start + 4 * len(indices[f]):end].any()
    assert int(byte_offsets[-1]) == raw.size


def test_preprocess_tuple_shape(host):
    raw = [["1,2", "", "3"], ["4", "5", "6"]]
    (dbo, out_off, extra_off, task_mapping, task_tiles, data, scala) = host.preprocess(raw, 0)
    assert len(dbo) == 3 and dbo[0] == 0
    assert extra_off == [0, 0, 0] and task_mapping == [] and task_tiles == [0, 0]
    assert scala == [3, 3, 3, 3]                      # (num_inputs, num_segments) per feature
    assert data[0].tolist() == [0, 2, 2, 3] and data[1].tolist() == [1, 2, 3]
    assert data[2].tolist() == [0, 1, 2, 3] and data[3].tolist() == [4, 5, 6]
