"""TEST INFRASTRUCTURE ONLY -- CPU checker for the fused-embedding path.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
import this module; the product (``recflex_amd``) never does.

Functions and what they restate (paths relative to the reference repository):

``pooled_sum_torch``
    The oracle named by the reference's own check ``examples/test.py:68-86``
    (``F.embedding(indices, table).sum(0)`` per sample, features side by side): per feature
    ``torch.nn.functional.embedding_bag(mode="sum")`` on CPU fp32, then ``torch.cat(dim=1)``.
    The arithmetic lives in PyTorch (reference pin ``torch==2.2.0``, ``README.md:41``; this
    image has 2.10).  Pinned by tests/test_oracle.py against a brute-force Python loop, the
    closed forms "all-ones table -> bag length" (the reference's tuning tables are
    ``torch.ones``, ``RecFlex/tuning/measure.py:41``) and "row r holds r -> sum of indices",
    and against the C restatement ``oracle.c`` bit for bit.
``pooled_sum_c``
    ctypes front end of ``oracle.c`` (sequential fp32 sum in plain C; fp32 / fp16 / int8 rows).
``decode_table``
    fp16 / int8 row-wise tables -> fp32.  These element types do not exist in the reference
    (``MetaData.data_type`` is always ``"float"``, ``RecFlex/code_emitter/schedule_base.py:23-25``),
    so their numerics are defined here -- "parity unpinned" with respect to the reference;
    the decode is pinned by closed-form tests.
``parse_lines_python``
    Pure-Python restatement of the line splitter
    ``examples/csrc/warp_per_sample_preprocess.cu:9-38``.
``sample_batch_ids_legacy``
    ``np.random.seed(seed)`` + ``np.random.choice(n, k, replace=False)`` + sort, as
    ``RecFlex/parser.py:34-40``.
``padded_sched_num`` / ``pad_sched_params`` / ``solve_local`` / ``solve_global`` /
``reduce_block_times``
    The tuner's arithmetic: ``RecFlex/tuning/tuner.py:83-91`` (padding of the candidate list to
    fill the GPU), ``:154-160`` (argmin per feature and occupancy), ``:194-205`` (argmin over
    occupancies) and ``RecFlex/rec_modules.py:96-109`` (sum of block times per candidate).

``oracle/_ref`` does not exist: the reference path needs nvcc, CUB and a torch CUDA extension,
none of which this image has.
"""

import ctypes
import os
import subprocess
from typing import Dict, List, Sequence, Tuple

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_lib = None

DTYPE_IDS = {"float": 0, "half": 1, "int8": 2}


def build(force: bool = False) -> str:
    if force or not os.path.exists(_LIB_PATH) or \
            os.path.getmtime(_LIB_PATH) < os.path.getmtime(os.path.join(_HERE, "oracle.c")):
        subprocess.run(["make", "-C", _HERE, "-B", "liboracle.so"], check=True,
                       stdout=subprocess.DEVNULL)
    return _LIB_PATH


def _load():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        lib = ctypes.CDLL(_LIB_PATH)
        lib.oracle_pool_feature.restype = ctypes.c_int
        lib.oracle_pool_feature.argtypes = [
            ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_int, ctypes.c_int,
            ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_int64,
            ctypes.c_int]
        lib.oracle_parse_lines.restype = ctypes.c_int64
        lib.oracle_parse_lines.argtypes = [ctypes.c_char_p, ctypes.c_int64, ctypes.c_int,
                                           ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p]
        lib.oracle_half_to_float.restype = ctypes.c_float
        lib.oracle_half_to_float.argtypes = [ctypes.c_uint16]
        _lib = lib
    return _lib


# ------------------------------------------------------------------------------------------------
# table formats
# ------------------------------------------------------------------------------------------------

def int8_row_stride(dim: int) -> int:
    return (dim + 4 + 15) // 16 * 16


def decode_table(table: np.ndarray, dim: int, data_type: str) -> np.ndarray:
    """Host table in its storage format -> fp32 ``[rows, dim]``.
    float: ``[rows, dim]`` float32.  half: ``[rows, dim]`` float16 (exact widening).
    int8: ``[rows, stride]`` uint8; per row ``dim`` codes, fp16 scale, fp16 bias;
    ``value = fp32(code) * fp32(scale) + fp32(bias)`` (separate multiply and add)."""
    if data_type == "float":
        assert table.dtype == np.float32 and table.shape[1] == dim
        return table
    if data_type == "half":
        assert table.dtype == np.float16 and table.shape[1] == dim
        return table.astype(np.float32)
    if data_type == "int8":
        assert table.dtype == np.uint8 and table.shape[1] == int8_row_stride(dim)
        codes = table[:, :dim].astype(np.float32)
        sb = np.ascontiguousarray(table[:, dim:dim + 4]).view(np.float16).astype(np.float32)
        prod = codes * sb[:, 0:1]
        return (prod + sb[:, 1:2]).astype(np.float32)
    raise ValueError(data_type)


# ------------------------------------------------------------------------------------------------
# pooling
# ------------------------------------------------------------------------------------------------

def pooled_sum_torch(tables_fp32: Sequence[np.ndarray], indices: Sequence[np.ndarray],
                     offsets: Sequence[np.ndarray]) -> np.ndarray:
    """``[batch, sum(dim)]`` fp32: per-feature ``embedding_bag(mode="sum")`` then concat."""
    import torch
    import torch.nn.functional as F
    outs = []
    for w, idx, off in zip(tables_fp32, indices, offsets):
        w = torch.from_numpy(np.ascontiguousarray(w, dtype=np.float32))
        idx = torch.from_numpy(np.asarray(idx).astype(np.int64))
        off = torch.from_numpy(np.asarray(off).astype(np.int64))
        outs.append(F.embedding_bag(idx, w, off, mode="sum", include_last_offset=True))
    return torch.cat(outs, dim=1).numpy()


def pooled_sum_c(tables: Sequence[np.ndarray], dims: Sequence[int], data_types: Sequence[str],
                 indices: Sequence[np.ndarray], offsets: Sequence[np.ndarray]) -> np.ndarray:
    """Same result through ``oracle.c``; tables in their storage format."""
    lib = _load()
    batch = len(offsets[0]) - 1
    dim_sum = int(sum(dims))
    out = np.empty((batch, dim_sum), dtype=np.float32)
    col = 0
    for t, d, dt, idx, off in zip(tables, dims, data_types, indices, offsets):
        t = np.ascontiguousarray(t)
        idx = np.ascontiguousarray(idx, dtype=np.int32)
        off = np.ascontiguousarray(off, dtype=np.int32)
        stride = t.shape[1] * t.dtype.itemsize
        rc = lib.oracle_pool_feature(t.ctypes.data, DTYPE_IDS[dt], t.shape[0], int(d), stride,
                                     idx.ctypes.data, off.ctypes.data, batch, out.ctypes.data,
                                     dim_sum, col)
        if rc != 0:
            raise RuntimeError(f"oracle_pool_feature failed with {rc}")
        col += int(d)
    return out


def pooled_sum_python(tables_fp32: Sequence[np.ndarray], indices: Sequence[np.ndarray],
                      offsets: Sequence[np.ndarray]) -> np.ndarray:
    """Brute force with Python loops and fp32 scalars (tiny inputs only)."""
    batch = len(offsets[0]) - 1
    cols = []
    for w, idx, off in zip(tables_fp32, indices, offsets):
        out = np.zeros((batch, w.shape[1]), dtype=np.float32)
        for b in range(batch):
            for p in range(int(off[b]), int(off[b + 1])):
                for d in range(w.shape[1]):
                    out[b, d] = np.float32(out[b, d] + w[int(idx[p]), d])
        cols.append(out)
    return np.concatenate(cols, axis=1)


def within_tolerance(got: np.ndarray, want: np.ndarray, rtol: float, atol: float) -> Tuple[bool, float, float]:
    """True if every element is within ``rtol`` relative OR ``atol`` absolute of the oracle.
    Also returns the largest absolute and relative error seen."""
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    err = np.abs(got - want)
    ok = (err <= atol) | (err <= rtol * np.abs(want))
    rel = err / np.maximum(np.abs(want), 1e-30)
    max_rel = float(np.max(np.where(err <= atol, 0.0, rel))) if err.size else 0.0
    return bool(np.all(ok)), float(err.max()) if err.size else 0.0, max_rel


# ------------------------------------------------------------------------------------------------
# text front end
# ------------------------------------------------------------------------------------------------

def parse_lines_python(lines: Sequence[str]) -> Tuple[np.ndarray, np.ndarray]:
    indices: List[int] = []
    offsets = [0]
    for line in lines:
        index, count = 0, 0
        for ch in line:
            if ch < '0' or ch > '9':
                indices.append(index)
                count += 1
                index = 0
            else:
                index = index * 10 + (ord(ch) - ord('0'))
        if len(line) > 0:
            indices.append(index)
            count += 1
        offsets.append(offsets[-1] + count)
    return np.array(indices, dtype=np.int32), np.array(offsets, dtype=np.int32)


def parse_lines_c(lines: Sequence[str]) -> Tuple[np.ndarray, np.ndarray]:
    lib = _load()
    text = "\n".join(lines).encode()
    cap = len(text) + 1
    indices = np.empty(cap, dtype=np.int32)
    offsets = np.empty(len(lines) + 1, dtype=np.int32)
    n = lib.oracle_parse_lines(text, len(text), len(lines), indices.ctypes.data, cap,
                               offsets.ctypes.data)
    if n < 0:
        raise RuntimeError("oracle_parse_lines failed")
    return indices[:n].copy(), offsets


def sample_batch_ids_legacy(num_batches: int, sample_batch_nums: int, seed: int = 0) -> np.ndarray:
    state = np.random.get_state()
    try:
        np.random.seed(seed)
        k = min(sample_batch_nums, num_batches)
        return np.sort(np.random.choice(num_batches, k, replace=False))
    finally:
        np.random.set_state(state)


# ------------------------------------------------------------------------------------------------
# tuner arithmetic
# ------------------------------------------------------------------------------------------------

def padded_sched_num(orig_num: int, max_concurrent_blocks: int) -> int:
    return (orig_num + max_concurrent_blocks - 1) // orig_num * orig_num


def pad_sched_params(sched_params: list, padded_num: int) -> list:
    out = list(sched_params)
    for i in range(padded_num - len(sched_params)):
        out.append(sched_params[i % len(sched_params)])
    return out


def solve_local(measured_times: Dict[int, Dict[int, List[float]]], occupancies: Sequence[int]
                ) -> List[List[int]]:
    """Per occupancy (outer list, in the given order): argmin candidate index of every feature."""
    feats = sorted(measured_times.keys())
    return [[int(np.argmin(measured_times[f][occ])) for f in feats] for occ in occupancies]


def solve_global(kernel_times: Sequence[float], occupancies: Sequence[int]) -> int:
    return occupancies[int(np.argmin(kernel_times))]


def reduce_block_times(task_mapping: Sequence[Tuple[int, int]], times: Sequence[float],
                       timing_schedules: int) -> List[float]:
    """Sum of the per-block times of each of the first ``timing_schedules`` features, walking
    the (feature-sorted) task mapping as rec_modules.py:96-109 does."""
    out = [0.0] * timing_schedules
    block = 0
    for feat in range(timing_schedules):
        while block < len(task_mapping) and task_mapping[block][0] == feat:
            out[feat] += times[block]
            block += 1
    return out
