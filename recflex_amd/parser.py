"""Readers of the model / dataset text formats and of rocprofv3 kernel statistics.

Formats and function names follow ``RecFlex/parser.py:19-85``:

* ``schedule_config.txt``: one line per feature, comma-separated schedule class names;
* ``table_config.txt``: one line per feature ``rows,dim`` -- extended here with an optional
  third field, the table element type (``float`` / ``half`` / ``int8``);
* dataset directory: ``batch_sizes.txt`` (one int per line) and ``f{i}.txt`` (one line per
  sample, comma-separated indices, empty line = empty bag); batch ``k`` is the line range given
  by the running sum of the batch sizes;
* ``parse_knl_total_time`` reads the total time of a kernel from a rocprofv3
  ``*_kernel_stats.csv`` (the reference shells out to ``nsys stats``).
"""

import csv
import glob
import os
from typing import Dict, List, Tuple

import numpy as np


def parse_schedule_types(config_fname: str, schedule_mapping: Dict[str, type],
                         sep: str = ',') -> List[List[type]]:
    """Unknown class names map to ``None`` exactly as ``dict.get`` does in the reference
    (parser.py:24)."""
    feat_schedule_types = []
    with open(config_fname) as f:
        for line in f.readlines():
            feat_schedule_types.append([schedule_mapping.get(name) for name in line.strip().split(sep)])
    return feat_schedule_types


def sample_batch_ids(num_batches: int, sample_batch_nums: int, seed: int = 0) -> np.ndarray:
    """Sorted ids of the sampled batches: legacy ``np.random.seed(seed)`` followed by
    ``np.random.choice(n, k, replace=False)`` (parser.py:34-40), so the same seed picks the same
    batches as the reference."""
    rng = np.random.RandomState(seed)
    k = min(sample_batch_nums, num_batches)
    return np.sort(rng.choice(num_batches, k, replace=False))


def parse_raw_data_batches(batch_sizes_fname: str, data_fnames: List[str], sample_batch_nums: int = 128,
                           seed: int = 0, feat_major: bool = True) -> List[List[List[str]]]:
    '''
    Return: (num_feats, sample_batch_nums, batch_size) (feat_major=True)
            (sample_batch_nums, num_feats, batch_size) (feat_major=False)
    '''
    with open(batch_sizes_fname) as f:
        batch_sizes = [int(line.strip()) for line in f.readlines() if line.strip()]
    line_offsets = np.cumsum([0] + batch_sizes)
    ids = sample_batch_ids(len(batch_sizes), sample_batch_nums, seed)

    num_feats = len(data_fnames)
    per_feat: List[List[List[str]]] = []
    for fname in data_fnames:
        with open(fname) as f:
            lines = f.read().splitlines()
        # a writer that joins lines with '\n' loses trailing empty bags; restore them
        total = int(line_offsets[-1])
        if len(lines) < total:
            lines.extend([""] * (total - len(lines)))
        per_feat.append([lines[line_offsets[b]:line_offsets[b + 1]] for b in ids])

    if feat_major:
        return per_feat
    return [[per_feat[f][i] for f in range(num_feats)] for i in range(len(ids))]


def parse_table_shapes(config_fname: str, sep: str = ',') -> List[Tuple[int, int]]:
    """``(rows, dim)`` per feature; a third field (data type) is ignored here, see
    ``parse_table_dtypes``."""
    table_shapes = []
    with open(config_fname) as f:
        for line in f.readlines():
            if not line.strip():
                continue
            fields = line.strip().split(sep)
            table_shapes.append((int(fields[0]), int(fields[1])))
    return table_shapes


def parse_table_dtypes(config_fname: str, sep: str = ',') -> List[str]:
    """Table element type per feature: third field of ``table_config.txt``, ``float`` if absent."""
    from recflex_amd.code_emitter.schedule_base import canonical_data_type
    dtypes = []
    with open(config_fname) as f:
        for line in f.readlines():
            if not line.strip():
                continue
            fields = line.strip().split(sep)
            dtypes.append(canonical_data_type(fields[2]) if len(fields) > 2 else "float")
    return dtypes


def _stats_files(report: str) -> List[str]:
    if os.path.isfile(report):
        return [report]
    pats = [os.path.join(report, "**", "*kernel_stats.csv"), report + "*kernel_stats.csv"]
    out: List[str] = []
    for pat in pats:
        out.extend(glob.glob(pat, recursive=True))
    return sorted(set(out))


def parse_knl_total_time(knl: str, report: str, reptype: str = "kernel_stats") -> int:
    """Total time (ns) of all kernels whose name contains ``knl`` in the rocprofv3
    ``--kernel-trace --stats`` output found at ``report`` (a csv file, or a directory /
    prefix that holds ``*_kernel_stats.csv``)."""
    files = _stats_files(report)
    if not files:
        raise FileNotFoundError(f"no *kernel_stats.csv under {report}")
    total = 0
    for fname in files:
        with open(fname, newline='') as f:
            for row in csv.DictReader(f):
                if knl in row.get("Name", ""):
                    total += int(float(row["TotalDurationNs"]))
    return total


def parse_knl_calls_and_average(knl: str, report: str) -> Tuple[int, float]:
    """(number of calls, average duration in ns) of the kernels whose name contains ``knl``."""
    calls, total = 0, 0.0
    for fname in _stats_files(report):
        with open(fname, newline='') as f:
            for row in csv.DictReader(f):
                if knl in row.get("Name", ""):
                    calls += int(row["Calls"])
                    total += float(row["TotalDurationNs"])
    return calls, (total / calls if calls else 0.0)


# kernels a library may launch ahead of the fused one within a call; their time belongs to it
AUX_KERNELS = ("BindKnl", "OutlierKnl", "ScratchClearKnl")


def _trace_files(report: str) -> List[str]:
    if os.path.isfile(report):
        return [report]
    pats = [os.path.join(report, "**", "*kernel_trace.csv"), report + "*kernel_trace.csv"]
    out: List[str] = []
    for pat in pats:
        out.extend(glob.glob(pat, recursive=True))
    return sorted(set(out))


def parse_knl_call_durations(knl: str, report: str, aux: Tuple[str, ...] = AUX_KERNELS) -> List[int]:
    """Duration (ns) of every call, in the order of execution, from a rocprofv3
    ``--kernel-trace`` output (``*_kernel_trace.csv`` at ``report``: a csv file, or a directory /
    prefix that holds one).  A call is one dispatch of the kernel whose name is ``knl`` plus the
    dispatches of the ``aux`` kernels that ran since the call before (the binding and outlier
    kernels a library launches ahead of its fused kernel)."""
    files = _trace_files(report)
    if not files:
        raise FileNotFoundError(f"no *kernel_trace.csv under {report}")
    rows = []
    for fname in files:
        with open(fname, newline='') as f:
            for row in csv.DictReader(f):
                name = row.get("Kernel_Name", "")
                if name == knl or name in aux:
                    rows.append((int(row["Start_Timestamp"]), int(row["End_Timestamp"]), name))
    rows.sort()
    calls, pending = [], 0
    for start, end, name in rows:
        if name == knl:
            calls.append(pending + end - start)
            pending = 0
        else:
            pending += end - start
    return calls


def parse_knl_batch_times(knl: str, report: str, passes: int, skip_passes: int = 1) -> List[float]:
    """For a program that ran the same sequence of batches ``passes`` times: per batch, the
    median over the passes after the first ``skip_passes`` (warm-up: cold caches, clocks still
    rising) of the call's duration in ns."""
    calls = parse_knl_call_durations(knl, report)
    if passes <= skip_passes or not calls or len(calls) % passes != 0:
        raise ValueError(f"{len(calls)} calls of {knl} do not make {passes} passes "
                         f"(of which {skip_passes} warm-up) over one sequence of batches")
    n = len(calls) // passes
    kept = np.asarray(calls, dtype=np.float64).reshape(passes, n)[skip_passes:]
    return np.median(kept, axis=0).tolist()


def parse_first_knl_total_time(report: str, reptype: str = "kernel_stats") -> int:
    """Total time (ns) of the kernel with the largest total time."""
    best = 0
    for fname in _stats_files(report):
        with open(fname, newline='') as f:
            for row in csv.DictReader(f):
                best = max(best, int(float(row["TotalDurationNs"])))
    return best
