"""Synthetic lookup datasets in the on-disk text format of the fused-embedding path.

Writes ``batch_sizes.txt`` (one batch size per line) and one ``f{i}.txt`` per feature (one line
per sample: comma-separated row indices, empty line = absent feature / empty bag) from a
``data_config.txt`` (``type,count,params...``) and a ``table_config.txt`` (``rows,dim[,dtype]``).

Same command line, file formats and distribution families as the reference generator
(``data_synthesis/data_generate.py:27-40,145-164`` and ``data_synthesis/README.md:7-14``):

* ``one-hot,n,coverage``                          one index per present sample;
* ``multi-hot,n,mean,std,max,coverage``           pooling factor ~ normal truncated to [0, max];
* ``multi-hot-static,n,hot,coverage``             fixed pooling factor;
* ``multi-hot-one-side,n,mean,std,coverage``      normal truncated to [0, inf);
* indices drawn with replacement from a per-group power-law (``numpy.random.power(a=3)``)
  probability vector over the table rows;
* batch sizes: ``floor(exp(N(ln mean, ln std)))`` folded into ``[1, max]``.

The random streams are this implementation's own (``numpy.random.Generator``, one child stream
per feature), so files are reproducible for a given ``--seed_base`` but not byte-identical to
the reference's (whose streams depend on the scipy version in use); existing files are kept,
which makes an interrupted run resumable.
"""

import argparse
import math
import os
import sys
from typing import List, Tuple

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

from recflex_amd.parser import parse_table_shapes  # noqa: E402


def parse_args():
    parser = argparse.ArgumentParser()
    parser.add_argument("-c", "--config_path", type=str, required=True)
    parser.add_argument("-t", "--table_config_path", type=str, required=True)
    parser.add_argument("-n", "--num_processes", type=int, default=64)   # accepted, unused
    parser.add_argument("-s", "--seed_base", type=int, default=1000)
    parser.add_argument("--num_queries", type=int, default=128)
    parser.add_argument("--query_mean", type=int, default=256)
    parser.add_argument("--query_stddev", type=int, default=128)
    parser.add_argument("--query_max", type=int, default=512)
    parser.add_argument("-o", "--output_dir", type=str, required=True)
    return parser.parse_args()


def parse_data_config(config_path: str) -> List[Tuple[str, int, List[float]]]:
    groups = []
    with open(config_path) as f:
        for line in f:
            fields = [x.strip() for x in line.strip().split(",")]
            if len(fields) < 3:
                continue
            groups.append((fields[0], int(fields[1]), [float(x) for x in fields[2:]]))
    return groups


def truncated_normal(rng: np.random.Generator, mean: float, std: float, lo: float, hi: float,
                     size: int) -> np.ndarray:
    """Rejection sampling of N(mean, std) restricted to [lo, hi], truncated to integers."""
    out = np.empty(size, dtype=np.float64)
    filled = 0
    while filled < size:
        draw = rng.normal(mean, std, max(2 * (size - filled), 16))
        draw = draw[(draw >= lo) & (draw <= hi)]
        take = min(len(draw), size - filled)
        out[filled:filled + take] = draw[:take]
        filled += take
    return out.astype(np.int64)


def generate_batch_sizes(rng: np.random.Generator, mean: int, std: int, maximum: int, n: int) -> List[int]:
    raw = np.exp(rng.normal(math.log(mean), math.log(std), n)).astype(np.int64)
    sizes = []
    for bs in raw:
        if bs <= maximum:
            sizes.append(max(1, int(bs)))
        else:
            splits = (bs + maximum - 1) // maximum
            last = int(bs % maximum) or maximum
            sizes.append(last if rng.integers(1, splits + 1) == splits else maximum)
    return sizes


def pooling_factors(rng: np.random.Generator, kind: str, params: List[float], n: int) -> Tuple[np.ndarray, float]:
    if kind == "one-hot":
        (coverage,) = params
        return np.ones(n, dtype=np.int64), coverage
    if kind == "multi-hot-static":
        hot, coverage = params
        return np.full(n, int(hot), dtype=np.int64), coverage
    if kind == "multi-hot":
        mean, std, maximum, coverage = params
        return truncated_normal(rng, mean, std, 0, maximum, n), coverage
    if kind == "multi-hot-one-side":
        mean, std, coverage = params
        return truncated_normal(rng, mean, std, 0, np.inf, n), coverage
    raise ValueError(f"unknown feature type {kind!r}")


def write_feature(fname: str, rng: np.random.Generator, hot: np.ndarray, absent: np.ndarray,
                  probabilities: np.ndarray) -> None:
    hot = np.where(absent, 0, hot)
    flat = rng.choice(len(probabilities), int(hot.sum()), replace=True, p=probabilities)
    tmp = fname + ".tmp"
    with open(tmp, "w") as f:
        pos = 0
        for h in hot:
            f.write(",".join(map(str, flat[pos:pos + h])) + "\n")
            pos += h
    os.replace(tmp, fname)


def main():
    args = parse_args()
    os.makedirs(args.output_dir, exist_ok=True)
    groups = parse_data_config(args.config_path)
    rows = [r for r, _ in parse_table_shapes(args.table_config_path)]
    root = np.random.SeedSequence(args.seed_base)

    bs_fname = os.path.join(args.output_dir, "batch_sizes.txt")
    if os.path.exists(bs_fname):
        with open(bs_fname) as f:
            batch_sizes = [int(l) for l in f if l.strip()]
    else:
        rng = np.random.default_rng(root.spawn(1)[0])
        batch_sizes = generate_batch_sizes(rng, args.query_mean, args.query_stddev, args.query_max,
                                           args.num_queries)
        with open(bs_fname + ".tmp", "w") as f:
            f.writelines(f"{bs}\n" for bs in batch_sizes)
        os.replace(bs_fname + ".tmp", bs_fname)
    total = int(sum(batch_sizes))

    feat_id = 0
    for g, (kind, count, params) in enumerate(groups):
        grng = np.random.default_rng(np.random.SeedSequence([args.seed_base, 1, g]))
        # as in the reference, the features of one group share their pooling factors, their
        # absent samples and the row popularity; only the drawn indices differ
        hot, coverage = pooling_factors(grng, kind, params, total)
        absent = grng.random(total) > coverage
        p = grng.power(3.0, rows[feat_id])
        p /= p.sum()
        for _ in range(count):
            fname = os.path.join(args.output_dir, f"f{feat_id}.txt")
            if not os.path.exists(fname):
                print(f"Generating {fname}", flush=True)
                frng = np.random.default_rng(np.random.SeedSequence([args.seed_base, 2, feat_id]))
                if len(p) != rows[feat_id]:
                    raise ValueError(f"features of group {g} must share the table row count")
                write_feature(fname, frng, hot, absent, p)
            feat_id += 1
    if feat_id != len(rows):
        raise ValueError(f"data config describes {feat_id} features, table config {len(rows)}")


if __name__ == "__main__":
    main()
