"""Writes tests/golden/pooled_small.npz: a small mixed-type model (fp32, fp16, int8 tables,
ragged bags with empties) with the pooled output of the pinned CPU oracle.  The reference ships
no vectors for this path, so these are this repository's own; run from the repository root:

    python tests/golden/make_golden.py
"""

import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import oracle  # noqa: E402


def main():
    rng = np.random.default_rng(20241125)
    specs = [("float", 8, 64), ("half", 16, 40), ("int8", 16, 50), ("float", 3, 9), ("int8", 20, 33)]
    batch = 24
    out = {"num_features": np.int32(len(specs)), "dims": np.array([d for _, d, _ in specs], np.int32),
           "data_types": np.array([t for t, _, _ in specs])}
    tables, idxs, offs = [], [], []
    for f, (dt, dim, rows) in enumerate(specs):
        w = (rng.standard_normal((rows, dim)) * 0.01).astype(np.float32)
        if dt == "half":
            t = w.astype(np.float16)
        elif dt == "int8":
            stride = oracle.int8_row_stride(dim)
            t = np.zeros((rows, stride), np.uint8)
            lo, hi = w.min(1, keepdims=True), w.max(1, keepdims=True)
            bias = lo.astype(np.float16)
            scale = ((hi - lo) / 255).astype(np.float16)
            t[:, :dim] = np.clip(np.rint((w - bias.astype(np.float32)) / scale.astype(np.float32)), 0, 255)
            t[:, dim:dim + 4] = np.concatenate([scale, bias], axis=1).view(np.uint8)
        else:
            t = w
        lens = rng.integers(0, 9, batch)
        lens[f::5] = 0
        off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        idx = rng.integers(0, rows, off[-1]).astype(np.int32)
        tables.append(t); idxs.append(idx); offs.append(off)
        out[f"table{f}"] = t
        out[f"indices{f}"] = idx
        out[f"offsets{f}"] = off
    out["expected"] = oracle.pooled_sum_c(tables, out["dims"].tolist(), [t for t, _, _ in specs], idxs, offs)
    np.savez_compressed(os.path.join(ROOT, "tests", "golden", "pooled_small.npz"), **out)
    print("wrote pooled_small.npz", out["expected"].shape)


if __name__ == "__main__":
    main()
