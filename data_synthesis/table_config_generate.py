"""Write a ``table_config.txt`` (``rows,dim[,dtype]`` per feature) for a ``data_config.txt``.

    python table_config_generate.py -c data_config.txt -t table_config.txt [-d DIM] [--dtype half] [--seed S]

Row counts and the weighted choice of embedding dims per feature type follow the reference's
generator (``data_synthesis/table_config_generate.py:16-23,42-51``): one-hot tables have 1024 rows
and dims {4..128} weighted 8:8:4:2:1:1, multi-hot and multi-hot-static 4096 rows and weights
2:2:2:1:1:1, multi-hot-one-side 16384 rows.  ``-d`` fixes the dim of every table.  Additions:
``--dtype`` appends the element type column (float, half, int8) and ``--seed`` makes the draw
reproducible (the reference draws from the unseeded global ``random`` stream).
"""

import argparse
import random

DIM_CHOICES = (4, 8, 16, 32, 64, 128)
TABLE_RULES = {
    # feature type: (rows, weights of DIM_CHOICES)
    "one-hot": (1024, (8, 8, 4, 2, 1, 1)),
    "multi-hot": (4096, (2, 2, 2, 1, 1, 1)),
    "multi-hot-static": (4096, (2, 2, 2, 1, 1, 1)),
    "multi-hot-one-side": (4096 * 4, (2, 2, 2, 1, 1, 1)),
}


def table_shapes(data_config_path: str, rng: random.Random, fixed_dim: int = None):
    shapes = []
    with open(data_config_path) as f:
        for line in f:
            if not line.strip():
                continue
            kind, count = line.split(",")[:2]
            if kind not in TABLE_RULES:
                raise ValueError(f"unknown feature type {kind!r}")
            rows, weights = TABLE_RULES[kind]
            dims = rng.choices(DIM_CHOICES, weights, k=int(count))
            shapes.extend((rows, fixed_dim or dim) for dim in dims)
    return shapes


if __name__ == "__main__":
    parser = argparse.ArgumentParser()
    parser.add_argument("-c", "--data_config_path", type=str, required=True)
    parser.add_argument("-t", "--table_config_path", type=str, required=True)
    parser.add_argument("-d", "--fixed_embed_dim", type=int)
    parser.add_argument("--dtype", type=str, choices=["float", "half", "int8"])
    parser.add_argument("--seed", type=int)
    args = parser.parse_args()
    rng = random.Random(args.seed)
    with open(args.table_config_path, "w") as f:
        for rows, dim in table_shapes(args.data_config_path, rng, args.fixed_embed_dim):
            f.write(f"{rows},{dim}" + (f",{args.dtype}" if args.dtype else "") + "\n")
