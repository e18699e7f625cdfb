"""Run a tuned (or freshly built) model end to end on its dataset and optionally check the
results.

    python test.py -m models/test -o models/test/output/optimal [--check] [-g OCC]
                   [--sample_batch_nums N] [--seed S] [--recompile]

Flags as in the reference's ``examples/test.py:37-50``.  ``-o`` is a directory holding
``build/librecom.so`` (e.g. ``<model>/output/optimal`` left by ``tune.py``); if the library is
missing it is built there with default schedules chosen from the data (the reference builds
with an empty schedule list at this point, ``test.py:117-118``, which cannot work).
``--check`` compares every sample of every feature with ``F.embedding(indices, table).sum(0)``
within ``atol = rtol = 1e-4`` for fp32 tables, exactly the reference's check
(``test.py:68-86``); fp16 / int8 tables are compared after decoding the rows to fp32.
"""

import argparse
import os
import sys
import time
from typing import List

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

import numpy as np
import torch
import torch.nn.functional as F

from recflex_amd.rec_modules import FeatProcessEmbed
from recflex_amd.parser import parse_raw_data_batches, parse_table_shapes
from recflex_amd.utils import import_from_path, find_file, compile_build
from recflex_amd.hip_helper import HipProfiler
from recflex_amd.schedules import default_schedule
from recflex_amd.model_build import DEFAULT_XCD_SEGMENTS

from tune import create_tuner


def parse_args() -> argparse.Namespace:
    parser = argparse.ArgumentParser()
    parser.add_argument("-m", "--model_dir", type=str, required=True)
    parser.add_argument("-o", "--output_dir", type=str, required=True)
    parser.add_argument("-n", "--num_processes", type=int, default=8)
    parser.add_argument("-b", "--block_threads", type=int, default=256)
    parser.add_argument("-g", "--occupancy", type=int)
    parser.add_argument("--sample_batch_nums", type=int, default=1)
    parser.add_argument("--seed", type=int, default=0)
    parser.add_argument("--recompile", action="store_true", default=False)
    parser.add_argument("--check", action="store_true", default=False)
    parser.add_argument("--debug", action="store_true", default=False)
    return parser.parse_args()


def build_targets(args: argparse.Namespace, tuner) -> str:
    build_dir = os.path.join(args.output_dir, "build")
    if not os.path.exists(f"{build_dir}/librecom.so") or args.recompile:
        mean_lens = [float(np.mean([len(i) / max(1, len(o) - 1) for i, o in feat])) for feat in tuner.batches]
        feat_schedules = [default_schedule(meta, pf, tuner.basic.block_threads)
                          for meta, pf in zip(tuner.metas, mean_lens)]
        tuner.emit_codes(args.output_dir, feat_schedules, args.occupancy, debug=args.debug,
                         xcd_segments=DEFAULT_XCD_SEGMENTS)
        compile_build(build_dir)
    return build_dir


def decode_table(table: torch.Tensor, dim: int) -> torch.Tensor:
    """Host table in its storage format -> fp32 [rows, dim]."""
    if table.dtype == torch.float32:
        return table
    if table.dtype == torch.float16:
        return table.float()
    codes = table[:, :dim].float()
    sb = table[:, dim:dim + 4].contiguous().view(torch.float16).float()
    return codes * sb[:, 0:1] + sb[:, 1:2]


def check_results(results: torch.Tensor, h_embed_tables: List[torch.Tensor], raw_data: List[List[str]]):
    dim_sum = sum(t.shape[1] for t in h_embed_tables)
    results = torch.reshape(results, [-1, dim_sum]).cpu()
    dim_offset = 0
    for raw, table in zip(raw_data, h_embed_tables):
        next_dim_offset = dim_offset + table.shape[1]
        for sid, row in enumerate(raw):
            indices = [] if row == "" else list(map(int, row.strip().split(',')))
            pooling = F.embedding(torch.LongTensor(indices), table).sum(0)
            assert torch.allclose(pooling, results[sid, dim_offset:next_dim_offset], atol=1e-4, rtol=1e-4), \
                f"sample {sid}, columns [{dim_offset}, {next_dim_offset})"
        dim_offset = next_dim_offset


def measure(model: FeatProcessEmbed, raw_data_batches: List[List[List[str]]], check: bool = False) -> float:
    if check:
        dims = model.embed_layer.lib.embed_dims
        h_embed_tables = [decode_table(t.cpu(), d) for t, d in zip(model.embed_layer.embed_tables, dims)]
    prof = HipProfiler()
    prof.start()
    accum_time_ms = 0
    for raw_data in raw_data_batches:
        start = time.perf_counter()
        output = model(raw_data)
        torch.cuda.synchronize()
        end = time.perf_counter()
        if check:
            check_results(output, h_embed_tables, raw_data)
        accum_time_ms += (end - start) * 1000
    prof.stop()
    return accum_time_ms


def main():
    args = parse_args()
    os.makedirs(args.output_dir, exist_ok=True)
    tuner = create_tuner(args)
    build_dir = build_targets(args, tuner)

    recom_host = import_from_path("recom_host", find_file(build_dir, "recom_host*.so"))
    table_shapes = parse_table_shapes(tuner.basic.table_config_fname)
    raw_data_batches = parse_raw_data_batches(tuner.basic.batch_sizes_fname, tuner.basic.data_fnames,
                                              args.sample_batch_nums, seed=args.seed, feat_major=False)

    model = FeatProcessEmbed(recom_host, torch.device("cuda", torch.cuda.current_device()),
                             table_shapes=table_shapes, librecom_path=f"{build_dir}/librecom.so")
    t = measure(model, raw_data_batches, args.check)
    print(f"Accumulated end-to-end time (ms): {t}")
    if args.check:
        print("check passed")


if __name__ == "__main__":
    main()
