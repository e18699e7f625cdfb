"""Fused embedding + MLP end to end: host preprocess outside the timed region, then
``RecomModel`` (fused lookup, reshape, ReLU MLP, sigmoid) per batch.

    python end_to_end.py -t models/test/table_config.txt -b models/test/output/optimal/build \\
                         -d models/test/data [-l 1024 256 128] [--sample_batch_nums N] [-o out.txt]

Flags as in the reference's ``examples/end_to_end.py:25-35``; the embedding layer runs the gfx950
fused kernel of ``<build_dir>/librecom.so``, the MLP is stock PyTorch-ROCm.
"""

import argparse
import os
import sys
import time
from typing import List

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

import torch

from recflex_amd.hip_helper import HipProfiler
from recflex_amd.parser import parse_raw_data_batches, parse_table_shapes
from recflex_amd.rec_modules import FeatPreprocess, RecomModel, load_library
from recflex_amd.utils import find_file, import_from_path


def parse_args() -> argparse.Namespace:
    parser = argparse.ArgumentParser()
    parser.add_argument("-l", "--mlp_unit_nums", type=int, nargs="+", default=[1024, 256, 128])
    parser.add_argument("-t", "--table_config_fname", type=str, required=True)
    parser.add_argument("-b", "--build_dir", type=str, required=True)
    parser.add_argument("-d", "--data_dir", type=str, required=True)
    parser.add_argument("-o", "--output", type=str)
    parser.add_argument("--sample_batch_nums", type=int, default=128)
    parser.add_argument("--seed", type=int, default=0)
    return parser.parse_args()


def measure(preprocess: FeatPreprocess, recom_model: RecomModel, max_concurrent_blocks: int,
            raw_data_batches: List[List[List[str]]]) -> float:
    accum_time_ms = 0.0
    for raw_data in raw_data_batches:
        preprocess_result = preprocess(raw_data, max_concurrent_blocks)
        torch.cuda.synchronize()
        start = time.perf_counter()
        output = recom_model(*preprocess_result)
        torch.cuda.synchronize()
        accum_time_ms += (time.perf_counter() - start) * 1000
    return accum_time_ms


def main():
    args = parse_args()
    lib = load_library(f"{args.build_dir}/librecom.so")
    recom_host = import_from_path("recom_host", find_file(args.build_dir, "recom_host*.so"))

    table_shapes = parse_table_shapes(args.table_config_fname)
    data_fnames = [f"{args.data_dir}/f{feat_id}.txt" for feat_id in range(len(table_shapes))]
    raw_data_batches = parse_raw_data_batches(f"{args.data_dir}/batch_sizes.txt", data_fnames,
                                              args.sample_batch_nums, seed=args.seed, feat_major=False)

    dev = torch.device("cuda", torch.cuda.current_device())
    recom_model = RecomModel(args.mlp_unit_nums, dev, table_shapes=table_shapes, librecom=lib)
    preprocess = FeatPreprocess(recom_host, dev, output_units=recom_model.embed_layer.output_units)

    prof = HipProfiler()
    prof.start()
    t = measure(preprocess, recom_model, recom_model.embed_layer.max_concurrent_blocks, raw_data_batches)
    prof.stop()

    print(f"Accumulated end-to-end time (ms): {t}")
    if args.output:
        with open(args.output, "w") as f:
            f.write(str(t))


if __name__ == "__main__":
    main()
