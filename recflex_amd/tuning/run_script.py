"""Profiling driver: runs the fused kernel of a built model over the sampled batches, to be
wrapped in ``rocprofv3 --kernel-trace --stats`` (reference: ``RecFlex/tuning/run_script.py:21-55``
under ``nsys profile``).  ``--data_dir`` is either a dataset directory in the text format
(``batch_sizes.txt`` + ``f{i}.txt``) or a directory of per-feature ``f{i}.npz`` files written by
the tuner."""

import argparse
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

if __name__ == "__main__":
    parser = argparse.ArgumentParser()
    parser.add_argument("--table_config_fname", type=str, required=True)
    parser.add_argument("--build_dir", type=str, required=True)
    parser.add_argument("--data_dir", type=str, required=True)
    parser.add_argument("--spec_feat_id", type=int)
    parser.add_argument("--sample_batch_nums", type=int, required=True)
    parser.add_argument("--seed", type=int, default=0)
    parser.add_argument("--repeats", type=int, default=1)
    parser.add_argument("--tile_bytes", type=int, default=0)
    parser.add_argument("--xcd_segments", type=int, default=0)
    args = parser.parse_args()

    import torch
    from recflex_amd.hip_helper import HipProfiler
    from recflex_amd.host import RecomHost
    from recflex_amd.parser import parse_raw_data_batches, parse_table_dtypes, parse_table_shapes
    from recflex_amd.rec_modules import FeatEmbed
    from recflex_amd.tuning.measure import load_batches, make_table

    table_shapes = parse_table_shapes(args.table_config_fname)
    data_types = parse_table_dtypes(args.table_config_fname)
    feat_ids = list(range(len(table_shapes)))
    if args.spec_feat_id is not None:
        feat_ids = [args.spec_feat_id]
    dev = torch.device("cuda", torch.cuda.current_device())
    tables = [make_table(table_shapes[f], data_types[f], dev, ones=False) for f in feat_ids]
    layer = FeatEmbed(dev, embed_tables=tables, librecom=f"{args.build_dir}/librecom.so")

    if os.path.exists(os.path.join(args.data_dir, "batch_sizes.txt")):
        host = RecomHost()
        fnames = [f"{args.data_dir}/f{f}.txt" for f in feat_ids]
        raw = parse_raw_data_batches(f"{args.data_dir}/batch_sizes.txt", fnames,
                                     args.sample_batch_nums, seed=args.seed, feat_major=True)
        per_feat = [[host.parse_lines(lines) for lines in batches] for batches in raw]
    else:
        per_feat = [load_batches(f"{args.data_dir}/f{f}.npz")[:args.sample_batch_nums] for f in feat_ids]

    device_batches = []
    for k in range(len(per_feat[0])):
        device_batches.append(([torch.from_numpy(b[k][0]).to(dev) for b in per_feat],
                               [torch.from_numpy(b[k][1]).to(dev) for b in per_feat]))
    torch.cuda.synchronize()

    prof = HipProfiler()
    prof.start()
    for _ in range(args.repeats):
        for d_idx, d_off in device_batches:
            output = layer.forward_indices(d_idx, d_off, tile_bytes=args.tile_bytes,
                                           xcd_segments=args.xcd_segments)
    torch.cuda.synchronize()
    prof.stop()
