"""Spread the local-stage results of a compressed model back over the features of the full model.

    python decompress.py -i compress/A -o models/A [--naive]

``compress/A/feat_map.txt`` (written by ``compress.py``) says which original features each
representative stands for; the per-feature result directories ``output/f{k}`` of the compressed
model (``output/naive/f{k}`` with ``--naive``) are copied to ``output/f{j}`` of the full model for
every ``j`` in cluster ``k``, and the compressed model's compile cache (``output/.cache``) with
them.  A following ``tune.py -m models/A --interference replicate`` finds
the libraries and measurements there and goes straight to the global stage.

Same command line and behaviour as the reference's ``examples/decompress.py:14-54``.  (The
in-model local stage keeps one result per occupancy for the whole model instead of per-feature
directories; it shares builds between like features through the compile cache and needs no
compression.)
"""

import argparse
import os
import shutil
from typing import List


def parse_clusters(feat_map_path: str) -> List[List[int]]:
    with open(feat_map_path) as f:
        return [[int(tok) for tok in line.split(",")] for line in f if line.strip()]


def restore_output(src_root: str, dst_root: str, clusters: List[List[int]]) -> int:
    copied = 0
    os.makedirs(dst_root, exist_ok=True)
    for rep_id, members in enumerate(clusters):
        src = os.path.join(src_root, f"f{rep_id}")
        if not os.path.isdir(src):
            raise FileNotFoundError(f"{src}: no local-stage results for representative {rep_id}")
        for feat_id in members:
            shutil.copytree(src, os.path.join(dst_root, f"f{feat_id}"), dirs_exist_ok=True)
            copied += 1
    # the compile cache goes along: the full model's tuner keeps a library it finds only if the
    # cache holds the build of that directory's source under the current device headers
    cache = os.path.join(src_root, ".cache")
    if os.path.isdir(cache):
        shutil.copytree(cache, os.path.join(dst_root, ".cache"), dirs_exist_ok=True)
    return copied


def main():
    parser = argparse.ArgumentParser()
    parser.add_argument("-i", "--input_model_dir", type=str, required=True)
    parser.add_argument("-o", "--output_model_dir", type=str, required=True)
    parser.add_argument("--naive", action="store_true", default=False)
    args = parser.parse_args()
    clusters = parse_clusters(os.path.join(args.input_model_dir, "feat_map.txt"))
    sub = ("output", "naive") if args.naive else ("output",)
    src_root = os.path.join(args.input_model_dir, *sub)
    if args.naive and not os.path.isdir(src_root):
        print(f"{src_root} does not exist: nothing to restore")
        return
    n = restore_output(src_root, os.path.join(args.output_model_dir, *sub), clusters)
    print(f"restored results of {n} features from {len(clusters)} representatives")


if __name__ == "__main__":
    main()
