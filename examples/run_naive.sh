#!/bin/bash
# Ablation: per-feature tuning without interference (every candidate alone on the device), the
# counterpart of the reference's examples/run_naive.sh.  Expects compress/$1 (see run_model.sh).
set -e
cd "$(dirname "$0")"
m=$1
python tune.py -m compress/$m -o compress/$m/output -n 16 --local_only --naive
python decompress.py -i compress/$m -o models/$m --naive
python tune.py -m models/$m -o models/$m/output -n 16 --naive
