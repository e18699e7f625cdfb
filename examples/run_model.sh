#!/bin/bash
# Tune model $1 the way the reference's examples/run_model.sh does: local stage on the compressed
# model (one representative per cluster of like features, candidates timed against copies of
# themselves), results spread back, then the global stage on the full model.  One MI355X.
set -e
cd "$(dirname "$0")"
m=$1
mkdir -p compress
python compress.py -m models/$m -o compress/$m
python tune.py -m compress/$m -o compress/$m/output -n 16 --local_only --interference replicate
python decompress.py -i compress/$m -o models/$m
python tune.py -m models/$m -o models/$m/output -n 16 --interference replicate
