#!/bin/bash
# Smallest complete run on one MI355X (the counterpart of the reference's examples/test.sh):
# generate a tiny dataset for models/test, tune it, check the tuned kernel, run it end to end.
set -e
cd "$(dirname "$0")"
mdir=models/test
python ../data_synthesis/data_generate.py -c $mdir/data_config.txt -t $mdir/table_config.txt --num_queries 32 -o $mdir/data
python tune.py -m $mdir -o $mdir/output -n 8 --occupancies 2,4,8 --profiler events --build_climb_trials 16
python test.py -m $mdir -o $mdir/output/optimal --check --sample_batch_nums 4
python end_to_end.py -t $mdir/table_config.txt -b $mdir/output/optimal/build -d $mdir/data --sample_batch_nums 8
