#!/bin/bash
# Ablation: thread binding fixed at emit time from the mean / the maximum workload of the sampled
# batches instead of computed per batch on the device (reference: examples/run_fixed_thread.sh).
set -e
cd "$(dirname "$0")"
for m in "$@"; do
  python tune.py -m models/$m -o models/$m/output -n 16 --fixed_thread_binding --thread_binding_choice mean
  python tune.py -m models/$m -o models/$m/output -n 16 --fixed_thread_binding --thread_binding_choice max
done
