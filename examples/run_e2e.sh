#!/bin/bash
# End-to-end (fused embedding + MLP) GPU time of tuned models under rocprofv3, summed over kernels
# (reference: examples/run_e2e.sh, with nsys).  Appends "<model>,<ms>" to end_to_end/result.txt.
set -e
cd "$(dirname "$0")"
outdir=end_to_end
mkdir -p $outdir
for m in "$@"; do
  rocprofv3 --kernel-trace --stats --output-format csv -d $outdir/$m -o $m -- \
    python3 end_to_end.py -t models/$m/table_config.txt -b models/$m/output/optimal/build -d models/$m/data
  python3 - "$m" $outdir/$m >> $outdir/result.txt <<'PY'
import csv, glob, sys
total = 0.0
for path in glob.glob(sys.argv[2] + "/**/*kernel_stats.csv", recursive=True):
    with open(path, newline="") as f:
        total += sum(float(row["TotalDurationNs"]) for row in csv.DictReader(f))
print(f"{sys.argv[1]},{total / 1e6}")
PY
done
