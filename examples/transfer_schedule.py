"""Carry a tuned schedule over to another built-in workload of the same family.

    python transfer_schedule.py --from_workload refa --from_schedule ../recflex_amd/tuned/refa_schedule.json \\
        --to_workload reff4 -o reff4_from_refa.json
    python tune.py --workload reff4 --launch_only --incumbent reff4_from_refa.json ...

The second command lets the tuner's global stage time the result against the default mix."""

import argparse
import json
import os
import sys

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))

from recflex_amd import prebuilt                                    # noqa: E402
from recflex_amd.code_emitter import CodeEmitter                    # noqa: E402
from recflex_amd.tuning.transfer import transfer_schedule           # noqa: E402


def main() -> None:
    parser = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    parser.add_argument("--from_workload", required=True, help="built-in workload the schedule was tuned for")
    parser.add_argument("--from_schedule", required=True, help="its schedule.json")
    parser.add_argument("--to_workload", required=True, help="built-in workload to write a schedule for")
    parser.add_argument("--agree", type=float, default=0.8,
                        help="share of a kind's features that must have got the same pick")
    parser.add_argument("-o", "--output", required=True)
    args = parser.parse_args()

    src, dst = prebuilt.model_spec(args.from_workload), prebuilt.model_spec(args.to_workload)
    with open(args.from_schedule) as f:
        doc = json.load(f)
    tuned = doc["schedules"] if isinstance(doc, dict) else doc
    feats = lambda spec: [(ft.dim, ft.data_type, ft.mean_bag) for ft in spec.workload.features]
    entries, counts = transfer_schedule(feats(src), CodeEmitter(src.feat_schedules).serialize_config(), tuned,
                                        feats(dst), CodeEmitter(dst.feat_schedules).serialize_config(),
                                        agree=args.agree)
    with open(args.output, "w") as f:
        json.dump({"occupancy": doc.get("occupancy") if isinstance(doc, dict) else None,
                   "schedules": entries}, f, indent=1)
    print(f"{args.output}: {counts['changed']} of {len(entries)} features changed, {counts['kept']} kept "
          f"their default on the source's word, {counts['unknown_kind']} of a kind the source does not have")


if __name__ == "__main__":
    main()
