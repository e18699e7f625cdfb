"""HBM traffic per launch of the prebuilt libraries, as hardware counters gave it.

A live benchmark run cannot read the memory counters; ``rocprofv3 --pmc FETCH_SIZE`` and
``--pmc WRITE_SIZE`` runs of ``bench.py`` can.  This module turns the two counter files of such
runs into one record per model in ``benchaid/hbm_traffic.json`` and hands the figure
back to ``bench.py`` -- but only for the very library it was measured on: every record carries a
key over the model's emitted source and the device headers, and a library built from anything
else gets ``None``.

    python -m benchaid.hbm_traffic record --model c3_tuned \\
        --fetch-csv prof/pmc_fetch_c3/x_counter_collection.csv \\
        --write-csv prof/pmc_write_c3/x_counter_collection.csv --copy-bytes 805306368

``FETCH_SIZE`` / ``WRITE_SIZE`` are what the L2 caches exchange with the memory side, in units
that a plain copy of known size calibrates: the runs hold one device-to-device copy of
``--copy-bytes`` bytes by a kernel of a name no library shares, ``CalibrationCopyKnl``
(``bench.py --copy-calibration``), and each counter is scaled by bytes copied / counter reading
of that dispatch.
"""

import argparse
import csv
import glob
import hashlib
import json
import os
from typing import Dict, List, Optional, Tuple

from recflex_amd.code_emitter.build_basic import BasicBuilder
from recflex_amd import prebuilt

CALIBRATION_KERNEL = "CalibrationCopyKnl"      # launched by gather_probe.calibration_copy

RECORD_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "hbm_traffic.json")


def library_key(model: str) -> Optional[str]:
    """Key of what the model's kernels are built from: its emitted ``process.hip`` and the
    device-code headers (``csrc/include/*.h``; the C-ABI header only shapes host code).  ``None``
    if the model was never emitted here."""
    src = os.path.join(prebuilt.model_dir(model), "process.hip")
    if not os.path.exists(src):
        return None
    basic = BasicBuilder()
    h = hashlib.sha256()
    for path in [src] + [p for p in basic.device_headers() if os.path.dirname(p) == basic.include]:
        with open(path, "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:24]


def load_records() -> Dict[str, dict]:
    if not os.path.exists(RECORD_PATH):
        return {}
    with open(RECORD_PATH) as f:
        return json.load(f)


def recorded_traffic(model: str) -> Optional[dict]:
    """Memory-side bytes per launch of ``FusedKnl`` of this model (``bytes``, ``read_bytes``,
    ``written_bytes``, ``source``), if counters were taken on the library as it is built now;
    ``None`` otherwise."""
    rec = load_records().get(model)
    if not rec or rec.get("key") != library_key(model):
        return None
    return {"bytes": float(rec["bytes"]), "read_bytes": float(rec["read_bytes"]),
            "written_bytes": float(rec["written_bytes"]),
            "source": "recorded in benchaid/hbm_traffic.json for this library (key over its emitted "
                      "source and the device headers)" + (": " + rec["note"] if rec.get("note") else "")}


def recorded_traffic_bytes(model: str) -> Optional[float]:
    rec = recorded_traffic(model)
    return rec["bytes"] if rec else None


def _counter_files(path: str) -> List[str]:
    if os.path.isfile(path):
        return [path]
    return sorted(glob.glob(os.path.join(path, "**", "*counter_collection.csv"), recursive=True))


def read_counter(path: str, counter: str) -> Dict[str, List[float]]:
    """kernel name -> value of ``counter`` per dispatch, from rocprofv3 ``--pmc`` csv output."""
    out: Dict[str, List[float]] = {}
    for fname in _counter_files(path):
        with open(fname, newline="") as f:
            for row in csv.DictReader(f):
                if row.get("Counter_Name") == counter:
                    out.setdefault(row["Kernel_Name"], []).append(float(row["Counter_Value"]))
    if not out:
        raise ValueError(f"no {counter} readings under {path}")
    return out


def _fused_and_copy(readings: Dict[str, List[float]], copy_substr: str,
                    skip_first: int = 0) -> Tuple[float, int, float]:
    """(mean reading of FusedKnl after its first ``skip_first`` dispatches, the dispatches that
    count, reading of the one calibration copy)."""
    fused = (readings.get("FusedKnl") or [])[skip_first:]
    if not fused:
        raise ValueError("the counter file holds no FusedKnl dispatch")
    copies = [v for name, vals in readings.items() if copy_substr in name for v in vals]
    if not copies:
        raise ValueError(f"the counter file holds no kernel named *{copy_substr}* to calibrate with")
    if len(copies) != 1:
        raise ValueError(f"{len(copies)} dispatches named *{copy_substr}*: the calibration needs exactly one")
    return sum(fused) / len(fused), len(fused), copies[0]


def traffic_from_counter_files(fetch_csv: str, write_csv: str, copy_bytes: int,
                               copy_substr: str = CALIBRATION_KERNEL, skip_first: int = 0) -> dict:
    """Bytes per launch of FusedKnl from a FETCH_SIZE and a WRITE_SIZE run (files or directories
    of rocprofv3 ``--pmc`` csv output), each counter scaled by its reading for the calibration
    copy of ``copy_bytes`` bytes in the same run; the first ``skip_first`` FusedKnl dispatches of
    each run (warm-up launches) are left out of the mean."""
    fetch, n_fetch, copy_fetch = _fused_and_copy(read_counter(fetch_csv, "FETCH_SIZE"), copy_substr, skip_first)
    write, n_write, copy_write = _fused_and_copy(read_counter(write_csv, "WRITE_SIZE"), copy_substr, skip_first)
    fetch_factor = copy_bytes / copy_fetch          # bytes per counter unit
    write_factor = copy_bytes / copy_write
    return {
        "fetch_reading": fetch, "write_reading": write,
        "fetch_bytes_per_unit": fetch_factor, "write_bytes_per_unit": write_factor,
        "read_bytes": fetch * fetch_factor, "written_bytes": write * write_factor,
        "bytes": fetch * fetch_factor + write * write_factor,
        "dispatches": [n_fetch, n_write],
        "calibration": f"the {copy_substr} dispatch = a copy of {copy_bytes} bytes",
    }


def record(model: str, fetch_csv: str, write_csv: str, copy_bytes: int,
           copy_substr: str = CALIBRATION_KERNEL, skip_first: int = 0, note: str = "") -> dict:
    key = library_key(model)
    if key is None:
        raise FileNotFoundError(f"{prebuilt.model_dir(model)}/process.hip: build the model first")
    rec = dict(traffic_from_counter_files(fetch_csv, write_csv, copy_bytes, copy_substr, skip_first), key=key)
    if note:
        rec["note"] = note
    records = load_records()
    records[model] = rec
    with open(RECORD_PATH, "w") as f:
        json.dump(records, f, indent=1, sort_keys=True)
    return rec


def main() -> None:
    parser = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    sub = parser.add_subparsers(dest="cmd", required=True)
    rec = sub.add_parser("record", help="turn a FETCH_SIZE and a WRITE_SIZE run into a record")
    rec.add_argument("--model", required=True, help="prebuilt model name, e.g. c3_tuned")
    rec.add_argument("--fetch-csv", required=True)
    rec.add_argument("--write-csv", required=True)
    rec.add_argument("--copy-bytes", type=int, required=True)
    rec.add_argument("--copy-kernel", default=CALIBRATION_KERNEL, help="substring of the copy kernel's name")
    rec.add_argument("--skip-first", type=int, default=0, help="FusedKnl dispatches to leave out (warm-up)")
    rec.add_argument("--note", default="", help="how the runs were made, kept with the record")
    sub.add_parser("show", help="print the records and whether each matches the library as built now")
    args = parser.parse_args()
    if args.cmd == "record":
        print(json.dumps(record(args.model, args.fetch_csv, args.write_csv, args.copy_bytes,
                                args.copy_kernel, args.skip_first, args.note), indent=1))
    else:
        for model, r in load_records().items():
            print(f"{model}: {r['bytes'] / 1e6:.1f} MB per launch "
                  f"({'current' if r['key'] == library_key(model) else 'STALE: library changed'})")


if __name__ == "__main__":
    main()
