"""Write a ``schedule_config.txt`` (one line of candidate schedule classes per feature) for a
``data_config.txt``.

    python schedule_config_gen.py -c models/A/data_config.txt -s models/A/schedule_config.txt [--names gfx950]

``--names reference`` (default) writes the reference's class names, as its generator does
(``examples/schedule_config_gen.py:29-41``: ``OneHotSchedule`` for one-hot features,
``ReduceByKeySchedule,OneBlockMultiSampleSchedule,WarpPerSampleSchedule`` for multi-hot ones);
``--names gfx950`` writes the four 64-lane templates these names resolve to.
"""

import argparse

LINES = {
    "reference": {
        "one-hot": "OneHotSchedule",
        "multi-hot": "ReduceByKeySchedule,OneBlockMultiSampleSchedule,WarpPerSampleSchedule",
    },
    "gfx950": {
        "one-hot": "ThreadPerBagSchedule,SubWavefrontPerBagSchedule",
        "multi-hot": "SubWavefrontPerBagSchedule,WavefrontPerBagSchedule,BlockPerBagSchedule",
    },
}
MULTI_HOT_KINDS = ("multi-hot", "multi-hot-static", "multi-hot-one-side")


def schedule_lines(data_config_path: str, names: str):
    out = []
    with open(data_config_path) as f:
        for line in f:
            if not line.strip():
                continue
            kind, count = line.split(",")[:2]
            if kind == "one-hot":
                entry = LINES[names]["one-hot"]
            elif kind in MULTI_HOT_KINDS:
                entry = LINES[names]["multi-hot"]
            else:
                raise ValueError(f"unknown feature type {kind!r}")
            out.extend([entry] * int(count))
    return out


if __name__ == "__main__":
    parser = argparse.ArgumentParser()
    parser.add_argument("-c", "--data_config_path", type=str, required=True)
    parser.add_argument("-s", "--schedule_config_path", type=str, required=True)
    parser.add_argument("--names", type=str, default="reference", choices=sorted(LINES))
    args = parser.parse_args()
    with open(args.schedule_config_path, "w") as f:
        for entry in schedule_lines(args.data_config_path, args.names):
            f.write(entry + "\n")
