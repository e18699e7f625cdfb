"""A tuned model's choices carried over to a model of the same family.

The reference's example models A-F are drawn from the same generator families (dims, table
sizes, bag-length distributions); tuning the largest of them feature by feature takes hours.
What the tuner decided for one kind of feature -- row width and type, bag-length class, the
schedule the default heuristic gives it -- on a model it did tune can be adopted for the
features of the same kind in another model, where the picks for that kind agree.  The result is
a schedule file like any other; whether it beats the default mix on the new model is for the
tuner's global stage to measure (``examples/tune.py --launch_only --incumbent <file>``).
"""

import collections
import json
from typing import Dict, List, Sequence, Tuple


def feature_kind(dim: int, data_type: str, mean_bag: float, default_entry: dict) -> Tuple:
    """Features of one kind share row width, row type, bag-length class (exact below four
    lookups, steps of eight above) and the default heuristic's schedule and parameters."""
    bag_class = round(mean_bag) if mean_bag < 4 else int(mean_bag) // 8 * 8
    return (dim, data_type, bag_class, default_entry["schedule"],
            json.dumps(default_entry["params"], sort_keys=True))


def transfer_schedule(src_feats: Sequence[Tuple[int, str, float]], src_default: List[dict],
                      src_tuned: List[dict], dst_feats: Sequence[Tuple[int, str, float]],
                      dst_default: List[dict], agree: float = 0.8) -> Tuple[List[dict], Dict[str, int]]:
    """``*_feats``: (embed_dim, data_type, mean bag length) per feature; ``*_default`` /
    ``src_tuned``: schedule entries (``serialize_config`` form) per feature.  Returns the
    destination's entries -- the default's, with the source's tuned pick wherever at least
    ``agree`` of the source's features of that kind got the same pick -- and counts
    (``changed``, ``kept``, ``unknown_kind``)."""
    if not (len(src_feats) == len(src_default) == len(src_tuned)) or len(dst_feats) != len(dst_default):
        raise ValueError("one entry per feature, please")
    votes: Dict[Tuple, collections.Counter] = collections.defaultdict(collections.Counter)
    for feat, default, tuned in zip(src_feats, src_default, src_tuned):
        pick = json.dumps({"schedule": tuned["schedule"], "params": tuned["params"]}, sort_keys=True)
        votes[feature_kind(*feat, default)][pick] += 1
    rule = {}
    for kind, counter in votes.items():
        pick, n = counter.most_common(1)[0]
        if n >= agree * sum(counter.values()):
            rule[kind] = json.loads(pick)
    out, counts = [], {"changed": 0, "kept": 0, "unknown_kind": 0}
    for feat, default in zip(dst_feats, dst_default):
        entry = dict(default)
        pick = rule.get(feature_kind(*feat, default))
        if pick is None:
            counts["unknown_kind"] += 1
        elif pick["schedule"] == default["schedule"] and pick["params"] == default["params"]:
            counts["kept"] += 1
        else:
            entry.update(schedule=pick["schedule"], params=pick["params"])
            counts["changed"] += 1
        out.append(entry)
    return out, counts
