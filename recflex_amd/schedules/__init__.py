"""Schedule templates for the gfx950 fused embedding kernel.

``SCHEDULE_MAPPING`` plays the role of ``globals()`` of the reference's ``examples/tune.py``
(``tune.py:78`` passes it as ``schedule_mapping``): class name in ``schedule_config.txt`` ->
schedule class.
"""

from typing import Dict, NamedTuple, Tuple, Type

from recflex_amd.code_emitter.schedule_base import ScheduleBase, MetaData
from .team import (TeamParams, TeamScheduleBase, ThreadPerBagSchedule, ThreadPerBagParams,
                   SubWavefrontPerBagSchedule, SubWavefrontPerBagParams,
                   WavefrontPerBagSchedule, WavefrontPerBagParams, OneHotBagSchedule,
                   OneHotBagParams, next_pow2)
from .block_per_bag import BlockPerBagSchedule, BlockPerBagParams, SplitBagSchedule
from .reference_names import (OneHotSchedule, OneHotMultiBlockSchedule, WarpPerSampleSchedule,
                              OneBlockMultiSampleSchedule, MultiBlockPerSampleSchedule,
                              ReduceByKeySchedule, OneHotParams, OneHotMultiBlockParams,
                              WarpPerSampleParams, OneBlockMultiSampleParams,
                              MultiBlockPerSampleParams, ReduceByKeyParams)

SCHEDULE_MAPPING: Dict[str, Type[ScheduleBase]] = {
    cls.__name__: cls
    for cls in (ThreadPerBagSchedule, SubWavefrontPerBagSchedule, WavefrontPerBagSchedule,
                OneHotBagSchedule, BlockPerBagSchedule, SplitBagSchedule, OneHotSchedule, OneHotMultiBlockSchedule,
                WarpPerSampleSchedule, OneBlockMultiSampleSchedule,
                MultiBlockPerSampleSchedule, ReduceByKeySchedule)
}

PARAM_TYPES: Dict[str, Type[NamedTuple]] = {
    "ThreadPerBagSchedule": ThreadPerBagParams,
    "SubWavefrontPerBagSchedule": SubWavefrontPerBagParams,
    "WavefrontPerBagSchedule": WavefrontPerBagParams,
    "BlockPerBagSchedule": BlockPerBagParams,
    "SplitBagSchedule": BlockPerBagParams,
    "OneHotBagSchedule": OneHotBagParams,
    "OneHotSchedule": OneHotBagParams,
    "OneHotMultiBlockSchedule": OneHotBagParams,
    "WarpPerSampleSchedule": TeamParams,
    "OneBlockMultiSampleSchedule": TeamParams,
    "MultiBlockPerSampleSchedule": BlockPerBagParams,
    "ReduceByKeySchedule": BlockPerBagParams,
}


def default_schedule(meta: MetaData, mean_bag_len: float = 1.0, block_threads: int = 256,
                     one_hot: bool = False) -> Tuple[ScheduleBase, NamedTuple]:
    """Untuned starting point for one feature from its row size and mean bag length
    (``one_hot``: no bag of the feature is known to hold more than one lookup -- the row-copy
    template): enough
    column lanes that a lane owns one or two 16-byte vectors, lookup lanes only for long bags,
    and two to four independent row loads in flight per lane -- fewer for fp16 and int8 rows,
    whose 8 or 16 fp32 accumulators per 16-byte vector would otherwise push the fused kernel past
    the registers that four or five workgroups per CU leave it (measured on C4 and C5: 2 % and
    17 % faster than with four loads in flight everywhere)."""
    if one_hot:
        sched = OneHotBagSchedule(meta, block_threads)
        return sched, sched.default_params()
    v = meta.row_vectors
    x = min(64, next_pow2(v))
    if v > 1 and x * meta.vec_bytes >= 256 and mean_bag_len < 8:
        x //= 2                      # short bags of wide rows: two vectors per lane
    vpl = -(-v // x)
    acc_floats = vpl * meta.elems_per_vector          # accumulators of one bag per lane
    if mean_bag_len <= 1.5:
        bags = 4 if 4 * acc_floats <= 16 else (2 if 2 * acc_floats <= 16 else 1)
        team = x
        if team == 1:
            return ThreadPerBagSchedule(meta, block_threads), ThreadPerBagParams(1, bags, vpl)
        if team == 64:
            return WavefrontPerBagSchedule(meta, block_threads), WavefrontPerBagParams(64, 1, vpl)
        return (SubWavefrontPerBagSchedule(meta, block_threads),
                SubWavefrontPerBagParams(x, 1, 1, bags, vpl))
    items = 4 if acc_floats <= 8 else 2
    if mean_bag_len >= 96 and meta.payload_bytes >= 512 and vpl * meta.elems_per_vector < 16:
        # long bags of wide rows: fewer column lanes, each with 16 accumulators (4 fp32 or 2 fp16
        # vectors), so that four (two) times as many lookups are in flight per wavefront -- the
        # move the production-build climb makes first on C3 (fp32, D=128) and C4 (fp16, D=256)
        vpl = max(1, 16 // meta.elems_per_vector)
        x = max(1, next_pow2(v) // vpl)
        vpl = -(-v // x)
        items = 2
    if mean_bag_len < 24:
        y = 1
    elif mean_bag_len < 96:
        y = max(1, min(4, 64 // x))
    else:
        y = max(1, 64 // x)
    if mean_bag_len >= 512 and next_pow2(v) >= 4:
        # the whole workgroup on one bag, one row vector per lane -- and several workgroups per
        # bag when the batch holds so few bags that one of them is a good part of a workgroup's
        # share (8 features x 64 bags x 4 000 lookups: 105 us against 203 us with a team per bag)
        return (SplitBagSchedule(meta, block_threads),
                BlockPerBagParams(min(64, next_pow2(v)), 4 if meta.elems_per_vector <= 4 else 2,
                                  4 * block_threads))
    team = x * y
    if team == 1:
        return ThreadPerBagSchedule(meta, block_threads), ThreadPerBagParams(items, 1, vpl)
    if team == 64:
        return WavefrontPerBagSchedule(meta, block_threads), WavefrontPerBagParams(x, items, vpl)
    return (SubWavefrontPerBagSchedule(meta, block_threads),
            SubWavefrontPerBagParams(x, y, items, 1, vpl))


def schedule_from_config(entry: dict, meta: MetaData, block_threads: int = 256
                         ) -> Tuple[ScheduleBase, NamedTuple]:
    """Inverse of ``CodeEmitter.serialize_config`` for one feature:
    ``{"schedule": ClassName, "params": {...}}`` -> (schedule object, params tuple)."""
    name = entry["schedule"]
    if name not in SCHEDULE_MAPPING:
        raise KeyError(f"unknown schedule class {name!r}")
    return SCHEDULE_MAPPING[name](meta, block_threads), PARAM_TYPES[name](**entry["params"])
