"""Schedule templates under the module paths the reference's scripts import them from
(``examples/schedules/*.py`` of the reference: ``from schedules.one_hot import OneHotSchedule,
OneHotParams`` and its five siblings); the implementations live in ``recflex_amd.schedules``.

The six submodules hold nothing of their own, so they are made here instead of kept as files:
each is a module object that carries the schedule class and the parameter tuple of its name."""

import sys
import types

import recflex_amd.schedules as _impl
from recflex_amd.schedules import *  # noqa: F401,F403

_SUBMODULES = {
    "one_hot": "OneHot",
    "one_hot_multi_block": "OneHotMultiBlock",
    "warp_per_sample": "WarpPerSample",
    "one_block_multi_sample": "OneBlockMultiSample",
    "multi_block_per_sample": "MultiBlockPerSample",
    "reduce_by_key": "ReduceByKey",
}

for _mod, _stem in _SUBMODULES.items():
    _m = types.ModuleType(f"{__name__}.{_mod}", f"{_stem}Schedule and {_stem}Params of recflex_amd.schedules")
    setattr(_m, f"{_stem}Schedule", getattr(_impl, f"{_stem}Schedule"))
    setattr(_m, f"{_stem}Params", getattr(_impl, f"{_stem}Params"))
    sys.modules[_m.__name__] = _m
    globals()[_mod] = _m
