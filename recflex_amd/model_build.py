"""Emit and build the fused-kernel library of one model outside the tuner: used by tests,
``bench.py`` and the example scripts.  Same steps as ``Tuner.emit_codes`` followed by
``compile_build`` in the reference (``RecFlex/tuning/tuner.py:101-110``, ``RecFlex/utils.py:27-36``).
"""

import json
import os
from typing import List, NamedTuple, Optional, Sequence, Tuple

from .code_emitter import CodeEmitter, MetaData, ScheduleBase
from .schedules import default_schedule, schedule_from_config
from .utils import compile_build

FeatSchedules = List[Tuple[ScheduleBase, NamedTuple]]


# Tile walk of a model that was not tuned: the tile space in 8 x 16 segments, one XCD each
# (with the per-batch tile size, measured against the flat walk: C3 125 vs 131 us, C4 4.92 vs
# 5.02 ms, C5 and C2 unchanged)
DEFAULT_XCD_SEGMENTS = 16


def emit_model(output_dir: str, feat_schedules: FeatSchedules, occupancy: Optional[int] = None,
               inline: bool = True, timing: bool = False, tune: bool = False,
               fixed_task_block_nums: List[int] = None, tile_bytes: int = None,
               debug: bool = False, host: bool = True, xcd_aware: bool = True,
               lookup_overhead_bytes: int = None, xcd_segments: int = DEFAULT_XCD_SEGMENTS,
               outliers: bool = False, bind_once: bool = None, tile_order: List[int] = None,
               drawn_tail: int = 0) -> None:
    os.makedirs(output_dir, exist_ok=True)
    emitter = CodeEmitter(feat_schedules)
    if host:
        emitter.emit_host(f"{output_dir}/preprocess.cpp", fixed_task_block_nums=fixed_task_block_nums)
    emitter.emit(f"{output_dir}/process.hip", occupancy=occupancy, timing=timing, inline=inline,
                 tune=tune, fixed_task_block_nums=fixed_task_block_nums, tile_bytes=tile_bytes,
                 xcd_aware=xcd_aware, lookup_overhead_bytes=lookup_overhead_bytes, xcd_segments=xcd_segments,
                 outliers=outliers, bind_once=bind_once, tile_order=tile_order, drawn_tail=drawn_tail)
    emitter.emit_cmake_list(f"{output_dir}/CMakeLists.txt", code_fname="process.hip",
                            host_fname="preprocess.cpp" if host else None, debug=debug)
    emitter.dump_key(f"{output_dir}/schedule.json")


def build_model(output_dir: str, feat_schedules: FeatSchedules, rebuild: bool = True,
                **emit_kwargs) -> str:
    """Returns the path of ``librecom.so``.  With ``rebuild=False`` an existing library is kept
    (the reference's resume-by-files rule, tuner.py:117)."""
    lib = f"{output_dir}/build/librecom.so"
    if rebuild or not os.path.exists(lib):
        emit_model(output_dir, feat_schedules, **emit_kwargs)
        if os.path.exists(lib):
            os.remove(lib)          # compile even if make would call the old library current
        compile_build(f"{output_dir}/build")
    return lib


def default_feat_schedules(metas: Sequence[MetaData], mean_bag_lens: Sequence[float],
                           block_threads: int = 256, one_hot: Sequence[bool] = None) -> FeatSchedules:
    """``one_hot[f]``: no bag of feature ``f`` holds more than one lookup, as far as is known."""
    one_hot = one_hot or [False] * len(metas)
    return [default_schedule(m, l, block_threads, one_hot=h)
            for m, l, h in zip(metas, mean_bag_lens, one_hot)]


def feat_schedules_from_entries(entries: Sequence[dict], block_threads: int = 256) -> FeatSchedules:
    """The schedules that ``CodeEmitter.serialize_config`` wrote as a list of entries."""
    return [schedule_from_config(e, MetaData(e["embed_dim"], e.get("data_type", "float")), block_threads)
            for e in entries]


def load_feat_schedules(schedule_json: str, block_threads: int = 256) -> FeatSchedules:
    """Read back what ``CodeEmitter.dump_key`` / ``serialize_config`` wrote."""
    with open(schedule_json) as f:
        return feat_schedules_from_entries(json.load(f), block_threads)
