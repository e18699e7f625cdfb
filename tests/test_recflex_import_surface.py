"""The reference's package name is importable: the import lines of scripts written against the
reference (``examples/tune.py:12-14``, ``examples/test.py:20-25``, ``examples/end_to_end.py:19-22``,
``RecFlex/tuning/run_script.py:14-18``, ``RecFlex/tuning/tuner.py:16-21`` there) run unchanged and
yield this build's objects; ``BasicConfig`` / ``TuneConfig`` take the reference's field names
(``RecFlex/tuning/tuner.py:24-46``)."""

import subprocess
import sys

import pytest

from helpers import ROOT

REFERENCE_IMPORT_LINES = """
from RecFlex.tuning import Tuner, TuneConfig, BasicConfig
from RecFlex.utils import get_data_fnames, compile_build
from RecFlex.cuda_helper import CudaInfoQuerier
from RecFlex.code_emitter import ScheduleBase
from RecFlex.rec_modules import FeatProcessEmbed
from RecFlex.parser import parse_raw_data_batches, parse_table_shapes
from RecFlex.utils import import_from_path, find_file, compile_build
from RecFlex.cuda_helper import CudaProfiler
from RecFlex.rec_modules import FeatPreprocess, RecomModel
from RecFlex.utils import import_from_path, find_file
from RecFlex.code_emitter import CodeEmitter, ScheduleBase, MetaData
from RecFlex.utils import find_file, compile_build, os_check
from RecFlex.task_manager import TaskManager
from RecFlex.parser import parse_raw_data_batches, parse_table_shapes, parse_schedule_types, parse_knl_total_time
from RecFlex.tuning.measure import measure_single_feat, nsys_profile, measure_task_blocks, measure_naive_candidate
from RecFlex.code_emitter import ScheduleBase, ScheduleVars, PreprocessVars, InputStats, MetaData
from RecFlex.code_emitter.codegen import CodeEmitter
from RecFlex.code_emitter.schedule_base import ScheduleBase
from RecFlex.code_emitter.build_basic import BasicBuilder
from RecFlex import TaskManager
"""


def test_reference_import_lines_resolve_to_this_build():
    ns = {}
    exec(REFERENCE_IMPORT_LINES, ns)
    import recflex_amd.code_emitter
    import recflex_amd.hip_helper
    import recflex_amd.rec_modules
    import recflex_amd.tuning
    assert ns["FeatProcessEmbed"] is recflex_amd.rec_modules.FeatProcessEmbed
    assert ns["RecomModel"] is recflex_amd.rec_modules.RecomModel
    assert ns["Tuner"] is recflex_amd.tuning.Tuner
    assert ns["CodeEmitter"] is recflex_amd.code_emitter.CodeEmitter
    assert ns["CudaInfoQuerier"] is recflex_amd.hip_helper.HipInfoQuerier
    assert ns["CudaProfiler"] is recflex_amd.hip_helper.HipProfiler
    assert ns["nsys_profile"] is recflex_amd.tuning.measure.rocprof_profile
    # the submodules are the very module objects (module-level state is shared)
    import RecFlex.rec_modules
    import RecFlex.tuning.tuner
    assert RecFlex.rec_modules is recflex_amd.rec_modules
    assert RecFlex.tuning.tuner is recflex_amd.tuning.tuner
    assert sys.modules["RecFlex.cuda_helper"] is recflex_amd.hip_helper


SCHEDULE_IMPORT_LINES = """
from schedules.reduce_by_key import ReduceByKeySchedule, ReduceByKeyParams
from schedules.multi_block_per_sample import MultiBlockPerSampleSchedule, MultiBlockPerSampleParams
from schedules.one_block_multi_sample import OneBlockMultiSampleSchedule, OneBlockMultiSampleParams
from schedules.warp_per_sample import WarpPerSampleSchedule, WarpPerSampleParams
from schedules.one_hot import OneHotSchedule, OneHotParams
from schedules.one_hot_multi_block import OneHotMultiBlockSchedule, OneHotMultiBlockParams
"""


def test_schedule_import_lines_of_the_example_scripts_resolve():
    """``examples/tune.py:16-21`` of the reference, run from the examples directory as there."""
    code = ("import sys; sys.path[:0] = ['.', %r]\n" % ROOT + SCHEDULE_IMPORT_LINES +
            "import recflex_amd.schedules as impl\n"
            "assert OneHotSchedule is impl.OneHotSchedule and ReduceByKeyParams is impl.ReduceByKeyParams\n"
            "assert issubclass(WarpPerSampleSchedule, impl.ScheduleBase)\n")
    subprocess.run([sys.executable, "-c", code], cwd=f"{ROOT}/examples", check=True)


def test_config_tuples_take_the_reference_field_names():
    from RecFlex.tuning import BasicConfig, TuneConfig
    basic = BasicConfig(batch_sizes_fname="b.txt", data_fnames=["f0.txt"], schedule_config_fname="s.txt",
                        table_config_fname="t.txt", codegen_dir="out", subdirs=[], includes=[], links=[],
                        host_links=[], block_threads=256, sample_batch_nums=128)
    assert basic._fields[:11] == ("batch_sizes_fname", "data_fnames", "schedule_config_fname",
                                  "table_config_fname", "codegen_dir", "subdirs", "includes", "links",
                                  "host_links", "block_threads", "sample_batch_nums")
    assert BasicConfig("b", ["f"], "s", "t", "o").block_threads == 256
    assert BasicConfig("b", ["f"], "s", "t", "o").sample_batch_nums == 128
    tune = TuneConfig(occupancies=[1, 2], gpu_ids=[0], sm_count=256, num_processes=8, inline=True,
                      recompile=False, remeasure=False, debug=False)
    assert tune._fields[:8] == ("occupancies", "gpu_ids", "sm_count", "num_processes", "inline",
                                "recompile", "remeasure", "debug")
    assert TuneConfig([1], [0], 256).num_processes == 8 and TuneConfig([1], [0], 256).inline is True


def test_importing_the_package_does_not_load_torch():
    """Like the reference's ``RecFlex/__init__.py``, the package itself pulls in TaskManager only."""
    out = subprocess.run([sys.executable, "-c",
                          "import sys; import RecFlex; print('torch' in sys.modules, RecFlex.TaskManager.__name__)"],
                         cwd=ROOT, capture_output=True, text=True, check=True).stdout.split()
    assert out == ["False", "TaskManager"]


def test_run_script_file_is_the_profiled_program():
    """``python RecFlex/tuning/run_script.py`` is the program of ``recflex_amd/tuning/run_script.py``
    (same flags as the reference's, ``RecFlex/tuning/run_script.py:22-29``)."""
    proc = subprocess.run([sys.executable, "RecFlex/tuning/run_script.py", "--help"], cwd=ROOT,
                          capture_output=True, text=True)
    assert proc.returncode == 0
    for flag in ("--table_config_fname", "--build_dir", "--data_dir", "--spec_feat_id",
                 "--sample_batch_nums", "--seed"):
        assert flag in proc.stdout
