"""The reference's package name over this build: ``from RecFlex.rec_modules import ...``,
``from RecFlex.tuning import Tuner, TuneConfig, BasicConfig``, ``from RecFlex import TaskManager``
and the other import lines of scripts written against the reference
(``examples/tune.py:12-14``, ``examples/test.py:20-25``, ``examples/end_to_end.py:19-22``,
``RecFlex/tuning/run_script.py:14-18`` there) resolve to the modules of ``recflex_amd``.

``RecFlex.<module>`` *is* ``recflex_amd.<module>`` -- the same module object, so module-level
state such as the library chosen by ``rec_modules.load_library`` is shared and every class has
one identity -- for ``rec_modules``, ``code_emitter`` (``.codegen``, ``.schedule_base``,
``.build_basic``), ``tuning`` (``.tuner``, ``.measure``, ``.run_script``), ``parser``, ``utils``,
``task_manager`` and whatever else ``recflex_amd`` holds; ``RecFlex.cuda_helper`` is
``recflex_amd.hip_helper``, whose ``CudaInfoQuerier`` / ``CudaProfiler`` are the HIP classes.
A finder on ``sys.meta_path`` does the mapping, so there are no stub files to keep in step; the
only file besides this one is ``tuning/run_script.py``, which can be run as a program.

Like the reference's ``RecFlex/__init__.py:12`` this file imports only ``TaskManager``; torch is
loaded when a submodule that needs it is.
"""

import importlib
import importlib.abc
import importlib.machinery
import importlib.util
import sys

from recflex_amd.task_manager import TaskManager  # noqa: F401

# reference module name -> module of this build, where the names differ
_RENAMED = {"cuda_helper": "hip_helper"}


def _target_name(fullname: str) -> str:
    parts = fullname.split(".")[1:]
    parts[0] = _RENAMED.get(parts[0], parts[0])
    return ".".join(["recflex_amd"] + parts)


class _AliasFinder(importlib.abc.MetaPathFinder, importlib.abc.Loader):
    """``RecFlex.a.b`` -> the module object ``recflex_amd.a.b``."""

    def find_spec(self, fullname, path=None, target=None):
        if not fullname.startswith(__name__ + "."):
            return None
        try:
            if importlib.util.find_spec(_target_name(fullname)) is None:
                return None
        except ModuleNotFoundError:
            return None
        return importlib.machinery.ModuleSpec(fullname, self)

    def create_module(self, spec):
        return importlib.import_module(_target_name(spec.name))

    def exec_module(self, module):
        pass            # already executed under its own name


if not any(type(f).__name__ == "_AliasFinder" for f in sys.meta_path):
    sys.meta_path.insert(0, _AliasFinder())
