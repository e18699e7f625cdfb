"""``RecFlex/tuning/run_script.py`` of the reference -- the program a profiler is wrapped around --
as a file that can be run: it is ``recflex_amd/tuning/run_script.py`` (same flags).  As a module,
``RecFlex.tuning.run_script`` is mapped to that module by the package's finder and this file is
not read."""

import os
import runpy
import sys

_ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
if _ROOT not in sys.path:
    sys.path.insert(0, _ROOT)

if __name__ == "__main__":
    runpy.run_module("recflex_amd.tuning.run_script", run_name="__main__", alter_sys=True)
