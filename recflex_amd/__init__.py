"""MI355X (gfx950) implementation of the RecFlex fused-embedding path.

Package layout follows the reference's ``RecFlex`` package (rec_modules, code_emitter, tuning,
parser, utils, task_manager; ``hip_helper`` stands in for ``cuda_helper``), plus ``schedules``
(the four 64-lane schedule templates), ``workloads`` (seeded synthetic inputs) and ``csrc``
(HIP device headers and the CPU text front end).
"""

from .task_manager import TaskManager
