"""Memory-level-parallelism probe (``csrc/mlp_probe.hip``): a stand-alone HIP program that times a
gather of uniformly random rows of a 4 GiB table at several grid sizes and with scalar-cache
prefetches, and prints one line per setting.

    python -m benchaid.mlp_probe            # builds the program if needed, runs it, prints its table

What it showed on an MI355X: a single workgroup on one CU fetches random 128-byte lines at
76 GB/s, 32 workgroups at 62 GB/s each, the whole chip at 6.6-6.8 TB/s (26 GB/s per CU) -- the
ceiling of a gather without reuse is on the memory side, not in a CU's miss handling; prefetching
the next lines through the scalar data cache makes the gather 2.4-4 x slower, ``s_atc_probe``
changes nothing.
"""

import os
import subprocess
import sys

from recflex_amd.code_emitter.build_basic import BasicBuilder

AID_DIR = os.path.dirname(os.path.abspath(__file__))


def exe_path() -> str:
    return os.path.join(AID_DIR, "build", "mlp_probe")


def build(force: bool = False) -> str:
    basic = BasicBuilder()
    exe = exe_path()
    if force or not os.path.exists(exe):
        os.makedirs(os.path.dirname(exe), exist_ok=True)
        flags = [f for f in basic.hip_flags if f not in ("-shared", "-fPIC")]
        tmp = exe + f".tmp{os.getpid()}"
        subprocess.run([basic.hipcc, *flags, "-O3", os.path.join(AID_DIR, "csrc", "mlp_probe.hip"), "-o", tmp],
                       check=True)
        os.replace(tmp, exe)
    return exe


def main() -> int:
    return subprocess.run([build()], timeout=600).returncode


if __name__ == "__main__":
    sys.exit(main())
