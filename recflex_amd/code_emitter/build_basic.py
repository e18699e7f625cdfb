"""Locations and compiler settings shared by every emitted library, and the build of the
model-independent host library ``librecflex_host.so``.

Reference counterpart: ``RecFlex/code_emitter/build_basic.py:17-28`` (``BasicBuilder`` builds
``libsched_basic.so`` once and hands its include directory and path to the generated
CMakeLists).  Here the device side is header-only (``csrc/include/*.hip.h``), so only the CPU
text front end is a prebuilt library.
"""

import os
import shutil
import subprocess
from typing import List

import recflex_amd

GPU_ARCH = "gfx950"


class BasicBuilder:
    def __init__(self):
        self.package_dir = os.path.dirname(os.path.abspath(recflex_amd.__file__))
        self.csrc_dir = os.path.join(self.package_dir, "csrc")
        self.include = os.path.join(self.csrc_dir, "include")
        # include/recflex_hip.h sits at the repository root, beside the package
        self.abi_include = os.path.join(os.path.dirname(self.package_dir), "include")
        self.host_source = os.path.join(self.csrc_dir, "host", "recflex_host.cpp")
        self.hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
        self.cxx = shutil.which("g++") or "g++"
        # gfx950 only; packed fp32 instructions are disabled on purpose
        self.hip_flags: List[str] = [
            f"--offload-arch={GPU_ARCH}", "-std=c++17", "-shared", "-fPIC",
            "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
            "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
        ]
        # e.g. RECFLEX_HIP_EXTRA_FLAGS="-DRFX_PREFETCH_GROUPS=0" for an experiment
        self.hip_flags += os.environ.get("RECFLEX_HIP_EXTRA_FLAGS", "").split()
        self.host_flags: List[str] = ["-std=c++17", "-shared", "-fPIC", "-Wall"]

    def device_headers(self) -> List[str]:
        """The headers every emitted ``process.hip`` is built from."""
        names = sorted(n for n in os.listdir(self.include) if n.endswith(".h"))
        return [os.path.join(self.include, n) for n in names] + \
               [os.path.join(self.abi_include, "recflex_hip.h")]

    def host_lib_path(self, dirname: str = "build") -> str:
        return os.path.join(self.csrc_dir, dirname, "librecflex_host.so")

    def build(self, dirname: str = "build", force: bool = False) -> str:
        """Build ``librecflex_host.so`` if missing (or ``force``); returns its path."""
        lib = self.host_lib_path(dirname)
        if force or not os.path.exists(lib):
            os.makedirs(os.path.dirname(lib), exist_ok=True)
            tmp = lib + f".tmp{os.getpid()}"
            cmd = [self.cxx, *self.host_flags, "-O2", f"-I{self.abi_include}", self.host_source, "-o", tmp]
            subprocess.run(cmd, check=True)
            os.replace(tmp, lib)
        return lib
