"""Small helpers with the names of ``RecFlex/utils.py:21-64`` (``os_check``, ``compile_build``,
``find_file``, ``import_from_path``, ``get_data_fnames``).

``import_from_path`` differs in one case: the host front end built by this package is a plain
C-ABI shared object, not a CPython extension, so a path ending in ``recom_host.so`` yields a
``recflex_amd.host.RecomHost`` wrapper (same ``preprocess`` method) instead of a module import.
"""

import fnmatch
import importlib.util
import os
import shutil
import subprocess
import sys
from types import ModuleType
from typing import List


def os_check(command: str) -> None:
    status = os.system(command)
    if status != 0:
        raise Exception(f"Process exit status {status}, command: {command}")


def compile_build(build_dir: str, make_dir: bool = True) -> None:
    """Configure and build the generated project that lives in ``build_dir/..``."""
    print(f"Building {build_dir}")
    if make_dir:
        os.makedirs(build_dir, exist_ok=True)
    if shutil.which("cmake") is None:
        raise Exception("cmake not found on PATH")
    for cmd in (["cmake", ".."], ["make"]):
        proc = subprocess.run(cmd, cwd=build_dir, stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                              text=True)
        if proc.returncode != 0:
            raise Exception(f"Process exit status {proc.returncode}, command: {' '.join(cmd)} "
                            f"(in {build_dir})\n{proc.stdout[-4000:]}")


def find_file(directory: str, pattern: str) -> str:
    for root, _, files in os.walk(directory):
        for filename in sorted(fnmatch.filter(files, pattern)):
            return os.path.join(root, filename)
    raise Exception(f"Cannot find {pattern} under {directory}")


def import_from_path(module_name: str, module_path: str):
    base = os.path.basename(module_path)
    if base.startswith("recom_host") and base.endswith(".so") and ".cpython-" not in base:
        from recflex_amd.host import RecomHost
        return RecomHost(module_path)
    spec = importlib.util.spec_from_file_location(module_name, module_path)
    module: ModuleType = importlib.util.module_from_spec(spec)
    sys.modules[module_name] = module
    spec.loader.exec_module(module)
    return module


def get_data_fnames(data_dir: str) -> List[str]:
    data_fnames: List[str] = []
    while os.path.exists(os.path.join(data_dir, f"f{len(data_fnames)}.txt")):
        data_fnames.append(os.path.join(data_dir, f"f{len(data_fnames)}.txt"))
    return data_fnames
