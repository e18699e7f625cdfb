"""Shared pieces of the parity tests: run a prebuilt model through the C ABI on the GPU and
compare with the CPU oracle."""

import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

from oracle import oracle  # noqa: E402  (the checker; tests are allowed to use it)

# tolerances of the path: fp32 tables within 1e-5 relative or 1e-6 absolute of the oracle;
# fp16 / int8 tables within 1e-3 relative (or 1e-6 absolute) of dequantise-then-fp32-sum
TOL = {"float": (1e-5, 1e-6), "half": (1e-3, 1e-6), "int8": (1e-3, 1e-6)}


def require_lib(name: str) -> str:
    """Path of a prebuilt model library; GPU tests fail loudly if it was not built in-tree."""
    from recflex_amd import prebuilt
    path = prebuilt.lib_path(name)
    if not os.path.exists(path):
        raise RuntimeError(f"{path} is missing: run `python -c 'import __graft_entry__ as g; g.build()'` "
                           "before the GPU tests (no CPU fallback exists)")
    return path


def oracle_output(wl, host_tables, indices, offsets):
    dims = [f.dim for f in wl.features]
    dts = [f.data_type for f in wl.features]
    return oracle.pooled_sum_c(host_tables, dims, dts, indices, offsets)


def check_against_oracle(wl, got: np.ndarray, want: np.ndarray):
    """Per feature column slab, with that feature's tolerance.  Returns a list of failures."""
    failures = []
    col = 0
    for f, spec in enumerate(wl.features):
        rtol, atol = TOL[spec.data_type]
        ok, max_abs, max_rel = oracle.within_tolerance(got[:, col:col + spec.dim],
                                                       want[:, col:col + spec.dim], rtol, atol)
        if not ok:
            failures.append((f, spec, max_abs, max_rel))
        col += spec.dim
    return failures
