"""GPU: the two command-line entry points, run as a user runs them -- each as a fresh program.

``examples/tune.py -m <model>`` (reference ``examples/tune.py:96-127``: local stage, global stage,
``<model>/output/optimal``) and then ``examples/test.py -m <model> -o <model>/output/optimal
--check`` (reference ``examples/test.py:106-131``: the text front end, the fused kernel and the
reference's own check of every sample against ``F.embedding(...).sum(0)``).  The model directory
is a copy of ``tests/golden/model_test`` whose ``output/`` was filled by ``tune.py
--compile_only`` ahead of time, so this machine measures, lets the global stage build the one
mix the measurements elect, and times it under rocprofv3 (tune.py's default profiler)."""

import json
import os
import shutil
import subprocess
import sys

import pytest

from helpers import ROOT

pytestmark = pytest.mark.gpu


def _run(script, *args, timeout=900):
    cmd = [sys.executable, os.path.join(ROOT, "examples", script), *args]
    print("[case]", " ".join(cmd), flush=True)
    # a child process of its own, never a replacement of this one
    done = subprocess.run(cmd, cwd=os.path.join(ROOT, "examples"), stdout=subprocess.PIPE,
                          stderr=subprocess.STDOUT, text=True, timeout=timeout)
    print(done.stdout[-3000:], flush=True)
    return done


def test_tune_then_test_entry_points(tmp_path):
    from recflex_amd import prebuilt
    src = os.path.join(prebuilt.entry_fixture_dir(), "model")
    if not os.path.exists(os.path.join(src, "output", "tournament", "o4", "build", "librecom.so")):
        raise RuntimeError(f"{src} is not built: run __graft_entry__.build() first")
    if shutil.which("hipcc") is None and not os.path.exists("/opt/rocm/bin/hipcc"):
        pytest.skip("the global stage builds the elected mix and needs hipcc")
    model = str(tmp_path / "model")
    shutil.copytree(src, model)

    tuned = _run("tune.py", "-m", model, *prebuilt.ENTRY_TUNE_FLAGS)
    assert tuned.returncode == 0, tuned.stdout[-3000:]
    optimal = os.path.join(model, "output", "optimal")
    doc = json.load(open(os.path.join(optimal, "schedule.json")))
    assert doc["occupancy"] == 4 and len(doc["schedules"]) == 6
    assert os.path.exists(os.path.join(optimal, "build", "librecom.so"))
    # the local stage measured every feature's admitted candidates, the global stage both contenders
    result = json.load(open(os.path.join(model, "output", "tournament", "o4", "result.json")))
    assert len(result["times"]) == 6 and all(len(t) > 0 for t in result["times"])
    for contender in ("all", "default"):
        assert os.path.exists(os.path.join(model, "output", contender, "o4", "report_kernel_trace.csv")), contender

    checked = _run("test.py", "-m", model, "-o", optimal, "--check", "--sample_batch_nums", "3")
    assert checked.returncode == 0, checked.stdout[-3000:]
    assert "check passed" in checked.stdout
    assert "Accumulated end-to-end time (ms):" in checked.stdout
