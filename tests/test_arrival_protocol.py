"""CPU: the arrival protocol of split bags and outlier tiles (``rfx_arrival.h``) as a thread model
under ThreadSanitizer.  The device code and this model instantiate the same function templates;
here the slots are plain memory and the arrival counter a release/acquire atomic, so the
sanitizer sees exactly what the protocol's order has to guarantee: every part's slot stores
happen before the last arrival's slot loads, and only the last arrival combines.  The model must
be clean in the protocol's order and must be reported as racy when a step is moved."""

import os
import shutil
import subprocess

import pytest

from helpers import ROOT

SRC = os.path.join(ROOT, "tests", "cpu", "arrival_protocol_model.cpp")
INC = os.path.join(ROOT, "recflex_amd", "csrc", "include")


def _build_and_run(tmp_path, name, *defines):
    exe = str(tmp_path / name)
    subprocess.run(["g++", "-std=c++17", "-O1", "-g", "-fsanitize=thread", "-pthread", f"-I{INC}",
                    *defines, SRC, "-o", exe], check=True)
    env = dict(os.environ, TSAN_OPTIONS="halt_on_error=0 exitcode=66")
    return subprocess.run([exe], env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True,
                          timeout=300)


@pytest.fixture(scope="module")
def tsan_works(tmp_path_factory):
    if shutil.which("g++") is None:
        pytest.skip("no g++")
    d = tmp_path_factory.mktemp("tsan_probe")
    (d / "p.cpp").write_text("int main() { return 0; }\n")
    built = subprocess.run(["g++", "-fsanitize=thread", str(d / "p.cpp"), "-o", str(d / "p")],
                           stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
    if built.returncode != 0 or subprocess.run([str(d / "p")], stdout=subprocess.DEVNULL,
                                               stderr=subprocess.DEVNULL).returncode != 0:
        pytest.skip("ThreadSanitizer does not run on this machine")


def test_protocol_order_is_race_free_and_sums_in_part_order(tmp_path, tsan_works):
    done = _build_and_run(tmp_path, "model")
    assert done.returncode == 0, done.stdout[-3000:]
    assert "data race" not in done.stdout
    assert "0 wrong values or counters" in done.stdout


@pytest.mark.parametrize("define", ["-DARRIVE_BEFORE_STORES", "-DCOMBINE_BY_ANYONE"])
def test_a_moved_step_is_reported(tmp_path, tsan_works, define):
    """The checker has teeth: announcing the arrival before the slots are stored, or letting a
    part other than the last arrival combine, is a data race."""
    done = _build_and_run(tmp_path, "broken", define)
    assert done.returncode != 0 and "data race" in done.stdout, done.stdout[-2000:]
