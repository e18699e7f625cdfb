"""CPU: the workgroup's list of mid-size bags (``rfx_mid_queue.h``) as a thread model under
ThreadSanitizer.  The device code and this model instantiate the same function templates; here a
thread plays a wavefront.  Every bag must be summed exactly once, by whoever takes it, with what
its producer wrote before the push in view; the model must be clean as the protocol stands and
must fail when a step is weakened or moved."""

import os
import shutil
import subprocess

import pytest

from helpers import ROOT

SRC = os.path.join(ROOT, "tests", "cpu", "mid_queue_model.cpp")
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


def test_every_bag_is_summed_once_and_race_free(tmp_path, tsan_works):
    done = _build_and_run(tmp_path, "model")
    assert done.returncode == 0, done.stdout[-3000:]
    assert "data race" not in done.stdout
    assert "0 bags summed not exactly once" in done.stdout


def test_an_unordered_entry_is_a_data_race(tmp_path, tsan_works):
    """Entry stored and loaded without release / acquire: the taker reads what the producer wrote
    before the push without any ordering."""
    done = _build_and_run(tmp_path, "relaxed", "-DRELAXED_ENTRY")
    assert done.returncode != 0 and "data race" in done.stdout, done.stdout[-2000:]


def test_a_claim_in_two_steps_hands_a_bag_out_twice(tmp_path, tsan_works):
    """Compare and store as two steps instead of one compare-and-swap: two wavefronts take the
    same entry."""
    done = _build_and_run(tmp_path, "claim", "-DNON_ATOMIC_CLAIM")
    assert done.returncode != 0, done.stdout[-2000:]
    assert "data race" in done.stdout or "summed not exactly once" in done.stdout
