"""The workspace rules of the library (which scratch buffer a recorded step may keep
using, when an old one may be freed) are plain bookkeeping in
aether-ml_amd/csrc/ws_ledger.h; tests/cpu/ws_ledger_check.cpp drives them on the host
with a fake allocator."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_workspace_ledger_rules(tmp_path):
    exe = str(tmp_path / "ws_ledger_check")
    src = os.path.join(ROOT, "tests", "cpu", "ws_ledger_check.cpp")
    inc = os.path.join(ROOT, "aether-ml_amd", "csrc")
    subprocess.run(["g++", "-std=c++17", "-O1", "-Wall", "-Werror", "-I", inc, src, "-o", exe], check=True)
    r = subprocess.run([exe], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout + r.stderr
    names = [line.split()[1] for line in r.stdout.splitlines() if line.startswith("ok ")]
    assert names == ["reuse", "grow_frees_old", "no_growth_while_recording", "live_recordings_keep_their_workspace",
                     "retired_freed_with_last_recording", "alloc_failure", "reset"]


def test_sample_runs_cover_the_batch_below_the_descriptor_limit(tmp_path):
    """aether-ml_amd/csrc/sample_runs.h: how a batch whose tensors reach 2^31 bytes is cut into runs of whole samples
    (tests/cpu/sample_runs_check.cpp walks the runs of several shapes and checks cover, order and extent)."""
    exe = str(tmp_path / "sample_runs_check")
    src = os.path.join(ROOT, "tests", "cpu", "sample_runs_check.cpp")
    inc = os.path.join(ROOT, "aether-ml_amd", "csrc")
    subprocess.run(["g++", "-std=c++17", "-O1", "-Wall", "-Werror", "-I", inc, src, "-o", exe], check=True)
    r = subprocess.run([exe], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout + r.stderr
    assert len([line for line in r.stdout.splitlines() if line.startswith("ok ")]) == 11


def test_dgrad_parts_list_every_contribution_once(tmp_path):
    """aether-ml_amd/csrc/dgrad_parts.h: the problems a dgrad is made of (stride classes, and their parts when the classes
    are cut along their borders) and the parts of a padded fprop.  tests/cpu/dgrad_parts_check.cpp enumerates, for 14 + 6
    geometries, every (pixel, filter tap) pair of every problem and compares with the definitions of the input gradient
    (CNN_classes_cupy.py:136-153) and of the forward pass (:92-116)."""
    exe = str(tmp_path / "dgrad_parts_check")
    src = os.path.join(ROOT, "tests", "cpu", "dgrad_parts_check.cpp")
    inc = os.path.join(ROOT, "aether-ml_amd", "csrc")
    subprocess.run(["g++", "-std=c++17", "-O1", "-Wall", "-Werror", "-I", inc, src, "-o", exe], check=True)
    r = subprocess.run([exe], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout + r.stderr
    assert len([line for line in r.stdout.splitlines() if line.startswith("ok ")]) == 20
