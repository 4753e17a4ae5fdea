"""Box lowering (modelexpress_amd/csrc/mxp_lower.hpp) checked without a GPU: tests/c/lower_check.cpp
lowers random pitched boxes of every operation to segments and work items and replays on the CPU the
addressing place_kernel performs over those tables - every destination byte written exactly once from
the source byte the box pairs it with, stores whole and aligned to their unit, loads element aligned
(a tensor's offset in a safetensors file promises no more), the reciprocal division exact, a wide tile
no larger than one batch.  The boxes play the part of `paired_runs` of the reference
(refit/reshard/slice_plan.py:259-339): the decomposition may differ, the bytes moved may not."""

import subprocess
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
SRC = ROOT / "tests" / "c" / "lower_check.cpp"
BIN = ROOT / "tests" / "c" / "lower_check"


@pytest.fixture(scope="module")
def checker():
    deps = [SRC, ROOT / "modelexpress_amd" / "csrc" / "mxp_lower.hpp", ROOT / "modelexpress_amd" / "csrc" / "mxp_device.h"]
    if not BIN.exists() or BIN.stat().st_mtime < max(p.stat().st_mtime for p in deps):
        cmd = ["g++", "-std=c++17", "-O2", "-Wall", "-Wextra", "-D__HIP_PLATFORM_AMD__", f"-I{ROOT / 'include'}",
               f"-I{ROOT / 'modelexpress_amd' / 'csrc'}", "-I/opt/rocm/include", str(SRC), "-o", str(BIN)]
        r = subprocess.run(cmd, capture_output=True, text=True)
        assert r.returncode == 0, r.stderr
    return BIN


@pytest.mark.parametrize("first", [0, 300, 600])
def test_lowered_tables_move_exactly_the_box(checker, first):
    r = subprocess.run([str(checker), str(first), "300"], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr
    assert "300 boxes lowered and replayed" in r.stdout


OVERLAP_SRC = ROOT / "tests" / "c" / "overlap_check.cpp"
OVERLAP_BIN = ROOT / "tests" / "c" / "overlap_check"


@pytest.fixture(scope="module")
def overlap_checker():
    deps = [OVERLAP_SRC, ROOT / "modelexpress_amd" / "csrc" / "mxp_overlap.hpp", ROOT / "modelexpress_amd" / "csrc" / "mxp_internal.hpp"]
    if not OVERLAP_BIN.exists() or OVERLAP_BIN.stat().st_mtime < max(p.stat().st_mtime for p in deps):
        cmd = ["g++", "-std=c++17", "-O2", "-Wall", "-Wextra", "-D__HIP_PLATFORM_AMD__", f"-I{ROOT / 'include'}",
               f"-I{ROOT / 'modelexpress_amd' / 'csrc'}", "-I/opt/rocm/include", str(OVERLAP_SRC), "-o", str(OVERLAP_BIN)]
        r = subprocess.run(cmd, capture_output=True, text=True)
        assert r.returncode == 0, r.stderr
    return OVERLAP_BIN


@pytest.mark.parametrize("first", [0, 20000])
def test_clipped_writes_leave_exactly_what_the_later_write_spares(overlap_checker, first):
    """modelexpress_amd/csrc/mxp_overlap.hpp: "later write wins" settled at plan time (the outcome of the serial
    copy loop of engines/vllm/refit/installer.py:419-424 and refit/reshard/receiver.py:939-955)."""
    r = subprocess.run([str(overlap_checker), str(first), "20000"], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr
    assert "20000 pairs clipped and replayed" in r.stdout
