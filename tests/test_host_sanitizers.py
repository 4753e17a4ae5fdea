"""The host side of the library under AddressSanitizer and UndefinedBehaviorSanitizer (CPU build, no GPU).

The safetensors parser, the planner and the CRC32C code (csrc/mxp_ckpt.cpp, mxp_plan.cpp, mxp_crc32c.cpp) are
compiled with ``g++ -fsanitize=address,undefined`` into tests/c/abi_replay; the box-lowering and overlap
checkers (tests/c/lower_check.cpp, overlap_check.cpp: csrc/mxp_lower.hpp, mxp_overlap.hpp) likewise.  The
inputs are the ones most likely to break host code: a session of the parser property tests (arbitrary bytes
and structured headers), the reference's planner vectors, the random planner models, the Megatron layouts and
the full-scale DeepSeek-V3 plan is run once with every host-side ABI call recorded (tests/abi_trace.py), and
the trace is replayed through the sanitized build, which must return what the product build returned, report
nothing and leak nothing."""

import os
import subprocess
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
CSRC = ROOT / "modelexpress_amd" / "csrc"
CDIR = ROOT / "tests" / "c"
SAN = ["-fsanitize=address,undefined", "-fno-sanitize-recover=undefined", "-fno-omit-frame-pointer", "-g", "-O1"]
COMMON = ["g++", "-std=c++17", "-Wall", "-Wextra", "-D__HIP_PLATFORM_AMD__", f"-I{ROOT / 'include'}", f"-I{CSRC}", "-I/opt/rocm/include"]
RECORDED = ["test_parser_fuzz.py", "test_planner_vectors.py", "test_planner_random.py", "test_planner_host.py",
            "test_megatron_layouts.py", "test_artifact_crc32c.py", "test_abi.py"]


def _env():
    env = dict(os.environ)
    env["ASAN_OPTIONS"] = "detect_leaks=1:abort_on_error=0:halt_on_error=1"
    env["UBSAN_OPTIONS"] = "print_stacktrace=1:halt_on_error=1"
    return env


def _clean(r):
    assert r.returncode == 0, (r.stdout[-2000:], r.stderr[-4000:])
    assert "AddressSanitizer" not in r.stderr and "runtime error" not in r.stderr and "LeakSanitizer" not in r.stderr, r.stderr[-4000:]


def _build(out: Path, sources, deps=()):
    newest = max(p.stat().st_mtime for p in [*sources, *deps, Path(__file__)])
    if not out.exists() or out.stat().st_mtime < newest:
        r = subprocess.run([*COMMON, *SAN, *map(str, sources), "-o", str(out), "-lpthread"], capture_output=True, text=True)
        assert r.returncode == 0, r.stderr[-4000:]
    return out


@pytest.fixture(scope="module")
def replay_binary():
    headers = [*CSRC.glob("*.hpp"), *CSRC.glob("*.h"), ROOT / "include" / "mxp.h"]
    return _build(CDIR / "abi_replay_san", [CDIR / "abi_replay.cpp", CSRC / "mxp_ckpt.cpp", CSRC / "mxp_plan.cpp", CSRC / "mxp_crc32c.cpp"], headers)


def test_parser_planner_and_crc_replayed_under_sanitizers(replay_binary, tmp_path, mxp):
    trace = tmp_path / "abi.trace"
    env = dict(os.environ, MXP_ABI_TRACE=str(trace))
    cmd = [sys.executable, "-m", "pytest", "-q", "-x", "-m", "not gpu", "-p", "no:cacheprovider", f"--basetemp={tmp_path / 'session'}",
           *[str(ROOT / "tests" / f) for f in RECORDED]]
    rec = subprocess.run(cmd, capture_output=True, text=True, env=env, cwd=str(ROOT), timeout=900)
    assert rec.returncode == 0, rec.stdout[-3000:]
    lines = trace.read_text().splitlines()
    kinds = {ln.split()[0] for ln in lines}
    assert {"ckpt_open", "plan_create", "plan_add_param", "plan_add_stacked", "plan_add_expert", "plan_add_virtual",
            "plan_add_virtual_shard", "plan_build", "crc32c", "file_crc32c"} <= kinds, kinds
    assert sum(ln.startswith("ckpt_open") for ln in lines) > 500 and sum(ln.startswith("plan_build") for ln in lines) > 80
    r = subprocess.run([str(replay_binary), str(trace)], capture_output=True, text=True, env=_env(), timeout=900)
    _clean(r)
    assert f"{len(lines)} calls replayed" in r.stdout


def test_lowering_and_overlap_checkers_under_sanitizers():
    lower = _build(CDIR / "lower_check_san", [CDIR / "lower_check.cpp"], [CSRC / "mxp_lower.hpp", CSRC / "mxp_device.h"])
    overlap = _build(CDIR / "overlap_check_san", [CDIR / "overlap_check.cpp"], [CSRC / "mxp_overlap.hpp", CSRC / "mxp_internal.hpp"])
    r = subprocess.run([str(lower), "0", "120"], capture_output=True, text=True, env=_env(), timeout=600)
    _clean(r)
    assert "120 boxes lowered and replayed" in r.stdout
    r = subprocess.run([str(overlap), "0", "4000"], capture_output=True, text=True, env=_env(), timeout=600)
    _clean(r)
    assert "4000 pairs clipped and replayed" in r.stdout
