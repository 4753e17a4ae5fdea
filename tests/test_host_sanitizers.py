"""The host side of the library under AddressSanitizer and UndefinedBehaviorSanitizer (CPU build, no GPU).

The safetensors parser, the planner and the CRC32C code (csrc/mxp_ckpt.cpp, mxp_plan.cpp, mxp_crc32c.cpp) are
compiled with ``g++ -fsanitize=address,undefined`` into tests/c/abi_replay; the box-lowering and overlap
checkers (tests/c/lower_check.cpp, overlap_check.cpp: csrc/mxp_lower.hpp, mxp_overlap.hpp) likewise.  The
inputs are the ones most likely to break host code: a session of the parser property tests (arbitrary bytes
and structured headers), the reference's planner vectors, the random planner models, the Megatron layouts and
the full-scale DeepSeek-V3 plan is run once with every host-side ABI call recorded (tests/abi_trace.py), and
the trace is replayed through the sanitized build, which must return what the product build returned, report
nothing and leak nothing.

The engine itself (csrc/mxp_engine.cpp: reader threads, pinned ring, slot events, stream ordering, error path) is
the one concurrent piece of the library.  It is built for the CPU against a stand-in for the HIP runtime
(tests/c/cpu_hip: streams are worker threads, events complete when their worker reaches them, "device" memory is
host memory, the kernel launches are executed by meaning) and driven by tests/c/engine_hosttest.cpp through every
ingest mode under ``-fsanitize=thread`` and again under ``-fsanitize=address,undefined``.  That the harness sees
what it is there to see is checked too: with events that claim completion early the same run must end in a data
race report."""

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


HIP_ON_CPU = CDIR / "cpu_hip"
ENGINE_SOURCES = [CDIR / "engine_hosttest.cpp", HIP_ON_CPU / "cpu_hip.cpp", HIP_ON_CPU / "cpu_kernels.cpp", CSRC / "mxp_engine.cpp",
                  CSRC / "mxp_ckpt.cpp", CSRC / "mxp_plan.cpp", CSRC / "mxp_crc32c.cpp"]
TSAN = ["-fsanitize=thread", "-fno-omit-frame-pointer", "-g", "-O1"]


@pytest.fixture(scope="module")
def engine_binaries():
    """engine_hosttest built twice (ThreadSanitizer; AddressSanitizer + UndefinedBehaviorSanitizer), side by side."""
    deps = [*CSRC.glob("*.hpp"), *CSRC.glob("*.h"), *(ROOT / "include").glob("*.h"), HIP_ON_CPU / "hip" / "hip_runtime.h", Path(__file__)]
    newest = max(p.stat().st_mtime for p in [*ENGINE_SOURCES, *deps])
    base = ["g++", "-std=c++17", "-Wall", f"-I{HIP_ON_CPU}", f"-I{ROOT / 'include'}", f"-I{CSRC}"]  # the stand-in's hip/hip_runtime.h, not ROCm's
    outs = {"tsan": (CDIR / "engine_hosttest_tsan", TSAN), "asan": (CDIR / "engine_hosttest_asan", SAN)}
    running = []
    for out, flags in outs.values():
        if not out.exists() or out.stat().st_mtime < newest:
            running.append(subprocess.Popen([*base, *flags, *map(str, ENGINE_SOURCES), "-o", str(out), "-lpthread"],
                                            stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True))
    for proc in running:
        _o, err = proc.communicate(timeout=900)
        assert proc.returncode == 0, err[-4000:]
    return {k: v[0] for k, v in outs.items()}


def _tsan_env(**extra):
    return dict(os.environ, TSAN_OPTIONS="halt_on_error=0:second_deadlock_stack=1", **extra)


def _skip_if_tsan_cannot_map(r):
    if "unexpected memory mapping" in r.stderr:  # the sanitizer's own start-up check against the kernel's address layout
        pytest.skip("ThreadSanitizer cannot run on this kernel's address-space layout")


def test_engine_ring_and_streams_under_thread_sanitizer(engine_binaries, tmp_path):
    r = subprocess.run([str(engine_binaries["tsan"]), str(tmp_path)], capture_output=True, text=True, env=_tsan_env(), timeout=900)
    _skip_if_tsan_cannot_map(r)
    assert r.returncode == 0, (r.stdout[-2000:], r.stderr[-6000:])
    assert "ThreadSanitizer" not in r.stderr, r.stderr[-6000:]
    assert r.stdout.startswith("ok: 63 placements and 581 view copies checked"), r.stdout


def test_engine_ring_and_streams_under_address_sanitizer(engine_binaries, tmp_path):
    r = subprocess.run([str(engine_binaries["asan"]), str(tmp_path)], capture_output=True, text=True, env=_env(), timeout=900)
    _clean(r)
    assert r.stdout.startswith("ok: 63 placements and 581 view copies checked"), r.stdout


def test_thread_sanitizer_reports_a_ring_slot_reused_too_early(engine_binaries, tmp_path):
    """The harness's own check: events that claim completion before their stream got there let the readers overwrite
    slots whose copies are still queued; the run must not pass."""
    r = subprocess.run([str(engine_binaries["tsan"]), str(tmp_path)], capture_output=True, text=True,
                       env=_tsan_env(CPU_HIP_EVENTS_COMPLETE_EARLY="1"), timeout=900)
    _skip_if_tsan_cannot_map(r)
    assert r.returncode != 0
    assert "ThreadSanitizer: data race" in r.stderr and "pread" in r.stderr, r.stderr[-3000:]
