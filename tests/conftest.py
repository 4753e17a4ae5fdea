import ctypes
import os
import subprocess
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")
    trace = os.environ.get("MXP_ABI_TRACE")
    if trace:  # test_host_sanitizers.py runs a session of its own with this set: record the host-side ABI calls
        import abi_trace

        abi_trace.install(trace)


@pytest.fixture(scope="session")
def oracle():
    """The CPU oracle module (test infrastructure)."""
    from oracle import oracle as mod

    return mod


@pytest.fixture(scope="session")
def oracle_c():
    """The C part of the oracle, built on demand if no library is present."""
    from oracle import cbind

    return cbind.load()


@pytest.fixture(scope="session")
def mxp():
    """The product library through its ctypes binding; built on demand if absent."""
    from modelexpress_amd import _lib

    if not _lib.LIB_PATH.exists():
        from modelexpress_amd.build import build_library

        build_library()
    _lib.lib()
    return _lib


@pytest.fixture(scope="session")
def gpu_engine(mxp):
    import torch

    if not torch.cuda.is_available():
        pytest.fail("a gpu-marked test ran without a GPU; the HIP path has no fallback")
    from modelexpress_amd.engine import PlacementEngine

    eng = PlacementEngine(0, ring_slots=4, slot_bytes=1 << 20, reader_threads=4, streams=2)
    yield eng
    eng.close()


@pytest.fixture(scope="session")
def gpu_engine_band(mxp):
    """Engine that stages whole row bands for strided slices (device gather) and uses slots
    small enough that tensors are split across several chunks."""
    import torch

    if not torch.cuda.is_available():
        pytest.fail("a gpu-marked test ran without a GPU; the HIP path has no fallback")
    from modelexpress_amd.engine import PlacementEngine

    eng = PlacementEngine(0, ring_slots=3, slot_bytes=1 << 16, reader_threads=3, streams=2, pack_strided_on_host=False)
    yield eng
    eng.close()
