"""``HipPlacementStrategy`` registered in the reference's own chain.

The scenarios run in a child process (tests/refchain_standin.py) because the package binds to
the reference's contract classes when it is first imported: the child installs a stand-in of
``modelexpress.adapter`` / ``modelexpress.load_strategy`` first, whose chain loop follows
load_strategy/__init__.py:79-136 and whose identity rule follows load_strategy/base.py:53-60.
"""

import json
import subprocess
import sys
from pathlib import Path

import pytest

SCRIPT = Path(__file__).resolve().parent / "refchain_standin.py"


def _run(scenario: str, workdir) -> dict:
    proc = subprocess.run([sys.executable, str(SCRIPT), scenario, str(workdir)], capture_output=True, text=True,
                          timeout=300)
    assert proc.returncode == 0, proc.stderr[-4000:]
    return json.loads(proc.stdout.strip().splitlines()[-1])


def _assert_bound(out: dict) -> None:
    assert out["bound"] and out["same_strategy_failed"] and out["same_engine_adapter"]
    assert out["same_load_strategy_base"] and out["strategy_is_reference_subclass"] and out["requires_is_base_default"]


def test_unbound_without_the_reference():
    from modelexpress_amd import adapter

    assert adapter.BOUND_TO_REFERENCE is False  # nothing named `modelexpress` is importable in this build


def test_adapter_without_the_capability_is_merely_ineligible(tmp_path):
    out = _run("ineligible", tmp_path)
    _assert_bound(out)
    assert out["is_available"] == {"bare": False, "duck": False}  # no AttributeError out of the eligibility pass
    assert out["placing_overrides"] is True
    assert out["chain_log"] == [["eligible", ["default"]], ["loaded", "default"]]
    assert out["native_calls"] == 1 and out["same_model"]


def test_clean_miss_reaches_the_reference_chain_as_its_own_exception(tmp_path):
    out = _run("clean_miss", tmp_path)
    _assert_bound(out)
    assert out["chain_log"] == [["eligible", ["hip_placement", "default"]], ["strategy_failed", "hip_placement", False],
                                ["loaded", "default"]]
    assert out["reinit_calls"] == 0 and out["native_calls"] == 1 and out["same_model"]


@pytest.mark.gpu
def test_success_in_the_reference_chain(tmp_path):
    out = _run("success", tmp_path)
    _assert_bound(out)
    assert out["eligible_with_plain_backend"] is True
    assert out["chain_log"] == [["eligible", ["hip_placement", "default"]], ["loaded", "hip_placement"]]
    assert out["bit_exact"] and out["same_model"] and out["ctx_tensors"]
    assert out["register_tensors_calls"] == 1  # as ModelStreamerStrategy does, model_streamer_strategy.py:96
    assert out["reinit_calls"] == 0 and out["native_calls"] == 0


@pytest.mark.gpu
def test_mutated_failure_reinitialises_through_the_reference_chain(tmp_path):
    """A shard truncated between planning and ingest: the chain must see ITS StrategyFailed with
    mutated=True, call reinit_for_retry once, and run the next strategy on the fresh model."""
    out = _run("mutated", tmp_path)
    _assert_bound(out)
    assert out["chain_log"] == [["eligible", ["hip_placement", "default"]], ["strategy_failed", "hip_placement", True],
                                ["loaded", "default"]]
    assert out["reinit_calls"] == 1 and out["native_calls"] == 1
    assert out["fresh_model_returned"] and out["native_loaded_over_fresh_model"] and out["fresh_model_clean"]
