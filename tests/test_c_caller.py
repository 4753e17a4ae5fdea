"""The library driven from plain C (tests/c/abi_driver.c, built with gcc by
``python -m modelexpress_amd.build --abi-driver``): what a foreign-function binding does
through include/mxp.h, with no Python or torch in the calling process."""

import subprocess
from pathlib import Path

import pytest

from helpers import oracle_place, tiny_layouts
from modelexpress_amd import synth

DRIVER = Path(__file__).parent / "c" / "abi_driver"


def _setup(tmp_path, name, tp_rank):
    layout, tp, ep, shards, ck_kw = tiny_layouts()[name]
    synth.write_checkpoint(layout.checkpoint(**ck_kw), str(tmp_path), n_shards=shards, seed=21)
    rv = layout.rank_view(tp_size=tp, tp_rank=tp_rank)
    lines = [f"{p.name} {p.dtype} {len(p.shape)} " + " ".join(str(d) for d in p.shape) for p in rv.params]
    lines += [f"stacked {fused} {member}" for fused, member, *_ in rv.stacked_params_mapping]
    pf = tmp_path / "params.txt"
    pf.write_text("\n".join(lines) + "\n")
    return rv, tp, pf


def _need_driver():
    if DRIVER.exists():
        return
    try:  # normally prebuilt by `python -m modelexpress_amd.build --abi-driver`; one gcc call otherwise
        from modelexpress_amd.build import build_abi_driver

        build_abi_driver()
    except Exception as e:  # noqa: BLE001
        pytest.fail(f"{DRIVER} is not built and could not be built here: {e}")


def test_c_caller_reports_a_missing_device_as_an_error(tmp_path):
    import torch

    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    _need_driver()
    rv, tp, pf = _setup(tmp_path, "llama_tp4", 1)
    r = subprocess.run([str(DRIVER), str(tmp_path), str(tp), "1", str(pf)], capture_output=True, text=True, timeout=60)
    assert r.returncode == 1 and "mxp_engine_create" in r.stderr  # parse and plan succeeded, no device: a clean error


@pytest.mark.gpu
def test_c_caller_places_a_rank_bit_exact(oracle, tmp_path):
    _need_driver()
    rv, tp, pf = _setup(tmp_path, "llama_tp4", 3)
    want = oracle_place(oracle, str(tmp_path), rv, tp_size=tp, tp_rank=3)
    r = subprocess.run([str(DRIVER), str(tmp_path), str(tp), "3", str(pf)], capture_output=True, text=True, timeout=100)
    assert r.returncode == 0, r.stderr
    rows = [line.split() for line in r.stdout.strip().splitlines()]
    assert [row[0] for row in rows] == [p.name for p in rv.params]
    for (name, nbytes, csum, digest), p in zip(rows, rv.params):
        assert int(nbytes) == len(want[name].tobytes()) == p.nbytes
        assert csum == oracle.safe_checksum(want[name]), name
        assert digest == oracle.tensor_digest(want[name]), name
