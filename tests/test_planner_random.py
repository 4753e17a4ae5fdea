"""Seeded random models: the product planner against the CPU oracle on shapes neither was
written around (odd extents, 1-D / 3-D / 4-D tensors, TP on any axis, fused groups with
unequal members on either axis, premerged pairs, fp32 sources into bf16 parameters)."""

import numpy as np
import pytest
import torch
from safetensors.torch import save_file

from helpers import apply_plan_numpy
from modelexpress_amd.engine import Checkpoint, ParamSpec, PlacementPlan

DT = {"F32": torch.float32, "BF16": torch.bfloat16, "U8": torch.uint8, "I16": torch.int16}


def _rand(rng, shape, dt):
    n = int(np.prod(shape)) if shape else 1
    if dt == "F32":
        return torch.from_numpy(rng.standard_normal(n).astype(np.float32)).reshape(shape)
    if dt == "BF16":
        return torch.from_numpy(rng.standard_normal(n).astype(np.float32)).reshape(shape).to(torch.bfloat16)
    if dt == "U8":
        return torch.from_numpy(rng.integers(0, 256, n, dtype=np.uint8)).reshape(shape)
    return torch.from_numpy(rng.integers(-3000, 3000, n, dtype=np.int16)).reshape(shape)


def build_random_model(seed, tmp_path):
    """Writes the seeded random checkpoint; returns (directory, {param: (dtype, shape)}, tp, rank, cast)."""
    rng = np.random.default_rng(1000 + seed)
    tp = int(rng.choice([1, 2, 3, 4]))
    rank = int(rng.integers(0, tp))
    cast = bool(rng.integers(0, 2))
    src_dt = "F32" if cast else str(rng.choice(["BF16", "U8", "I16", "F32"]))
    dst_dt = "BF16" if cast else src_dt
    tensors, params = {}, {}

    def dims(nd):
        return [int(rng.integers(1, 7)) for _ in range(nd)]

    # direct tensors, TP-sharded on a random axis or replicated
    for k in range(int(rng.integers(1, 5))):
        nd = int(rng.integers(0, 5))
        local = dims(nd)
        full = list(local)
        if nd and tp > 1 and rng.integers(0, 3):
            full[int(rng.integers(0, nd))] *= tp
        tensors[f"d{k}.weight"] = _rand(rng, full, src_dt)
        params[f"d{k}.weight"] = (dst_dt, tuple(local))
    # fused groups (q/k/v and gate/up) on axis 0 or 1, members global or already local
    for k in range(int(rng.integers(1, 4))):
        group = ("q_proj", "k_proj", "v_proj") if rng.integers(0, 2) else ("gate_proj", "up_proj")
        fused = "qkv_proj" if len(group) == 3 else "gate_up_proj"
        axis = int(rng.integers(0, 2))
        other = int(rng.integers(1, 6))
        member_global = tp > 1 and bool(rng.integers(0, 2))
        locals_ = [int(rng.integers(1, 5)) for _ in group]
        if len(group) == 2 and tp > 1 and member_global and axis == 0 and locals_[0] == locals_[1]:
            locals_[1] += 1  # keep clear of the premerged shape pattern; tested separately below
        total = 0
        for m, n_local in zip(group, locals_):
            ext = n_local * (tp if member_global else 1)
            shape = [ext, other] if axis == 0 else [other, ext]
            tensors[f"f{k}.{m}.weight"] = _rand(rng, shape, src_dt)
            total += n_local
        params[f"f{k}.{fused}.weight"] = (dst_dt, (total, other) if axis == 0 else (other, total))
    # one premerged [gate; up] tensor
    if tp > 1 and rng.integers(0, 2):
        half, other = int(rng.integers(1, 4)), int(rng.integers(1, 5))
        tensors["p.gate_up_proj.weight"] = _rand(rng, [2 * half * tp, other], src_dt)
        params["p.gate_up_proj.weight"] = (dst_dt, (2 * half, other))

    path = tmp_path / "ck"
    path.mkdir()
    save_file({n: t.contiguous() for n, t in tensors.items()}, str(path / "model.safetensors"))
    return path, params, tp, rank, cast


def oracle_result(oracle, path, params, tp, rank, cast):
    """The oracle's parameters, or None where it refuses the model (ambiguous shapes)."""
    oparams = {n: oracle.OTensor.zeros(shape, dt) for n, (dt, shape) in params.items()}
    try:
        oracle.MdlOracle(oparams, tp, rank, allow_cast=cast).load_weights(oracle.load_checkpoint(str(path)))
    except oracle.CoverageError:
        return None
    return oparams


@pytest.mark.parametrize("seed", range(40))
def test_random_model(seed, oracle, mxp, tmp_path):
    path, params, tp, rank, cast = build_random_model(seed, tmp_path)
    OT = oracle.OTensor
    oparams = {n: OT.zeros(shape, dt) for n, (dt, shape) in params.items()}
    try:
        oracle.MdlOracle(oparams, tp, rank, allow_cast=cast).load_weights(oracle.load_checkpoint(str(path)))
        oracle_ok = True
    except oracle.CoverageError:
        oracle_ok = False
    ck = Checkpoint(str(path))
    specs = [ParamSpec(n, dt, tuple(shape)) for n, (dt, shape) in params.items()]
    if not oracle_ok:  # ambiguous shapes (e.g. two axes that both look sharded): both sides must refuse
        with pytest.raises(mxp.MxpError):
            PlacementPlan(ck, specs, tp_size=tp, tp_rank=rank, allow_cast=cast)
        return
    plan = PlacementPlan(ck, specs, tp_size=tp, tp_rank=rank, allow_cast=cast)
    got = apply_plan_numpy(ck, plan)
    for n in params:
        assert got[n].tobytes() == oparams[n].tobytes(), (seed, n, tp, rank)
