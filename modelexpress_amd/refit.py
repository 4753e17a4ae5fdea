"""Refit of resident parameters from a new checkpoint version (plan -> stage -> apply).

Mirrors the shape of the reference's generator-engine refit boundary
(modelexpress_rl/inference/adapter.py:59-93: ``create_transfer_plan`` /
``validate_transfer_plan`` / ``stage_weight`` -- transfer and verify with the live weights
untouched -- / ``apply_weight`` / ``release_staged_weight`` / ``close``) for a source that
is a safetensors checkpoint on local storage instead of a set of RDMA publishers:

* plan: the placement plan of the resident layout against the new checkpoint; an fp32
  checkpoint into bf16 parameters plans the round-to-nearest-even cast
  (refit/reshard/transfer_plan.py:49-61: dtype mismatch -> staged, then converted);
* stage: ingest + slice + cast into staging buffers, then recompute the per-parameter
  ``tensor_digest`` on the device and compare it with the digests the publisher stamped
  (modelexpress_rl/inference/nixl_staged_transfer.py:529-549): a mismatch, or a digest that
  is required but missing, raises and leaves the live weights as they were;
* apply: one batched device copy of staging into the live parameters, with the
  checksums of what was installed.

``in_place=True`` skips the staging copy (stage writes the live parameters directly):
that waives the "untouched until verified" guarantee and is therefore explicit.
"""

from __future__ import annotations

import contextlib
import json
import logging
from dataclasses import dataclass, field
from typing import Any

import torch

from . import envs
from .adapter import PlacementLayout
from ._lib import DTYPE_SIZE
from .mla import IncompleteRefit
from .engine import Checkpoint, PlacementEngine, PlacementPlan
from .timing import RefitTimingRecorder


logger = logging.getLogger("modelexpress_amd.refit")


@dataclass(frozen=True)
class RefitInputs:
    """One version to install: where it is and what it must digest to."""

    version_id: str
    checkpoint_path: str
    layout_signature: str = ""
    expected_digests: dict = field(default_factory=dict)  # parameter name -> 32 hex chars
    require_digests: bool = False
    # parameter name -> [(shard_offset, shape, digest or None), ...]: the digest of each publisher's
    # region of the parameter, the granularity the reference stamps and checks
    # (modelexpress_rl/inference/nixl_staged_transfer.py:529-549: one digest per source shard)
    expected_shard_digests: dict = field(default_factory=dict)

    @property
    def physical_fingerprint(self) -> tuple:
        """The assumptions whose drift invalidates a cached plan (adapter.py:40-56)."""
        return (self.layout_signature, self.checkpoint_path)


@dataclass
class RefitPlan:
    inputs: RefitInputs
    ckpt: Checkpoint
    plan: PlacementPlan
    fingerprint: tuple


@dataclass
class StagedWeights:
    plan: RefitPlan
    buffers: list  # staging tensors, or the live parameters when in_place
    checksums: list
    digests: list
    stats: dict
    in_place: bool


def _null():
    return contextlib.nullcontext()


def coverage_floor() -> float:
    """The fraction of engine parameter bytes a gated refit must install; outside [0, 1] is an
    error rather than a gate that passes or rejects everything (refit/reshard/receiver.py:236-259)."""
    floor = float(envs.MX_RESHARD_COVERAGE_FLOOR)
    if not 0.0 <= floor <= 1.0:
        raise ValueError(f"MX_RESHARD_COVERAGE_FLOOR must be a fraction in [0.0, 1.0], got {floor}")
    return floor


def log_coverage(param_layout: dict, all_params, *, rank: int = 0, copies_captured: int = 0, unsupported=(),
                 plan_stats: dict | None = None) -> dict:
    """What a refit will write against what the engine holds, as one ``MX_REFIT_COVERAGE`` JSON record
    (refit/reshard/receiver.py:661-755, schema ``refit-coverage-v1``).  ``param_layout`` maps every engine
    parameter to ``(shape, torch dtype or safetensors dtype name)``; ``all_params`` names the ones this refit
    writes.  Coverage is a byte ratio: half the parameters can be far from half the bytes.  INFO when
    complete, WARNING otherwise; with ``MX_RESHARD_REQUIRE_FULL_COVERAGE`` set, coverage below
    ``MX_RESHARD_COVERAGE_FLOOR`` raises ``IncompleteRefit``.  Returns the record."""
    installed = set(all_params)
    dest_bytes = engine_bytes = 0
    missed = []
    for name, (shape, dtype) in param_layout.items():
        count = 1
        for dim in shape:
            count *= int(dim)
        width = DTYPE_SIZE[dtype] if isinstance(dtype, str) else torch.empty(0, dtype=dtype).element_size()
        engine_bytes += count * width
        if name in installed:
            dest_bytes += count * width
        else:
            missed.append(name)
    coverage = (dest_bytes / engine_bytes) if engine_bytes else 0.0
    unsupported = list(unsupported or [])
    stats = plan_stats or {}
    record = {
        "schema": "refit-coverage-v1",
        "rank": rank,
        "params_installed": len(list(all_params)),
        "engine_params": len(param_layout),
        "dest_bytes": dest_bytes,
        "engine_bytes": engine_bytes,
        "coverage_pct": round(100.0 * coverage, 4),
        "params_never_written": len(missed),
        "params_never_written_sample": sorted(missed)[:10],
        "copies_captured": copies_captured,
        "unsupported": len(unsupported),
        "unsupported_sample": [str(u)[:120] for u in unsupported[:10]],
        # the plan's economics ride on the same record: bytes over the wire (here: over PCIe) against useful bytes
        "planned_wire_bytes": int(stats.get("planned_wire_bytes", 0)),
        "extra_wire_bytes": int(stats.get("extra_wire_bytes", 0)),
        "descriptors": int(stats.get("descriptors", 0)),
        "converts": int(stats.get("converts", 0)),
        "fallback": int(stats.get("fallback", 0)),
    }
    complete = not missed and not unsupported and not record["fallback"]
    logger.log(logging.INFO if complete else logging.WARNING, "MX_REFIT_COVERAGE %s", json.dumps(record))
    if envs.MX_RESHARD_REQUIRE_FULL_COVERAGE and coverage < coverage_floor():
        raise IncompleteRefit(
            f"refit covers {100.0 * coverage:.2f}% of the engine's parameter bytes ({dest_bytes} of {engine_bytes}); "
            f"{len(missed)} of {len(param_layout)} params would keep their previous values, e.g. {sorted(missed)[:5]}. "
            f"No digest gate can detect this - bytes that are never requested are never checked. "
            f"Set MX_RESHARD_REQUIRE_FULL_COVERAGE=0 for an intentionally partial refit.")
    return record


class HipRefitAdapter:
    """Refit executor for one rank's resident parameters."""

    supported_payload_formats = frozenset({"safetensors"})

    def __init__(self, layout: PlacementLayout, *, device: int = 0, engine: PlacementEngine | None = None,
                 in_place: bool = False):
        self.timing: RefitTimingRecorder | None = None  # the record of the cycle in progress
        self._plans_built = 0
        self.coverage: dict | None = None  # the MX_REFIT_COVERAGE record of the last plan
        self.layout = layout
        self.device = device
        self.in_place = in_place
        self._own_engine = engine is None
        self.engine = engine or PlacementEngine(device)

    def create_transfer_plan(self, inputs: RefitInputs) -> RefitPlan:
        lay = self.layout
        self.timing = RefitTimingRecorder(backend="hip_placement", version=inputs.version_id, tp_rank=lay.tp_rank,
                                          tp_size=lay.tp_size, cold=self._plans_built == 0)
        # the NaN image of the casts is platform-defined upstream (torch's device kernels give 0x7FC0, its
        # AVX-512 CPU kernels 0xFFFF): the record says which one this cycle wrote
        self.timing.extra["cast_nan_bits"] = f"0x{self.engine.nan_bits:04x}"
        with self.timing.span("transfer_planning"):
            ck = Checkpoint(inputs.checkpoint_path)
            plan = PlacementPlan(ck, lay.params, tp_size=lay.tp_size, tp_rank=lay.tp_rank,
                                 stacked_params_mapping=lay.stacked_params_mapping, expert_mapping=lay.expert_mapping,
                                 skip_prefixes=lay.skip_prefixes, allow_cast=True)
        self._plans_built += 1
        # What this refit will write against everything the engine holds; with the gate on, an
        # incomplete plan stops here, before any byte moves.
        info = plan.param_info()
        self.engine.prepare(plan)  # lowers the plan for this engine: its byte totals are complete afterwards
        totals = plan.totals()
        self.coverage = log_coverage(
            {p["name"]: (p["shape"], p["dtype"]) for p in info}, [p["name"] for p in info if p["bytes_written"] == p["nbytes"]],
            rank=lay.tp_rank, copies_captured=sum(p["n_writes"] for p in info),
            plan_stats={"planned_wire_bytes": totals["h2d_bytes"], "extra_wire_bytes": totals["h2d_bytes"] - totals["placed_bytes"],
                        "descriptors": sum(p["n_writes"] for p in info)})
        return RefitPlan(inputs, ck, plan, inputs.physical_fingerprint)

    def validate_transfer_plan(self, plan: Any, inputs: RefitInputs) -> bool:
        return isinstance(plan, RefitPlan) and plan.fingerprint == inputs.physical_fingerprint

    def stage_weight(self, plan: RefitPlan) -> StagedWeights:
        eng = self.engine
        rec = self.timing or RefitTimingRecorder(backend="hip_placement", version=plan.inputs.version_id, cold=False)
        self.timing = rec
        with rec.span("setup_registration"):
            buffers = list(self.layout.destinations) if self.in_place else eng.allocate(plan.plan)
        with rec.span("wire_transfer"):
            # checksums and tensor_digest sums are accumulated by the placement kernel itself: what is
            # verified below is what was written, with no second pass over the staged buffers
            eng.set_fused_digests(True)
            try:
                stats = eng.execute(plan.plan, buffers)
            finally:
                eng.set_fused_digests(False)
            sums = eng.checksums(plan.plan)
        rec.bytes = stats["placed_bytes"]
        with rec.span("receive_sync"):
            digests = eng.digests(plan.plan)
            staged = StagedWeights(plan, buffers, sums, digests, stats, self.in_place)
            self._verify(staged)
        return staged

    def _verify(self, staged: StagedWeights) -> None:
        inputs = staged.plan.inputs
        names = [p.name for p in staged.plan.plan.params]
        for name, got in zip(names, staged.digests):
            want = inputs.expected_digests.get(name)
            if want is None:
                if inputs.require_digests:
                    raise RuntimeError(f"refit {inputs.version_id}: no published digest for {name}; refusing to install")
                continue
            if want != got:
                raise RuntimeError(f"refit {inputs.version_id}: digest mismatch for {name}: "
                                   f"published {want}, staged {got}")
        if not inputs.expected_shard_digests:
            return
        params = {p.name: (p, buf) for p, buf in zip(staged.plan.plan.params, staged.buffers)}
        regions, wanted = [], []
        for name, shards in inputs.expected_shard_digests.items():
            if name not in params:
                raise RuntimeError(f"refit {inputs.version_id}: source {name!r} is not a parameter of this plan")
            spec, buf = params[name]
            itemsize = DTYPE_SIZE[spec.dtype]
            for offset, shape, digest in shards:
                if not digest:
                    raise RuntimeError(f"source {name!r} did not publish a verification digest")
                region, _ = self.engine.shard_region(buf, spec.shape, offset, shape, itemsize)
                regions.append(region)
                wanted.append((name, tuple(offset), digest))
        got = self.engine.digest(regions, [r.numel() for r in regions]) if regions else []
        for (name, offset, want), have in zip(wanted, got):
            if want != have:
                raise RuntimeError(f"staged weight digest mismatch for source {name!r} at offset {offset}")

    def apply_weight(self, staged: StagedWeights) -> dict:
        names = [p.name for p in staged.plan.plan.params]
        rec = self.timing
        try:
            if staged.in_place:
                return dict(zip(names, staged.checksums))
            sizes = [p.nbytes for p in staged.plan.plan.params]
            with (rec.span("installation") if rec else _null()):
                sums = self.engine.copy_batch(staged.buffers, list(self.layout.destinations), sizes)
                torch.cuda.synchronize(self.device)
            if sums != staged.checksums:
                raise RuntimeError(f"refit {staged.plan.inputs.version_id}: installed bytes differ from the staged ones")
            return dict(zip(names, sums))
        finally:
            if rec is not None:
                rec.emit()

    def release_staged_weight(self, staged: StagedWeights) -> None:
        if not staged.in_place:
            staged.buffers.clear()

    def close(self) -> None:
        if self._own_engine:
            self.engine.close()
