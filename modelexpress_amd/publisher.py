"""Trainer-side staging of one weight version: the snapshot a publisher serves.

Mirrors the rank-local part of the reference's FSDP trainer adapter
(modelexpress_rl/train/engines/fsdp/adapter.py:100-264, publisher.py:40-44): every floating-point tensor
of the state dict gets a persistent arena in the wire dtype (bf16) and each step copies the live tensors
into them - ``arena.copy_(src)``, which casts only when the dtypes differ (adapter.py:196-211) - or, for
``IN_PLACE``, serves the live storage when it already is contiguous wire-dtype memory that has not moved.
The layout (tensor set, shapes) is fixed at the first stage and must not change afterwards.

Here the whole snapshot is one device launch: the copies are lowered once into a view plan
(``mxp_view_plan``) and every later step only launches it; digests of the served buffers
(refit/reshard/verify.py:186-196, opt-in publication) come from one batched launch as well.
Registration with a transport, manifests and rendezvous are outside this module.
"""

from __future__ import annotations

from typing import Any

import torch

from . import _lib as L
from . import envs
from .engine import CAST_CODES, PlacementEngine
from .load_strategy import safetensors_dtype_of

WIRE_DTYPE = torch.bfloat16  # publisher.py:40-44

COPY_TO_DEVICE = "copy_to_device"
IN_PLACE = "in_place"


class WireStager:
    """Stages one rank's state dict for publication; see the module docstring."""

    supported_staging_modes = frozenset({COPY_TO_DEVICE, IN_PLACE})

    def __init__(self, engine: PlacementEngine, *, publish_digests: bool | None = None):
        self.engine = engine
        self._publish_digests = publish_digests  # None: follow MX_RESHARD_PUBLISH_DIGEST, read at every stage
        self._initialized = False
        self._staging_mode: str | None = None
        self._expected_layout: dict[str, tuple] = {}
        self._arenas: dict[str, torch.Tensor] = {}
        self._registered_addrs: dict[str, int] = {}
        self._plan = None
        self._plan_key: tuple | None = None
        self.skipped: list[str] = []  # non-floating tensors of the last stage (publisher.py: skipped, not published)

    # ---- capture and layout rules ----
    def _capture(self, tensors: Any) -> dict:
        if not isinstance(tensors, dict):
            raise TypeError("tensors must be a state_dict (dict[str, Tensor])")
        self.skipped = [n for n, t in tensors.items() if not t.is_floating_point()]
        shards = {n: t.detach() for n, t in tensors.items() if t.is_floating_point()}
        if not shards:
            raise ValueError("no local shards to publish")
        return shards

    @staticmethod
    def _require_in_place_servable(name: str, t: torch.Tensor) -> None:
        if t.dtype != WIRE_DTYPE:
            raise NotImplementedError(f"{name}: IN_PLACE serves the source dtype but wire is {WIRE_DTYPE}; use COPY_TO_DEVICE to cast")
        if not t.is_contiguous():
            raise NotImplementedError(f"{name}: IN_PLACE requires a contiguous local shard; use COPY_TO_DEVICE for this tensor")

    def initialize(self, shards: dict, staging_mode: str) -> None:
        if self._initialized:
            return
        if staging_mode not in self.supported_staging_modes:
            raise NotImplementedError(f"WireStager does not support {staging_mode} staging")
        self._expected_layout = {n: tuple(t.shape) for n, t in shards.items()}
        if staging_mode == COPY_TO_DEVICE:
            self._arenas = {n: torch.empty(t.shape, dtype=WIRE_DTYPE, device=t.device) for n, t in shards.items()}
            self._registered_addrs = {n: a.data_ptr() for n, a in self._arenas.items()}
        else:
            for n, t in shards.items():
                self._require_in_place_servable(n, t)
            self._registered_addrs = {n: t.data_ptr() for n, t in shards.items()}
        self._staging_mode = staging_mode
        self._initialized = True

    def _require_same_layout(self, shards: dict) -> None:
        expected, names = frozenset(self._expected_layout), frozenset(shards)
        if names != expected:
            raise ValueError(f"tensor set changed since initialize (missing={sorted(expected - names)[:5]} "
                             f"extra={sorted(names - expected)[:5]})")
        for n, t in shards.items():
            if tuple(t.shape) != self._expected_layout[n]:
                raise ValueError(f"{n}: shard geometry changed since initialize (was {self._expected_layout[n]}, now {tuple(t.shape)}); "
                                 "a trainer must keep a fixed shard layout across steps")

    # ---- one version ----
    def stage(self, tensors: Any, staging_mode: str = COPY_TO_DEVICE, *, stream: int = 0) -> dict:
        """Returns ``{"served": name -> served tensor, "total_bytes", "tensor_count", "digests" (or None)}``.
        The copies are queued on ``stream``; the caller orders its publication after them."""
        if staging_mode not in self.supported_staging_modes:
            raise NotImplementedError(f"WireStager does not support {staging_mode} staging")
        shards = self._capture(tensors)
        self.initialize(shards, staging_mode)
        if staging_mode != self._staging_mode:
            raise ValueError(f"WireStager initialized for {self._staging_mode} staging; cannot stage {staging_mode}")
        self._require_same_layout(shards)
        if staging_mode == COPY_TO_DEVICE:
            self._snapshot_into_arenas(shards, stream)
            served = dict(self._arenas)
        else:
            for n, t in shards.items():
                self._require_in_place_servable(n, t)
                if t.data_ptr() != self._registered_addrs[n]:
                    raise NotImplementedError(f"{n}: source storage moved since registration; IN_PLACE requires stable storage, "
                                              "use COPY_TO_DEVICE")
            served = shards
        digests = None
        if envs.MX_RESHARD_PUBLISH_DIGEST if self._publish_digests is None else self._publish_digests:
            names = list(served)
            digests = dict(zip(names, self.engine.digest([served[n] for n in names], stream=stream)))
        wire = torch.empty((), dtype=WIRE_DTYPE).element_size()
        return {"served": served, "tensor_count": len(served), "total_bytes": sum(t.numel() * wire for t in served.values()),
                "digests": digests}

    def _snapshot_into_arenas(self, shards: dict, stream: int) -> None:
        """``arena.copy_(src)`` for every shard, as one launch; contiguous sources whose addresses did not move
        since the last step replay the lowered plan."""
        key = tuple((n, t.data_ptr(), t.dtype, tuple(t.stride())) for n, t in shards.items())
        if key != self._plan_key:
            if self._plan is not None:
                self._plan.close()
            arr = (L.ViewCopy * len(shards))()
            for o, (n, t) in zip(arr, shards.items()):
                arena = self._arenas[n]
                src_dt = safetensors_dtype_of(t)
                cast = 0 if t.dtype == WIRE_DTYPE else CAST_CODES.get((src_dt, "BF16"), 0)
                if t.dtype != WIRE_DTYPE and not cast:
                    raise NotImplementedError(f"{n}: no conversion from {src_dt} to the wire dtype")
                o.src, o.dst, o.ndim, o.elem_size, o.cast, o.contiguous_dst = t.data_ptr(), arena.data_ptr(), t.dim(), 2, cast, 1
                for d in range(t.dim()):
                    o.shape[d], o.src_strides[d] = t.shape[d], t.stride(d)
            self._plan = self.engine.view_plan(arr, len(shards))
            self._plan_key = key
        self._plan.run(stream=stream)

    def close(self) -> None:
        if self._plan is not None:
            self._plan.close()
            self._plan = None
