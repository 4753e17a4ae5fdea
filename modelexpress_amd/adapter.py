"""Engine adapter boundary used by the load strategies.

Mirrors modelexpress/adapter.py:19-196 of the reference: ``StrategyFailed(mutated)``,
``UnsupportedCapability``, and ``@gated_capability`` methods that a strategy lists in
its ``requires`` tuple and that are compared by identity, so a strategy is eligible only
when the concrete engine adapter overrides them.  Only the capabilities the weight
placement path uses are declared; ``placement_layout`` is the one addition: it hands the
engine's rank-local parameter table and destination tensors to the HIP placement engine,
so weights are written straight into ``param.data`` instead of flowing through a Python
``(name, tensor)`` iterator.
"""

from __future__ import annotations

import functools
import os
from dataclasses import dataclass, field
from typing import TYPE_CHECKING, Iterator, Sequence

import torch

if TYPE_CHECKING:
    from .load_strategy import LoadResult


class UnsupportedCapability(NotImplementedError):
    """Raised by default bodies for adapter capabilities."""


class StrategyFailed(RuntimeError):
    """Expected strategy miss that lets the chain try the next strategy.

    ``mutated=True`` when the strategy may have changed model weights before failing:
    the chain then asks the adapter to re-initialise the model (adapter.py:24-34).
    """

    def __init__(self, message: str, *, mutated: bool = False):
        super().__init__(message)
        self.mutated = mutated


def gated_capability(method):
    """An optional adapter method engines must override to support it (adapter.py:37-51)."""

    @functools.wraps(method)
    def default(self, *args, **kwargs):
        raise UnsupportedCapability(method.__name__)

    default.__gated_capability__ = True
    return default


@dataclass
class PlacementLayout:
    """What the placement engine needs to know about one serving rank.

    ``params`` are ``ParamSpec`` rows in the order of ``destinations``; each destination
    is the engine's own parameter storage (a contiguous device tensor), written in place
    and never replaced.  ``stacked_params_mapping`` and ``expert_mapping`` are what the
    reference's direct loader reads off the model object
    (engines/vllm/refit/installer.py:489-497,773-797).
    """

    params: Sequence
    destinations: Sequence[torch.Tensor]
    tp_size: int = 1
    tp_rank: int = 0
    stacked_params_mapping: Sequence | None = None
    expert_mapping: Sequence | None = None
    skip_prefixes: Sequence[str] = ()
    expected_checksums: dict = field(default_factory=dict)  # name -> 8 hex chars, optional manifest


class EngineAdapter:
    """Engine-specific boundary used by shared loading strategies (adapter.py:54-196)."""

    @gated_capability
    def get_device_id(self) -> int:
        """Return the local device id owned by this adapter instance."""
        ...

    @gated_capability
    def apply_weight_iter(self, result: "LoadResult", weights_iter: Iterator[tuple[str, torch.Tensor]]) -> "LoadResult":
        """Apply a stream of named tensors to the engine model (may mutate weights)."""
        ...

    @gated_capability
    def build_model_streamer_weight_iter(self, model_uri: str, model: torch.nn.Module | None = None
                                         ) -> Iterator[tuple[str, torch.Tensor]]:
        """Return the engine-native streamer weight iterator."""
        ...

    @gated_capability
    def placement_layout(self, result: "LoadResult") -> PlacementLayout:
        """Describe this rank's parameters and hand over their storage for in-place placement."""
        ...

    @gated_capability
    def load_via_native(self, result: "LoadResult") -> "LoadResult":
        """Load the model using the engine's native disk/checkpoint loader."""
        ...

    @gated_capability
    def reinit_for_retry(self, result: "LoadResult") -> "LoadResult":
        """Replace a possibly-mutated model with a fresh engine model instance."""
        ...

    def get_unique_id(self) -> str:
        if torch.distributed.is_available() and torch.distributed.is_initialized():
            return f"rank-{torch.distributed.get_rank()}"
        return f"pid-{os.getpid()}"

    def get_target_device(self) -> torch.device:
        return torch.device(f"cuda:{self.get_device_id()}")

    def is_cuda_alike(self) -> bool:
        return False

    def after_weight_iter_load(self, result: "LoadResult") -> "LoadResult":
        """Run engine post-processing after apply_weight_iter() succeeds."""
        return result

    def after_placement(self, result: "LoadResult") -> "LoadResult":
        """Run engine post-processing after an in-place placement succeeds."""
        return result

    def after_native_load(self, result: "LoadResult") -> "LoadResult":
        return result
