"""Engine adapter boundary used by the load strategies.

The contract is the reference's (modelexpress/adapter.py:19-196): ``StrategyFailed(mutated)``,
``UnsupportedCapability``, and ``@gated_capability`` methods that a strategy lists in its
``requires`` tuple and that are compared by identity, so a strategy is eligible only when the
concrete engine adapter overrides them.

When the reference package can be imported, these names ARE the reference's classes: its
chain catches ``modelexpress.adapter.StrategyFailed`` (load_strategy/__init__.py:95-103) and
compares ``requires`` with methods of its own ``EngineAdapter`` (load_strategy/base.py:53-60),
so a strategy registered there must raise and subclass exactly those.  Without the reference
(this repository on its own) local mirrors with the same behaviour are used.
``BOUND_TO_REFERENCE`` says which.

``placement_layout`` is the one capability this package adds: it hands the engine's
rank-local parameter table and destination tensors to the HIP placement engine, so weights
are written straight into ``param.data`` instead of flowing through a Python
``(name, tensor)`` iterator.  It is attached to whichever ``EngineAdapter`` is in use (the
reference's class does not declare it), together with the ``after_placement`` hook.
"""

from __future__ import annotations

import functools
import os
from dataclasses import dataclass, field
from typing import TYPE_CHECKING, Iterator, Sequence

import torch

if TYPE_CHECKING:
    from .load_strategy import LoadResult


def _reference_contract():
    """The reference's adapter module, or None when it cannot be imported here."""
    try:
        import modelexpress.adapter as ref
    except Exception:  # noqa: BLE001 - absent, or its own import-time checks fail (protobuf pin, missing engine)
        return None
    wanted = ("StrategyFailed", "UnsupportedCapability", "gated_capability", "EngineAdapter")
    return ref if all(hasattr(ref, n) for n in wanted) else None


_ref = _reference_contract()
BOUND_TO_REFERENCE = _ref is not None

if BOUND_TO_REFERENCE:
    UnsupportedCapability = _ref.UnsupportedCapability
    StrategyFailed = _ref.StrategyFailed
    gated_capability = _ref.gated_capability
    EngineAdapter = _ref.EngineAdapter
else:
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

        def after_native_load(self, result: "LoadResult") -> "LoadResult":
            return result


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


@gated_capability
def placement_layout(self, result: "LoadResult") -> PlacementLayout:
    """Describe this rank's parameters and hand over their storage for in-place placement."""
    ...


def after_placement(self, result: "LoadResult") -> "LoadResult":
    """Run engine post-processing after an in-place placement succeeds."""
    return result


# The capability this package adds lives on the adapter base class in use, so the identity
# rule (base.py:53-60) reads it like any other gated capability.  A base class that already
# declares them (a reference that has adopted the capability) keeps its own.
if not hasattr(EngineAdapter, "placement_layout"):
    EngineAdapter.placement_layout = placement_layout
if not hasattr(EngineAdapter, "after_placement"):
    EngineAdapter.after_placement = after_placement
del placement_layout, after_placement
