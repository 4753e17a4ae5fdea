"""Prioritized chain of loading strategies with the HIP placement strategy in it.

Mirrors the reference's ``modelexpress/load_strategy`` package for the weight-placement
path: ``LoadStrategy`` (base.py:37-76), ``LoadContext`` / ``LoadResult``
(context.py:39-87), ``LoadStrategyChain.run`` (__init__.py:45-136) and the streamer
strategy (model_streamer_strategy.py:38-107).  Same contract:

* a strategy returns a ``LoadResult`` only on success;
* ``StrategyFailed(mutated=False)`` for a clean miss, ``mutated=True`` once model bytes may
  have changed -- the chain then rolls back and asks the adapter to re-initialise;
* any other exception is logged, rolled back and the chain moves on;
* no strategy left -> ``RuntimeError``.

When the reference package can be imported, ``LoadStrategy``, ``LoadContext``, ``LoadResult``,
``_as_load_result`` and ``register_tensors`` ARE the reference's (load_strategy/base.py,
context.py), and ``StrategyFailed`` / ``EngineAdapter`` come from its adapter module (see
``adapter.py``): the strategies below then subclass and raise exactly what the reference's own
chain dispatches on.  Otherwise local mirrors with the same behaviour are used.

``HipPlacementStrategy`` takes the slot the reference gives ``ModelStreamerStrategy``
(after InstantTensor, before GDS): same activation variable (``MX_MODEL_URI``), same URI
resolution order, but the bytes go file -> pinned ring -> HBM -> placement kernels ->
``param.data`` inside libmxplace.so instead of through a Python tensor iterator.
``HipStreamerStrategy`` keeps the iterator shape for engines that only expose
``load_weights``.
"""

from __future__ import annotations

import logging
from abc import ABC, abstractmethod
from dataclasses import dataclass, field
from typing import Any, Callable, ClassVar, Generic, Iterator, Sequence, TypeVar

import torch
from torch import nn

from . import envs
from .accelerators import AcceleratorBackend, HipAcceleratorBackend
from .adapter import EngineAdapter, PlacementLayout, StrategyFailed, UnsupportedCapability

logger = logging.getLogger("modelexpress_amd.load_strategy")

T = TypeVar("T")

from .manifest import TensorRecord  # noqa: E402

_TORCH_DTYPE = {
    "F64": torch.float64, "F32": torch.float32, "F16": torch.float16, "BF16": torch.bfloat16,
    "F8_E4M3": torch.float8_e4m3fn, "F8_E5M2": torch.float8_e5m2, "I64": torch.int64, "I32": torch.int32,
    "I16": torch.int16, "I8": torch.int8, "U8": torch.uint8, "BOOL": torch.bool,
}
_ST_DTYPE = {v: k for k, v in _TORCH_DTYPE.items()}


def safetensors_dtype_of(t: torch.Tensor) -> str:
    """The safetensors dtype string of a torch tensor (inverse of gds_loader.py:36-49)."""
    try:
        return _ST_DTYPE[t.dtype]
    except KeyError as exc:
        raise ValueError(f"dtype {t.dtype} has no safetensors name") from exc


def _reference_load_strategy():
    """(base module, context module) of the reference's load_strategy package, or None."""
    from . import adapter as _adapter

    if not _adapter.BOUND_TO_REFERENCE:
        return None
    try:
        from modelexpress.load_strategy import base as ref_base
    except Exception:  # noqa: BLE001 - the reference's own import-time requirements
        return None
    try:
        from modelexpress.load_strategy import context as ref_ctx
    except Exception:  # noqa: BLE001
        ref_ctx = ref_base  # base re-exports both classes (base.py:19)
    ok = hasattr(ref_base, "LoadStrategy") and hasattr(ref_ctx, "LoadContext") and hasattr(ref_ctx, "LoadResult")
    return (ref_base, ref_ctx) if ok else None


_ref = _reference_load_strategy()

if _ref is not None:
    LoadStrategy = _ref[0].LoadStrategy
    LoadContext = _ref[1].LoadContext
    LoadResult = _ref[1].LoadResult
    _as_load_result = getattr(_ref[0], "_as_load_result", None)
    # ModelStreamerStrategy registers the loaded tensors itself (model_streamer_strategy.py:96)
    _register_tensors = getattr(_ref[0], "register_tensors", None)

    @dataclass
    class SourceIdentity:
        """Stand-alone identity record for callers of this package's own chain."""

        model_name: str = ""
else:
    _register_tensors = None
    _as_load_result = None

    @dataclass
    class LoadResult(Generic[T]):
        """Stable envelope passed through strategies and adapter hooks (context.py:39-52)."""

        value: T
        model: nn.Module | None = None
        publishable: bool = True
        metadata: dict[str, Any] = field(default_factory=dict)


    @dataclass
    class SourceIdentity:
        """The part of the reference's identity message the load path reads."""

        model_name: str = ""


    @dataclass
    class LoadContext:
        """Shared state passed to all loading strategies (context.py:55-87, load-path fields)."""

        model_config: Any
        load_config: Any = None
        target_device: torch.device = field(default_factory=lambda: torch.device("cuda", 0))
        global_rank: int = 0
        worker_rank: int = 0
        device_id: int = 0
        identity: SourceIdentity = field(default_factory=SourceIdentity)
        adapter: EngineAdapter | None = None
        accelerator_backend: AcceleratorBackend = field(default_factory=HipAcceleratorBackend)
        tensors: dict[str, torch.Tensor] = field(default_factory=dict)
        source_ready_fn: Callable[[], bool] | None = None


    class LoadStrategy(ABC):
        """Base class for weight-loading strategies (base.py:37-76)."""

        name: str
        requires: ClassVar[tuple] = ()

        def is_available(self, ctx: LoadContext) -> bool:
            if not self.requires:
                return True
            if ctx.adapter is None:
                return False
            cls = type(ctx.adapter)
            return all(getattr(cls, m.__name__) is not m for m in self.requires)

        @abstractmethod
        def load(self, result: LoadResult, ctx: LoadContext) -> LoadResult:
            """Attempt to load weights and return the updated result."""

        def rollback(self, ctx: LoadContext) -> None:
            """Clean up strategy-owned state after a failed load attempt."""
            return None



if _as_load_result is None:
    def _as_load_result(result_or_model) -> LoadResult:
        if isinstance(result_or_model, LoadResult):
            return result_or_model
        return LoadResult(value=result_or_model, model=result_or_model)


def _resolve_model_uri(ctx: LoadContext) -> str:
    """model_streamer_strategy.py:27-35: env first, then the engine's model config."""
    if model_uri := envs.MX_MODEL_URI:
        return model_uri
    for attr in ("model_weights", "model", "model_path"):
        value = getattr(ctx.model_config, attr, None)
        if value:
            return value
    return ""


def log_tensor_summary(checksums: dict, label: str, shapes: dict | None = None) -> None:
    """Per-tensor ``[CHECKSUM]`` lines at DEBUG, the format a source log and a target log
    are diffed on (tensor_utils.py:363-382).  The values come from the placement kernel,
    so logging them costs no extra device pass."""
    if not logger.isEnabledFor(logging.DEBUG):
        return
    for name, value in checksums.items():
        shape, dtype = (shapes or {}).get(name, ("?", "?"))
        logger.debug(f"[CHECKSUM] {label} | {name} | shape={shape} dtype={dtype} | {value}")


def _engine_from_env(device: int):
    from .engine import PlacementEngine

    pack = envs.MXP_PACK_STRIDED
    return PlacementEngine(
        device, ring_slots=envs.MXP_RING_SLOTS, slot_bytes=envs.MXP_SLOT_MIB << 20,
        reader_threads=envs.MXP_READER_THREADS, streams=envs.MXP_STREAMS, nan_bits=envs.MXP_NAN_BITS,
        use_o_direct=envs.MXP_O_DIRECT, pack_strided_on_host=None if pack == "" else pack == "1")


def _hip_placement_supported(backend) -> bool:
    """The backend's own answer when it has one (``HipAcceleratorBackend``); for a backend that
    predates the question (the reference's CUDA backend serves ROCm builds of torch too,
    accelerators/cuda.py:49-50) the same check is made here."""
    probe = getattr(backend, "supports_hip_placement", None)
    if callable(probe):
        return bool(probe())
    return HipAcceleratorBackend().supports_hip_placement() and bool(getattr(torch.version, "hip", None))


class HipPlacementStrategy(LoadStrategy):
    """Place weights with the HIP engine, straight into the engine's parameters."""

    name = "hip_placement"
    requires = (EngineAdapter.placement_layout,)

    def __init__(self):
        self._engine = None
        self._plan = None
        self._ckpt = None

    def is_available(self, ctx: LoadContext) -> bool:
        # Identity rule of base.py:53-60, tolerant of adapters that do not derive from the
        # base class the capability was attached to: a missing method means "not overridden".
        if ctx.adapter is None:
            return False
        cls = type(ctx.adapter)
        if not all(getattr(cls, m.__name__, m) is not m for m in self.requires):
            return False
        if not _hip_placement_supported(ctx.accelerator_backend):
            logger.info(f"[Worker {ctx.global_rank}] HIP placement library or device not available, skipping")
            return False
        model_uri = envs.MX_MODEL_URI or ""
        if not model_uri:
            logger.info(f"[Worker {ctx.global_rank}] MX_MODEL_URI not set, skipping HIP placement")
            return False
        if "://" in model_uri and not model_uri.startswith("file://"):
            logger.info(f"[Worker {ctx.global_rank}] MX_MODEL_URI is not a local path, skipping HIP placement")
            return False
        return True

    def load(self, result: LoadResult, ctx: LoadContext) -> LoadResult:
        from . import _lib
        from .engine import Checkpoint, PlacementPlan

        result = _as_load_result(result)
        model_uri = _resolve_model_uri(ctx)
        if not model_uri:
            raise StrategyFailed("HIP placement model URI is not configured", mutated=False)
        if model_uri.startswith("file://"):
            model_uri = model_uri[len("file://"):]
        logger.info(f"[Worker {ctx.global_rank}] Attempting HIP placement from {model_uri}")
        # Everything up to and including the plan touches no model byte.
        try:
            layout: PlacementLayout = ctx.adapter.placement_layout(result)
            for spec, dst in zip(layout.params, layout.destinations):
                if not dst.is_contiguous() or dst.numel() * dst.element_size() != spec.nbytes:
                    raise ValueError(f"destination of {spec.name} is not a contiguous tensor of {spec.nbytes} bytes")
            self._ckpt = Checkpoint(model_uri)
            self._plan = PlacementPlan(
                self._ckpt, layout.params, tp_size=layout.tp_size, tp_rank=layout.tp_rank,
                stacked_params_mapping=layout.stacked_params_mapping, expert_mapping=layout.expert_mapping,
                skip_prefixes=layout.skip_prefixes, allow_cast=envs.MXP_ALLOW_CAST)
            self._engine = _engine_from_env(ctx.device_id)
        except Exception as e:
            logger.warning(f"[Worker {ctx.global_rank}] HIP placement planning failed, falling through: {e}")
            raise StrategyFailed(str(e), mutated=False) from e

        try:
            stats = self._engine.execute(self._plan, list(layout.destinations))
            sums = dict(zip([p.name for p in layout.params], self._engine.checksums(self._plan)))
        except _lib.MxpError as e:
            mutated = bool(getattr(e, "mutated", True))
            logger.warning(f"[Worker {ctx.global_rank}] HIP placement failed, falling through: {e}")
            raise StrategyFailed(str(e), mutated=mutated) from e
        except Exception as e:
            logger.warning(f"[Worker {ctx.global_rank}] HIP placement failed, falling through: {e}")
            raise StrategyFailed(str(e), mutated=True) from e

        if layout.expected_checksums and envs.MXP_VERIFY_CHECKSUMS:
            bad = [n for n, want in layout.expected_checksums.items() if sums.get(n) != want]
            if bad:
                raise StrategyFailed(f"checksum mismatch after placement for {bad[:10]}", mutated=True)
        try:
            result.metadata["placement_stats"] = stats
            result.metadata["checksums"] = sums
            result.metadata["manifest"] = [TensorRecord(p.name, p.nbytes, p.dtype, sums[p.name]) for p in layout.params]
            log_tensor_summary(sums, f"worker{ctx.global_rank}",
                               {p.name: (tuple(p.shape), p.dtype) for p in layout.params})
            logger.info(f"[Worker {ctx.global_rank}] HIP placement complete: "
                        f"{stats['placed_bytes'] / 1e9:.2f} GB in {stats['wall_seconds']:.3f}s")
            after = getattr(ctx.adapter, "after_placement", None)
            if callable(after):
                result = after(result)
        except Exception as e:
            raise StrategyFailed(str(e), mutated=True) from e
        ctx.tensors.update({p.name: d for p, d in zip(layout.params, layout.destinations)})
        if _register_tensors is not None:
            _register_tensors(result, ctx)
        return result

    def rollback(self, ctx: LoadContext) -> None:
        for h in (self._plan, self._ckpt, self._engine):
            if h is not None:
                h.close()
        self._plan = self._ckpt = self._engine = None


def iter_checkpoint_tensors(model_uri: str, device: int = 0) -> Iterator[tuple[str, torch.Tensor]]:
    """Yield ``(name, device tensor)`` for every tensor of a checkpoint, one shard file at
    a time through the pinned ring, the next file loading while the current one is consumed:
    the reference's per-file iterator (gds_loader.py:84-156)."""
    from .loader import MxHipLoader

    loader = MxHipLoader(device=device)
    try:
        yield from loader.load_iter(model_uri, use_tqdm=False)
    finally:
        loader.shutdown()


class HipStreamerStrategy(LoadStrategy):
    """Iterator-shaped variant: the adapter builds the ``(name, tensor)`` stream (normally
    with ``iter_checkpoint_tensors``) and applies it through its own ``load_weights``;
    failure semantics are those of model_streamer_strategy.py:69-95."""

    name = "model_streamer"
    requires = (EngineAdapter.apply_weight_iter, EngineAdapter.build_model_streamer_weight_iter)

    def is_available(self, ctx: LoadContext) -> bool:
        if not super().is_available(ctx):
            return False
        if not (envs.MX_MODEL_URI or ""):
            logger.info(f"[Worker {ctx.global_rank}] MX_MODEL_URI not set, skipping model streamer")
            return False
        return True

    def load(self, result: LoadResult, ctx: LoadContext) -> LoadResult:
        result = _as_load_result(result)
        model_uri = _resolve_model_uri(ctx)
        if not model_uri:
            raise StrategyFailed("ModelStreamer model URI is not configured", mutated=False)
        try:
            weights_iter = self._stream_weights(model_uri, ctx, result.model)
        except Exception as e:
            raise StrategyFailed(str(e), mutated=False) from e
        try:
            result = ctx.adapter.apply_weight_iter(result, weights_iter)
            logger.info(f"[Worker {ctx.global_rank}] Model streamer weight loading complete")
            result = ctx.adapter.after_weight_iter_load(result)
        except Exception as e:
            raise StrategyFailed(str(e), mutated=True) from e
        return result

    def _stream_weights(self, model_uri, ctx, model=None) -> Iterator[tuple[str, torch.Tensor]]:
        yield from ctx.adapter.build_model_streamer_weight_iter(model_uri, model=model)


class DefaultStrategy(LoadStrategy):
    """Last resort: the engine's native loader (default_strategy.py)."""

    name = "default"
    requires = (EngineAdapter.load_via_native,)

    def load(self, result: LoadResult, ctx: LoadContext) -> LoadResult:
        result = _as_load_result(result)
        try:
            result = ctx.adapter.load_via_native(result)
            return ctx.adapter.after_native_load(result)
        except Exception as e:
            raise StrategyFailed(str(e), mutated=True) from e


class LoadStrategyChain:
    """Prioritized chain of model loading strategies (__init__.py:45-136)."""

    @staticmethod
    def default_strategies() -> list:
        # The reference's order is RDMA, ServerCache, InstantTensor, ModelStreamer, GDS,
        # Default (__init__.py:71-78); the two placement strategies stand where
        # ModelStreamer does.
        return [HipPlacementStrategy(), HipStreamerStrategy(), DefaultStrategy()]

    @staticmethod
    def run(model: nn.Module, ctx: LoadContext, strategies: Sequence[LoadStrategy] | None = None) -> nn.Module:
        all_strategies = list(strategies) if strategies is not None else LoadStrategyChain.default_strategies()
        eligible = [s for s in all_strategies if s.is_available(ctx)]
        logger.info(f"Eligible loaders: {[s.name for s in eligible]}")
        result = LoadResult(value=model, model=model)
        for strategy in eligible:
            logger.info(f"[Worker {ctx.global_rank}] Trying strategy: {strategy.name}")
            try:
                result = strategy.load(result, ctx)
                result.metadata["weight_loading_strategy"] = strategy.name
                return result.value
            except StrategyFailed as e:
                logger.warning(f"[Worker {ctx.global_rank}] Strategy {strategy.name} failed, trying next: {e}")
                strategy.rollback(ctx)
                if e.mutated:
                    result = LoadStrategyChain._reinit_for_retry(result, ctx, strategy)
                continue
            except Exception as e:  # noqa: BLE001 - the chain keeps the engine alive
                logger.warning(f"[Worker {ctx.global_rank}] Strategy {strategy.name} raised unexpected error, "
                               f"trying next: {e}")
                strategy.rollback(ctx)
        raise RuntimeError(
            f"[Worker {ctx.global_rank}] No loading strategy succeeded for model '{ctx.identity.model_name}'")

    @staticmethod
    def _reinit_for_retry(result: LoadResult, ctx: LoadContext, strategy: LoadStrategy) -> LoadResult:
        if ctx.adapter is None:
            raise RuntimeError(f"[Worker {ctx.global_rank}] Strategy '{strategy.name}' mutated the model but no "
                               "adapter can reinitialize it")
        try:
            return ctx.adapter.reinit_for_retry(result)
        except UnsupportedCapability as exc:
            raise RuntimeError(f"[Worker {ctx.global_rank}] Strategy '{strategy.name}' mutated the model but adapter "
                               "does not support retry reinitialization") from exc


def layout_from_module(model: nn.Module, *, tp_size: int = 1, tp_rank: int = 0, expert_mapping=None,
                       skip_prefixes: Sequence[str] = ()) -> PlacementLayout:
    """Build a ``PlacementLayout`` from a torch module the way the reference's direct loader
    inspects one: ``named_parameters()`` for names, shapes, dtypes and storage,
    ``stacked_params_mapping`` and ``get_expert_mapping()`` when the model exposes them
    (engines/vllm/refit/installer.py:489-497,773-797)."""
    from .engine import ParamSpec

    params, dests = [], []
    for name, p in model.named_parameters():
        params.append(ParamSpec(name, safetensors_dtype_of(p), tuple(p.shape)))
        dests.append(p.data)
    raw = getattr(model, "stacked_params_mapping", None)
    stacked = [(str(e[0]), str(e[1])) for e in raw] if raw else None
    if expert_mapping is None and callable(getattr(model, "get_expert_mapping", None)):
        expert_mapping = list(model.get_expert_mapping())
    return PlacementLayout(params, dests, tp_size, tp_rank, stacked, expert_mapping, tuple(skip_prefixes))
