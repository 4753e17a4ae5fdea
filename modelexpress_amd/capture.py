"""Geometry capture: which slice of each full source tensor an engine's own weight loader reads,
and where in which parameter it lands - the producer of the ``RecordedCopy`` descriptors that
``reshard.execute_recorded_copies`` runs on the device.

Same contract as the reference's capture (modelexpress/refit/reshard/geometry.py:259-309): the
model's ``load_weights`` is dry-run once per source with a placeholder that holds no data; the
view / slice calls the loader makes on it are collected as an op-chain, and ``copy_`` - the sink -
records ``(parameter, offset, shape, stride, dtype)`` of the destination and moves nothing.
A loader that needs the source's values (arithmetic, a dtype conversion, mask indexing) marks that
one source unsupported, with the operator that defeated it, and never yields a wrong copy.

The placeholder here (``SourceProbe``) is an alias of a real ``meta`` tensor: shapes, strides and
multi-output views (``chunk``, ``unbind``) come from torch itself, only the allowlist below and the
``copy_`` sink are handled in ``__torch_function__``, and any operator that reaches
``__torch_dispatch__`` is by construction one that would have read data.
"""

from __future__ import annotations

import functools
import logging
from dataclasses import dataclass, field
from typing import Any, Callable

import torch

from .reshard import RecordedCopy, UnsupportedReshard

logger = logging.getLogger("modelexpress_amd.capture")

# Pure view / slice / shape calls a weight loader may make on a source, by the method name the
# op-chain replays them with (geometry.py:60-82; ``unbind`` serves vLLM's fused-expert loader).
VIEW_OPS: dict[Callable, str] = {
    torch.Tensor.narrow: "narrow", torch.Tensor.view: "view", torch.Tensor.reshape: "reshape",
    torch.Tensor.__getitem__: "__getitem__", torch.Tensor.unsqueeze: "unsqueeze", torch.Tensor.squeeze: "squeeze",
    torch.Tensor.transpose: "transpose", torch.Tensor.t: "t", torch.Tensor.permute: "permute",
    torch.Tensor.flatten: "flatten", torch.Tensor.contiguous: "contiguous", torch.Tensor.chunk: "chunk",
    torch.Tensor.unbind: "unbind",
    # the same calls spelled as functions (torch.narrow(w, ...)): replayed as the method
    torch.narrow: "narrow", torch.reshape: "reshape", torch.unsqueeze: "unsqueeze", torch.squeeze: "squeeze",
    torch.transpose: "transpose", torch.t: "t", torch.permute: "permute", torch.flatten: "flatten", torch.chunk: "chunk",
    torch.unbind: "unbind",
}


@dataclass
class CaptureResult:
    """refit/reshard/types.py: the recorded copies plus what could not be captured."""

    copies: list = field(default_factory=list)
    unsupported: list = field(default_factory=list)   # source names
    unattributed: int = 0                             # copy_ calls outside any stamped weight_loader
    unsupported_reasons: dict = field(default_factory=dict)


def summarize_unsupported(reasons: dict, limit: int | None = 3) -> list:
    """Distinct causes with the number of sources each one defeated, most frequent first. Every message
    names its own source after `` on lazy ``, so that tail is dropped before grouping."""
    counts: dict[str, int] = {}
    for text in (reasons or {}).values():
        cause = str(text).split(" on lazy ", 1)[0].strip()
        counts[cause] = counts.get(cause, 0) + 1
    ranked = sorted(counts.items(), key=lambda kv: (-kv[1], kv[0]))
    return ranked if limit is None else ranked[:limit]


class _Recorder:
    def __init__(self) -> None:
        self.copies: list = []
        self.unattributed = 0
        self.current: str | None = None  # the parameter whose weight_loader is running


class SourceProbe(torch.Tensor):
    """A ``meta`` view of one full source tensor that remembers how the loader reached it."""

    _probe_name: str
    _probe_ops: tuple
    _probe_rec: Any
    _probe_meta: torch.Tensor

    @staticmethod
    def __new__(cls, meta: torch.Tensor, name: str, ops: tuple = (), recorder: Any = None):
        t = torch.Tensor._make_subclass(cls, meta, False)
        t._probe_meta, t._probe_name, t._probe_ops, t._probe_rec = meta, name, tuple(ops), recorder
        return t

    @classmethod
    def for_source(cls, name: str, dtype: torch.dtype, shape, recorder: Any = None) -> "SourceProbe":
        return cls(torch.empty(tuple(int(s) for s in shape), dtype=dtype, device="meta"), name, (), recorder)

    @classmethod
    def __torch_function__(cls, func, types, args=(), kwargs=None):
        kwargs = kwargs or {}
        if func is torch.Tensor.copy_:
            dest = args[0]
            src = args[1] if len(args) > 1 else kwargs.get("src")
            if isinstance(src, cls) and not isinstance(dest, cls):
                rec = src._probe_rec
                if rec is not None and rec.current is not None:
                    rec.copies.append(RecordedCopy(src._probe_name, src._probe_ops, rec.current, int(dest.storage_offset()),
                                                   tuple(int(s) for s in dest.shape), tuple(int(s) for s in dest.stride()),
                                                   dest.dtype))
                elif rec is not None:
                    rec.unattributed += 1
                return dest  # record only: nothing is copied, whatever device `dest` is on
        op_name = VIEW_OPS.get(func)
        if op_name is not None and args and isinstance(args[0], cls):
            me = args[0]
            out = func(me._probe_meta, *args[1:], **kwargs)
            op = (op_name, tuple(args[1:]), tuple(sorted(kwargs.items())))
            if isinstance(out, torch.Tensor):
                return cls(out, me._probe_name, me._probe_ops + (op,), me._probe_rec)
            if isinstance(out, (tuple, list)):  # chunk / unbind: one probe per output, indexed on replay
                return tuple(cls(o, me._probe_name, me._probe_ops + (op, ("__getitem__", (i,), ())), me._probe_rec)
                             for i, o in enumerate(out))
            raise UnsupportedReshard(f"{op_name!r} on lazy {me._probe_name!r} returned a non-tensor ({type(out).__name__}); cannot defer.")
        with torch._C.DisableTorchFunctionSubclass():  # metadata reads resolve here; anything else reaches __torch_dispatch__
            return func(*args, **kwargs)

    @classmethod
    def __torch_dispatch__(cls, func, types, args=(), kwargs=None):
        for a in list(args) + list((kwargs or {}).values()):
            if isinstance(a, cls):
                raise UnsupportedReshard(f"unsupported op {func} on lazy {a._probe_name!r} (chain={a._probe_ops}); "
                                         f"supported: {sorted(VIEW_OPS.values())} + copy_.")
        return func(*args, **(kwargs or {}))


def _stamp_loaders(model: torch.nn.Module, recorder: _Recorder, default_weight_loader: Callable | None) -> list:
    """Wraps every parameter's ``weight_loader`` (or the framework's default one) so that ``copy_`` knows
    which parameter is being written.  The wrapper passes its arguments through untouched: vLLM's
    fused-expert loader is called by keyword only."""
    saved = []
    for name, param in model.named_parameters():
        original = getattr(param, "weight_loader", None)
        inner = original if original is not None else default_weight_loader
        if inner is None:
            continue

        def make(inner=inner, name=name):
            @functools.wraps(inner)
            def stamped(*a, **kw):
                recorder.current = name
                try:
                    return inner(*a, **kw)
                finally:
                    recorder.current = None
            return stamped

        param.weight_loader = make()
        saved.append((param, original))
    return saved


def capture_geometry(model: torch.nn.Module, manifest, default_weight_loader: Callable | None = None) -> CaptureResult:
    """Dry-runs ``model.load_weights`` (ideally on a ``meta`` twin of the engine's model) once per entry of
    ``manifest`` - ``(name, dtype, shape)`` of every full source tensor - and returns the recorded copies.
    One source at a time, so an unsupported loader is charged to that source only."""
    recorder = _Recorder()
    saved = _stamp_loaders(model, recorder, default_weight_loader)
    result = CaptureResult()
    try:
        for name, dtype, shape in manifest:
            try:
                model.load_weights([(name, SourceProbe.for_source(name, dtype, shape, recorder))])
            except UnsupportedReshard as exc:
                result.unsupported.append(name)
                result.unsupported_reasons[name] = str(exc)
                recorder.copies = [c for c in recorder.copies if c.src_name != name]  # nothing partial survives
    finally:
        for param, original in saved:
            if original is None:
                try:
                    del param.weight_loader
                except AttributeError:
                    pass
            else:
                param.weight_loader = original
    result.copies = recorder.copies
    result.unattributed = recorder.unattributed
    logger.info("reshard capture: %d copies, %d unsupported source(s), %d unattributed copy_", len(result.copies),
                len(result.unsupported), result.unattributed)
    for reason, count in summarize_unsupported(result.unsupported_reasons):
        logger.warning("reshard capture: %d source(s) unsupported, cause: %s", count, reason)
    return result
