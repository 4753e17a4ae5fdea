"""Device execution of recorded scatter copies.

Mirrors the data model of the reference's reshard receiver: a ``RecordedCopy`` says "read
``src_name`` sliced by ``op_chain`` and write it into ``param_name`` at
``as_strided(dest_shape, dest_stride, dest_offset)``" (modelexpress/refit/reshard/types.py:57-71).
The op-chain is replayed on a zero-storage tensor to a strided source view, as the reference
does (refit/reshard/slice_plan.py:136-164, ``_replay_view``); the copies then run through
``mxp_copy_views``: pitched boxes (all of them in one launch), the LDS transpose for a transposed innermost dimension,
or element runs - instead of the reference's per-run descriptors and per-view ``copy_``
(slice_plan.py:259-339, receiver.py:919-960).  A dtype difference between source and
parameter is converted on the way ("raw-copy vs convert-via-staging", types.py:62-63).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping, Sequence

import torch

from .engine import CAST_CODES, PlacementEngine
from .load_strategy import safetensors_dtype_of

OpChain = Sequence[tuple]  # ((op_name, args, kwargs), ...)


class UnsupportedReshard(RuntimeError):
    """The op-chain is not a pure strided view of its source, or the copy cannot be placed."""


@dataclass
class RecordedCopy:
    src_name: str
    op_chain: OpChain
    param_name: str
    dest_offset: int
    dest_shape: tuple
    dest_stride: tuple
    dest_dtype: Any = None


def replay_view(op_chain: OpChain, global_shape: Sequence[int]) -> tuple:
    """``(storage_offset, shape, stride)`` of the view the op-chain selects in a row-major source of
    ``global_shape``.  Raises ``UnsupportedReshard`` when an op copies (the result no longer
    shares the source's storage) or does not return a tensor."""
    src = torch.empty(tuple(int(g) for g in global_shape), device="meta")
    t: Any = src
    for op_name, args, kw in op_chain:
        t = getattr(t, op_name)(*args, **dict(kw))
    if not isinstance(t, torch.Tensor):
        raise UnsupportedReshard(f"op-chain resolved to non-tensor {type(t).__name__}")
    if t is not src and t._base is not src:
        raise UnsupportedReshard("op-chain includes a copy (not a pure view)")
    return int(t.storage_offset()), tuple(int(s) for s in t.shape), tuple(int(s) for s in t.stride())


def execute_recorded_copies(engine: PlacementEngine, copies: Sequence[RecordedCopy], sources: Mapping[str, torch.Tensor],
                            params: Mapping[str, torch.Tensor], *, stream: int = 0) -> int:
    """Runs every copy on the device; returns the number of bytes written.  ``sources`` holds the
    full (contiguous) source tensors, ``params`` the destination parameters; both stay where they are."""
    resolved = []
    for c in copies:  # resolve everything before the first byte moves
        if c.src_name not in sources:
            raise UnsupportedReshard(f"source '{c.src_name}' is not available")
        if c.param_name not in params:
            raise UnsupportedReshard(f"parameter '{c.param_name}' is not available")
        src, dst = sources[c.src_name], params[c.param_name]
        if not src.is_contiguous():
            raise UnsupportedReshard(f"source '{c.src_name}' is not contiguous")
        off, shape, stride = replay_view(c.op_chain, src.shape)
        if tuple(c.dest_shape) != shape:
            raise UnsupportedReshard(f"{c.param_name}: dest {tuple(c.dest_shape)} != resolved view {shape}")
        sd, dd = safetensors_dtype_of(src), safetensors_dtype_of(dst)
        cast = 0
        if sd != dd:
            cast = CAST_CODES.get((sd, dd), 0)
            if not cast:
                raise UnsupportedReshard(f"{c.param_name}: no conversion from {sd} to {dd}")
        span = c.dest_offset + sum((n - 1) * st for n, st in zip(shape, c.dest_stride) if n > 0) + 1
        if any(n == 0 for n in shape):
            continue
        if c.dest_offset < 0 or span > dst.untyped_storage().nbytes() // dst.element_size() - dst.storage_offset():
            raise UnsupportedReshard(f"{c.param_name}: destination view leaves the parameter's storage")
        resolved.append((src.data_ptr() + off * src.element_size(), dst.data_ptr() + c.dest_offset * dst.element_size(),
                         shape, stride, tuple(int(s) for s in c.dest_stride), dst.element_size(), cast))
    # One call moves every view whose destination span is clear of the others'; a view whose span
    # (first to last byte it can touch, holes included - the conservative test of
    # refit/reshard/receiver.py:289-321) meets an earlier one's starts a new call, so overlapping
    # views land in plan order as the reference's sequential fallback does.
    written = 0
    batch: list[dict] = []
    spans: list[tuple[int, int]] = []
    for sp, dp, shape, ss, ds, es, cast in resolved:
        lo = dp
        hi = dp + (sum((n - 1) * st for n, st in zip(shape, ds)) + 1) * es
        if any(lo < b and a < hi for a, b in spans):
            engine.copy_views(batch, stream=stream)
            batch, spans = [], []
        batch.append({"src": sp, "dst": dp, "shape": shape, "elem_size": es, "src_strides": ss, "dst_strides": ds, "cast": cast})
        spans.append((lo, hi))
        n = es
        for v in shape:
            n *= v
        written += n
    if batch:
        engine.copy_views(batch, stream=stream)  # one launch for every row / element box, one per kind of transposed view
    return written
