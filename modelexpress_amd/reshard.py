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


class ReslicePlan:
    """Recorded copies resolved once and replayed every refit step.

    The reference builds its plan once and re-derives nothing per step that the plan and the
    registered buffer addresses fix (refit/reshard/receiver.py:787-801, cached descriptors): here the
    op-chains are replayed to strided views, checked and split into calls when the plan is built, and
    the descriptor arrays handed to the library are rebuilt only when a source or parameter moved.
    A model with thousands of per-expert sources costs a few hundred milliseconds to resolve and
    nothing per step after that: each call's views are lowered into a device-resident ``mxp_view_plan``."""

    def __init__(self, copies: Sequence[RecordedCopy], sources: Mapping[str, torch.Tensor], params: Mapping[str, torch.Tensor]):
        self.entries: list[tuple] = []  # (src_name, src_elem_offset, param_name, dst_elem_offset, shape, src_strides, dst_strides, es_src, es_dst, cast)
        self.bytes = 0
        self._src_meta: dict[str, tuple] = {}
        self._param_meta: dict[str, tuple] = {}
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
            if any(n == 0 for n in shape):
                continue
            span = c.dest_offset + sum((n - 1) * st for n, st in zip(shape, c.dest_stride)) + 1
            if c.dest_offset < 0 or span > dst.untyped_storage().nbytes() // dst.element_size() - dst.storage_offset():
                raise UnsupportedReshard(f"{c.param_name}: destination view leaves the parameter's storage")
            self.entries.append((c.src_name, off, c.param_name, int(c.dest_offset), shape, stride, tuple(int(s) for s in c.dest_stride),
                                 src.element_size(), dst.element_size(), cast))
            n = dst.element_size()
            for v in shape:
                n *= v
            self.bytes += n
            self._src_meta[c.src_name] = (tuple(src.shape), src.dtype)
            self._param_meta[c.param_name] = (tuple(dst.shape), dst.dtype)
        self.batches = self._split_by_overlap()
        self._key: tuple | None = None
        self._arrays: list = []

    def _split_by_overlap(self) -> list:
        """Indices of ``entries`` grouped into calls.  One call moves every view whose destination span is
        clear of the others'; a view whose span (first to last element it can touch, holes included - the
        conservative test of refit/reshard/receiver.py:289-321) meets an earlier one's starts a new call, so
        overlapping views land in plan order as the reference's sequential fallback does."""
        import bisect

        def span(e):
            _s, _so, param, do, shape, _ss, ds, _es_s, es_d, _c = e
            return param, do * es_d, (do + sum((n - 1) * st for n, st in zip(shape, ds)) + 1) * es_d

        spans = [span(e) for e in self.entries]
        order = sorted(range(len(spans)), key=lambda i: spans[i])
        if all(spans[a][0] != spans[b][0] or spans[a][2] <= spans[b][1] for a, b in zip(order, order[1:])):
            return [list(range(len(spans)))] if spans else []
        batches, cur, taken = [], [], {}  # taken: parameter -> sorted, pairwise disjoint [(lo, hi)]
        for i, (param, lo, hi) in enumerate(spans):
            held = taken.setdefault(param, [])
            k = bisect.bisect_left(held, (lo, hi))
            if (k > 0 and held[k - 1][1] > lo) or (k < len(held) and held[k][0] < hi):
                batches.append(cur)
                cur, taken = [], {param: []}
                held, k = taken[param], 0
            held.insert(k, (lo, hi))
            cur.append(i)
        if cur:
            batches.append(cur)
        return batches

    def replay(self, *, stream: int = 0) -> int:
        """``run`` again on the tensors of the last ``run``, which the caller guarantees are where they were
        (buffers registered once, as the reference's are): launches only, no per-tensor checks."""
        if self._key is None:
            raise UnsupportedReshard("replay before the first run")
        for plan in self._arrays:
            plan.run(stream=stream)
        return self.bytes

    def close(self) -> None:
        for plan in self._arrays:
            plan.close()
        self._arrays = []

    def _build_arrays(self, engine, sources, params) -> None:
        from . import _lib as L

        self.close()
        for batch in self.batches:
            arr = (L.ViewCopy * max(1, len(batch)))()
            for o, i in zip(arr, batch):
                src_name, so, param, do, shape, ss, ds, es_s, es_d, cast = self.entries[i]
                o.src = sources[src_name].data_ptr() + so * es_s
                o.dst = params[param].data_ptr() + do * es_d
                o.ndim, o.elem_size, o.cast = len(shape), es_d, cast
                for d, n in enumerate(shape):
                    o.shape[d], o.src_strides[d], o.dst_strides[d] = n, ss[d], ds[d]
            self._arrays.append(engine.view_plan(arr, len(batch)))  # lowered and uploaded here, once

    def run(self, engine: PlacementEngine, sources: Mapping[str, torch.Tensor], params: Mapping[str, torch.Tensor], *,
            stream: int = 0) -> int:
        """Moves every copy; returns the bytes written.  The tensors may live elsewhere than when the plan was
        built, but must have the shapes and dtypes it was built for."""
        key = []
        for held, meta, is_source in ((sources, self._src_meta, True), (params, self._param_meta, False)):
            for name, (shape, dtype) in meta.items():
                t = held.get(name)
                if t is None or tuple(t.shape) != shape or t.dtype != dtype or (is_source and not t.is_contiguous()):
                    raise UnsupportedReshard(f"'{name}' is missing or changed shape, dtype or layout since the plan was built")
                key.append(t.data_ptr())
        key.append(id(engine))
        if tuple(key) != self._key:
            self._build_arrays(engine, sources, params)
            self._key = tuple(key)
        for plan in self._arrays:
            plan.run(stream=stream)  # launches only: one kernel for every row / element box, one per kind of transposed view
        return self.bytes


def execute_recorded_copies(engine: PlacementEngine, copies: Sequence[RecordedCopy], sources: Mapping[str, torch.Tensor],
                            params: Mapping[str, torch.Tensor], *, stream: int = 0) -> int:
    """Runs every copy on the device; returns the number of bytes written.  ``sources`` holds the
    full (contiguous) source tensors, ``params`` the destination parameters; both stay where they are."""
    return ReslicePlan(copies, sources, params).run(engine, sources, params, stream=stream)
