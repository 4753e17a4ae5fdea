"""Python handles over the C ABI: Checkpoint, PlacementPlan, PlacementEngine.

PyTorch appears here only as the owner of device memory and streams: destination
parameters are torch tensors whose ``data_ptr()`` is handed to the library, and all
arithmetic happens in libmxplace.so.
"""

from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from typing import Iterable, Sequence

from . import _lib as L


@dataclass(frozen=True)
class TensorEntry:
    name: str
    dtype: str
    shape: tuple
    file_index: int
    file_offset: int
    nbytes: int


@dataclass(frozen=True)
class ParamSpec:
    """One parameter of the serving rank: what the engine allocated for it."""

    name: str
    dtype: str
    shape: tuple

    @property
    def nbytes(self) -> int:
        n = L.DTYPE_SIZE[self.dtype]
        for d in self.shape:
            n *= int(d)
        return n


@dataclass(frozen=True)
class VirtualTensor:
    """A checkpoint tensor assembled from boxes of real tensors.  ``shards`` rows are
    ``(source_tensor_name, source_offset, shard_offset, shape)`` with per-dimension tuples."""

    name: str
    shape: tuple
    shards: tuple


# MXP_CAST_* of include/mxp.h
CAST_CODES = {("F32", "BF16"): 1, ("BF16", "F32"): 2, ("F16", "F32"): 3, ("F32", "F16"): 4, ("F8_E4M3", "BF16"): 5,
              ("F16", "BF16"): 6, ("BF16", "F16"): 7}


@dataclass(frozen=True)
class WriteEntry:
    tensor: str
    param: str
    kind: str
    cast: int  # 0 or a CAST_CODES value
    src_offset: int
    src_pitch: int
    dst_offset: int
    dst_pitch: int
    rows: int
    row_bytes: int
    paired_runs: int


class Checkpoint:
    """A parsed safetensors checkpoint (directory or single file)."""

    def __init__(self, model_path: str):
        self._h = C.c_void_p()
        L.check(L.lib().mxp_ckpt_open(str(model_path).encode(), C.byref(self._h)))
        self.path = str(model_path)

    def close(self) -> None:
        if self._h:
            L.lib().mxp_ckpt_close(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:  # noqa: BLE001 - interpreter shutdown
            pass

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def __len__(self) -> int:
        return int(L.lib().mxp_ckpt_tensor_count(self._h))

    def tensors(self) -> list[TensorEntry]:
        out = []
        info = L.TensorInfo()
        for i in range(len(self)):
            L.check(L.lib().mxp_ckpt_tensor_info(self._h, i, C.byref(info)))
            out.append(TensorEntry(info.name.decode(), L.DTYPES[info.dtype], tuple(info.shape[: info.ndim]),
                                   info.file_index, info.file_offset, info.nbytes))
        return out

    def files(self) -> list[dict]:
        """The shard files.  ``staging_pad``: a caller that stages a whole file in device memory for
        ``execute_resident`` does best to put its first byte that many bytes past a 256-byte boundary: the
        data section then starts on one, and strided row gathers touch no line more than they need
        (measured on the Llama-3-8B rank share: 1.5 points of HBM peak)."""
        out = []
        info = L.FileInfo()
        for i in range(int(L.lib().mxp_ckpt_file_count(self._h))):
            L.check(L.lib().mxp_ckpt_file_info(self._h, i, C.byref(info)))
            out.append({"path": info.path.decode(), "file_size": info.file_size, "data_start": info.data_start,
                        "n_tensors": info.n_tensors, "staging_pad": (-int(info.data_start)) % 256 if info.data_start % 8 == 0 else 0})
        return out

    def find(self, name: str) -> int:
        return int(L.lib().mxp_ckpt_find(self._h, name.encode()))


class PlacementPlan:
    """Destination map of one rank, built from the rank's parameter table.

    ``stacked_params_mapping`` is a list of ``(fused_suffix, member_suffix)`` pairs in
    pack order (None = built-in qkv / gate_up groups); ``expert_mapping`` rows are
    ``(param_prefix, weight_prefix, expert_id, shard[, local_id])`` where a missing
    ``local_id`` means the global id, -1 means "not on this rank", -2 "unknown".
    """

    def __init__(self, ckpt: Checkpoint, params: Iterable[ParamSpec], *, tp_size: int = 1, tp_rank: int = 0,
                 stacked_params_mapping: Sequence | None = None, expert_mapping: Sequence | None = None,
                 skip_prefixes: Sequence[str] = (), virtual_tensors: Sequence[VirtualTensor] = (),
                 allow_cast: bool = False, allow_unmapped: bool = False,
                 allow_uncovered: bool = False, fp8_block_check: bool = True,
                 nonlocal_experts_unmapped: bool = False):
        lib = L.lib()
        self.ckpt = ckpt
        flags = 0
        flags |= L.PLAN_ALLOW_CAST_F32_BF16 if allow_cast else 0
        flags |= L.PLAN_ALLOW_UNMAPPED if allow_unmapped else 0
        flags |= L.PLAN_ALLOW_UNCOVERED if allow_uncovered else 0
        flags |= 0 if fp8_block_check else L.PLAN_NO_FP8_BLOCK_CHECK
        flags |= L.PLAN_NONLOCAL_EXPERTS_UNMAPPED if nonlocal_experts_unmapped else 0
        self._h = C.c_void_p()
        L.check(lib.mxp_plan_create(ckpt._h, tp_size, tp_rank, flags, C.byref(self._h)))
        self.tp_size, self.tp_rank = tp_size, tp_rank
        self.params = list(params)
        for p in self.params:
            shape = (C.c_int64 * max(1, len(p.shape)))(*[int(d) for d in p.shape])
            L.check(lib.mxp_plan_add_param(self._h, p.name.encode(), L.DTYPE_CODE[p.dtype], len(p.shape), shape))
        for fused, member in stacked_params_mapping or ():
            L.check(lib.mxp_plan_add_stacked(self._h, str(fused).encode(), str(member).encode()))
        for row in expert_mapping or ():
            p_pre, w_pre, eid, shard = row[:4]
            local = int(row[4]) if len(row) > 4 else int(eid)
            L.check(lib.mxp_plan_add_expert(self._h, p_pre.encode(), w_pre.encode(), int(eid), shard.encode(), local))
        for pre in skip_prefixes:
            L.check(lib.mxp_plan_add_skip_prefix(self._h, pre.encode()))
        for v in virtual_tensors:
            nd = len(v.shape)
            arr = lambda t: (C.c_int64 * max(1, nd))(*[int(x) for x in t])  # noqa: E731
            vi = L.check(lib.mxp_plan_add_virtual(self._h, v.name.encode(), nd, arr(v.shape)))
            for source, src_off, shard_off, shape in v.shards:
                L.check(lib.mxp_plan_add_virtual_shard(self._h, vi, source.encode(), arr(src_off), arr(shard_off),
                                                       arr(shape)))
        L.check(lib.mxp_plan_build(self._h))

    def close(self) -> None:
        if self._h:
            L.lib().mxp_plan_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:  # noqa: BLE001
            pass

    def writes(self) -> list[WriteEntry]:
        lib = L.lib()
        tensors = self.ckpt.tensors()
        out = []
        info = L.WriteInfo()
        for i in range(int(lib.mxp_plan_write_count(self._h))):
            L.check(lib.mxp_plan_write_info(self._h, i, C.byref(info)))
            out.append(WriteEntry(tensors[info.tensor_index].name, self.params[info.param_index].name,
                                  L.WRITE_KINDS[info.kind], int(info.cast), info.src_offset, info.src_pitch,
                                  info.dst_offset, info.dst_pitch, info.rows, info.row_bytes, info.paired_runs))
        return out

    def param_info(self) -> list[dict]:
        lib = L.lib()
        out = []
        info = L.ParamInfo()
        for i in range(int(lib.mxp_plan_param_count(self._h))):
            L.check(lib.mxp_plan_param_info(self._h, i, C.byref(info)))
            out.append({"name": info.name.decode(), "dtype": L.DTYPES[info.dtype],
                        "shape": tuple(info.shape[: info.ndim]), "nbytes": info.nbytes,
                        "bytes_written": info.bytes_written, "n_writes": info.n_writes})
        return out

    def totals(self) -> dict:
        vals = [C.c_uint64() for _ in range(4)]
        L.check(L.lib().mxp_plan_totals(self._h, *[C.byref(v) for v in vals]))
        keys = ("file_bytes", "h2d_bytes", "placed_bytes", "kernel_algorithmic_bytes")
        return {k: int(v.value) for k, v in zip(keys, vals)}


def _ptr_array(ptrs: Sequence[int]):
    return (C.c_void_p * max(1, len(ptrs)))(*[C.c_void_p(int(p)) for p in ptrs])


class PlacementEngine:
    """Device-side executor: pinned ring + streams + kernels of one GPU."""

    def __init__(self, device: int = 0, *, ring_slots: int = 0, slot_bytes: int = 0, reader_threads: int = 0,
                 streams: int = 0, tile_bytes: int = 0, nan_bits: int = 0, use_o_direct: bool = False,
                 pack_strided_on_host: bool | None = None):
        pack = 0 if pack_strided_on_host is None else (1 if pack_strided_on_host else 2)
        opts = L.EngineOptions(device=device, ring_slots=ring_slots, slot_bytes=slot_bytes,
                               reader_threads=reader_threads, streams=streams, tile_bytes=tile_bytes,
                               nan_bits=nan_bits, pack_strided_on_host=pack, use_o_direct=int(use_o_direct))
        self._h = C.c_void_p()
        L.check(L.lib().mxp_engine_create(C.byref(opts), C.byref(self._h)))
        self.device = device
        self.nan_bits = nan_bits or 0x7FC0  # the bf16 image this engine gives every fp32 / fp16 NaN

    def close(self) -> None:
        if self._h:
            L.lib().mxp_engine_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:  # noqa: BLE001
            pass

    # ---- buffers ----
    def allocate(self, plan: PlacementPlan, fill: int | None = None) -> list:
        """One uint8 torch tensor per parameter of ``plan`` on this engine's device."""
        import torch

        dev = torch.device("cuda", self.device)
        out = []
        for p in plan.params:
            n = max(p.nbytes, 1)
            t = torch.empty(n, dtype=torch.uint8, device=dev) if fill is None else torch.full(
                (n,), fill, dtype=torch.uint8, device=dev)
            out.append(t[: p.nbytes] if p.nbytes != n else t)
        return out

    # ---- placement ----
    def prepare(self, plan: PlacementPlan) -> None:
        L.check(L.lib().mxp_prepare(self._h, plan._h))

    def execute(self, plan: PlacementPlan, dst: Sequence, *, after_stream: int | None = None) -> dict:
        """Ingest from storage into ``dst`` (torch tensors or raw device addresses).

        The engine's streams first wait for what is already queued on ``after_stream`` (a raw
        ``hipStream_t``; default: the calling thread's current torch stream), so pending work on
        the destinations lands before the placed bytes, as it would ahead of ``copy_``."""
        ptrs = _ptr_array([_addr(t) for t in dst])
        stats = L.ExecStats()
        if after_stream is None:
            after_stream = _current_stream(self.device)
        rc = L.lib().mxp_execute_after(self._h, plan._h, ptrs, C.c_void_p(after_stream), C.byref(stats))
        if rc < 0:
            err = L.MxpError(int(rc), L.lib().mxp_last_error().decode("utf-8", "replace"))
            err.mutated = bool(stats.mutated)
            raise err
        return stats.as_dict()

    def execute_resident(self, plan: PlacementPlan, staged_files: Sequence, dst: Sequence, *, stream: int = 0,
                         timed: bool = False) -> dict | None:
        """Placement from shard files already staged in HBM; one launch.  ``staged_files`` and ``dst`` are
        torch tensors / raw addresses, or pointer tables built once with ``pointer_table`` (a serving loop
        that refits into the same buffers every step then spends nothing on converting them again)."""
        fptrs = staged_files if isinstance(staged_files, C.Array) else _ptr_array([_addr(t) for t in staged_files])
        dptrs = dst if isinstance(dst, C.Array) else _ptr_array([_addr(t) for t in dst])
        stats = L.ExecStats() if timed else None
        L.check(L.lib().mxp_execute_resident(self._h, plan._h, fptrs, dptrs, C.c_void_p(stream),
                                             C.byref(stats) if timed else None))
        return stats.as_dict() if timed else None

    @staticmethod
    def pointer_table(buffers: Sequence):
        """The ``void*`` array the C ABI takes for ``buffers`` (torch tensors or raw addresses).  The table
        holds addresses only: the caller keeps the buffers alive and in place."""
        return _ptr_array([_addr(t) for t in buffers])

    def set_direct_placement(self, min_bytes: int = 0) -> None:
        """Ingest copies contiguous unconverted pieces of at least ``min_bytes`` straight to their final address
        (0 = the default, 64 KiB); a negative value sends every byte through the bounce slot and the kernel."""
        L.check(L.lib().mxp_engine_set_direct_placement(self._h, int(min_bytes)))

    def set_launch_timing(self, on: bool = True) -> None:
        """Asynchronous resident launches record an event pair around their placement kernel (no synchronisation)."""
        L.check(L.lib().mxp_engine_set_launch_timing(self._h, 1 if on else 0))

    def launch_times(self, n: int = 256) -> list[float]:
        """Kernel durations (ms) of the most recent ``n`` timed resident launches, oldest first; waits for them."""
        out = (C.c_float * max(1, n))()
        got = C.c_int32()
        L.check(L.lib().mxp_engine_launch_times(self._h, out, n, C.byref(got)))
        return [float(out[i]) for i in range(got.value)]

    def set_fused_digests(self, on: bool = True) -> None:
        """Placements also accumulate the ``tensor_digest`` sums of every parameter inside the placement kernel."""
        L.check(L.lib().mxp_engine_set_fused_digests(self._h, 1 if on else 0))

    def digests(self, plan: PlacementPlan) -> list[str]:
        """The ``tensor_digest`` of every parameter as the last execute of ``plan`` left it (fused digests on)."""
        n = len(plan.params)
        out = (C.c_uint8 * (16 * max(1, n)))()
        L.check(L.lib().mxp_plan_digests(self._h, plan._h, out, n))
        return [bytes(out[16 * i: 16 * i + 16]).hex() for i in range(n)]

    def checksums(self, plan: PlacementPlan) -> list[str]:
        n = len(plan.params)
        out = (C.c_uint32 * max(1, n))()
        L.check(L.lib().mxp_plan_checksums(self._h, plan._h, out, n))
        return [format(out[i], "08x") for i in range(n)]

    # ---- stand-alone operators ----
    def checksum32(self, buffers: Sequence, nbytes: Sequence[int] | None = None, *, stream: int = 0) -> list[str]:
        n = len(buffers)
        sizes = [_nbytes(t) for t in buffers] if nbytes is None else list(nbytes)
        out = (C.c_uint32 * max(1, n))()
        L.check(L.lib().mxp_checksum32(self._h, _ptr_array([_addr(t) for t in buffers]),
                                       (C.c_uint64 * max(1, n))(*sizes), n, out, C.c_void_p(stream)))
        return [format(out[i], "08x") for i in range(n)]

    def checksum32_static(self, buffers: Sequence, nbytes: Sequence[int] | None = None, *, stream: int = 0) -> list[str]:
        """``checksum32`` through the entry point that allocates nothing (at most 1024 buffers, about 12 GiB)."""
        n = len(buffers)
        sizes = [_nbytes(t) for t in buffers] if nbytes is None else list(nbytes)
        out = (C.c_uint32 * max(1, n))()
        L.check(L.lib().mxp_checksum32_static(self._h, _ptr_array([_addr(t) for t in buffers]),
                                              (C.c_uint64 * max(1, n))(*sizes), n, out, C.c_void_p(stream)))
        return [format(out[i], "08x") for i in range(n)]

    def verify_plan(self, buffers: Sequence, nbytes: Sequence[int] | None = None) -> "VerifyPlan":
        """``buffers`` lowered once for repeated ``checksums()`` / ``digests()`` passes."""
        return VerifyPlan(self, buffers, nbytes)

    def digest(self, buffers: Sequence, nbytes: Sequence[int] | None = None, *, stream: int = 0,
               with_scalars: bool = False):
        n = len(buffers)
        sizes = [_nbytes(t) for t in buffers] if nbytes is None else list(nbytes)
        out = (C.c_uint8 * (16 * max(1, n)))()
        sc = (C.c_uint64 * (7 * max(1, n)))()
        L.check(L.lib().mxp_digest(self._h, _ptr_array([_addr(t) for t in buffers]),
                                   (C.c_uint64 * max(1, n))(*sizes), n, out, sc, C.c_void_p(stream)))
        hexes = [bytes(out[16 * i: 16 * i + 16]).hex() for i in range(n)]
        if with_scalars:
            return hexes, [[int(sc[7 * i + k]) for k in range(7)] for i in range(n)]
        return hexes

    def cast_f32_bf16(self, src, dst, n_elems: int, *, stream: int = 0, checksum: bool = True) -> str | None:
        out = C.c_uint32()
        L.check(L.lib().mxp_cast_f32_bf16(self._h, C.c_void_p(_addr(src)), C.c_void_p(_addr(dst)), n_elems,
                                          C.byref(out) if checksum else None, C.c_void_p(stream)))
        return format(out.value, "08x") if checksum else None

    def cast(self, src, dst, n_elems: int, src_dtype: str, dst_dtype: str, *, stream: int = 0,
             checksum: bool = True) -> str | None:
        """``dst.copy_(src)`` across dtypes for the supported pairs (``CAST_CODES``)."""
        code = CAST_CODES.get((src_dtype, dst_dtype))
        if code is None:
            raise ValueError(f"no conversion from {src_dtype} to {dst_dtype}")
        out = C.c_uint32()
        L.check(L.lib().mxp_cast(self._h, C.c_void_p(_addr(src)), C.c_void_p(_addr(dst)), n_elems, code,
                                 C.byref(out) if checksum else None, C.c_void_p(stream)))
        return format(out.value, "08x") if checksum else None

    def gather2d(self, src, src_pitch: int, dst, dst_pitch: int, rows: int, row_bytes: int, *, stream: int = 0,
                 checksum: bool = True) -> str | None:
        out = C.c_uint32()
        L.check(L.lib().mxp_gather2d(self._h, C.c_void_p(_addr(src)), src_pitch, C.c_void_p(_addr(dst)), dst_pitch,
                                     rows, row_bytes, C.byref(out) if checksum else None, C.c_void_p(stream)))
        return format(out.value, "08x") if checksum else None

    def place_boxes(self, boxes: Sequence[dict], n_groups: int = 1, *, stream: int = 0,
                    checksums: bool = True) -> list[str] | None:
        """n pitched boxes in one launch.  Each box is a dict with ``src``, ``dst`` (tensors or
        device addresses), ``rows``, ``row_bytes`` and optionally ``src_pitch``, ``dst_pitch``,
        ``csum_index``, ``csum_group``, ``cast``."""
        arr = (L.Box * max(1, len(boxes)))()
        for i, b in enumerate(boxes):
            arr[i] = L.Box(src=_addr(b["src"]), dst=_addr(b["dst"]), src_pitch=b.get("src_pitch", 0),
                           dst_pitch=b.get("dst_pitch", 0), rows=b["rows"], row_bytes=b["row_bytes"],
                           csum_index=b.get("csum_index", 0), csum_group=b.get("csum_group", 0),
                           cast=int(b.get("cast", 0)))
        out = (C.c_uint32 * max(1, n_groups))()
        L.check(L.lib().mxp_place_boxes(self._h, arr, len(boxes), n_groups, out if checksums else None,
                                        C.c_void_p(stream)))
        return [format(out[i], "08x") for i in range(n_groups)] if checksums else None

    def shard_region(self, full, global_shape: Sequence[int], shard_offset: Sequence[int], shape: Sequence[int],
                     itemsize: int, out=None, *, stream: int = 0):
        """The sub-box of an assembled full tensor that one publisher owns, as a contiguous
        device buffer with its checksum (refit/reshard/verify.py:158-183).  ``full`` holds
        the row-major bytes of the whole tensor."""
        import torch

        if not len(global_shape) == len(shard_offset) == len(shape):
            raise ValueError(f"rank mismatch: global_shape {tuple(global_shape)}, shard_offset "
                             f"{tuple(shard_offset)} and shape {tuple(shape)} must have equal rank")
        n = itemsize
        for d in shape:
            n *= int(d)
        if out is None:
            out = torch.empty(max(n, 1), dtype=torch.uint8, device=torch.device("cuda", self.device))[:n]
        # merge trailing dims that are taken whole, keep the next one as the row index
        dims = [(int(g), int(o), int(s)) for g, o, s in zip(global_shape, shard_offset, shape)]
        run_src = run_dst = itemsize
        while dims and dims[-1][1] == 0 and dims[-1][2] == dims[-1][0]:
            g, _o, s = dims.pop()
            run_src *= g
            run_dst *= s
        base = _addr(full)
        boxes = []
        if not dims:
            boxes.append({"src": base, "dst": out, "rows": 1, "row_bytes": run_dst, "csum_index": 0})
        else:
            g, o, s = dims.pop()  # innermost sliced dim: a contiguous piece of s * run bytes per outer index
            piece = s * run_dst
            src_stride = g * run_src
            strides, acc = [], src_stride
            for gg, _oo, _ss in reversed(dims):
                strides.append(acc)
                acc *= gg
            strides.reverse()
            import itertools

            for k, idx in enumerate(itertools.product(*[range(ss) for _g, _o, ss in dims])):
                off = o * run_src + sum((i + oo) * st for i, (_gg, oo, _ss), st in zip(idx, dims, strides))
                boxes.append({"src": base + off, "dst": _addr(out) + k * piece, "rows": 1, "row_bytes": piece,
                              "csum_index": k * piece})
        sums = self.place_boxes(boxes, 1, stream=stream)
        return out, sums[0]

    def permute_copy(self, src, dst, shape: Sequence[int], perm: Sequence[int], elem_size: int, *,
                     src_strides: Sequence[int] | None = None, stream: int = 0, checksum: bool = True) -> str | None:
        """``dst = src.permute(perm).contiguous()`` on the device (row gather or LDS transpose)."""
        n = len(shape)
        shp = (C.c_int64 * max(1, n))(*[int(v) for v in shape])
        prm = (C.c_int32 * max(1, n))(*[int(v) for v in perm])
        strides = None if src_strides is None else (C.c_int64 * max(1, n))(*[int(v) for v in src_strides])
        out = C.c_uint32()
        L.check(L.lib().mxp_permute_copy(self._h, C.c_void_p(_addr(src)), C.c_void_p(_addr(dst)), n, shp, strides, prm,
                                         elem_size, C.byref(out) if checksum else None, C.c_void_p(stream)))
        return format(out.value, "08x") if checksum else None

    def copy_view(self, src, dst, shape: Sequence[int], elem_size: int, *, src_strides: Sequence[int] | None = None,
                  dst_strides: Sequence[int] | None = None, cast: int = 0, stream: int = 0,
                  checksum: bool = True) -> str | None:
        """``dst.as_strided(shape, dst_strides).copy_(src.as_strided(shape, src_strides))`` on the device
        (strides in elements, ``None`` = contiguous).  ``src`` / ``dst`` address the first element of each
        view; ``cast`` is a ``CAST_CODES`` value and ``elem_size`` then the destination element's size."""
        n = len(shape)
        shp = (C.c_int64 * max(1, n))(*[int(v) for v in shape])
        ss = None if src_strides is None else (C.c_int64 * max(1, n))(*[int(v) for v in src_strides])
        ds = None if dst_strides is None else (C.c_int64 * max(1, n))(*[int(v) for v in dst_strides])
        out = C.c_uint32()
        L.check(L.lib().mxp_copy_view(self._h, C.c_void_p(_addr(src)), C.c_void_p(_addr(dst)), n, shp, ss, ds,
                                      elem_size, cast, C.byref(out) if checksum else None, C.c_void_p(stream)))
        return format(out.value, "08x") if checksum else None

    def copy_views(self, views: Sequence[dict], *, stream: int = 0) -> None:
        """Many ``copy_view`` calls in one go (keys: src, dst, shape, elem_size and optionally src_strides,
        dst_strides, cast): all row / element boxes run in one launch, transposed views in one launch per element type and conversion."""
        L.check(L.lib().mxp_copy_views(self._h, self.views_array(views), len(views), C.c_void_p(stream)))

    @staticmethod
    def views_array(views: Sequence[dict]):
        """The ``_lib.ViewCopy`` array of ``views`` (the dicts ``copy_views`` takes), for callers that run the
        same views again (``copy_views_array``, ``view_plan``) and need not rebuild it per call."""
        arr = (L.ViewCopy * max(1, len(views)))()
        for v, o in zip(views, arr):
            shape = [int(x) for x in v["shape"]]
            o.src, o.dst, o.ndim, o.elem_size, o.cast = _addr(v["src"]), _addr(v["dst"]), len(shape), int(v["elem_size"]), int(v.get("cast", 0))
            for d, n in enumerate(shape):
                o.shape[d] = n
            for key, flag in (("src_strides", "contiguous_src"), ("dst_strides", "contiguous_dst")):
                st = v.get(key)
                setattr(o, flag, 1 if st is None else 0)
                for d, x in enumerate(st or ()):
                    getattr(o, key)[d] = int(x)
        return arr

    def describe_views(self, views: Sequence[dict]) -> list:
        """How ``copy_views`` would run each view (nothing is launched): ``("boxes" | "transpose" | "staged_tile",
        tile rows, tile row bytes)`` per view."""
        n = len(views)
        kinds, rows, row_bytes = ((C.c_int32 * max(1, n))() for _ in range(3))
        L.check(L.lib().mxp_describe_views(self._h, self.views_array(views), n, kinds, rows, row_bytes))
        return [(("boxes", "transpose", "staged_tile")[kinds[k]], rows[k], row_bytes[k]) for k in range(n)]

    def copy_views_array(self, arr, n: int, *, stream: int = 0) -> None:
        """``copy_views`` on an ``_lib.ViewCopy`` array the caller built (and may keep between calls)."""
        L.check(L.lib().mxp_copy_views(self._h, arr, n, C.c_void_p(stream)))

    def view_plan(self, arr, n: int) -> "ViewPlan":
        """The views of an ``_lib.ViewCopy`` array lowered once; ``ViewPlan.run`` only launches."""
        return ViewPlan(self, arr, n)

    def copy_batch(self, srcs: Sequence, dsts: Sequence, nbytes: Sequence[int] | None = None, *, stream: int = 0,
                   checksums: bool = True) -> list[str] | None:
        """n contiguous device copies in one launch (optionally with destination checksums)."""
        n = len(srcs)
        sizes = [_nbytes(t) for t in dsts] if nbytes is None else list(nbytes)
        out = (C.c_uint32 * max(1, n))()
        L.check(L.lib().mxp_copy_batch(self._h, _ptr_array([_addr(t) for t in srcs]),
                                       _ptr_array([_addr(t) for t in dsts]), (C.c_uint64 * max(1, n))(*sizes), n,
                                       out if checksums else None, C.c_void_p(stream)))
        return [format(out[i], "08x") for i in range(n)] if checksums else None

    def measure_gather(self, rows: int, row_bytes: int, src_pitch: int | None = None, col_offset: int = 0, repeats: int = 5,
                       cast: int = 0) -> float:
        """Bytes per second (read + written) that a bare kernel of the placement kernel's workgroup shape reaches
        on ``rows`` rows of ``row_bytes`` destination bytes gathered out of a ``src_pitch`` (default: contiguous):
        what the memory system of this box gives the shape, for comparison with the library's own kernels.
        ``cast``: 0, or ``CAST_CODES[("F32", "BF16")]`` for fp32 rows (twice as long in the source) stored as bf16."""
        out = C.c_double()
        src_row = row_bytes * 2 if cast else row_bytes
        L.check(L.lib().mxp_measure_gather(self._h, rows, row_bytes, src_row if src_pitch is None else src_pitch, col_offset,
                                           cast, repeats, C.byref(out)))
        return float(out.value)

    def measure_h2d(self, nbytes: int = 256 << 20, repeats: int = 5) -> float:
        out = C.c_double()
        L.check(L.lib().mxp_measure_h2d(self._h, nbytes, repeats, C.byref(out)))
        return float(out.value)


def set_transpose_form(form: int) -> None:
    """Measurement switch: 1 = every transposed view runs in the wavefront-autonomous form, 0 = the library picks."""
    L.check(L.lib().mxp_set_transpose_form(int(form)))


def measure_read(paths: Sequence[str], *, threads: int = 16, request_bytes: int = 16 << 20, direct: bool = True) -> dict:
    """Plain read rate of ``paths`` (no GPU work): what a cold ingest of the same files is compared with."""
    arr = (C.c_char_p * len(paths))(*[str(p).encode() for p in paths])
    total, rate = C.c_uint64(), C.c_double()
    L.check(L.lib().mxp_measure_read(arr, len(paths), threads, request_bytes, 1 if direct else 0, C.byref(total), C.byref(rate)))
    return {"bytes": int(total.value), "bytes_per_second": float(rate.value)}


class VerifyPlan:
    """Handle of ``mxp_verify_plan``: a fixed set of device buffers lowered once for repeated ``checksum32`` /
    ``tensor_digest`` passes; a run is one launch, a small reduction into pinned memory and an event wait."""

    def __init__(self, engine: "PlacementEngine", buffers: Sequence, nbytes: Sequence[int] | None = None):
        self._engine = engine
        self.n = len(buffers)
        sizes = [_nbytes(t) for t in buffers] if nbytes is None else list(nbytes)
        self._keep = list(buffers)  # the plan holds raw addresses: keep the tensors alive with it
        self._h = C.c_void_p()
        L.check(L.lib().mxp_verify_plan_create(engine._h, _ptr_array([_addr(t) for t in buffers]),
                                               (C.c_uint64 * max(1, self.n))(*sizes), self.n, C.byref(self._h)))
        self._sums = (C.c_uint32 * max(1, self.n))()
        self._dig = (C.c_uint8 * (16 * max(1, self.n)))()

    def checksums_raw(self, *, stream: int = 0):
        """One pass; the ``n`` checksums as the plan's own ``uint32`` ctypes array (rewritten by the next pass)."""
        L.check(L.lib().mxp_verify_plan_checksums(self._engine._h, self._h, self._sums, C.c_void_p(stream)))
        return self._sums

    def checksums(self, *, stream: int = 0) -> list[str]:
        sums = self.checksums_raw(stream=stream)
        return [format(sums[i], "08x") for i in range(self.n)]

    def digests_raw(self, *, stream: int = 0):
        """One pass; the ``n`` 16-byte digests as the plan's own ``uint8`` ctypes array (rewritten by the next pass)."""
        L.check(L.lib().mxp_verify_plan_digests(self._engine._h, self._h, self._dig, None, C.c_void_p(stream)))
        return self._dig

    def digests(self, *, stream: int = 0) -> list[str]:
        raw = bytes(self.digests_raw(stream=stream))
        return [raw[16 * i: 16 * i + 16].hex() for i in range(self.n)]

    def close(self) -> None:
        if self._h:
            L.lib().mxp_verify_plan_destroy(self._h)
            self._h = C.c_void_p()
            self._keep = []

    def __del__(self):
        try:
            self.close()
        except Exception:  # noqa: BLE001
            pass


class ViewPlan:
    """Handle of ``mxp_view_plan``: descriptor tables resident on the device for a fixed set of view copies
    at fixed addresses.  ``run`` allocates nothing, copies nothing from the host and does not synchronise."""

    def __init__(self, engine: PlacementEngine, arr, n: int):
        self._engine = engine
        self._h = C.c_void_p()
        L.check(L.lib().mxp_view_plan_create(engine._h, arr, n, C.byref(self._h)))
        out = C.c_uint64()
        L.check(L.lib().mxp_view_plan_bytes(self._h, C.byref(out)))
        self.bytes = int(out.value)

    def run(self, *, stream: int = 0) -> None:
        L.check(L.lib().mxp_view_plan_run(self._engine._h, self._h, C.c_void_p(stream)))

    def close(self) -> None:
        if self._h:
            L.lib().mxp_view_plan_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:  # noqa: BLE001
            pass


def digest_from_scalars(scalars: Sequence[int]) -> str:
    sc = (C.c_uint64 * 7)(*[int(v) & ((1 << 64) - 1) for v in scalars])
    out = (C.c_uint8 * 16)()
    L.check(L.lib().mxp_digest_from_scalars(sc, out))
    return bytes(out).hex()


def _current_stream(device: int) -> int:
    """The raw handle of the calling thread's current torch stream on ``device`` (0 = the default stream)."""
    try:
        import torch
    except ImportError:  # a caller that hands over raw device addresses needs no torch: the default stream
        return 0
    if not torch.cuda.is_available():
        return 0
    return int(torch.cuda.current_stream(device).cuda_stream)


def _addr(t) -> int:
    if isinstance(t, int):
        return t
    return int(t.data_ptr())


def _nbytes(t) -> int:
    return int(t.numel() * t.element_size())
