"""Records the host-side C-ABI calls a test session makes (checkpoint parse, planner, CRC32C) as a text
trace that tests/c/abi_replay.cpp replays against a build of the same sources under AddressSanitizer and
UndefinedBehaviorSanitizer.  Installed by conftest.py when MXP_ABI_TRACE names the trace file.

One call per line: the function (without its ``mxp_`` prefix), what it returned, then its arguments.
Strings travel hex-encoded (``-`` = NULL), handles as small ids handed out at open / create, integer arrays
as comma lists.  A small file or directory given to ``mxp_ckpt_open`` is copied beside the trace first: tests
rewrite one path many times, and the replay must see what the call saw."""

from __future__ import annotations

import ctypes as C
import os
import shutil


def _hex(b) -> str:
    if b is None:
        return "-"
    if isinstance(b, str):
        b = b.encode()
    return "x" + bytes(b).hex()


def _ints(arr, n) -> str:
    return ",".join(str(int(arr[i])) for i in range(n)) if n > 0 else "-"


class TracingLib:
    """Stands in for the ctypes library handle: forwards everything, writes a line for the traced calls."""

    def __init__(self, real, trace_path: str):
        self._real = real
        self._out = open(trace_path, "a", buffering=1)
        self._blobs = trace_path + ".blobs"
        os.makedirs(self._blobs, exist_ok=True)
        self._ids: dict[int, int] = {}  # live handle address -> id
        self._next = 1
        self._n_blobs = 0

    # -- handle bookkeeping --
    def _new(self, holder) -> str:
        addr = holder.value
        if not addr:
            return "-"
        self._ids[addr] = self._next
        self._next += 1
        return str(self._ids[addr])

    def _id(self, h) -> str:
        addr = h.value if isinstance(h, C.c_void_p) else h
        return str(self._ids.get(addr, "-")) if addr else "-"

    def _drop(self, h) -> str:
        addr = h.value if isinstance(h, C.c_void_p) else h
        return str(self._ids.pop(addr, "-")) if addr else "-"

    def _snapshot(self, path: bytes) -> bytes:
        p = path.decode("utf-8", "surrogateescape")
        if os.path.isfile(p) and os.path.getsize(p) <= (1 << 20):
            self._n_blobs += 1
            copy = os.path.join(self._blobs, f"{self._n_blobs}.safetensors")
            shutil.copyfile(p, copy)
            return copy.encode()
        if os.path.isdir(p):  # a small directory is copied too: a test may rewrite its files before the next open
            entries = [e for e in os.scandir(p)]
            if len(entries) <= 64 and all(e.is_file() for e in entries) and sum(e.stat().st_size for e in entries) <= (4 << 20):
                self._n_blobs += 1
                copy = os.path.join(self._blobs, str(self._n_blobs))
                shutil.copytree(p, copy)
                return copy.encode()
        return path

    def _w(self, *tokens) -> None:
        self._out.write(" ".join(str(t) for t in tokens) + "\n")

    # -- traced entry points --
    def mxp_ckpt_open(self, path, out):
        seen = self._snapshot(path)
        rc = self._real.mxp_ckpt_open(path, out)
        self._w("ckpt_open", rc, self._new(out._obj) if rc == 0 else "-", _hex(seen))
        return rc

    def mxp_ckpt_close(self, h):
        self._w("ckpt_close", 0, self._drop(h))
        return self._real.mxp_ckpt_close(h)

    def mxp_plan_create(self, ck, tp, rank, flags, out):
        rc = self._real.mxp_plan_create(ck, tp, rank, flags, out)
        self._w("plan_create", rc, self._new(out._obj) if rc == 0 else "-", self._id(ck), int(tp), int(rank), int(flags))
        return rc

    def mxp_plan_destroy(self, h):
        self._w("plan_destroy", 0, self._drop(h))
        return self._real.mxp_plan_destroy(h)

    def mxp_plan_add_param(self, pl, name, dtype, ndim, shape):
        rc = self._real.mxp_plan_add_param(pl, name, dtype, ndim, shape)
        self._w("plan_add_param", rc, self._id(pl), _hex(name), int(dtype), int(ndim), _ints(shape, min(int(ndim), len(shape))))
        return rc

    def mxp_plan_add_stacked(self, pl, fused, member):
        rc = self._real.mxp_plan_add_stacked(pl, fused, member)
        self._w("plan_add_stacked", rc, self._id(pl), _hex(fused), _hex(member))
        return rc

    def mxp_plan_add_expert(self, pl, p_pre, w_pre, eid, shard, local):
        rc = self._real.mxp_plan_add_expert(pl, p_pre, w_pre, eid, shard, local)
        self._w("plan_add_expert", rc, self._id(pl), _hex(p_pre), _hex(w_pre), int(eid), _hex(shard), int(local))
        return rc

    def mxp_plan_add_skip_prefix(self, pl, prefix):
        rc = self._real.mxp_plan_add_skip_prefix(pl, prefix)
        self._w("plan_add_skip_prefix", rc, self._id(pl), _hex(prefix))
        return rc

    def mxp_plan_add_virtual(self, pl, name, ndim, shape):
        rc = self._real.mxp_plan_add_virtual(pl, name, ndim, shape)
        self._w("plan_add_virtual", rc, self._id(pl), _hex(name), int(ndim), _ints(shape, min(int(ndim), len(shape))))
        return rc

    def mxp_plan_add_virtual_shard(self, pl, vi, source, src_off, shard_off, shape):
        rc = self._real.mxp_plan_add_virtual_shard(pl, vi, source, src_off, shard_off, shape)
        n = len(shape)
        self._w("plan_add_virtual_shard", rc, self._id(pl), int(vi), _hex(source), n, _ints(src_off, n), _ints(shard_off, n), _ints(shape, n))
        return rc

    def mxp_plan_build(self, pl):
        rc = self._real.mxp_plan_build(pl)
        self._w("plan_build", rc, self._id(pl))
        return rc

    def mxp_crc32c(self, seed, data, n):
        rc = self._real.mxp_crc32c(seed, data, n)
        if int(n) <= (1 << 16):
            self._w("crc32c", rc, int(seed), _hex(bytes(data[: int(n)])) if int(n) else "-")
        return rc

    def mxp_file_crc32c(self, path, chunk, whole, crcs, max_chunks, n_out):
        rc = self._real.mxp_file_crc32c(path, chunk, whole, crcs, max_chunks, n_out)
        self._w("file_crc32c", rc, _hex(path), int(chunk), int(max_chunks), whole._obj.value if rc == 0 else 0,
                n_out._obj.value if rc == 0 else 0)
        return rc

    def __getattr__(self, name):
        return getattr(self._real, name)


def install(trace_path: str) -> None:
    """Loads the product library and puts the tracer in front of it for this process."""
    from modelexpress_amd import _lib

    real = _lib.lib()
    if not isinstance(real, TracingLib):
        _lib._lib = TracingLib(real, trace_path)
