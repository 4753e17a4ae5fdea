"""Seeded synthetic safetensors checkpoints, on disk or staged straight into HBM.

Every tensor's bytes are a pure function of ``(base_seed, tensor name, element index)``
computed by the library's generator, which runs the same integer arithmetic on the host
and on the device: a checkpoint written to files and one generated directly into device
memory hold identical bytes, so full-size runs need no 16 GB host copy.
"""

from __future__ import annotations

import ctypes as C
import json
import mmap
import struct
import zlib
from pathlib import Path

from . import _lib as L
from .models import FP8_FINITE, SCALE, TensorSpec


def tensor_seed(base_seed: int, name: str) -> int:
    return ((base_seed * 0x9E3779B97F4A7C15) ^ (zlib.crc32(name.encode()) * 0x100000001B3)) & ((1 << 64) - 1)


def _kind(t: TensorSpec) -> int:
    if t.dtype in ("F8_E4M3", "F8_E5M2"):
        return FP8_FINITE
    if t.name.endswith("scale_inv") or t.name.endswith("_scale"):
        return SCALE
    return t.kind


def split_shards(tensors: list, n_shards: int) -> list:
    """Contiguous split of the tensor list into ``n_shards`` groups of similar byte size."""
    n_shards = max(1, min(n_shards, len(tensors)))
    total = sum(t.nbytes for t in tensors)
    target = total / n_shards
    shards, cur, acc = [], [], 0
    for i, t in enumerate(tensors):
        cur.append(t)
        acc += t.nbytes
        remaining_shards = n_shards - len(shards) - 1
        remaining_tensors = len(tensors) - i - 1
        if remaining_shards > 0 and (acc >= target * (len(shards) + 1) or remaining_tensors == remaining_shards):
            shards.append(cur)
            cur = []
    if cur:
        shards.append(cur)
    return shards


def shard_header(tensors: list, align: int = 64) -> tuple:
    """safetensors header bytes (8-byte length + JSON padded with spaces so the data
    section starts on an ``align`` boundary) and each tensor's offset in the data section."""
    entries, offsets, pos = {}, [], 0
    for t in tensors:
        entries[t.name] = {"dtype": t.dtype, "shape": list(t.shape), "data_offsets": [pos, pos + t.nbytes]}
        offsets.append(pos)
        pos += t.nbytes
    entries["__metadata__"] = {"format": "pt"}
    body = json.dumps(entries, separators=(",", ":")).encode()
    pad = (-(8 + len(body))) % align
    body += b" " * pad
    return struct.pack("<Q", len(body)) + body, offsets, pos


def write_checkpoint(tensors: list, out_dir: str, *, n_shards: int = 1, seed: int = 0, threads: int = 8,
                     with_index: bool | None = None) -> dict:
    """Write ``tensors`` (TensorSpec list) as safetensors shards into ``out_dir``.

    Returns ``{"files": [...], "total_bytes": n}``.  One shard is named
    ``model.safetensors``; several get ``model-0000i-of-0000n.safetensors`` plus
    ``model.safetensors.index.json`` unless ``with_index`` is False.
    """
    lib = L.lib()
    out = Path(out_dir)
    out.mkdir(parents=True, exist_ok=True)
    shards = split_shards(tensors, n_shards)
    if with_index is None:
        with_index = len(shards) > 1
    weight_map, files, total = {}, [], 0
    for si, shard in enumerate(shards):
        fname = "model.safetensors" if len(shards) == 1 else f"model-{si + 1:05d}-of-{len(shards):05d}.safetensors"
        header, offsets, data_bytes = shard_header(shard)
        path = out / fname
        size = len(header) + data_bytes
        with open(path, "wb+") as f:
            f.truncate(size)
            f.write(header)
            f.flush()
            if data_bytes:
                with mmap.mmap(f.fileno(), size) as mm:
                    base = C.addressof(C.c_char.from_buffer(mm))
                    for t, off in zip(shard, offsets):
                        n_elems = t.nbytes // L.DTYPE_SIZE[t.dtype]
                        L.check(lib.mxp_synth_host(C.c_void_p(base + len(header) + off), n_elems,
                                                   L.DTYPE_CODE[t.dtype], _kind(t), tensor_seed(seed, t.name), threads))
                    del base
        for t in shard:
            weight_map[t.name] = fname
        files.append(str(path))
        total += size
    if with_index:
        with open(out / "model.safetensors.index.json", "w") as f:
            json.dump({"metadata": {"total_size": sum(t.nbytes for t in tensors)}, "weight_map": weight_map}, f)
    return {"files": files, "total_bytes": total}


def write_headers_only(tensors: list, out_dir: str, *, n_shards: int = 1) -> dict:
    """Sparse shard files with real headers and unwritten (zero) data: enough for the
    checkpoint parser and planner when the contents are generated on the device."""
    out = Path(out_dir)
    out.mkdir(parents=True, exist_ok=True)
    shards = split_shards(tensors, n_shards)
    weight_map, files = {}, []
    for si, shard in enumerate(shards):
        fname = "model.safetensors" if len(shards) == 1 else f"model-{si + 1:05d}-of-{len(shards):05d}.safetensors"
        header, _offsets, data_bytes = shard_header(shard)
        with open(out / fname, "wb") as f:
            f.write(header)
            f.truncate(len(header) + data_bytes)
        for t in shard:
            weight_map[t.name] = fname
        files.append(str(out / fname))
    if len(shards) > 1:
        with open(out / "model.safetensors.index.json", "w") as f:
            json.dump({"metadata": {}, "weight_map": weight_map}, f)
    return {"files": files}


def stage_on_device(ckpt, tensors: list, *, seed: int = 0, device: int = 0, stream: int = 0) -> list:
    """One uint8 device tensor per shard file of ``ckpt`` holding that file's bytes, the
    tensor data generated on the device with the same seeds ``write_checkpoint`` uses.
    (Header bytes are left zero: placement never reads them.)"""
    import torch

    lib = L.lib()
    by_name = {t.name: t for t in tensors}
    files = ckpt.files()
    dev = torch.device("cuda", device)
    # Each file sits `staging_pad` bytes into its allocation, so that its data section (and with it
    # every tensor whose offset in the data section is a multiple of 256) starts on a 256-byte boundary.
    staged = []
    for f in files:
        pad = int(f["staging_pad"])
        staged.append(torch.zeros(int(f["file_size"]) + pad, dtype=torch.uint8, device=dev)[pad:])
    with torch.cuda.device(dev):
        for e in ckpt.tensors():
            spec = by_name[e.name]
            if e.file_offset % L.DTYPE_SIZE[e.dtype]:
                raise ValueError(f"tensor {e.name} is not element-aligned in its file")
            n_elems = e.nbytes // L.DTYPE_SIZE[e.dtype]
            L.check(lib.mxp_synth_device(C.c_void_p(staged[e.file_index].data_ptr() + e.file_offset), n_elems,
                                         L.DTYPE_CODE[e.dtype], _kind(spec), tensor_seed(seed, e.name),
                                         C.c_void_p(stream)))
        torch.cuda.synchronize(dev)
    return staged
