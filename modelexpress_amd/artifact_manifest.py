"""File and chunk CRC32C checksums of an artifact directory, the checksum half of the
reference's artifact manifest (modelexpress_common/src/artifact_manifest.rs:56-117,260-324;
Python twin modelexpress/metadata/artifact_manifest.py): regular files sorted by manifest
path, a whole-file checksum per file, fixed-size chunks numbered across files."""

from __future__ import annotations

import ctypes as C
import os
from dataclasses import dataclass
from pathlib import Path

from . import _lib as L


@dataclass(frozen=True)
class ManifestFile:
    path: str
    file_index: int
    size: int
    checksum: str


@dataclass(frozen=True)
class ManifestChunk:
    chunk_index: int
    file_index: int
    file_offset: int
    length: int
    checksum: str


def crc32c(data: bytes, seed: int = 0) -> str:
    buf = (C.c_char * max(1, len(data))).from_buffer_copy(data or b"\0")
    return format(L.lib().mxp_crc32c(seed, buf, len(data)), "08x")


def build_checksums(root: str, chunk_size: int) -> tuple:
    """``(files, chunks)`` for every regular file under ``root``."""
    if chunk_size <= 0:
        raise ValueError("chunk_size must be positive")
    base = Path(root).resolve()
    paths = sorted((p.resolve().as_posix() for p in base.rglob("*") if p.is_file() and not p.is_symlink()))
    files, chunks = [], []
    for index, path in enumerate(paths):
        size = os.path.getsize(path)
        n_max = max(1, -(-size // chunk_size))
        crcs = (C.c_uint32 * n_max)()
        whole, n = C.c_uint32(), C.c_uint64()
        L.check(L.lib().mxp_file_crc32c(path.encode(), chunk_size, C.byref(whole), crcs, n_max, C.byref(n)))
        files.append(ManifestFile(path, index, size, format(whole.value, "08x")))
        for k in range(n.value):
            off = k * chunk_size
            chunks.append(ManifestChunk(len(chunks), index, off, min(chunk_size, size - off), format(crcs[k], "08x")))
    return files, chunks
