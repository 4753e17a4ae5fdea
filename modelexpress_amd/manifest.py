"""Tensor manifests for compatibility validation between a source and a target.

Structural checks follow the reference's receive path (modelexpress/nixl_transfer.py:835-897):
a tensor present on both sides must have the same byte size and dtype string, and a
difference in the name sets is an error when an exact match is required and a warning
otherwise.  Content checks add what the reference logs or stamps per tensor: the
position-weighted checksum (tensor_utils.py:27-44, ``[CHECKSUM]`` lines of
``log_tensor_summary``, :363-382) and the blake2b digest (refit/reshard/verify.py:79-155).
"""

from __future__ import annotations

import json
import logging
from dataclasses import asdict, dataclass
from typing import Iterable, Sequence

logger = logging.getLogger("modelexpress_amd.manifest")


class ManifestMismatchError(RuntimeError):
    """Source and target tensors are not compatible (name, size, dtype or content)."""


@dataclass(frozen=True)
class TensorRecord:
    name: str
    nbytes: int
    dtype: str                 # safetensors dtype name
    checksum: str | None = None  # 8 hex chars
    digest: str | None = None    # 32 hex chars


def build_manifest(engine, params: Sequence, buffers: Sequence, *, checksums: Sequence[str] | None = None,
                   with_digest: bool = True) -> list[TensorRecord]:
    """Records for finished parameter buffers.  ``params`` carry ``name``, ``dtype``, ``nbytes``;
    checksums default to one batched device pass over the buffers, digests likewise."""
    sizes = [p.nbytes for p in params]
    sums = list(checksums) if checksums is not None else engine.checksum32(list(buffers), sizes)
    digs = engine.digest(list(buffers), sizes) if with_digest else [None] * len(sizes)
    return [TensorRecord(p.name, p.nbytes, p.dtype, s, d) for p, s, d in zip(params, sums, digs)]


def compare_manifests(source: Iterable[TensorRecord], local: Iterable[TensorRecord], *, require_exact_match: bool = False,
                      check_content: bool = True) -> int:
    """Raises ``ManifestMismatchError`` as the reference's matcher does; returns the number of
    matched tensors.  Content is compared only where both sides carry the field."""
    local_by = {t.name: t for t in local}
    source = list(source)
    matched = 0
    for s in source:
        t = local_by.get(s.name)
        if t is None:
            continue
        if t.nbytes != s.nbytes:
            raise ManifestMismatchError(f"Tensor '{s.name}' size mismatch: source={s.nbytes} bytes, local={t.nbytes} bytes")
        if t.dtype != s.dtype:
            raise ManifestMismatchError(f"Tensor '{s.name}' dtype mismatch: source={s.dtype!r}, local={t.dtype!r}")
        if check_content:
            for field in ("checksum", "digest"):
                a, b = getattr(s, field), getattr(t, field)
                if a is not None and b is not None and a != b:
                    raise ManifestMismatchError(f"Tensor '{s.name}' {field} mismatch: source={a}, local={b}")
        matched += 1
    src_names = {s.name for s in source}
    local_only = sorted(set(local_by) - src_names)
    source_only = sorted(src_names - set(local_by))
    if local_only or source_only:
        if require_exact_match:
            raise ManifestMismatchError(
                f"Tensor name mismatch: {len(local_only)} local-only (first: {local_only[:5]}), "
                f"{len(source_only)} source-only (first: {source_only[:5]})")
        logger.warning("Tensor name mismatch between source manifest and local registration: %d local-only, %d source-only",
                       len(local_only), len(source_only))
    if not matched and require_exact_match:
        raise ManifestMismatchError("No matching tensors found")
    return matched


def dumps(records: Iterable[TensorRecord]) -> str:
    return json.dumps([asdict(r) for r in records], separators=(",", ":"))


def loads(text: str) -> list[TensorRecord]:
    return [TensorRecord(**d) for d in json.loads(text)]
