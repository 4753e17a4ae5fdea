"""Normalized stage timing for refit cycles.

Keeps the reference's stage vocabulary and record prefix (modelexpress/refit/timing.py:23-35:
ten fixed stages, one JSON record prefixed ``MX_REFIT_TIMING``) so harnesses that parse the
reference's records can read these too.  On this path ``wire_transfer`` is the ingest
(file -> pinned ring -> HBM, with the slice / cast / checksum kernels running inside it),
``receive_sync`` the digest verification, ``installation`` the batched device copy into
the live parameters.
"""

from __future__ import annotations

import contextlib
import json
import logging
import time
from typing import Any, Iterator

logger = logging.getLogger("modelexpress_amd.timing")

MX_REFIT_TIMING_PREFIX = "MX_REFIT_TIMING"
REFIT_TIMING_STAGES = (
    "control_discovery", "source_preparation", "setup_registration", "transfer_planning", "wire_transfer",
    "receive_sync", "transformation", "installation", "post_install", "rollout_readiness",
)


class RefitTimingRecorder:
    """Collects repeated spans per stage and emits one JSON record."""

    def __init__(self, *, backend: str, version, tp_rank: int | None = None, tp_size: int | None = None,
                 cold: bool | None = None, clock=time.perf_counter):
        self.backend, self.version, self.tp_rank, self.tp_size, self.cold = backend, version, tp_rank, tp_size, cold
        self.bytes = 0
        self.extra: dict[str, Any] = {}  # further facts of the cycle, emitted with the record
        self._clock = clock
        self._started = clock()
        self._stages = {s: {"duration_s": 0.0, "count": 0, "statuses": []} for s in REFIT_TIMING_STAGES}

    @contextlib.contextmanager
    def span(self, stage: str, status: str = "ok") -> Iterator[None]:
        if stage not in self._stages:
            raise ValueError(f"unknown refit timing stage {stage!r}")
        t0 = self._clock()
        try:
            yield
        except BaseException:
            self.add_duration(stage, self._clock() - t0, status="error")
            raise
        else:
            self.add_duration(stage, self._clock() - t0, status=status)

    def add_duration(self, stage: str, duration_s: float, status: str = "ok") -> None:
        if stage not in self._stages:
            raise ValueError(f"unknown refit timing stage {stage!r}")
        if duration_s < 0:
            raise ValueError("duration_s must be non-negative")
        item = self._stages[stage]
        item["duration_s"] += float(duration_s)
        item["count"] += 1
        if status not in item["statuses"]:
            item["statuses"].append(status)

    def as_dict(self) -> dict[str, Any]:
        total = self._clock() - self._started
        return {
            "backend": self.backend, "version": self.version, "tp_rank": self.tp_rank, "tp_size": self.tp_size,
            "cold_warm": None if self.cold is None else ("cold" if self.cold else "warm"), "bytes": self.bytes,
            "total_s": round(total, 6), **self.extra,
            "stages": {s: {"duration_s": round(v["duration_s"], 6), "count": v["count"], "statuses": v["statuses"]}
                       for s, v in self._stages.items() if v["count"]},
        }

    def emit(self) -> str:
        line = f"{MX_REFIT_TIMING_PREFIX} {json.dumps(self.as_dict(), sort_keys=True)}"
        logger.warning(line)  # WARNING so harnesses capture it without raising the log level
        return line
