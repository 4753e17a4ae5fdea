"""Registry of the environment variables this package reads.

Same pattern as the reference's ``modelexpress/envs.py:216-411``: one zero-argument
callable per variable, evaluated live on every attribute read, so tests can
``monkeypatch.setenv`` and callers see the new value without re-importing.
"""

from __future__ import annotations

import os
from typing import Any, Callable

_TRUTHY = ("1", "true", "yes", "on")


def _env_int(name: str, default: int) -> int:
    raw = os.environ.get(name, "").strip()
    if not raw:
        return default
    try:
        return int(raw, 0)
    except ValueError:
        return default


def _env_float(name: str, default: float) -> float:
    raw = os.environ.get(name, "").strip()
    if not raw:
        return default
    try:
        return float(raw)
    except ValueError:
        return default


def _env_bool(name: str, default: bool) -> bool:
    raw = os.environ.get(name)
    if raw is None or not raw.strip():
        return default
    return raw.strip().lower() in _TRUTHY


environment_variables: dict[str, Callable[[], Any]] = {
    # The checkpoint to place; same variable and precedence as the reference's streamer
    # strategy (load_strategy/model_streamer_strategy.py:27-35).
    "MX_MODEL_URI": lambda: os.environ.get("MX_MODEL_URI"),
    # Pinned ring geometry and I/O (0 = library default).
    "MXP_RING_SLOTS": lambda: _env_int("MXP_RING_SLOTS", 0),
    "MXP_SLOT_MIB": lambda: _env_int("MXP_SLOT_MIB", 0),
    "MXP_READER_THREADS": lambda: _env_int("MXP_READER_THREADS", 0),
    "MXP_STREAMS": lambda: _env_int("MXP_STREAMS", 0),
    "MXP_O_DIRECT": lambda: _env_bool("MXP_O_DIRECT", False),
    # "", "1" (readers pack strided rows) or "0" (stage row bands, gather on device).
    "MXP_PACK_STRIDED": lambda: os.environ.get("MXP_PACK_STRIDED", "").strip(),
    # bf16 image of NaN in the refit cast (0 = 0x7FC0).
    "MXP_NAN_BITS": lambda: _env_int("MXP_NAN_BITS", 0),
    # Fail the load when a checksum differs from the manifest the caller supplied.
    "MXP_VERIFY_CHECKSUMS": lambda: _env_bool("MXP_VERIFY_CHECKSUMS", True),
    # Read by the library itself (not through this registry), once per process: when set, every ingest prints one line
    # on stderr with the times of its phases (first chunk read, last chunk read, readers done, streams idle).
    "MXP_INGEST_TRACE": lambda: os.environ.get("MXP_INGEST_TRACE"),
    # Allow fp32 checkpoints to be cast into bf16 parameters (refit).
    "MXP_ALLOW_CAST": lambda: _env_bool("MXP_ALLOW_CAST", False),
    # Coverage gate of a refit, same names and defaults as the reference (modelexpress/envs.py:266-272):
    # refuse a refit that writes less than the floor fraction of the engine's parameter bytes.
    "MX_RESHARD_REQUIRE_FULL_COVERAGE": lambda: _env_bool("MX_RESHARD_REQUIRE_FULL_COVERAGE", False),
    "MX_RESHARD_COVERAGE_FLOOR": lambda: _env_float("MX_RESHARD_COVERAGE_FLOOR", 0.995),
    # Publishers stamp every served tensor with its digest (modelexpress/envs.py:304); off by default, read live.
    "MX_RESHARD_PUBLISH_DIGEST": lambda: _env_bool("MX_RESHARD_PUBLISH_DIGEST", False),
}


def __getattr__(name: str) -> Any:
    if name in environment_variables:
        return environment_variables[name]()
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")


def __dir__() -> list[str]:
    return sorted(environment_variables)


def is_set(name: str) -> bool:
    return name in os.environ
