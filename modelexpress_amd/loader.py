"""Whole-tensor loader with the interface of the reference's ``MxGdsLoader``
(modelexpress/gds_loader.py:52-160): ``load(model_path) -> {name: device tensor}`` and
``load_iter(model_path)`` yielding ``(name, device tensor)`` per shard file, the next file being
ingested while the current one is consumed (the reference's one-worker prefetch, :135-152).
Here a file travels through the pinned ring and the placement kernel instead of cuFile, and
tensors come out as ``raw.view(dtype).reshape(shape)`` of one device buffer each (:327-328).
"""

from __future__ import annotations

import logging
import time
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path
from typing import Iterator

import torch

logger = logging.getLogger("modelexpress_amd.loader")


class MxHipLoader:
    def __init__(self, accelerator_backend=None, *, device: int | None = None):
        self._accelerator_backend = accelerator_backend
        self._device_id = device
        self._engine = None

    # ------------------------------------------------------------------ public API
    def load(self, model_path: str) -> dict[str, torch.Tensor]:
        """Load all tensors from model_path to the GPU."""
        return dict(self.load_iter(model_path, use_tqdm=False))

    def load_iter(self, model_path: str, *, use_tqdm: bool = True, revision: str | None = None
                  ) -> Iterator[tuple[str, torch.Tensor]]:
        from .engine import Checkpoint

        load_start = time.perf_counter()
        model_path = self._resolve_model_path(model_path, revision=revision)
        if self._device_id is None:
            self._device_id = (self._accelerator_backend.current_device() if self._accelerator_backend is not None
                               else torch.cuda.current_device())
        self._ensure_engine()
        top = Checkpoint(model_path)
        try:
            files = [f["path"] for f in top.files()]
            wanted = {t.name for t in top.tensors()}
        finally:
            top.close()
        if not files:
            return
        pbar = None
        if use_tqdm:
            from tqdm import tqdm

            pbar = tqdm(total=len(files), desc="Loading safetensors through the HIP placement engine", unit="file")
        pool = ThreadPoolExecutor(max_workers=1)  # the engine handle is used by this one worker only
        try:
            pending = pool.submit(self._load_file_tensors, files[0], wanted)
            for i in range(len(files)):
                loaded = pending.result()
                if pbar is not None:
                    pbar.update(1)
                if i + 1 < len(files):
                    pending = pool.submit(self._load_file_tensors, files[i + 1], wanted)
                yield from loaded.items()
            logger.info("HIP load complete in %.2fs", time.perf_counter() - load_start)
        finally:
            if pbar is not None:
                pbar.close()
            pool.shutdown(wait=True)

    def shutdown(self) -> None:
        if self._engine is not None:
            self._engine.close()
            self._engine = None

    # ------------------------------------------------------------------ helpers
    @staticmethod
    def _resolve_model_path(model_path: str, revision: str | None = None) -> str:
        """A local directory or file; hub identifiers are not resolved here (no network path in this engine)."""
        p = Path(model_path)
        if p.exists():
            return str(p.resolve())
        raise FileNotFoundError(f"model path '{model_path}' does not exist locally"
                                + (f" (revision {revision})" if revision else ""))

    def _ensure_engine(self) -> None:
        if self._engine is None:
            from .load_strategy import _engine_from_env

            self._engine = _engine_from_env(self._device_id)

    def _load_file_tensors(self, file_path: str, wanted: set) -> dict[str, torch.Tensor]:
        from .engine import Checkpoint, ParamSpec, PlacementPlan
        from .load_strategy import _TORCH_DTYPE

        torch.cuda.set_device(self._device_id)
        ck = Checkpoint(file_path)
        try:
            entries = [t for t in ck.tensors() if t.name in wanted]  # file order = offset order (gds_loader.py:297-300)
            plan = PlacementPlan(ck, [ParamSpec(t.name, t.dtype, t.shape) for t in entries], allow_unmapped=True)
            try:
                dst = self._engine.allocate(plan)
                self._engine.execute(plan, dst)
            finally:
                plan.close()
            return {t.name: buf.view(_TORCH_DTYPE[t.dtype]).reshape(t.shape) for t, buf in zip(entries, dst)}
        finally:
            ck.close()
