"""Accelerator backend for ROCm devices.

Mirrors the reference's ``AcceleratorBackend`` protocol (modelexpress/accelerators/base.py:16-72)
and the place new vendors plug in (accelerators/__init__.py:41-61).  On ROCm builds of
PyTorch the device type is still ``"cuda"``, so torch calls are the same as the CUDA
backend's (accelerators/cuda.py:15-62); what differs is the capability policy: no
GPUDirect Storage, no CUDA VMM arena, no NIXL pool registration, no RDMA P2P.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Protocol, runtime_checkable

import torch

NIXL_ACCELERATOR_MEM_TYPE = "VRAM"


@runtime_checkable
class AcceleratorBackend(Protocol):
    @property
    def name(self) -> str: ...
    @property
    def torch_device_type(self) -> str: ...
    @property
    def nixl_mem_type(self) -> str: ...
    def set_device(self, device_id: int) -> None: ...
    def current_device(self) -> int: ...
    def synchronize(self, device_id: int | None = None) -> None: ...
    def empty_cache(self) -> None: ...
    def torch_device(self, device_id: int) -> torch.device: ...
    def is_accel_tensor(self, tensor: torch.Tensor) -> bool: ...
    def supports_rdma_p2p(self) -> bool: ...
    def supports_pool_reg(self) -> bool: ...
    def supports_vmm(self) -> bool: ...
    def supports_gds(self) -> bool: ...


@dataclass(frozen=True)
class HipAcceleratorBackend:
    """ROCm / HIP implementation of the accelerator backend boundary."""

    @property
    def name(self) -> str:
        return "rocm"

    @property
    def torch_device_type(self) -> str:
        return "cuda"

    @property
    def nixl_mem_type(self) -> str:
        return NIXL_ACCELERATOR_MEM_TYPE

    def set_device(self, device_id: int) -> None:
        torch.cuda.set_device(device_id)

    def current_device(self) -> int:
        return int(torch.cuda.current_device())

    def synchronize(self, device_id: int | None = None) -> None:
        if device_id is None:
            torch.cuda.synchronize()
        else:
            torch.cuda.synchronize(device_id)

    def empty_cache(self) -> None:
        torch.cuda.empty_cache()

    def torch_device(self, device_id: int) -> torch.device:
        return torch.device(self.torch_device_type, device_id)

    def is_accel_tensor(self, tensor: torch.Tensor) -> bool:
        return bool(tensor.is_cuda)

    def supports_rdma_p2p(self) -> bool:
        return False

    def supports_pool_reg(self) -> bool:
        return False

    def supports_vmm(self) -> bool:
        return False

    def supports_gds(self) -> bool:
        return False

    def supports_hip_placement(self) -> bool:
        """Whether the HIP placement library is built and a device is visible."""
        from . import _lib

        try:
            _lib.lib()
        except ImportError:
            return False
        return torch.cuda.is_available()


def accelerator_backend_for(device: torch.device | str) -> AcceleratorBackend:
    """The backend for ``device`` (accelerators/__init__.py:41-61); only ROCm devices,
    which torch names ``cuda``, are served here."""
    torch_device = torch.device(device)
    if torch_device.type == "cuda":
        return HipAcceleratorBackend()
    raise ValueError(
        f"Unsupported accelerator backend for torch device {torch_device!s}; supported device types: cuda (ROCm)"
    )
