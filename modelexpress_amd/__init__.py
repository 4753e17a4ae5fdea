"""MI355X-native weight placement for the ModelExpress loading chain.

The compute lives in libmxplace.so (hand-written gfx950 kernels plus a C++ host engine,
C ABI in include/mxp.h).  This package is the host-side mirror of the reference's
loader interface: strategy chain, engine adapter, accelerator backend.
"""

from .adapter import EngineAdapter, PlacementLayout, StrategyFailed, UnsupportedCapability, gated_capability
from .accelerators import HipAcceleratorBackend, accelerator_backend_for

__all__ = [
    "EngineAdapter", "PlacementLayout", "StrategyFailed", "UnsupportedCapability", "gated_capability",
    "HipAcceleratorBackend", "accelerator_backend_for",
]
__version__ = "0.1.0"
