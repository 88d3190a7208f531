"""helium_amd — MI355X (gfx950) execution backend for helium, reached through libhelium_hip.so's C ABI."""
from ._ffi import HeliumError, lib  # noqa: F401  (raises ImportError when the library is not built)
from . import device  # noqa: F401
from .device import DeviceBuffer, Event, Stream  # noqa: F401
from .permute import PermuteDims  # noqa: F401
from . import allocator, backend, configs, fusion, fusion_search, ir, kernels  # noqa: F401
from .kernels import TileKernel  # noqa: F401

__all__ = ["HeliumError", "device", "DeviceBuffer", "Event", "Stream", "PermuteDims", "TileKernel", "ir", "fusion", "kernels", "backend", "configs", "fusion_search"]
