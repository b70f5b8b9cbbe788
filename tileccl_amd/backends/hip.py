"""The slice of the reference HAL this path uses: device properties and synchronisation.

Reference: ``/root/reference/tileccl/backends/base.py:72-234`` (interface) and
``backends/hip.py:458-490`` (``get_device_properties``).  The reference reads
``props.total_mem`` there, an attribute torch does not have, so on ROCm it falls into its
``except`` branch and reports ``compute_units=0``; this build queries the HIP runtime
through the C library instead and never reports zero CUs.
"""

from __future__ import annotations

import ctypes as C
from dataclasses import dataclass

import torch

from tileccl_amd import _lib


@dataclass(frozen=True)
class DeviceProperties:
    name: str
    compute_units: int
    clock_mhz: int
    wavefront_size: int
    lds_bytes: int
    xcds: int
    total_memory: int
    backend: str = "hip"


class HIPBackend:
    """Device queries and synchronisation for the single visible GPU."""

    name = "hip"

    def __init__(self) -> None:
        if not torch.cuda.is_available():
            raise RuntimeError("HIP backend unavailable: torch.cuda.is_available() is False")
        self._props: DeviceProperties | None = None

    def get_device_properties(self, device: int = 0) -> DeviceProperties:
        if self._props is None:
            info = _lib.DeviceInfo()
            _lib.check(_lib.load().tccl_device_query(device, C.byref(info)), "tccl_device_query")
            self._props = DeviceProperties(
                name=info.arch.decode(),
                compute_units=int(info.compute_units),
                clock_mhz=int(info.clock_khz) // 1000,
                wavefront_size=int(info.wavefront),
                lds_bytes=int(info.lds_bytes),
                xcds=int(info.xcds),
                total_memory=int(torch.cuda.get_device_properties(device).total_memory),
            )
        return self._props

    def synchronize(self) -> None:
        torch.cuda.synchronize()

    def get_device_count(self) -> int:
        return torch.cuda.device_count()


_backend: HIPBackend | None = None


def get_backend(name: str = "hip", force: bool = False) -> HIPBackend:
    """Cached backend instance (reference ``backends/__init__.py:75``); only ``"hip"`` exists."""
    global _backend
    if name != "hip":
        raise RuntimeError(f"Backend {name!r} is not available in this build (HIP only).")
    if _backend is None or force:
        _backend = HIPBackend()
    return _backend
