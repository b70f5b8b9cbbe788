"""One ``hipMalloc`` arena cut into ``world_size`` slices: the single-GPU symmetric heap.

Peer ranks are emulated as slices of the same HBM.  ``bases[r]`` is the address of rank
``r``'s slice, the quantity the reference obtains from one allocation per GPU plus peer
access or IPC (``/root/reference/tileccl/memory/symmetric_heap.py:239-343``,
``/root/reference/tileccl_v2/heap.py:225-264``).  "Remote" stores are ordinary global
stores into another slice, so no inter-GPU traffic exists.

The arena is allocated by the C library; torch sees a slice through the CUDA array
interface, which makes tensors *views* that never own the memory.
"""

from __future__ import annotations

import ctypes as C

import torch

from tileccl_amd import _lib

DEVICE = "cuda:0"  # every emulated rank lives on the one GPU


class _RawDeviceBytes:
    """Minimal ``__cuda_array_interface__`` exporter over [ptr, ptr+nbytes)."""

    def __init__(self, ptr: int, nbytes: int, owner: object) -> None:
        self._owner = owner  # keeps the arena alive while torch holds the view
        self.__cuda_array_interface__ = {
            "shape": (nbytes,),
            "typestr": "|u1",
            "data": (ptr, False),
            "version": 2,
            "strides": None,
        }


class Arena:
    """``world_size`` equally sized slices of one device allocation."""

    def __init__(self, slice_bytes: int, world_size: int) -> None:
        if slice_bytes <= 0:
            raise ValueError(f"Heap size must be positive, got {slice_bytes}")
        if world_size < 1:
            raise ValueError(f"world_size must be >= 1, got {world_size}")
        if world_size > _lib.MAX_WORLD:
            raise ValueError(f"world_size={world_size} exceeds the supported maximum {_lib.MAX_WORLD}")
        if not torch.cuda.is_available():
            raise RuntimeError("tileccl_amd needs a HIP device: torch.cuda.is_available() is False")
        lib = _lib.load()
        torch.cuda.init()
        handle = C.c_void_p()
        bases = (C.c_int64 * world_size)()
        with torch.cuda.device(0):
            _lib.check(lib.tccl_heap_create(slice_bytes, world_size, C.byref(handle), bases), "tccl_heap_create")
        self._handle = handle
        self.slice_bytes = int(slice_bytes)
        self.world_size = int(world_size)
        self.bases = [int(b) for b in bases]
        self._slices: list[torch.Tensor] | None = [
            torch.as_tensor(_RawDeviceBytes(b, self.slice_bytes, self), device=DEVICE) for b in self.bases
        ]
        self.heap_bases = torch.tensor(self.bases, dtype=torch.int64, device=DEVICE)
        self._users = 0

    def slice(self, rank: int) -> torch.Tensor:
        if self._slices is None:
            raise RuntimeError("SymmetricHeap has been cleaned up")
        return self._slices[rank]

    def acquire(self) -> "Arena":
        self._users += 1
        return self

    def release(self) -> None:
        """Drop one user; the last one frees the device memory."""
        self._users -= 1
        if self._users <= 0:
            self.destroy()

    def destroy(self) -> None:
        if self._handle is None:
            return
        torch.cuda.synchronize()
        self._slices = None
        self.heap_bases = None
        handle, self._handle = self._handle, None
        _lib.check(_lib.load().tccl_heap_destroy(handle), "tccl_heap_destroy")

    def __del__(self) -> None:  # pragma: no cover - interpreter shutdown order
        try:
            self.destroy()
        except Exception:
            pass
