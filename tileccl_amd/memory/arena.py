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
    """``world_size`` equally sized slices of one device allocation.

    Lifetime: every tensor handed out is a view of a slice tensor, and a slice tensor keeps
    the exporter it was built from -- and through it this object -- alive for as long as its
    storage exists.  ``release()`` by the last heap therefore only forgets the slice tensors;
    the device memory is freed when this object is collected, i.e. once no tensor views it
    any more.  (The reference's ``cleanup`` likewise only drops its reference to a
    torch-owned buffer, so tensors allocated earlier stay valid:
    ``/root/reference/tileccl/memory/symmetric_heap.py:1266-1316``.)
    """

    def __init__(self, slice_bytes: int, world_size: int) -> None:
        self._handle = None
        if slice_bytes <= 0:
            raise ValueError(f"Heap size must be positive, got {slice_bytes}")
        if world_size < 1:
            raise ValueError(f"world_size must be >= 1, got {world_size}")
        if world_size > _lib.MAX_WORLD:
            raise ValueError(f"world_size={world_size} exceeds the supported maximum {_lib.MAX_WORLD}")
        self.slice_bytes = int(slice_bytes)
        self.world_size = int(world_size)
        self._handle, self.bases = self._allocate(self.slice_bytes, self.world_size)
        self._slices: list[torch.Tensor] | None = [self._view(b, self.slice_bytes) for b in self.bases]
        self.heap_bases = self._device_bases(self.bases)
        self._users = 0

    # -- the three places that touch the device (replaced by a fake in the CPU tests) -----
    def _allocate(self, slice_bytes: int, world_size: int) -> tuple[object, list[int]]:
        if not torch.cuda.is_available():
            raise RuntimeError("tileccl_amd needs a HIP device: torch.cuda.is_available() is False")
        lib = _lib.load()
        torch.cuda.init()
        handle = C.c_void_p()
        bases = (C.c_int64 * world_size)()
        with torch.cuda.device(0):
            _lib.check(lib.tccl_heap_create(slice_bytes, world_size, C.byref(handle), bases), "tccl_heap_create")
        return handle, [int(b) for b in bases]

    def _view(self, base: int, nbytes: int) -> torch.Tensor:
        return torch.as_tensor(_RawDeviceBytes(base, nbytes, self), device=DEVICE)

    def _device_bases(self, bases: list[int]) -> torch.Tensor:
        return torch.tensor(bases, dtype=torch.int64, device=DEVICE)

    def _deallocate(self, handle: object) -> None:
        torch.cuda.synchronize()
        _lib.check(_lib.load().tccl_heap_destroy(handle), "tccl_heap_destroy")

    # -- users ------------------------------------------------------------------------------
    @property
    def live(self) -> bool:
        """The device allocation still exists."""
        return self._handle is not None

    def slice(self, rank: int) -> torch.Tensor:
        if self._slices is None:
            raise RuntimeError("SymmetricHeap has been cleaned up")
        return self._slices[rank]

    def acquire(self) -> "Arena":
        self._users += 1
        return self

    def release(self) -> None:
        """Drop one user.  After the last one the arena hands out nothing more; the device
        memory stays until the last tensor viewing it is gone (see the class docstring)."""
        self._users -= 1
        if self._users <= 0:
            self._slices = None
            self.heap_bases = None

    def __del__(self) -> None:
        handle, self._handle = getattr(self, "_handle", None), None
        if handle is None:
            return
        try:
            self._deallocate(handle)
        except Exception:  # interpreter shutdown: the driver reclaims the memory with the process
            pass
