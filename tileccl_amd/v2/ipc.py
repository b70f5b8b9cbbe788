"""Host-callable probes of the device-side signal primitives.

In the reference these are ``@triton.jit`` device functions
(``/root/reference/tileccl_v2/ipc.py:137-254``, ``tileccl/sync/primitives.py:357-500``); here
the device functions live in ``csrc/tccl_device.h`` and are inlined into the kernels.  Each
function below launches the primitive on one lane over one word, which is how their
semantics are tested: ``tile_signal`` sets 1 with release, ``tile_try_wait`` consumes
(1 -> 0) within a bounded number of probes, ``tile_try_poll`` observes without consuming,
``tile_signal_add`` returns the previous value, ``tile_wait_ge`` spins until the word
reaches a threshold or the (host-chosen) time limit expires.

``translate_ptr`` is the host twin of the device pointer translation
(``tileccl_v2/ipc.py:24-63``).
"""

from __future__ import annotations

import torch

from tileccl_amd import _launch, _lib


def _words(t: torch.Tensor) -> torch.Tensor:
    if t.dtype != torch.int32 or not t.is_cuda or not t.is_contiguous():
        raise ValueError("signal words must be a contiguous int32 device tensor")
    return t


def _result() -> torch.Tensor:
    return torch.zeros(1, dtype=torch.int32, device="cuda:0")


def translate_ptr(ptr: int, from_rank: int, to_rank: int, heap_bases) -> int:
    """``heap_bases[to_rank] + (ptr - heap_bases[from_rank])``."""
    bases = [int(b) for b in (heap_bases.tolist() if hasattr(heap_bases, "tolist") else heap_bases)]
    return bases[to_rank] + (int(ptr) - bases[from_rank])


def tile_signal(locks: torch.Tensor, tile_id: int) -> None:
    _lib.check(_lib.load().tccl_prim_signal(_launch.ptr(_words(locks)), tile_id, _launch.stream_ptr()), "tile_signal")


def tile_signal_add(signals: torch.Tensor, tile_id: int, value: int = 1) -> int:
    out = _result()
    rc = _lib.load().tccl_prim_signal_add(_launch.ptr(_words(signals)), tile_id, value, _launch.ptr(out), _launch.stream_ptr())
    _lib.check(rc, "tile_signal_add")
    return int(out.item())


def _try(locks: torch.Tensor, tile_id: int, max_spins: int, consume: bool) -> int:
    out = _result()
    rc = _lib.load().tccl_prim_try_wait(
        _launch.ptr(_words(locks)), tile_id, max_spins, int(consume), _launch.ptr(out), _launch.stream_ptr()
    )
    _lib.check(rc, "tile_try_wait")
    return int(out.item())


def tile_try_wait(locks: torch.Tensor, tile_id: int, MAX_SPINS: int = 1024) -> int:
    """1 if the flag was set (and is now consumed), 0 after ``MAX_SPINS`` empty probes."""
    return _try(locks, tile_id, MAX_SPINS, True)


def tile_try_poll(locks: torch.Tensor, tile_id: int, MAX_SPINS: int = 1024) -> int:
    """Like ``tile_try_wait`` but leaves the flag set."""
    return _try(locks, tile_id, MAX_SPINS, False)


def tile_wait(locks: torch.Tensor, tile_id: int, *, max_spins: int = 1 << 20) -> None:
    """Consume the flag (1 -> 0) once it is set (reference ipc.py:152-168).  The reference spins
    without end; here no device-side wait is unbounded, so after ``max_spins`` empty probes
    this raises instead."""
    if not _try(locks, tile_id, max_spins, True):
        raise RuntimeError(f"tile_wait: locks[{tile_id}] was not signalled within {max_spins} probes")


def tile_poll(locks: torch.Tensor, tile_id: int, *, max_spins: int = 1 << 20) -> None:
    """Wait until the flag is set without consuming it (reference ipc.py:192-209); bounded like ``tile_wait``."""
    if not _try(locks, tile_id, max_spins, False):
        raise RuntimeError(f"tile_poll: locks[{tile_id}] was not signalled within {max_spins} probes")


def tile_wait_ge(signals: torch.Tensor, tile_id: int, threshold: int, *, spin_limit_ns: int = 1_000_000) -> int:
    """1 once ``signals[tile_id] >= threshold``; 0 if ``spin_limit_ns`` passes first."""
    out = _result()
    rc = _lib.load().tccl_prim_wait_ge(
        _launch.ptr(_words(signals)), tile_id, threshold, spin_limit_ns, _launch.ptr(out), _launch.stream_ptr()
    )
    _lib.check(rc, "tile_wait_ge")
    return int(out.item())
