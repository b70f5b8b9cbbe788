"""Per-TileGroup signal, barrier and trace tensors.

Same names, fields and error texts as ``/root/reference/tileccl_v2/signal.py:14-66``: ``counter``,
``barrier`` and any ``extra`` counters are ``int32[n_groups]`` in the symmetric heap (so a peer's
copy sits at the same offset of the peer's slice); the trace tensors are plain device tensors.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Iterable

import torch

from tileccl_amd.v2.heap import SymmetricHeap

# Trace tensors outside the heap: name -> (one entry per group?, element type)
_TRACES = {
    "trace_comm_counter": (True, torch.int32),
    "trace_start_clock": (False, torch.int64),
    "trace_ready_clock": (True, torch.int64),
    "trace_done_clock": (True, torch.int64),
}


@dataclass
class TileGroupSignalState:
    counter: torch.Tensor
    barrier: torch.Tensor
    trace_comm_counter: torch.Tensor
    trace_start_clock: torch.Tensor
    trace_ready_clock: torch.Tensor
    trace_done_clock: torch.Tensor
    extra_counters: "dict[str, torch.Tensor]" = field(default_factory=dict)

    def extra(self, name: str) -> torch.Tensor:
        try:
            return self.extra_counters[name]
        except KeyError:
            raise KeyError(f"unknown TileGroup signal counter: {name}") from None

    def all_tensors(self) -> "list[torch.Tensor]":
        """Heap words first (counter, barrier, extras), then the traces."""
        return [self.counter, self.barrier, *self.extra_counters.values(), *(getattr(self, name) for name in _TRACES)]

    def reset(self) -> None:
        """Zero every word (device fill kernels on the current stream)."""
        for words in self.all_tensors():
            words.zero_()


def allocate_tile_group_signals(*, heap: SymmetricHeap, n_groups: int, device: "torch.device | str",
                                extra_counters: Iterable[str] = ()) -> TileGroupSignalState:
    if n_groups <= 0:
        raise ValueError("n_groups must be positive")
    # Allocation order in the heap: the named extras, then counter, then barrier.
    in_heap = {name: heap.allocate_tensor((n_groups,), dtype=torch.int32) for name in (*extra_counters, "counter", "barrier")}
    traces = {name: torch.empty((n_groups if per_group else 1,), dtype=dtype, device=device)
              for name, (per_group, dtype) in _TRACES.items()}
    counter, barrier = in_heap.pop("counter"), in_heap.pop("barrier")
    return TileGroupSignalState(counter=counter, barrier=barrier, extra_counters=in_heap, **traces)
