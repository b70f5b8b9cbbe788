"""Per-TileGroup signal, barrier and trace tensors.

Mirrors ``/root/reference/tileccl_v2/signal.py:14-66``: ``counter``, ``barrier`` and any
``extra`` counters are ``int32[n_groups]`` in the symmetric heap (so a peer's copy sits at
the same offset of the peer's slice); the trace tensors are plain device tensors.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Iterable

import torch

from tileccl_amd.v2.heap import SymmetricHeap


@dataclass
class TileGroupSignalState:
    counter: torch.Tensor
    barrier: torch.Tensor
    trace_comm_counter: torch.Tensor
    trace_start_clock: torch.Tensor
    trace_ready_clock: torch.Tensor
    trace_done_clock: torch.Tensor
    extra_counters: dict[str, torch.Tensor] = field(default_factory=dict)

    def extra(self, name: str) -> torch.Tensor:
        if name not in self.extra_counters:
            raise KeyError(f"unknown TileGroup signal counter: {name}")
        return self.extra_counters[name]

    def all_tensors(self) -> list[torch.Tensor]:
        return [
            self.counter,
            self.barrier,
            *self.extra_counters.values(),
            self.trace_comm_counter,
            self.trace_start_clock,
            self.trace_ready_clock,
            self.trace_done_clock,
        ]

    def reset(self) -> None:
        """Zero every word (device fill kernels on the current stream)."""
        for t in self.all_tensors():
            t.zero_()


def allocate_tile_group_signals(
    *, heap: SymmetricHeap, n_groups: int, device: torch.device | str, extra_counters: Iterable[str] = ()
) -> TileGroupSignalState:
    if n_groups <= 0:
        raise ValueError("n_groups must be positive")
    words = lambda: heap.allocate_tensor((n_groups,), dtype=torch.int32)  # noqa: E731
    extra = {name: words() for name in extra_counters}
    return TileGroupSignalState(
        counter=words(),
        barrier=words(),
        trace_comm_counter=torch.empty((n_groups,), dtype=torch.int32, device=device),
        trace_start_clock=torch.empty((1,), dtype=torch.int64, device=device),
        trace_ready_clock=torch.empty((n_groups,), dtype=torch.int64, device=device),
        trace_done_clock=torch.empty((n_groups,), dtype=torch.int64, device=device),
        extra_counters=extra,
    )
