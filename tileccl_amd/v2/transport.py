"""Direction and task size of the device-side peer transfers.

Mirrors ``/root/reference/tileccl_v2/transport.py:12-86``.  ``push``: the producer of a
TileGroup writes it into the peer's slice; ``pull``: the consumer reads it out of the
producer's slice.  Payloads move as packed 64-bit words of four 16-bit values.
"""

from __future__ import annotations

from dataclasses import dataclass
from enum import Enum

from tileccl_amd.v2.wg import WGPlan, build_wg_plan

PACKED_FP16_VALUES_PER_WORD = 4


class CommMode(Enum):
    PUSH = "push"
    PULL = "pull"


@dataclass(frozen=True)
class P2PTransportPlan:
    comm_mode: CommMode
    copy_elems: int
    reduce_elems: int | None = None
    packed_values_per_word: int = PACKED_FP16_VALUES_PER_WORD

    @property
    def push_mode(self) -> bool:
        return self.comm_mode is CommMode.PUSH

    @property
    def copy_qwords(self) -> int:
        return self.copy_elems // self.packed_values_per_word

    def build_wg_plan(self, *, total_sms: int, num_comm_wgs: int, max_group_elems: int) -> WGPlan:
        """Workgroup plan for a launch that moves groups of up to ``max_group_elems``."""
        return build_wg_plan(
            total_sms=total_sms,
            num_comm_wgs=num_comm_wgs,
            max_group_elems=max_group_elems,
            copy_elems=self.copy_elems,
            reduce_elems=self.reduce_elems,
            packed_values_per_word=self.packed_values_per_word,
        )


def normalize_comm_mode(comm_mode: str | CommMode) -> CommMode:
    """Accept a ``CommMode`` or its string value."""
    if isinstance(comm_mode, CommMode):
        return comm_mode
    for mode in CommMode:
        if mode.value == comm_mode:
            return mode
    allowed = ", ".join(mode.value for mode in CommMode)
    raise ValueError(f"unknown comm_mode={comm_mode!r}; expected one of {allowed}")


def build_p2p_transport_plan(
    *,
    comm_mode: str | CommMode,
    copy_elems: int,
    reduce_elems: int | None = None,
    packed_values_per_word: int = PACKED_FP16_VALUES_PER_WORD,
) -> P2PTransportPlan:
    if copy_elems <= 0:
        raise ValueError("copy_elems must be positive")
    if reduce_elems is not None and reduce_elems <= 0:
        raise ValueError("reduce_elems must be positive")
    if packed_values_per_word <= 0:
        raise ValueError("packed_values_per_word must be positive")
    return P2PTransportPlan(
        comm_mode=normalize_comm_mode(comm_mode),
        copy_elems=copy_elems,
        reduce_elems=reduce_elems,
        packed_values_per_word=packed_values_per_word,
    )
