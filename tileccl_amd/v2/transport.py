"""Direction and task size of the device-side peer transfers.

Same names, fields, defaults and error texts as ``/root/reference/tileccl_v2/transport.py:12-86``.
``push``: the producer of a TileGroup writes it into the peer's slice; ``pull``: the consumer
reads it out of the producer's slice.  Task sizes are counted in elements; ``copy_qwords`` is the
same size in packed 64-bit words of four 16-bit values, the unit the reference's kernels move.
"""

from __future__ import annotations

import enum
from dataclasses import dataclass, fields

from tileccl_amd.v2 import wg

PACKED_FP16_VALUES_PER_WORD = 4

CommMode = enum.Enum("CommMode", {"PUSH": "push", "PULL": "pull"}, module=__name__)


def normalize_comm_mode(comm_mode: "str | CommMode") -> CommMode:
    """A ``CommMode`` passes through; a string is looked up by value."""
    if type(comm_mode) is CommMode:
        return comm_mode
    found = [m for m in CommMode if m.value == comm_mode]
    if not found:
        raise ValueError(f"unknown comm_mode={comm_mode!r}; expected one of {', '.join(m.value for m in CommMode)}")
    return found[0]


@dataclass(frozen=True)
class P2PTransportPlan:
    comm_mode: CommMode
    copy_elems: int
    reduce_elems: "int | None" = None
    packed_values_per_word: int = PACKED_FP16_VALUES_PER_WORD

    push_mode = property(lambda self: self.comm_mode is CommMode.PUSH)
    copy_qwords = property(lambda self: self.copy_elems // self.packed_values_per_word)

    def build_wg_plan(self, *, total_sms: int, num_comm_wgs: int, max_group_elems: int) -> "wg.WGPlan":
        """Workgroup plan of a launch that moves groups of up to ``max_group_elems`` with these task sizes."""
        sizes = {f.name: getattr(self, f.name) for f in fields(self) if f.name != "comm_mode"}
        return wg.build_wg_plan(total_sms=total_sms, num_comm_wgs=num_comm_wgs, max_group_elems=max_group_elems, **sizes)


def build_p2p_transport_plan(*, comm_mode: "str | CommMode", copy_elems: int, reduce_elems: "int | None" = None,
                             packed_values_per_word: int = PACKED_FP16_VALUES_PER_WORD) -> P2PTransportPlan:
    """Check the sizes (each must be positive when given), resolve the mode, freeze the plan."""
    sizes = dict(copy_elems=copy_elems, reduce_elems=reduce_elems, packed_values_per_word=packed_values_per_word)
    for name, value in sizes.items():
        if value is not None and value <= 0:
            raise ValueError(f"{name} must be positive")
    return P2PTransportPlan(normalize_comm_mode(comm_mode), **sizes)
