"""Compute / communication workgroup split and per-group task geometry.

Mirrors ``/root/reference/tileccl_v2/wg.py:10-90``.  ``total_sms`` is the number of
workgroup slots of one launch (on MI355X: 256 CUs); ``num_comm_wgs`` of them move data,
the rest run the GEMM.  A group's payload is cut into tasks of ``copy_elems`` (copy) or
``reduce_elems`` (reduce) elements; a task is what one communication workgroup handles
at a time.
"""

from __future__ import annotations

from dataclasses import dataclass


def _cdiv(a: int, b: int) -> int:
    return -(-a // b)


@dataclass(frozen=True)
class WGPlan:
    total_sms: int
    num_comm_wgs: int
    max_group_elems: int
    copy_elems: int
    reduce_elems: int | None = None
    packed_values_per_word: int = 4

    @property
    def num_comp_wgs(self) -> int:
        return self.total_sms - self.num_comm_wgs

    @property
    def total_wgs(self) -> int:
        return self.num_comp_wgs + self.num_comm_wgs

    @property
    def grid(self) -> tuple[int]:
        return (self.total_wgs,)

    @property
    def copy_qwords(self) -> int:
        """64-bit words per copy task (``packed_values_per_word`` 16-bit values each)."""
        return self.copy_elems // self.packed_values_per_word

    @property
    def copy_tasks_per_group(self) -> int:
        return _cdiv(self.max_group_elems, self.copy_elems)

    @property
    def reduce_tasks_per_group(self) -> int:
        return 0 if self.reduce_elems is None else _cdiv(self.max_group_elems, self.reduce_elems)

    @property
    def tasks_per_group(self) -> int:
        return max(self.copy_tasks_per_group, self.reduce_tasks_per_group)


def build_wg_plan(
    *,
    total_sms: int,
    num_comm_wgs: int,
    max_group_elems: int,
    copy_elems: int,
    reduce_elems: int | None = None,
    packed_values_per_word: int = 4,
) -> WGPlan:
    """Validate the split and task sizes, then freeze them into a ``WGPlan``."""
    checks = (
        (total_sms <= 0, "total_sms must be positive"),
        (num_comm_wgs < 0, "num_comm_wgs must be non-negative"),
        (total_sms - num_comm_wgs <= 0, f"num_comm_wgs={num_comm_wgs} leaves no compute WGs"),
        (max_group_elems <= 0, "max_group_elems must be positive"),
        (copy_elems <= 0, "copy_elems must be positive"),
        (packed_values_per_word <= 0, "packed_values_per_word must be positive"),
    )
    for failed, message in checks:
        if failed:
            raise ValueError(message)
    if copy_elems % packed_values_per_word:
        raise ValueError("copy_elems must be divisible by packed_values_per_word")
    if max_group_elems % packed_values_per_word:
        raise ValueError("max_group_elems must be divisible by packed_values_per_word")
    if reduce_elems is not None and reduce_elems <= 0:
        raise ValueError("reduce_elems must be positive")
    return WGPlan(
        total_sms=total_sms,
        num_comm_wgs=num_comm_wgs,
        max_group_elems=max_group_elems,
        copy_elems=copy_elems,
        reduce_elems=reduce_elems,
        packed_values_per_word=packed_values_per_word,
    )
