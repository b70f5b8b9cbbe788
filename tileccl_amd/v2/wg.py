"""Compute / communication workgroup split and per-group task geometry.

Same names, fields, defaults and error texts as ``/root/reference/tileccl_v2/wg.py:10-90``.
``total_sms`` is the number of workgroup slots of one launch (on MI355X: 256 CUs);
``num_comm_wgs`` of them move data, the rest run the GEMM.  A group's payload is cut into tasks
of ``copy_elems`` (copy) or ``reduce_elems`` (reduce) elements; a task is what one communication
workgroup handles at a time.
"""

from __future__ import annotations

from dataclasses import dataclass


def _tasks(payload: int, per_task: "int | None") -> int:
    """Tasks needed for ``payload`` elements (none when the operation is not planned)."""
    return 0 if per_task is None else (payload + per_task - 1) // per_task


@dataclass(frozen=True)
class WGPlan:
    total_sms: int
    num_comm_wgs: int
    max_group_elems: int
    copy_elems: int
    reduce_elems: "int | None" = None
    packed_values_per_word: int = 4

    # workgroups
    num_comp_wgs = property(lambda p: p.total_sms - p.num_comm_wgs)
    total_wgs = property(lambda p: p.total_sms)  # compute + communication
    grid = property(lambda p: (p.total_sms,))
    # tasks: 64-bit words per copy task, and how many tasks the largest group takes
    copy_qwords = property(lambda p: p.copy_elems // p.packed_values_per_word)
    copy_tasks_per_group = property(lambda p: _tasks(p.max_group_elems, p.copy_elems))
    reduce_tasks_per_group = property(lambda p: _tasks(p.max_group_elems, p.reduce_elems))
    tasks_per_group = property(lambda p: max(p.copy_tasks_per_group, p.reduce_tasks_per_group))


def _reject(**values) -> None:
    """ValueError for the first quantity that is given and not positive."""
    for name, value in values.items():
        if value is not None and value <= 0:
            raise ValueError(f"{name} must be positive")


def build_wg_plan(*, total_sms: int, num_comm_wgs: int, max_group_elems: int, copy_elems: int,
                  reduce_elems: "int | None" = None, packed_values_per_word: int = 4) -> WGPlan:
    """Validate the split and task sizes, then freeze them into a ``WGPlan``."""
    _reject(total_sms=total_sms)
    if num_comm_wgs < 0:
        raise ValueError("num_comm_wgs must be non-negative")
    if num_comm_wgs >= total_sms:
        raise ValueError(f"num_comm_wgs={num_comm_wgs} leaves no compute WGs")
    _reject(max_group_elems=max_group_elems, copy_elems=copy_elems, packed_values_per_word=packed_values_per_word)
    for name, value in (("copy_elems", copy_elems), ("max_group_elems", max_group_elems)):
        if value % packed_values_per_word:
            raise ValueError(f"{name} must be divisible by packed_values_per_word")
    _reject(reduce_elems=reduce_elems)
    return WGPlan(total_sms, num_comm_wgs, max_group_elems, copy_elems, reduce_elems, packed_values_per_word)
