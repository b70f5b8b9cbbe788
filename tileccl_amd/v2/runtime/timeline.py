"""Lane timeline of a fused launch: events, JSON artifact, lane chart, device-trace bridge.

Same surface and JSON schema as ``/root/reference/tileccl_v2/runtime/timeline.py:13-214``
(``TimelineEvent``, ``TimelineRecorder.record_span / record_marker / to_payload /
from_payload / write_json / render_png``, schema ``tileccl.timeline.v1``), so artifacts are
interchangeable.  New here: ``record_device_trace`` turns the clocks a traced S2 launch
leaves in ``TileGroupSignalState`` (reference ``tileccl_v2/signal.py:20-23``) into lanes:
per TileGroup, "produce" = launch start .. the group's last tile stored, and "transfer" =
group complete .. its transfers stored.
"""

from __future__ import annotations

import json
import math
from dataclasses import dataclass, field
from pathlib import Path
from typing import Any, Iterable, Mapping, Sequence

SCHEMA = "tileccl.timeline.v1"
DEVICE_TICKS_PER_MS = 100_000.0  # the device wall clock read by the kernels counts at 100 MHz


@dataclass(frozen=True)
class TimelineEvent:
    name: str
    lane: str
    start_ms: float
    end_ms: float
    category: str = "span"
    rank: int | None = None
    label: str | None = None
    source: str = "runtime"
    tile_range: Mapping[str, Any] | None = None
    color: str | None = None
    metadata: Mapping[str, Any] = field(default_factory=dict)

    def __post_init__(self) -> None:
        lo, hi = float(self.start_ms), float(self.end_ms)
        if not (math.isfinite(lo) and math.isfinite(hi)):
            raise ValueError("TimelineEvent times must be finite")
        if hi < lo:
            raise ValueError(f"TimelineEvent {self.name!r} has end_ms < start_ms: {hi} < {lo}")
        if not self.source:
            raise ValueError("TimelineEvent source must not be empty")
        object.__setattr__(self, "start_ms", lo)
        object.__setattr__(self, "end_ms", hi)

    @property
    def duration_ms(self) -> float:
        return self.end_ms - self.start_ms

    def to_json(self) -> dict[str, Any]:
        out: dict[str, Any] = {
            "name": self.name,
            "lane": self.lane,
            "start_ms": self.start_ms,
            "end_ms": self.end_ms,
            "duration_ms": self.duration_ms,
            "category": self.category,
            "source": self.source,
        }
        optional = {"rank": self.rank, "label": self.label, "color": self.color}
        out.update({k: v for k, v in optional.items() if v is not None})
        if self.tile_range is not None:
            out["tile_range"] = dict(self.tile_range)
        if self.metadata:
            out["metadata"] = dict(self.metadata)
        # key order of the reference artifact: rank, label, tile_range, color, metadata
        order = ["name", "lane", "start_ms", "end_ms", "duration_ms", "category", "source", "rank", "label",
                 "tile_range", "color", "metadata"]
        return {k: out[k] for k in order if k in out}

    @classmethod
    def from_json(cls, payload: Mapping[str, Any]) -> "TimelineEvent":
        return cls(
            name=str(payload["name"]),
            lane=str(payload["lane"]),
            start_ms=float(payload["start_ms"]),
            end_ms=float(payload["end_ms"]),
            category=str(payload.get("category", "span")),
            rank=payload.get("rank"),
            label=payload.get("label"),
            source=str(payload.get("source", "runtime")),
            tile_range=payload.get("tile_range"),
            color=payload.get("color"),
            metadata=payload.get("metadata", {}),
        )


def _lanes_in_order(events: Iterable[TimelineEvent], lane_order: Sequence[str] | None = None) -> list[str]:
    if lane_order is not None:
        return list(lane_order)
    seen: dict[str, None] = {}
    for e in events:
        seen.setdefault(e.lane, None)
    return list(seen)


class TimelineRecorder:
    def __init__(self, *, benchmark: str, path_name: str, metadata: Mapping[str, Any] | None = None) -> None:
        self.benchmark = benchmark
        self.path_name = path_name
        self.metadata = dict(metadata or {})
        self._events: list[TimelineEvent] = []

    @property
    def events(self) -> tuple[TimelineEvent, ...]:
        return tuple(self._events)

    def record_span(self, *, name: str, lane: str, start_ms: float, end_ms: float, category: str = "span",
                    rank: int | None = None, label: str | None = None, source: str = "runtime",
                    tile_range: Mapping[str, Any] | None = None, color: str | None = None,
                    metadata: Mapping[str, Any] | None = None) -> TimelineEvent:
        event = TimelineEvent(name=name, lane=lane, start_ms=start_ms, end_ms=end_ms, category=category, rank=rank,
                              label=label, source=source, tile_range=tile_range, color=color, metadata=metadata or {})
        self._events.append(event)
        return event

    def record_marker(self, *, name: str, lane: str, at_ms: float, category: str = "marker", **kwargs) -> TimelineEvent:
        return self.record_span(name=name, lane=lane, start_ms=at_ms, end_ms=at_ms, category=category, **kwargs)

    # -- device trace -------------------------------------------------------------------
    def record_device_trace(self, *, start_clock: int, ready_clocks: Sequence[int], done_clocks: Sequence[int],
                            groups: Sequence[tuple[int, int, int]] | None = None, rank: int | None = None,
                            ticks_per_ms: float = DEVICE_TICKS_PER_MS) -> list[TimelineEvent]:
        """Lanes from the clocks of one traced TileGroup launch.

        ``start_clock`` is the launch's first stamp, ``ready_clocks[g]`` the moment group ``g``
        was complete (or first seen complete), ``done_clocks[g]`` the moment its transfers were
        stored; a zero clock means "not stamped" and yields no event.  ``groups`` are the
        plan's ``(row_start, row_end, tiles)`` triples, recorded as ``tile_range``.
        """
        if len(ready_clocks) != len(done_clocks):
            raise ValueError("ready_clocks and done_clocks must have one entry per TileGroup")
        if groups is not None and len(groups) != len(ready_clocks):
            raise ValueError("groups must have one entry per TileGroup")
        t0 = int(start_clock)
        made: list[TimelineEvent] = []
        for g, (ready, done) in enumerate(zip(ready_clocks, done_clocks)):
            rng = None
            if groups is not None:
                rng = {"row_start": int(groups[g][0]), "row_end": int(groups[g][1]), "tiles": int(groups[g][2])}
            if ready and t0 and ready >= t0:
                made.append(self.record_span(
                    name=f"group {g} produce", lane=f"group {g}", start_ms=0.0, end_ms=(ready - t0) / ticks_per_ms,
                    category="producer", rank=rank, label=f"g{g}", source="device_trace", tile_range=rng))
            if ready and done and done >= ready:
                made.append(self.record_span(
                    name=f"group {g} transfer", lane=f"group {g}", start_ms=(ready - t0) / ticks_per_ms,
                    end_ms=(done - t0) / ticks_per_ms, category="frontier", rank=rank, source="device_trace",
                    tile_range=rng))
        return made

    def record_signal_state(self, signals, plan=None, rank: int | None = None) -> list[TimelineEvent]:
        """``record_device_trace`` from a ``TileGroupSignalState`` (synchronises the device)."""
        return self.record_device_trace(
            start_clock=int(signals.trace_start_clock.cpu()[0]),
            ready_clocks=[int(x) for x in signals.trace_ready_clock.cpu().tolist()],
            done_clocks=[int(x) for x in signals.trace_done_clock.cpu().tolist()],
            groups=None if plan is None else list(plan.groups),
            rank=rank,
        )

    # -- artifacts ----------------------------------------------------------------------
    def to_payload(self) -> dict[str, Any]:
        return {
            "schema": SCHEMA,
            "benchmark": self.benchmark,
            "path_name": self.path_name,
            "metadata": self.metadata,
            "lane_order": _lanes_in_order(self._events),
            "events": [e.to_json() for e in self._events],
            "authenticity_checks": {
                "event_count": len(self._events),
                "all_events_have_source": all(bool(e.source) for e in self._events),
                "all_events_have_nonnegative_duration": all(e.end_ms >= e.start_ms for e in self._events),
            },
        }

    @classmethod
    def from_payload(cls, payload: Mapping[str, Any]) -> "TimelineRecorder":
        rec = cls(benchmark=str(payload["benchmark"]), path_name=str(payload["path_name"]),
                  metadata=payload.get("metadata", {}))
        rec._events.extend(TimelineEvent.from_json(e) for e in payload.get("events", []))
        return rec

    def write_json(self, path: Path) -> None:
        path = Path(path)
        path.parent.mkdir(parents=True, exist_ok=True)
        path.write_text(json.dumps(self.to_payload(), indent=2), encoding="utf-8")

    def render_png(self, path: Path, *, title: str | None = None, lane_order: Sequence[str] | None = None) -> None:
        render_timeline_png(self._events, Path(path), title=title or f"{self.benchmark}: {self.path_name}",
                            lane_order=lane_order)


def render_timeline_png(events: Sequence[TimelineEvent], path: Path, *, title: str,
                        lane_order: Sequence[str] | None = None) -> None:
    """A Gantt chart: one row per lane (first lane on top), one bar per span, a thin mark
    per zero-length event.  Categories share a colour taken from matplotlib's ``tab10``
    cycle in order of first appearance; an event's own ``color`` wins."""
    if not events:
        raise ValueError("Cannot render an empty timeline")
    import matplotlib

    matplotlib.use("Agg")
    import matplotlib.pyplot as plt

    lanes = _lanes_in_order(events, lane_order)
    palette = plt.get_cmap("tab10").colors
    shade: dict[str, object] = {}
    for e in events:
        shade.setdefault(e.category, palette[len(shade) % len(palette)])
    horizon = max(e.end_ms for e in events) or 1.0
    mark = horizon / 400.0  # width given to instantaneous events so that they stay visible
    fig, ax = plt.subplots(figsize=(11, 1.2 + 0.5 * len(lanes)), constrained_layout=True)
    for row, lane in enumerate(lanes):
        mine = [e for e in events if e.lane == lane]
        ax.broken_barh([(e.start_ms, e.duration_ms or mark) for e in mine], (row - 0.3, 0.6),
                       facecolors=[e.color or shade[e.category] for e in mine])
        for e in mine:
            text = e.label or e.name
            if e.duration_ms / horizon * 11 * 72 > 5.5 * len(text):  # the bar is wider than the text at 7 pt
                ax.annotate(text, (e.start_ms + e.duration_ms / 2, row), ha="center", va="center", fontsize=7)
    ax.set(title=title, xlabel="Elapsed time (ms)", xlim=(0, horizon * 1.02), ylim=(len(lanes) - 0.5, -0.5))
    ax.set_yticks(range(len(lanes)), labels=lanes)
    ax.xaxis.grid(True, linewidth=0.4)
    ax.legend(handles=[plt.Rectangle((0, 0), 1, 1, color=c) for c in shade.values()], labels=list(shade),
              loc="upper right", fontsize=7, ncols=min(len(shade), 4), frameon=False)
    path.parent.mkdir(parents=True, exist_ok=True)
    fig.savefig(path, dpi=150)
    plt.close(fig)
