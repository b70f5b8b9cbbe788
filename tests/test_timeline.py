"""TimelineRecorder: event validation, JSON schema round trip, device-trace bridge
(reference tileccl_v2/runtime/timeline.py:13-214; schema "tileccl.timeline.v1")."""

import json

import pytest

from tileccl_amd.v2.runtime import TimelineEvent, TimelineRecorder


def test_event_validation_messages():
    with pytest.raises(ValueError, match="times must be finite"):
        TimelineEvent(name="x", lane="l", start_ms=float("nan"), end_ms=1.0)
    with pytest.raises(ValueError, match=r"'x' has end_ms < start_ms: 1.0 < 2.0"):
        TimelineEvent(name="x", lane="l", start_ms=2.0, end_ms=1.0)
    with pytest.raises(ValueError, match="source must not be empty"):
        TimelineEvent(name="x", lane="l", start_ms=0.0, end_ms=1.0, source="")
    e = TimelineEvent(name="x", lane="l", start_ms=1, end_ms=3)
    assert isinstance(e.start_ms, float) and e.duration_ms == 2.0


def test_payload_schema_and_round_trip(tmp_path):
    rec = TimelineRecorder(benchmark="gate1", path_name="s2", metadata={"M": 4096})
    rec.record_span(name="gemm", lane="compute", start_ms=0.0, end_ms=0.04, category="compute", rank=0,
                    tile_range={"row_start": 0, "row_end": 1024})
    rec.record_marker(name="ready g0", lane="signals", at_ms=0.02, label="g0")
    rec.record_span(name="copy", lane="compute", start_ms=0.02, end_ms=0.05, source="device_trace")
    p = rec.to_payload()
    assert p["schema"] == "tileccl.timeline.v1" and p["benchmark"] == "gate1" and p["path_name"] == "s2"
    assert p["lane_order"] == ["compute", "signals"]  # first appearance
    assert p["authenticity_checks"] == {"event_count": 3, "all_events_have_source": True,
                                        "all_events_have_nonnegative_duration": True}
    first = p["events"][0]
    assert list(first) == ["name", "lane", "start_ms", "end_ms", "duration_ms", "category", "source", "rank", "tile_range"]
    assert p["events"][1]["duration_ms"] == 0.0 and p["events"][1]["category"] == "marker" and "rank" not in p["events"][1]
    out = tmp_path / "deep" / "t.json"
    rec.write_json(out)
    again = TimelineRecorder.from_payload(json.loads(out.read_text()))
    assert again.to_payload() == p and again.events == rec.events


def test_device_trace_to_lanes():
    rec = TimelineRecorder(benchmark="gate1", path_name="s2")
    groups = [(0, 1024, 256), (1024, 2048, 256), (2048, 3072, 256)]
    # 100 MHz clock: 100 ticks = 1 us.  Group 2 was never stamped.
    made = rec.record_device_trace(start_clock=1_000_000, ready_clocks=[1_003_000, 1_004_000, 0],
                                   done_clocks=[1_004_500, 1_005_000, 0], groups=groups, rank=0)
    assert [e.name for e in made] == ["group 0 produce", "group 0 transfer", "group 1 produce", "group 1 transfer"]
    produce, transfer = made[0], made[1]
    assert produce.start_ms == 0.0 and produce.end_ms == pytest.approx(0.03) and produce.category == "producer"
    assert transfer.start_ms == pytest.approx(0.03) and transfer.end_ms == pytest.approx(0.045)
    assert transfer.tile_range == {"row_start": 0, "row_end": 1024, "tiles": 256} and transfer.source == "device_trace"
    assert rec.to_payload()["lane_order"] == ["group 0", "group 1"]
    with pytest.raises(ValueError, match="one entry per TileGroup"):
        rec.record_device_trace(start_clock=1, ready_clocks=[1], done_clocks=[1, 2])


def test_render_png(tmp_path):
    pytest.importorskip("matplotlib")
    rec = TimelineRecorder(benchmark="b", path_name="p")
    with pytest.raises(ValueError, match="empty timeline"):
        rec.render_png(tmp_path / "e.png")
    rec.record_span(name="a", lane="x", start_ms=0.0, end_ms=1.0)
    rec.record_marker(name="m", lane="y", at_ms=0.5)
    rec.render_png(tmp_path / "t.png")
    assert (tmp_path / "t.png").stat().st_size > 1000
