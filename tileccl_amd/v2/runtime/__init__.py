"""Runtime helpers of the TileGroup path (reference ``tileccl_v2/runtime/__init__.py``)."""

from tileccl_amd.v2.runtime.timeline import TimelineEvent, TimelineRecorder

__all__ = ["TimelineEvent", "TimelineRecorder"]
