"""Named stage timers behind a flag: which share of a step goes to which part of the model.

Reference: the stage timers of the prefill profiler (benchmarks/profile_prefill.py:201-285: named stages timed with
device events, :302-375: their summary).  Here a part wraps the launches of a stage in ``with stage("name"):``;
unless a :func:`collect` block is active that costs one attribute test.  Inside one, two device events are recorded
around the stage on the current stream, and the summary adds their distances by name, so the work of the device is
what is measured, not the host's launches.  Captured graph replays hold no Python and so no stages: stage times are
those of eager steps.
"""

from __future__ import annotations

import contextlib

import torch

_collecting: "StageTimes | None" = None


class StageTimes:
    def __init__(self) -> None:
        self.pairs: list[tuple[str, torch.cuda.Event, torch.cuda.Event]] = []

    def summary(self) -> dict[str, dict[str, float]]:
        """name -> {"calls", "ms", "share"}; waits for the device."""
        torch.cuda.synchronize()
        totals: dict[str, list[float]] = {}
        for name, start, end in self.pairs:
            entry = totals.setdefault(name, [0, 0.0])
            entry[0] += 1
            entry[1] += start.elapsed_time(end)
        whole = sum(ms for _, ms in totals.values()) or 1.0
        return {name: {"calls": int(calls), "ms": round(ms, 4), "share": round(ms / whole, 4)}
                for name, (calls, ms) in sorted(totals.items(), key=lambda item: -item[1][1])}


class stage:
    """``with stage("attention"): ...`` around the launches of a stage."""

    __slots__ = ("name", "start")

    def __init__(self, name: str) -> None:
        self.name = name
        self.start = None

    def __enter__(self) -> "stage":
        if _collecting is not None:
            self.start = torch.cuda.Event(enable_timing=True)
            self.start.record()
        return self

    def __exit__(self, *exc) -> None:
        if self.start is not None and _collecting is not None:
            end = torch.cuda.Event(enable_timing=True)
            end.record()
            _collecting.pairs.append((self.name, self.start, end))


@contextlib.contextmanager
def collect():
    """Stages entered inside the block are timed; yields the :class:`StageTimes` to ask for the summary."""
    global _collecting
    previous, _collecting = _collecting, StageTimes()
    try:
        yield _collecting
    finally:
        _collecting = previous
