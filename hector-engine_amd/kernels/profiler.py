"""Per-kernel times from pairs of events, in the manner of the reference's engine profiler
(an event pair around every command, calls / total / average / share per op:
src/engine.cpp:299-316, :372-435).

While a profiler is active, every launch that goes through kernels.ops (and every library
matrix product of parts.linear) is bracketed by two events on the current stream. The events
are read when the table is asked for, not after each launch, so the launches still follow one
another without a wait in between. Steps run eagerly while profiling: a captured graph has no
place for events between its nodes.
"""
from __future__ import annotations

import contextlib
import functools

import torch

_active: "OpProfiler | None" = None


class OpProfiler:
    def __init__(self):
        self._pending: list[tuple[str, torch.cuda.Event, torch.cuda.Event]] = []
        self._totals: dict[str, list] = {}     # name -> [calls, milliseconds]

    @contextlib.contextmanager
    def span(self, name: str):
        start = torch.cuda.Event(enable_timing=True)
        stop = torch.cuda.Event(enable_timing=True)
        start.record()
        try:
            yield
        finally:
            stop.record()
            self._pending.append((name, start, stop))

    def collect(self) -> None:
        if self._pending:
            self._pending[-1][2].synchronize()
        for name, start, stop in self._pending:
            stop.synchronize()
            entry = self._totals.setdefault(name, [0, 0.0])
            entry[0] += 1
            entry[1] += start.elapsed_time(stop)
        self._pending.clear()

    def clear(self) -> None:
        self.collect()
        self._totals.clear()

    def rows(self) -> list[tuple[str, int, float, float, float]]:
        """(op, calls, total ms, average ms, share in %) by total time, largest first."""
        self.collect()
        total = sum(ms for _, ms in self._totals.values())
        return summarize({k: tuple(v) for k, v in self._totals.items()}, total)

    def format(self) -> str:
        return format_table(self.rows())


def summarize(totals: dict[str, tuple[int, float]], total_ms: float):
    rows = [(name, calls, ms, ms / calls, 100.0 * ms / total_ms if total_ms > 0 else 0.0)
            for name, (calls, ms) in totals.items() if calls > 0]
    return sorted(rows, key=lambda r: -r[2])


def format_table(rows) -> str:
    """The reference's table (src/engine.cpp:393-434): Op, Calls, Total(ms), Avg(ms), %."""
    if not rows:
        return "No profiling data"
    width = max(12, max(len(r[0]) for r in rows) + 2)
    lines = ["=== Engine Profile ===",
             f"{'Op':>{width}}{'Calls':>10}{'Total(ms)':>12}{'Avg(ms)':>12}{'%':>8}",
             "-" * (width + 42)]
    for name, calls, ms, avg, pct in rows:
        lines.append(f"{name:>{width}}{calls:>10}{ms:>12.2f}{avg:>12.3f}{pct:>7.1f}%")
    lines.append("-" * (width + 42))
    lines.append(f"{'TOTAL':>{width}}{'':>10}{sum(r[2] for r in rows):>12.2f}")
    return "\n".join(lines)


@contextlib.contextmanager
def active(profiler: "OpProfiler | None"):
    """Inside: launches are recorded by `profiler` (None: nothing is recorded)."""
    global _active
    before, _active = _active, profiler
    try:
        yield
    finally:
        _active = before


def span(name: str):
    """A context that times what runs inside under `name` when a profiler is active."""
    return _active.span(name) if _active is not None else contextlib.nullcontext()


def op(name: str):
    """Decorator of a launching function: one span per call while a profiler is active."""
    def deco(fn):
        @functools.wraps(fn)
        def timed(*args, **kwargs):
            if _active is None:
                return fn(*args, **kwargs)
            with _active.span(name):
                return fn(*args, **kwargs)
        return timed
    return deco
