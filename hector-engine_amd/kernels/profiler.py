"""Per-kernel times from pairs of events, in the manner of the reference's engine profiler
(an event pair around every command, calls / total / average / share per op:
src/engine.cpp:299-316, :372-435).

While a profiler is active, every launch that goes through kernels.ops (and every library
matrix product of parts.linear) is bracketed by two events on the current stream. The events
are read when the table is asked for, not after each launch, so the launches still follow one
another without a wait in between. Steps run eagerly while profiling: a captured graph has no
place for events between its nodes.

The same hooks serve a debugging mode in the manner of the reference's sync_after_each_op
(src/engine.cpp:318-334): inside sync_each_launch() the host waits for the GPU after every
launch, so that a fault a kernel raises asynchronously is reported with the name of the op
that caused it, not at some later call.
"""
from __future__ import annotations

import contextlib
import functools

import torch

_active: "OpProfiler | None" = None
_sync_each = False
# events of launches not yet read: collect() is called on the way once so many are waiting
MAX_PENDING = 4096


class LaunchFault(RuntimeError):
    """The GPU reported an error right after the named launch (sync_each_launch mode)."""


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
            if len(self._pending) >= MAX_PENDING:
                # a long profiled generation would pile up events without bound; the oldest
                # have long completed, so reading them costs no wait to speak of
                self._collect(len(self._pending) // 2)

    def collect(self) -> None:
        self._collect(len(self._pending))

    def _collect(self, count: int) -> None:
        """Reads the `count` oldest pending event pairs into the totals."""
        for name, start, stop in self._pending[:count]:
            stop.synchronize()
            entry = self._totals.setdefault(name, [0, 0.0])
            entry[0] += 1
            entry[1] += start.elapsed_time(stop)
        del self._pending[:count]

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


@contextlib.contextmanager
def sync_each_launch(on: bool = True):
    """Inside (with on): the host waits for the GPU after every launch and raises LaunchFault
    naming the op when the wait reports an error."""
    global _sync_each
    before, _sync_each = _sync_each, bool(on)
    try:
        yield
    finally:
        _sync_each = before


def _wait_after(name: str) -> None:
    try:
        torch.cuda.synchronize()
    except RuntimeError as exc:
        raise LaunchFault(f"the GPU reported an error after the launch of '{name}': {exc}") from exc


@contextlib.contextmanager
def _synced(name: str):
    with (_active.span(name) if _active is not None else contextlib.nullcontext()):
        yield
    _wait_after(name)


def span(name: str):
    """A context that times what runs inside under `name` when a profiler is active (and waits
    for it in sync_each_launch mode)."""
    if _sync_each:
        return _synced(name)
    return _active.span(name) if _active is not None else contextlib.nullcontext()


def op(name: str):
    """Decorator of a launching function: one span per call while a profiler is active."""
    def deco(fn):
        @functools.wraps(fn)
        def timed(*args, **kwargs):
            if _active is None and not _sync_each:
                return fn(*args, **kwargs)
            with span(name):
                return fn(*args, **kwargs)
        return timed
    return deco
