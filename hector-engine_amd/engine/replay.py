"""Trace replay: feeds given token ids through the engine's own step function,
step by step, and writes the logits at the wanted places. It samples nothing and
has no forward pass, cache or loader of its own. The reference's tools of the
same purpose feed ids one by one and write the per-position argmax
(tools/quant_bench/argmax_all_positions.cu:12-55) or feed one prompt and write
the last position's logits as float32 (tools/gemma4_dump_logits.cu:41-99).

Input, one JSON object a line:
    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}
For a step that wants something, <out>/<step>.f32 holds [wanted, vocab]
little-endian float32 in the order of the entries and of their `want`.
"""
from __future__ import annotations

import json
import os

from .engine import Engine, StepEntry


class TraceError(ValueError):
    pass


def run_trace(engine: Engine, lines, out_dir: str, report=None) -> int:
    """Runs every step read from `lines`; returns the number of steps."""
    os.makedirs(out_dir, exist_ok=True)
    slots: dict[str, int] = {}
    count = 0
    for line in lines:
        line = line.strip()
        if not line:
            continue
        try:
            obj = json.loads(line)
            step_no = obj["step"]
            raw_entries = obj["entries"]
        except (json.JSONDecodeError, KeyError, TypeError) as exc:
            raise TraceError(f"bad trace line {line[:80]!r}: {exc}") from None
        entries = []
        for e in raw_entries:
            rid = str(e["id"])
            if rid not in slots:
                slots[rid] = engine.acquire()
            entries.append(StepEntry(slots[rid], list(e["tokens"]), list(e.get("want", []))))
        logits = engine.step(entries) if entries else None
        if logits is not None:
            arr = logits.detach().to("cpu").numpy().astype("<f4", copy=False)
            arr.tofile(os.path.join(out_dir, f"{step_no}.f32"))
        for rid in obj.get("end", []):
            rid = str(rid)
            if rid not in slots:
                raise TraceError(f"step {step_no}: request '{rid}' ends but was never started")
            engine.release(slots.pop(rid))
        count += 1
        if report is not None:
            report(step_no)
    return count
