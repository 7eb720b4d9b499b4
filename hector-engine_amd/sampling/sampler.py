"""Sampling options and the batched sampler.

The options carry the reference's names, defaults and presets
(src/sampler.hpp:26-52): temperature (below 0.01 means greedy,
src/sampler.cpp:141), top_k (0 = off), top_p (1.0 = off), repetition_penalty,
frequency_penalty, presence_penalty, seed; penalties look back over the last
`penalty_window` generated tokens (src/sampler.hpp:134, src/sampler.cpp:41-91).
With top_k = 0 the whole vocabulary is sampled (the reference's kernel puts 50
in its place: src/sampler.cpp:172-174). All rows of a step are sampled by one
launch and only the chosen ids come back to the host.
"""
from __future__ import annotations

import dataclasses

import numpy as np
import torch

from ..kernels import ops
from .rng import uniform_u32

GREEDY_BELOW = 0.01


@dataclasses.dataclass
class SamplingConfig:
    temperature: float = 1.0
    top_k: int = 0
    top_p: float = 1.0
    repetition_penalty: float = 1.0
    frequency_penalty: float = 0.0
    presence_penalty: float = 0.0
    seed: int = 0
    penalty_window: int = 128

    @classmethod
    def greedy(cls):
        return cls(temperature=0.0, repetition_penalty=1.2)

    @classmethod
    def creative(cls, temp: float = 0.8, k: int = 50, p: float = 0.9):
        return cls(temperature=temp, top_k=k, top_p=p, repetition_penalty=1.15, frequency_penalty=0.1)

    @classmethod
    def balanced(cls, temp: float = 0.7, k: int = 40):
        return cls(temperature=temp, top_k=k, repetition_penalty=1.2)

    @classmethod
    def deterministic(cls):
        return cls(temperature=0.0)

    @property
    def is_greedy(self) -> bool:
        return self.temperature < GREEDY_BELOW

    @property
    def has_penalties(self) -> bool:
        return (self.repetition_penalty != 1.0 or self.frequency_penalty != 0.0
                or self.presence_penalty != 0.0)

    def validate(self) -> None:
        if self.temperature < 0:
            raise ValueError("temperature must not be negative")
        if self.top_k < 0:
            raise ValueError("top_k must not be negative")
        if not 0.0 < self.top_p <= 1.0:
            raise ValueError("top_p must lie in (0, 1]")
        if self.repetition_penalty <= 0:
            raise ValueError("repetition_penalty must be positive")
        if self.penalty_window < 0:
            raise ValueError("penalty_window must not be negative")


def window_counts(context: list[int], window: int, vocab: int) -> tuple[list[int], list[int]]:
    """Distinct ids of the last `window` context tokens with their counts, in
    order of first appearance (src/sampler.cpp:55-74)."""
    counts: dict[int, int] = {}
    for t in context[max(0, len(context) - window):]:
        if 0 <= t < vocab:
            counts[t] = counts.get(t, 0) + 1
    return list(counts.keys()), list(counts.values())


class PendingIds:
    """Ids on their way to the host: wait() gives them once their copy has arrived."""

    def __init__(self, host: torch.Tensor, event):
        self._host = host
        self._event = event

    def wait(self) -> list[int]:
        if self._event is not None:
            self._event.synchronize()
        return self._host.tolist()


READS_IN_FLIGHT = 64
# The longest penalty window that is kept on the device for runs of queued steps (the kernel
# counts its distinct ids in a hash table in LDS, linear in the window); longer windows are
# counted on the host, step by step.
WINDOW_ON_DEVICE_MAX = ops.PENALTY_WINDOW_MAX


class Sampler:
    def __init__(self, config: SamplingConfig, device):
        config.validate()
        self.config = config
        self.device = device
        self._ring: list[torch.Tensor | None] = [None] * READS_IN_FLIGHT   # pinned rows for read_later
        self._ring_next = 0

    def read_later(self, ids: torch.Tensor) -> PendingIds:
        """Starts the copy of device ids (int32 [rows]) to pinned host memory without waiting
        for it; at most READS_IN_FLIGHT such reads may be outstanding."""
        i = self._ring_next
        self._ring_next = (i + 1) % READS_IN_FLIGHT
        n = ids.numel()
        if self._ring[i] is None or self._ring[i].numel() < n:
            self._ring[i] = torch.empty(max(256, n), dtype=torch.int32).pin_memory()
        host = self._ring[i][:n]
        host.copy_(ids, non_blocking=True)
        event = torch.cuda.Event()
        event.record()
        return PendingIds(host, event)

    def sample(self, logits: torch.Tensor, sequences: list[int], steps: list[int],
               contexts: list[list[int]] | None = None) -> list[int]:
        """logits: fp32 [rows, vocab] on the device; sequences[r] and steps[r] key
        the row's random draw; contexts[r] are the row's generated tokens so far.
        Returns the chosen ids (one device-to-host copy, which synchronises)."""
        return self.sample_device(logits, sequences, steps, contexts).tolist()

    def uniforms_device(self, sequences: list[int], steps: list[int], count: int) -> torch.Tensor:
        """The random draws of `count` successive steps of these rows (steps[r], steps[r] + 1, ...)
        on the device, int32 bits [count, rows]: one upload for a run of steps."""
        cfg = self.config
        u = np.array([[uniform_u32(cfg.seed, s, t + j) for s, t in zip(sequences, steps)]
                      for j in range(count)], dtype=np.uint32)
        return torch.from_numpy(u.view(np.int32)).to(self.device)

    @property
    def window_on_device(self) -> bool:
        """Whether the penalties of these options can run from a window kept on the device."""
        return self.config.has_penalties \
            and 1 <= self.config.penalty_window <= min(WINDOW_ON_DEVICE_MAX, ops.PENALTY_WINDOW_MAX)

    def window_device(self, contexts: list[list[int]]):
        """The penalty windows of these rows on the device, for a run of steps whose tokens stay
        there: (ring int32 [rows, W], appended int32 [rows]), or None when the options have no
        penalties (or a window the kernel does not take). One upload; sample_device then appends
        each step's ids itself."""
        cfg = self.config
        W = cfg.penalty_window
        if not self.window_on_device:
            return None
        rows = len(contexts)
        host = np.zeros((rows, W + 1), dtype=np.int32)
        for r, ctx in enumerate(contexts):
            last = ctx[max(0, len(ctx) - W):]
            host[r, :len(last)] = last          # oldest first: the next token overwrites the oldest
            host[r, W] = len(last)
        dev = torch.from_numpy(host).to(self.device)
        return dev[:, :W].contiguous(), dev[:, W].contiguous()

    def sample_device(self, logits: torch.Tensor, sequences: list[int], steps: list[int],
                      contexts: list[list[int]] | None = None,
                      uniforms: torch.Tensor | None = None, window=None,
                      last_ids: torch.Tensor | None = None) -> torch.Tensor:
        """The same, the ids left on the device (int32 [rows]). With `uniforms` (a row of
        uniforms_device) and no penalties nothing is copied or waited for. window: what
        window_device gave, in place of `contexts`; last_ids: the ids the step before sampled,
        which the window has not seen yet (they are appended first). The penalties then change
        `logits` itself."""
        cfg = self.config
        rows, V = logits.shape
        if window is not None:
            ops.apply_penalties_window(logits, rows, window[0], window[1], last_ids, cfg.repetition_penalty,
                                       cfg.frequency_penalty, cfg.presence_penalty)
        elif cfg.has_penalties and contexts is not None and any(contexts):
            ids, counts, offsets = [], [], [0]
            for ctx in contexts:
                i, c = window_counts(ctx, cfg.penalty_window, V)
                ids += i
                counts += c
                offsets.append(len(ids))
            packed = torch.tensor([ids + offsets, counts + [0] * len(offsets)], dtype=torch.int32)
            packed = packed.to(self.device)
            n = len(ids)
            logits = logits.clone()     # penalties work on a copy (src/sampler.cpp:126-139)
            ops.apply_penalties(logits, rows, packed[0, :n].contiguous(), packed[1, :n].contiguous(),
                                packed[0, n:].contiguous(), cfg.repetition_penalty,
                                cfg.frequency_penalty, cfg.presence_penalty)
        out = torch.empty(rows, dtype=torch.int32, device=self.device)
        if cfg.is_greedy:
            ops.argmax_rows(out, logits, rows)
        else:
            if uniforms is None:
                uniforms = self.uniforms_device(sequences, steps, 1)[0]
            ops.sample_rows(out, logits, rows, uniforms, cfg.temperature, cfg.top_k, cfg.top_p)
        return out
