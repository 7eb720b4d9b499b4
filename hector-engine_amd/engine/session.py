"""A conversation in one slot of the cache: each turn's tokens continue what the slot holds.

The reference's session runs turn after turn against one cache (InferenceSession::run_turn,
src/inference_session.cpp:495-699): it notes the position before the turn (:513), refuses a turn
that does not fit with "context_full" and touches nothing (:530-534), builds the sampling
configuration anew for every turn (:538), and takes a turn back that failed before it gave
anything out (rewind, :682-693; src/kv_cache.hpp:93-96); reset() empties the cache (:321-324).
Here a turn is token ids in and token ids out: what closes a turn (a template's end-of-turn
tokens, :665-676) is the caller's and goes in with the next turn's tokens.
"""
from __future__ import annotations

import dataclasses
from typing import Callable

from ..cache import CacheError
from .generate import RUN_OF_STEPS, GenerationResult, _run_batch


class Session:
    """Holds one slot of `engine` from its construction to close().

    turn(tokens) feeds the tokens behind everything the slot holds and generates; the slot then
    holds the turn's tokens and the generated ones that were fed back. A token that ended the
    turn under its budget was sampled but not fed: it is kept and goes in front of the next turn's
    tokens, so that the next turn sees everything the caller has seen (:651-653)."""

    def __init__(self, engine, sampling=None, stop_ids=None, make_sampler=None):
        """make_sampler(config) -> an object with the library Sampler's interface, in place of
        Sampler(config, engine.device)."""
        from ..sampling import SamplingConfig
        self.engine = engine
        self.make_sampler = make_sampler
        self.sampling = sampling or SamplingConfig.deterministic()
        self.stop_ids = frozenset(int(t) for t in (getattr(engine, "stop_ids", ()) if stop_ids is None else stop_ids))
        self.slot: int | None = engine.acquire()
        self.unfed: list[int] = []
        self.turns = 0

    @property
    def position(self) -> int:
        """Tokens the slot holds."""
        return self.engine.length(self._slot())

    def _slot(self) -> int:
        if self.slot is None:
            raise RuntimeError("the session is closed")
        return self.slot

    def turn(self, tokens: list[int], max_new_tokens: int = 100, *, sampling=None, include_stop: bool = False,
             cancel: Callable[[], bool] | None = None, on_token: Callable[[int], None] | None = None,
             run_of_steps: int = RUN_OF_STEPS) -> GenerationResult:
        """One turn. sampling: this turn's configuration in place of the session's. A turn that does
        not fit into the slot's remaining room is refused ("context_full", nothing touched); a turn
        that fails is taken back (the slot holds what it held before) and the error raised."""
        engine, slot = self.engine, self._slot()
        feed = self.unfed + [int(t) for t in tokens]
        if not feed:
            raise ValueError("an empty turn: no tokens to feed")
        before = engine.length(slot)
        if max_new_tokens < 1 or before + len(feed) + 1 > engine.max_seq_len:
            reason = "max_tokens" if max_new_tokens < 1 else "context_full"
            return GenerationResult([], reason, len(feed))
        config = sampling or self.sampling
        # every turn draws its own random numbers: the same seed would repeat the first turn's
        config = dataclasses.replace(config, seed=config.seed + self.turns)
        if self.make_sampler is not None:
            sampler = self.make_sampler(config)
        else:
            from ..sampling import Sampler
            sampler = Sampler(config, engine.device)
        # Step by step where a queued step could not be taken back: a stop token read late has been
        # fed by the step queued behind it, and a group that keeps a window may have given a page away
        # by then.
        windowed = any(g.window > 0 for g in engine.cache.book.groups)
        stepwise = run_of_steps <= 1 or (config.has_penalties and not getattr(sampler, "window_on_device", False)) \
            or (windowed and bool(self.stop_ids))
        results: list[GenerationResult | None] = [None]
        try:
            _run_batch(engine, [feed], [0], results, max_new_tokens, self.stop_ids, include_stop, cancel,
                       sampler.sample, None if stepwise else sampler, run_of_steps,
                       None if on_token is None else (lambda _i, tok: on_token(tok)), None, held={0: slot})
            result = results[0]
            # the generated tokens that were fed back: all but one that ended the turn unfed
            last_unfed = result.finish_reason in ("max_tokens", "stop") or (
                result.finish_reason == "eos" and include_stop)
            kept = before + len(feed) + len(result.tokens) - (1 if last_unfed and result.tokens else 0)
            if engine.length(slot) > kept:
                # a step that was queued when the stop token was read has fed it: taken back
                engine.truncate(slot, kept)
        except BaseException:
            self._take_back(before)
            raise
        self.unfed = [result.tokens[-1]] if result.finish_reason in ("max_tokens", "stop") and result.tokens else []
        self.turns += 1
        return result

    def feed(self, tokens: list[int]) -> bool:
        """Puts tokens behind what the slot holds without generating (a system prompt, a turn of the
        other side). False, with nothing touched, if they do not fit."""
        from .engine import StepEntry
        engine, slot = self.engine, self._slot()
        feed = self.unfed + [int(t) for t in tokens]
        if not feed:
            return True
        before = engine.length(slot)
        if before + len(feed) > engine.max_seq_len:
            return False
        try:
            engine.step([StepEntry(slot, feed, [])])
        except BaseException:
            self._take_back(before)
            raise
        self.unfed = []
        return True

    def _take_back(self, length: int) -> None:
        try:
            self.engine.truncate(self.slot, length)
        except (CacheError, RuntimeError):
            # a cache that cannot be cut back (a window's pages given away, state per sequence):
            # the session starts again empty rather than hold half a turn
            self.reset()

    def rewind(self, length: int) -> None:
        """The slot keeps its first `length` tokens (Engine.truncate)."""
        self.engine.truncate(self._slot(), length)
        self.unfed = []

    def reset(self) -> None:
        """Forgets everything: a fresh slot."""
        self.engine.release(self._slot())
        self.slot = self.engine.acquire()
        self.unfed = []

    def close(self) -> None:
        if self.slot is not None:
            self.engine.release(self.slot)
            self.slot = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()
