"""The generation loop above the step function: batches of unequal prompts,
stop tokens, sequences that end earlier, and as many batches one after another
as there are requests.

Reference loop: prefill gives the first token; then, per token, stop checks,
record, sample the next (src/inference_session.cpp:597-660). A stop token ends
its sequence, is not fed back and is not part of the result (:611-615). Finish
reasons follow the reference's names (:59-67): "eos", "max_tokens", "stop"
(the sequence has filled its cache room; the reference stops at pos + 4 >=
max_seq, :616-619), "cancelled", and "context_full" for a request that is
refused at admission (:530-534).
"""
from __future__ import annotations

import dataclasses
import time
from typing import Callable


from ..cache.pages import blocks_for
from .engine import StepEntry


@dataclasses.dataclass
class GenerationResult:
    tokens: list[int]
    finish_reason: str
    prompt_tokens: int
    prefill_ms: float = 0.0
    decode_ms: float = 0.0


def plan_batch(pending: list[tuple[int, int]], max_new_tokens: int, free_pages: int,
               free_slots: int, max_seq_len: int, batch_size: int | None) -> tuple[list[int], list[int]]:
    """pending: (request index, prompt length) in order. Returns (admitted, refused)
    for the next batch: requests are admitted in order while slots and pages for
    prompt + max_new_tokens remain; a request that can never run is refused."""
    admitted, refused = [], []
    pages_left = free_pages
    limit = free_slots if batch_size is None else min(free_slots, batch_size)
    for idx, n in pending:
        if n < 1 or n + 1 > max_seq_len:
            refused.append(idx)
            continue
        need = blocks_for(min(n + max_new_tokens, max_seq_len))
        if need > free_pages and not admitted:
            refused.append(idx)          # would not fit even in an empty cache
            continue
        if len(admitted) >= limit or need > pages_left:
            break
        admitted.append(idx)
        pages_left -= need
    return admitted, refused


def after_token(token: int, generated: int, max_new_tokens: int, length: int, max_seq_len: int,
                stop_ids) -> tuple[bool, str | None]:
    """Decision after sampling `token` as the (generated+1)-th new token of a
    sequence whose cache holds `length` tokens. Returns (keep the token, finish
    reason or None to go on)."""
    if token in stop_ids:
        return False, "eos"
    if generated + 1 >= max_new_tokens:
        return True, "max_tokens"
    if length + 1 > max_seq_len:
        return True, "stop"              # no room to feed this token back
    return True, None


RUN_OF_STEPS = 8        # one-token steps queued ahead of the host's reading of their ids
LONGEST_RUN = 256       # steps after which a run of queued steps ends in any case


def generate(engine, prompts: list[list[int]], *, max_new_tokens: int = 100, sampling=None,
             stop_ids=None, include_stop: bool = False, batch_size: int | None = None,
             cancel: Callable[[], bool] | None = None, sample_fn=None, sampler=None,
             run_of_steps: int = RUN_OF_STEPS, on_token: Callable[[int, int], None] | None = None,
             on_prefill: Callable[[list[int], float], None] | None = None) -> list[GenerationResult]:
    """Generates for every prompt; returns results in the order of `prompts`.

    stop_ids: the token ids that end a sequence; None: the model's own (engine.stop_ids: the
    end-of-sequence ids of its generation_config.json or config.json), (): none.

    sampler: an object with the library Sampler's interface (config, sample, sample_device,
    uniforms_device, read_later) in place of one made from `sampling`; sample_fn: a plain
    function (logits, requests, steps, contexts) -> ids, which runs step by step.

    on_token(request index, token) is called for every token that becomes part of a result, in
    the order of each sequence (the reference hands text out as it comes through its on_text
    callback: src/inference_session.cpp:636-645; here the ids); with queued steps a token arrives
    when the host reads its step's ids, run_of_steps steps behind the queue. on_prefill(request indices, ms) is called
    once per batch after its prompt step (:603).

    run_of_steps: with a sampler, one-token steps are queued ahead of the host, each step's ids
    going into the next on the device (and into the penalty windows, which then live there for
    the run). The tokens are the same as step by step. When nothing can end a sequence inside a
    run but its token budget or its cache room (no stop ids, no `cancel`), the run never reaches
    past those, and the host reads a step's ids (and hands them to on_token) when
    run_of_steps - 1 further steps are queued behind it: the device does not wait for the host
    between steps. Otherwise the host reads the ids of a step while the next one runs, and
    queues nothing more once it has seen a stop token or `cancel` says so: a sequence that has
    sampled its stop token is stepped once more at most (the step that was already queued), then
    gives its slot back and leaves the batch. 1 or less: step by step."""
    from ..sampling import Sampler, SamplingConfig
    from ..sampling.sampler import READS_IN_FLIGHT
    if sample_fn is None:
        if sampler is None:
            sampler = Sampler(sampling or SamplingConfig.deterministic(), engine.device)
        sample_fn = sampler.sample
        if run_of_steps <= 1 or (sampler.config.has_penalties
                                 and not getattr(sampler, "window_on_device", False)):
            sampler = None          # step by step: each token on the host before the next
    else:
        sampler = None
    run_of_steps = min(run_of_steps, READS_IN_FLIGHT)
    if stop_ids is None:
        stop_ids = getattr(engine, "stop_ids", ())
    stop_ids = frozenset(int(s) for s in stop_ids)
    results: list[GenerationResult | None] = [None] * len(prompts)
    pending = [(i, len(p)) for i, p in enumerate(prompts)]
    if max_new_tokens < 1:
        return [GenerationResult([], "max_tokens", len(p)) for p in prompts]
    while pending:
        admitted, refused = plan_batch(pending, max_new_tokens, engine.cache.free_pages,
                                       engine.cache.book.slots.available, engine.max_seq_len,
                                       batch_size)
        for i in refused:
            results[i] = GenerationResult([], "context_full", len(prompts[i]))
        done = set(admitted) | set(refused)
        pending = [p for p in pending if p[0] not in done]
        if not admitted:
            if not refused:
                raise RuntimeError("the cache holds other sequences and no request fits beside them")
            continue
        _run_batch(engine, prompts, admitted, results, max_new_tokens, stop_ids, include_stop,
                   cancel, sample_fn, sampler, run_of_steps, on_token, on_prefill)
    return results


def steps_in_run(generated: list[int], lengths: list[int], max_new_tokens: int, max_seq_len: int,
                 run_of_steps: int) -> int:
    """How many one-token steps can be queued for sequences that have `generated` tokens (the
    one to feed included) and `lengths` cached tokens, so that none passes max_new_tokens or
    runs out of room whatever it samples: every step feeds one token and samples one."""
    room = min(max_seq_len - n for n in lengths)            # tokens that can still be fed
    budget = min(max_new_tokens - g for g in generated)     # tokens that may still be sampled
    return max(1, min(run_of_steps, room, budget))


def _run_of_steps(engine, sampler, slots: list[int], tokens: list[int], seqs: list[int],
                  steps: list[int], count: int, stop_ids=frozenset(), cancel=None,
                  contexts: list[list[int]] | None = None, ahead: int = RUN_OF_STEPS,
                  on_ids=None) -> list[list[int]]:
    """Feeds `tokens` and queues up to `count` one-token steps, each step's ids going into the
    next on the device; returns the sampled ids of the steps that ran, [steps][rows]. The host
    reads the ids of a step when `ahead` - 1 further steps have been queued behind it, so inside
    a run the device never waits for the host. With stop ids or `cancel`, the ids of step j are
    read while step j + 1 runs, and the run ends with the step that was queued when a stop token
    (or the cancellation) was seen. on_ids(j, ids) hands over the ids of step j once a later
    step's have been read: every step of the run but its last, whose ids the caller feeds next."""
    from ..sampling.sampler import READS_IN_FLIGHT
    # the penalty windows (the generated tokens, the ones fed now included) go to the device once
    window = sampler.window_device(contexts) if sampler.config.has_penalties and contexts is not None else None
    watch = bool(stop_ids) or cancel is not None
    depth = 1 if watch else max(1, min(ahead, READS_IN_FLIGHT) - 1)
    draws = max(1, ahead)          # random draws go up for so many steps at a time, while earlier steps run
    reads, ids, device_ids, uniforms = [], [], None, None

    def take() -> None:
        """Reads the oldest step not yet read."""
        ids.append(reads[len(ids)].wait())
        if on_ids is not None and len(ids) >= 2:
            on_ids(len(ids) - 2, ids[-2])

    for j in range(count):
        if not sampler.config.is_greedy and j % draws == 0:
            uniforms = sampler.uniforms_device(seqs, [t + j for t in steps], min(draws, count - j))
        entries = [StepEntry(s, [t], [0]) for s, t in zip(slots, tokens)]
        logits = engine.step(entries, device_tokens=device_ids)
        more = {} if window is None else {"window": window, "last_ids": device_ids}
        device_ids = sampler.sample_device(logits, seqs, [t + j for t in steps],
                                           uniforms=None if uniforms is None else uniforms[j % draws], **more)
        reads.append(sampler.read_later(device_ids))
        if j >= depth:
            take()
            if watch and (not stop_ids.isdisjoint(ids[-1]) or (cancel is not None and cancel())):
                break
    while len(ids) < len(reads):
        take()
    return ids


def _run_batch(engine, prompts, admitted, results, max_new_tokens, stop_ids, include_stop, cancel,
               sample_fn, sampler=None, run_of_steps: int = 1, on_token=None, on_prefill=None,
               held: dict[int, int] | None = None) -> None:
    """One batch from its prompt step to its last sequence's end. held: request -> a slot the
    caller holds and keeps (a session's turn: `prompts` then continue what the slots hold);
    without it the batch takes slots of its own and gives each back as its sequence ends."""
    slots = dict(held) if held is not None else {i: engine.acquire() for i in admitted}
    out: dict[int, list[int]] = {i: [] for i in admitted}
    t0 = time.perf_counter()
    try:
        logits = engine.step([StepEntry(slots[i], prompts[i], [len(prompts[i]) - 1]) for i in admitted])
        active = list(admitted)
        tokens = sample_fn(logits, active, [0] * len(active), [out[i] for i in active])
        prefill_ms = (time.perf_counter() - t0) * 1e3
        if on_prefill is not None:
            on_prefill(list(admitted), prefill_ms)
        t1 = time.perf_counter()

        def finish(i, reason):
            results[i] = GenerationResult(out[i], reason, len(prompts[i]), prefill_ms,
                                          (time.perf_counter() - t1) * 1e3)
            slot = slots.pop(i)
            if held is None:
                engine.release(slot)         # the slot goes back at once

        def decide(i, tok, length) -> bool:
            """Records a sampled token of request i whose cache held `length` tokens when it was
            sampled; True if the sequence goes on (the token is then to be fed)."""
            keep, reason = after_token(tok, len(out[i]), max_new_tokens, length, engine.max_seq_len, stop_ids)
            if keep or include_stop:
                out[i].append(tok)
                if on_token is not None:
                    on_token(i, tok)
            if reason is not None:
                finish(i, reason)
            return reason is None

        while active:
            if cancel is not None and cancel():
                for i in active:
                    finish(i, "cancelled")
                break
            feed = [(i, tok) for i, tok in zip(active, tokens) if decide(i, tok, engine.length(slots[i]))]
            active = [i for i, _ in feed]
            if not active:
                break
            count = 1 if sampler is None else steps_in_run(
                [len(out[i]) for i in active], [engine.length(slots[i]) for i in active],
                max_new_tokens, engine.max_seq_len, LONGEST_RUN)
            if count == 1:
                logits = engine.step([StepEntry(slots[i], [tok], [0]) for i, tok in feed])
                tokens = sample_fn(logits, active, [len(out[i]) for i in active], [out[i] for i in active])
                continue
            # all but the last step of the run are decided as their ids are read, each with the cache
            # length of its moment; a sequence that ends inside the run drops the rest of its ids
            before = {i: engine.length(slots[i]) for i in active}
            going = dict.fromkeys(active, True)
            row_of = list(active)

            def decide_step(j, row):
                for col, i in enumerate(row_of):
                    if going[i]:
                        going[i] = decide(i, row[col], before[i] + j + 1)

            run = _run_of_steps(engine, sampler, [slots[i] for i in active], [tok for _, tok in feed],
                                active, [len(out[i]) for i in active], count, stop_ids, cancel,
                                [out[i] for i in active], run_of_steps, decide_step)
            tokens = [run[-1][col] for col, i in enumerate(active) if going[i]]
            active = [i for i in active if going[i]]
    finally:
        for i in list(slots):
            slot = slots.pop(i)
            if held is None:
                engine.release(slot)
