"""The generation loop's decisions, with a fake engine on the CPU: admission,
batches one after another, stop tokens, sequences that end earlier and give
their slot back at once, the token budget and the cache-room stop."""
import pytest

import hector_engine_amd  # noqa: F401
from hector_engine_amd.cache import GroupPages, SlotBook
from hector_engine_amd.engine.generate import after_token, generate, plan_batch, steps_in_run

V = 50


class FakeCache:
    def __init__(self, pages, slots, max_blocks):
        self.book = SlotBook(slots, max_blocks, [GroupPages(pages, 0, "0")])

    @property
    def free_pages(self):
        return self.book.groups[0].pool.available


class FakeEngine:
    """next token of a sequence = (sum of its tokens + its length) % V."""

    device = "cpu"

    def __init__(self, pages=16, slots=3, max_blocks=4):
        self.cache = FakeCache(pages, slots, max_blocks)
        self.max_seq_len = max_blocks * 64
        self.history = {}
        self.log = []          # (slots in the step, tokens per slot)
        self.max_live = 0

    def acquire(self):
        s = self.cache.book.acquire()
        self.history[s] = []
        self.max_live = max(self.max_live, len(self.history))
        return s

    def release(self, s):
        self.cache.book.release(s)
        del self.history[s]

    def length(self, s):
        return self.cache.book.length[s]

    def truncate(self, s, length):
        self.cache.book.truncate(s, length)
        del self.history[s][length:]

    def step(self, entries, device_tokens=None):
        """device_tokens: as the engine takes them, the tokens of a one-token step in place of
        the entries' own (here a plain list: the fake has no device)."""
        self.log.append([(e.slot, len(e.tokens)) for e in entries])
        rows = []
        for k, e in enumerate(entries):
            new = self.length(e.slot) + len(e.tokens)
            self.cache.book.reserve(e.slot, new)
            self.cache.book.commit(e.slot, new)
            self.history[e.slot] += list(e.tokens) if device_tokens is None else [device_tokens[k]]
            if not e.want:
                continue
            assert list(e.want) == [len(e.tokens) - 1]
            h = self.history[e.slot]
            rows.append((sum(h) + len(h)) % V)
        self.cache.book.check_invariants()
        return rows


def pick(rows, sequences, steps, contexts):
    return list(rows)


class FakeSampler:
    """The library sampler's interface without a device: ids are plain lists, and a read of
    them is ready at once. `reads` counts how often the loop looked at a step's ids."""

    def __init__(self):
        from hector_engine_amd.sampling import SamplingConfig
        self.config = SamplingConfig.deterministic()
        self.waits = 0

    def sample(self, rows, sequences, steps, contexts=None):
        return list(rows)

    def sample_device(self, rows, sequences, steps, contexts=None, uniforms=None):
        return list(rows)

    def read_later(self, ids):
        outer = self

        class Ready:
            def wait(self):
                outer.waits += 1
                return list(ids)
        return Ready()


def expected(prompt, n, stop=()):
    h, out = list(prompt), []
    for _ in range(n):
        t = (sum(h) + len(h)) % V
        if t in stop:
            return out, "eos"
        out.append(t)
        h.append(t)
    return out, "max_tokens"


def test_plan_batch():
    # slots limit, page limit, refusals
    assert plan_batch([(0, 10), (1, 20), (2, 30)], 5, 100, 2, 256, None) == ([0, 1], [])
    assert plan_batch([(0, 10), (1, 20), (2, 30)], 5, 100, 3, 256, 2) == ([0, 1], [])
    assert plan_batch([(0, 100), (1, 100)], 60, 3, 8, 256, None) == ([0], [])      # 3 pages: one request of 160
    assert plan_batch([(0, 0), (1, 256), (2, 5)], 5, 100, 8, 256, None) == ([2], [0, 1])
    assert plan_batch([(0, 200)], 100, 2, 8, 256, None) == ([], [0])               # never fits
    # room is counted up to max_seq_len only
    assert plan_batch([(0, 250)], 100, 4, 8, 256, None) == ([0], [])


def test_after_token():
    assert after_token(7, 0, 5, 10, 64, {7}) == (False, "eos")
    assert after_token(3, 4, 5, 10, 64, {7}) == (True, "max_tokens")
    assert after_token(3, 0, 5, 64, 64, {7}) == (True, "stop")
    assert after_token(3, 0, 5, 63, 64, {7}) == (True, None)


def test_unequal_prompts_stop_tokens_and_early_finishers():
    eng = FakeEngine()
    prompts = [[1, 2, 3], [4] * 9, [7, 7, 7, 7, 7]]
    stop = {expected(prompts[1], 3)[0][2]}            # the third token of request 1 is a stop token
    res = generate(eng, prompts, max_new_tokens=6, stop_ids=stop, sample_fn=pick)
    for p, r in zip(prompts, res):
        want, reason = expected(p, 6, stop)
        assert r.tokens == want and r.finish_reason == reason and r.prompt_tokens == len(p)
    assert res[1].finish_reason == "eos" and len(res[1].tokens) == 2
    # the first step holds all prompts; after request 1 ended the steps hold two sequences
    assert [n for _, n in eng.log[0]] == [3, 9, 5]
    sizes = [len(step) for step in eng.log[1:]]
    assert sizes[:2] == [3, 3] and set(sizes[2:]) == {2}
    assert eng.cache.book.slots.available == 3 and eng.cache.free_pages == 16 and not eng.history


def test_more_requests_than_slots_run_batch_after_batch():
    eng = FakeEngine(slots=2)
    prompts = [[i + 1] * (i + 2) for i in range(5)]
    res = generate(eng, prompts, max_new_tokens=4, sample_fn=pick)
    for p, r in zip(prompts, res):
        assert (r.tokens, r.finish_reason) == expected(p, 4)
    assert eng.max_live == 2
    firsts = [step for step in eng.log if any(n > 1 for _, n in step)]
    assert [len(s) for s in firsts] == [2, 2, 1]       # three batches
    assert {s for step in eng.log for s, _ in step} == {0, 1}          # slots are used again


def test_include_stop_and_refusals_and_cache_room():
    eng = FakeEngine(max_blocks=1)                     # 64 positions per sequence
    p = [3, 1, 4]
    stop = {expected(p, 2)[0][1]}
    r = generate(eng, [p], max_new_tokens=5, stop_ids=stop, include_stop=True, sample_fn=pick)[0]
    assert r.finish_reason == "eos" and r.tokens == expected(p, 2)[0]
    long = [1] * 64
    r = generate(eng, [long, [2] * 60], max_new_tokens=10, sample_fn=pick)
    assert r[0].finish_reason == "context_full" and r[0].tokens == []
    want, _ = expected([2] * 60, 5)                    # 60 + 4 fed tokens fill the 64 positions
    assert r[1].finish_reason == "stop" and r[1].tokens == want
    assert eng.cache.book.slots.available == 3


def test_cancel_and_zero_budget():
    eng = FakeEngine()
    calls = {"n": 0}

    def cancel():
        calls["n"] += 1
        return calls["n"] > 2

    r = generate(eng, [[1, 2]], max_new_tokens=50, cancel=cancel, sample_fn=pick)[0]
    assert r.finish_reason == "cancelled" and len(r.tokens) == 2
    assert eng.cache.book.slots.available == 3
    assert generate(eng, [[1]], max_new_tokens=0, sample_fn=pick)[0].finish_reason == "max_tokens"


def test_slots_are_released_when_a_step_fails():
    eng = FakeEngine()

    def boom(rows, *a):
        raise RuntimeError("sampler failed")

    with pytest.raises(RuntimeError, match="sampler failed"):
        generate(eng, [[1, 2], [3]], max_new_tokens=3, sample_fn=boom)
    assert eng.cache.book.slots.available == 3 and eng.cache.free_pages == 16


def test_steps_in_run():
    """How many steps may be queued before the host sees a token: never past the token budget of
    any sequence, never past the room in its cache, at least one."""
    assert steps_in_run([1, 1], [10, 20], 100, 256, 8) == 8
    assert steps_in_run([1, 95], [10, 20], 100, 256, 8) == 5          # 5 more tokens may be sampled
    assert steps_in_run([1, 1], [10, 253], 100, 256, 8) == 3          # 3 more tokens can be fed
    assert steps_in_run([99], [10], 100, 256, 8) == 1
    assert steps_in_run([3], [256], 100, 256, 8) == 1                 # the loop ends such a sequence before
    assert steps_in_run([1], [10], 100, 256, 1) == 1


def test_a_stop_token_inside_a_run_of_queued_steps():
    """Three requests through two slots, eight steps queued at a time. Request 0 samples its stop
    token as its second token, early in a run: it is stepped once more at most (the step that was
    queued when the host read the token), then its slot and pages are back and the batch goes on
    without it; the waiting request starts when that batch has ended, in the slots it gave back;
    every result equals one step at a time."""
    prompts = [[1, 2, 3], [4] * 9, [7, 7, 7, 7, 7]]
    stop = {expected(prompts[0], 2)[0][1]}            # the second token of request 0
    assert all(t not in stop for p in prompts[1:] for t in expected(p, 12)[0])
    one = generate(FakeEngine(slots=2), prompts, max_new_tokens=12, stop_ids=stop, sampler=FakeSampler(),
                   run_of_steps=1)
    eng = FakeEngine(slots=2)
    many = generate(eng, prompts, max_new_tokens=12, stop_ids=stop, sampler=FakeSampler(), run_of_steps=8)
    assert [(r.tokens, r.finish_reason) for r in many] == [(r.tokens, r.finish_reason) for r in one]
    assert many[0].finish_reason == "eos" and len(many[0].tokens) == 1
    assert [(r.tokens, r.finish_reason) for r in many[1:]] == [expected(p, 12) for p in prompts[1:]]
    # step 0: both prompts. Request 0's first token is fed in step 1, which samples the stop token;
    # step 2 was queued before the host read it; from step 3 on request 1 runs alone.
    first_batch = [step for step in eng.log[:1 + 11]]
    assert [n for _, n in first_batch[0]] == [3, 9]
    assert [len(step) for step in first_batch[1:]] == [2, 2] + [1] * 9
    # the third request starts right after, alone, in the lowest slot
    assert eng.log[12] == [(0, 5)] and all(len(step) == 1 for step in eng.log[12:])
    assert len(eng.log) == 12 + 12
    assert eng.cache.book.slots.available == 2 and eng.cache.free_pages == 16 and not eng.history


def test_runs_without_stop_ids_read_their_ids_once():
    """Nothing can end a sequence inside a run but its budget: the run is never cut and reaches
    exactly to the budget."""
    eng, sampler = FakeEngine(), FakeSampler()
    prompts = [[1, 2, 3], [5, 5]]
    res = generate(eng, prompts, max_new_tokens=11, sampler=sampler, run_of_steps=8)
    assert [(r.tokens, r.finish_reason) for r in res] == [expected(p, 11) for p in prompts]
    assert len(eng.log) == 1 + 10            # the prompt step and ten one-token steps, none wasted
    assert eng.cache.book.slots.available == 3


def test_the_host_reads_ids_a_fixed_number_of_steps_behind_the_queue():
    """Without stop ids one run reaches to the budget, far beyond run_of_steps; the host has read
    (and handed out) the ids of step j by the time step j + run_of_steps is queued, and never
    looks at a step's ids before run_of_steps - 1 further steps are queued behind it: the device
    has work queued while the host waits. With stop ids the host is one step behind."""
    for ahead, stop in ((8, ()), (3, ()), (8, {(1 + 2 + 2) % V + 99})):       # the last: a stop id that never comes
        eng, sampler = FakeEngine(), FakeSampler()
        seen_at_step = []                 # tokens handed out when one-token step k was queued
        handed = []
        step = eng.step

        def logged_step(entries, device_tokens=None):
            if all(len(e.tokens) == 1 for e in entries):
                seen_at_step.append(len(handed))
            return step(entries, device_tokens)

        eng.step = logged_step
        r = generate(eng, [[1, 2]], max_new_tokens=40, sampler=sampler, run_of_steps=ahead,
                     stop_ids=stop, on_token=lambda i, tok: handed.append(tok))[0]
        assert (r.tokens, r.finish_reason) == expected([1, 2], 40) and handed == r.tokens
        assert len(seen_at_step) == 39     # one run: the prompt step gave the first token, none wasted
        lag = 2 if stop else ahead
        for k, n in enumerate(seen_at_step):
            # token 0 came from the prompt step; step k samples token k + 1. The loop hands a step's ids
            # out once the next step's ids are read, hence one step more than the reading itself.
            assert n >= min(1, k + 1) + max(0, k - lag), (k, n)
            assert n <= 1 + max(0, k - (1 if stop else ahead - 1)), (k, n)
        assert sampler.waits == 39


def test_cancel_is_seen_inside_a_run():
    eng = FakeEngine()
    calls = {"n": 0}

    def cancel():
        calls["n"] += 1
        return calls["n"] > 3

    r = generate(eng, [[1, 2]], max_new_tokens=50, cancel=cancel, sampler=FakeSampler(), run_of_steps=8)[0]
    assert r.finish_reason == "cancelled" and 1 <= len(r.tokens) <= 5
    assert r.tokens == expected([1, 2], len(r.tokens))[0]
    assert eng.cache.book.slots.available == 3 and eng.cache.free_pages == 16


def test_tokens_are_handed_out_as_they_come():
    """on_token sees every token of every result, per sequence in order and nothing else (a stop
    token only with include_stop); on_prefill once per batch with its requests. Step by step and
    with queued runs alike."""
    prompts = [[1, 2, 3], [4] * 9, [7, 7, 7, 7, 7]]
    stop = {expected(prompts[1], 3)[0][2]}
    for include_stop in (False, True):
        for kwargs in (dict(sample_fn=pick), dict(sampler=FakeSampler(), run_of_steps=8)):
            seen = {i: [] for i in range(3)}
            batches = []
            res = generate(FakeEngine(slots=2), prompts, max_new_tokens=6, stop_ids=stop,
                           include_stop=include_stop, on_token=lambda i, t: seen[i].append(t),
                           on_prefill=lambda ids, ms: batches.append(ids), **kwargs)
            assert [seen[i] for i in range(3)] == [r.tokens for r in res]
            assert (res[1].tokens[-1] in stop) == include_stop
            assert batches == [[0, 1], [2]]


def test_a_session_continues_its_slot_turn_after_turn():
    """Turns of a session against one long run: the second turn sees the first turn's tokens, the
    generated ones and the token that ended the first turn under its budget (sampled, not yet
    fed: it goes in front of the second turn's tokens). Step by step and with queued runs."""
    from hector_engine_amd.engine.session import Session
    p1, p2 = [1, 2, 3], [9, 8]
    for run_of_steps in (1, 8):
        eng = FakeEngine()
        with Session(eng, stop_ids=(), make_sampler=lambda config: FakeSampler()) as ses:
            assert ses.feed(p1[:2]) and ses.position == 2 and not ses.feed([1] * 300) and ses.position == 2
            r1 = ses.turn(p1[2:], 5, run_of_steps=run_of_steps)
            assert (r1.tokens, r1.finish_reason) == expected(p1, 5) and r1.prompt_tokens == 1
            assert ses.position == 3 + 4 and ses.unfed == [r1.tokens[-1]]
            r2 = ses.turn(p2, 6, run_of_steps=run_of_steps)
            assert (r2.tokens, r2.finish_reason) == expected(p1 + r1.tokens + p2, 6) and r2.prompt_tokens == 3
            assert eng.history[ses.slot] == p1 + r1.tokens + p2 + r2.tokens[:-1]
            seen = []
            r3 = ses.turn([4], 3, on_token=seen.append, run_of_steps=run_of_steps)
            assert seen == r3.tokens == expected(p1 + r1.tokens + p2 + r2.tokens + [4], 3)[0]
            assert ses.turns == 3 and eng.cache.book.slots.available == 2
        assert eng.cache.book.slots.available == 3 and eng.cache.free_pages == 16 and not eng.history


def test_a_session_takes_back_what_a_late_read_stop_token_fed():
    """With queued steps the stop token is read while the next step, which feeds it, is already
    queued. A session keeps its slot, so that step is taken back: the slot holds the turn's tokens
    and the generated ones before the stop token, and the next turn continues from there."""
    from hector_engine_amd.engine.session import Session
    p1 = [1, 2, 3]
    stop = {expected(p1, 3)[0][2]}                     # the third token of the first turn
    eng = FakeEngine()
    ses = Session(eng, stop_ids=stop, make_sampler=lambda config: FakeSampler())
    r1 = ses.turn(p1, 12, run_of_steps=8)
    assert (r1.tokens, r1.finish_reason) == expected(p1, 12, stop) and len(r1.tokens) == 2
    assert eng.history[ses.slot] == p1 + r1.tokens and ses.position == 5 and ses.unfed == []
    assert max(len(step) for step in eng.log) == 1 and len(eng.log) == 1 + 3      # the prompt, two tokens, the surplus step
    r2 = ses.turn([7], 4, run_of_steps=8)
    assert r2.tokens == expected(p1 + r1.tokens + [7], 4, stop)[0]
    # include_stop: the stop token is part of the result and still not fed
    ses.reset()
    r = ses.turn(p1, 12, include_stop=True, run_of_steps=8)
    assert r.tokens[:-1] == r1.tokens and r.tokens[-1] in stop and eng.history[ses.slot] == p1 + r1.tokens
    ses.close()
    assert eng.cache.book.slots.available == 3 and eng.cache.free_pages == 16
    with pytest.raises(RuntimeError, match="closed"):
        ses.turn([1])


def test_a_session_refuses_a_turn_without_room_and_takes_a_failed_turn_back():
    from hector_engine_amd.engine.session import Session
    eng = FakeEngine(max_blocks=1)                      # 64 positions
    ses = Session(eng, stop_ids=(), make_sampler=lambda config: FakeSampler())
    ses.turn([1] * 40, 4, run_of_steps=1)
    at = ses.position
    held = list(eng.history[ses.slot])
    r = ses.turn([2] * 30, 4)
    assert r.finish_reason == "context_full" and r.tokens == [] and ses.position == at and eng.history[ses.slot] == held
    with pytest.raises(ValueError, match="empty turn"):
        Session(eng, stop_ids=(), make_sampler=lambda config: FakeSampler()).turn([])
    # the step after the turn's third fails: the slot holds again what it held before the turn
    calls = {"n": 0}
    step = eng.step

    def failing(entries, device_tokens=None):
        calls["n"] += 1
        if calls["n"] == 3:
            raise RuntimeError("boom")
        return step(entries, device_tokens)
    eng.step = failing
    unfed = list(ses.unfed)
    with pytest.raises(RuntimeError, match="boom"):
        ses.turn([3, 4], 6, run_of_steps=1)
    assert ses.position == at and eng.history[ses.slot] == held and ses.unfed == unfed
    eng.step = step
    r = ses.turn([3, 4], 2, run_of_steps=1)
    assert r.tokens == expected(held + unfed + [3, 4], 2)[0]
    # the room ends inside a turn: "stop", and the next turn is refused
    r = ses.turn([5] * 8, 40, run_of_steps=1)
    assert r.finish_reason == "stop" and ses.position == 64 and len(ses.unfed) == 1
    assert ses.turn([1], 2).finish_reason == "context_full"
