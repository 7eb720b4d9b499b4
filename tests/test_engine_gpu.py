"""The engine against the plain implementation on the GPU, in 32-bit and in
bfloat16, for three tiny configurations: each request alone and whole; the last
32 tokens one by one; batches of unequal lengths whose shorter requests end
earlier, one batch after another so that slots are used again; long decoding;
the first tokens of a sequence; and that cutting, batching, padding and slot
numbers change nothing."""
import pytest
import torch

from tests.conftest import TINY
from tests.helpers import argmax_agrees_where_clear, close, rand_ids
from tests.plain import qwen2_plain as P

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]
NAMES = list(TINY)


@pytest.fixture(scope="module")
def engines(model_dirs):
    import hector_engine_amd as he
    cache = {}

    def get(name, dtype, **kw):
        key = (name, dtype, tuple(sorted(kw.items())))
        if key not in cache:
            opts = dict(max_tokens=4096, max_slots=8, max_seq_len=1024, beyond_max_positions=True)
            opts.update(kw)
            cache[key] = he.Engine(model_dirs[name], dtype=dtype, **opts)
        return cache[key]

    return get


def entry(slot, tokens, want):
    from hector_engine_amd.engine.engine import StepEntry
    return StepEntry(slot, list(tokens), list(want))


def plain_logits(plain_models, name, ids):
    cfg, w = plain_models[name]
    return P.forward(cfg, w, ids)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_each_request_alone_and_whole(engines, plain_models, name, dtype):
    eng = engines(name, dtype)
    vocab = plain_models[name][0]["vocab_size"]
    for seed, n in enumerate([1, 2, 13, 64, 65, 150]):
        ids = rand_ids(vocab, n, seed)
        s = eng.acquire()
        got = eng.step([entry(s, ids, range(n))])
        want = plain_logits(plain_models, name, ids)
        close(got, want, dtype)
        argmax_agrees_where_clear(got, want, 0.05 * want.abs().max().item())
        eng.release(s)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_last_32_tokens_one_by_one(engines, plain_models, name, dtype):
    eng = engines(name, dtype)
    vocab = plain_models[name][0]["vocab_size"]
    n = 200 if name == "C" else 100
    ids = rand_ids(vocab, n, 7)
    want = plain_logits(plain_models, name, ids)
    s = eng.acquire()
    whole = eng.step([entry(s, ids, range(n))]).clone()
    eng.release(s)
    s = eng.acquire()
    assert eng.step([entry(s, ids[:n - 32], [])]) is None
    rows = [eng.step([entry(s, [t], [0])]).clone() for t in ids[n - 32:]]
    eng.release(s)
    dec = torch.cat(rows)
    close(dec, want[n - 32:], dtype)
    if dtype == "float32":
        assert torch.equal(dec, whole[n - 32:])       # the 32-bit path does not depend on the cut
    else:
        close(dec, whole[n - 32:].cpu(), dtype)


def run_batches(eng, requests, batch_sizes):
    """requests: token lists. Batches of the given sizes run one after another; in a batch
    all prompts (the first half of each request, at least one token) go in one step, then
    every request feeds its own next given token each step; a request whose tokens are
    used up leaves the batch and gives its slot back. Returns each request's logits at
    all positions, and the slots used."""
    out = {i: [] for i in range(len(requests))}
    used = []
    nxt = 0
    for bs in batch_sizes:
        batch = list(range(nxt, min(nxt + bs, len(requests))))
        nxt += bs
        slots = {i: eng.acquire() for i in batch}
        used += list(slots.values())
        fed = {i: max(1, len(requests[i]) // 2) for i in batch}
        logits = eng.step([entry(slots[i], requests[i][:fed[i]], range(fed[i])) for i in batch])
        r = 0
        for i in batch:
            out[i].append(logits[r:r + fed[i]].clone())
            r += fed[i]
        live = list(batch)
        while True:
            for i in list(live):
                if fed[i] == len(requests[i]):
                    eng.release(slots.pop(i))
                    live.remove(i)
            if not live:
                break
            logits = eng.step([entry(slots[i], [requests[i][fed[i]]], [0]) for i in live])
            for r, i in enumerate(live):
                out[i].append(logits[r:r + 1].clone())
                fed[i] += 1
    return {i: torch.cat(v) for i, v in out.items()}, used


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_unequal_batches_early_finishers_and_slot_reuse(engines, plain_models, name, dtype):
    eng = engines(name, dtype, max_slots=4)
    vocab = plain_models[name][0]["vocab_size"]
    lengths = [6, 18, 26, 3, 14, 34, 60, 9, 130, 2]
    requests = [rand_ids(vocab, n, 20 + i) for i, n in enumerate(lengths)]
    got, used = run_batches(eng, requests, [3, 4, 3])
    assert set(used) <= {0, 1, 2, 3} and len(used) == 10          # four slots serve ten requests
    for i, ids in enumerate(requests):
        close(got[i], plain_logits(plain_models, name, ids), dtype)
    assert eng.cache.book.slots.available == 4 and eng.cache.free_pages == eng.cache.num_pages
    eng.cache.book.check_invariants()
    if dtype == "float32":
        # each request alone gives the same bits as in its batch
        for i in (0, 5, 8):
            s = eng.acquire()
            alone = eng.step([entry(s, requests[i], range(len(requests[i])))]).clone()
            eng.release(s)
            assert torch.equal(alone, got[i])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_a_batch_of_a_hundred_unequal_requests(engines, plain_models, name, dtype):
    """A hundred requests of 2 to 60 tokens in one batch: as they end, the one-token steps shrink from
    a hundred rows through every range of rows that has kernels and graphs of its own (above 64,
    33 to 64, 17 to 32, up to 16), and every request's logits still equal the plain implementation's."""
    eng = engines(name, dtype, max_slots=100, max_tokens=100 * 64)
    vocab = plain_models[name][0]["vocab_size"]
    g = torch.Generator().manual_seed(5)
    lengths = torch.randint(2, 61, (100,), generator=g).tolist()
    lengths[7], lengths[50] = 60, 60            # some last to the end
    requests = [rand_ids(vocab, n, 300 + i) for i, n in enumerate(lengths)]
    got, used = run_batches(eng, requests, [100])
    assert sorted(used) == list(range(100))
    for i, ids in enumerate(requests):
        close(got[i], plain_logits(plain_models, name, ids), dtype)
    assert eng.cache.book.slots.available == 100 and eng.cache.free_pages == eng.cache.num_pages
    eng.cache.book.check_invariants()


def test_random_configurations(tmp_path):
    """Forty random configurations of the architecture (head sizes 16 to 256, any head and group counts, widths
    and vocabularies of any size, 1 to 3 layers, tied or not, windows from any layer on): model folders with
    random weights, prompts of unequal lengths in one step and then token by token, in 32-bit and in bfloat16,
    against the plain implementation."""
    import random
    import hector_engine_amd as he
    from hector_engine_amd.registry import config_from_dict
    rng = random.Random(6)
    for case in range(40):
        hd, KVH = rng.choice([16, 32, 48, 64, 64, 80, 96, 128, 128, 256]), rng.randint(1, 4)
        H, L = KVH * rng.randint(1, 7), rng.randint(1, 3)
        cfg = {"architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "num_hidden_layers": L,
               "hidden_size": rng.choice([8 * rng.randint(2, 40), rng.randint(16, 300)]), "num_attention_heads": H,
               "num_key_value_heads": KVH, "head_dim": hd,
               "intermediate_size": rng.choice([8 * rng.randint(1, 60), rng.randint(8, 400)]),
               "vocab_size": rng.randint(20, 700), "rope_theta": rng.choice([1e4, 1e6, 5e4]),
               "rms_norm_eps": rng.choice([1e-6, 1e-5, 3e-6]), "max_position_embeddings": 512,
               "tie_word_embeddings": rng.random() < 0.5, "use_sliding_window": rng.random() < 0.5, "hidden_act": "silu"}
        if cfg["use_sliding_window"]:
            cfg.update(sliding_window=rng.choice([1, 3, 8, 70, 200]), max_window_layers=rng.randint(0, L))
        folder = str(tmp_path / f"c{case}")
        he.write_random_model(config_from_dict(dict(cfg)), case, folder, "bfloat16")
        pc, w = P.read_model(folder)
        reqs = [[rng.randrange(cfg["vocab_size"]) for _ in range(rng.randint(2, rng.choice([6, 40, 150])))]
                for _ in range(rng.randint(1, rng.choice([3, 20])))]
        want = [P.forward(pc, w, r) for r in reqs]
        for dtype in DTYPES:
            eng = he.Engine(folder, dtype=dtype, max_tokens=64 * 24 * 3, max_slots=24, max_seq_len=192)
            slots = [eng.acquire() for _ in reqs]
            fed = [rng.randint(1, len(r)) for r in reqs]
            logits = eng.step([entry(s, r[:f], range(f)) for s, r, f in zip(slots, reqs, fed)])
            got, r0 = [], 0
            for f in fed:
                got.append([logits[r0:r0 + f].clone()])
                r0 += f
            live = list(range(len(reqs)))
            while True:
                live = [i for i in live if fed[i] < len(reqs[i])]
                if not live:
                    break
                logits = eng.step([entry(slots[i], [reqs[i][fed[i]]], [0]) for i in live])
                for j, i in enumerate(live):
                    got[i].append(logits[j:j + 1].clone())
                    fed[i] += 1
            for i in range(len(reqs)):
                try:
                    close(torch.cat(got[i]), want[i], dtype)
                except AssertionError as e:
                    raise AssertionError(f"{dtype} {cfg}: {e}") from None


@pytest.mark.parametrize("dtype", DTYPES)
def test_random_traffic(engines, plain_models, dtype):
    """Sixty batches of random sizes (1 to 24 requests), random lengths and random cuts (a prompt whole or in
    two chunks, then token by token, shorter requests leaving early), over all configurations: every checked
    request equals the plain implementation, and in 32-bit it equals, bit for bit, the request run alone."""
    import random
    rng = random.Random(11)
    for round_ in range(60):
        name = rng.choice(NAMES)
        eng = engines(name, dtype, max_slots=24, max_tokens=24 * 256, max_seq_len=256)
        cfg = plain_models[name][0]
        longest = min(cfg.get("max_position_embeddings", 256), 250) - 1
        reqs = [[rng.randrange(cfg["vocab_size"]) for _ in range(rng.randint(1, rng.choice([8, 40, longest])))]
                for _ in range(rng.randint(1, 24))]
        slots = {i: eng.acquire() for i in range(len(reqs))}
        fed = {i: rng.randint(1, len(r)) for i, r in enumerate(reqs)}
        got = {i: [] for i in slots}
        first = {i: max(1, fed[i] // 2) if rng.random() < 0.3 else fed[i] for i in slots}
        for lo, hi in ((lambda i: 0, first.get), (first.get, fed.get)):        # the prompts, some in two chunks
            part = [i for i in slots if hi(i) > lo(i)]
            if not part:
                continue
            logits = eng.step([entry(slots[i], reqs[i][lo(i):hi(i)], range(hi(i) - lo(i))) for i in part])
            r = 0
            for i in part:
                got[i].append(logits[r:r + hi(i) - lo(i)].clone())
                r += hi(i) - lo(i)
        live = list(slots)
        while True:
            for i in list(live):
                if fed[i] == len(reqs[i]):
                    eng.release(slots.pop(i))
                    live.remove(i)
            if not live:
                break
            logits = eng.step([entry(slots[i], [reqs[i][fed[i]]], [0]) for i in live])
            for r, i in enumerate(live):
                got[i].append(logits[r:r + 1].clone())
                fed[i] += 1
        assert eng.cache.free_pages == eng.cache.num_pages
        for i in rng.sample(range(len(reqs)), min(len(reqs), 3)):
            whole = torch.cat(got[i])
            close(whole, plain_logits(plain_models, name, reqs[i]), dtype)
            if dtype == "float32":
                s = eng.acquire()
                alone = eng.step([entry(s, reqs[i], range(len(reqs[i])))]).clone()
                eng.release(s)
                assert torch.equal(alone, whole), (round_, name, i)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_long_decoding(engines, plain_models, name, dtype):
    """Five prompt tokens, then 250 single-token steps: page boundaries at 64, 128 and 192
    are crossed, and configuration C's window of 70 slides and gives pages back."""
    eng = engines(name, dtype)
    vocab = plain_models[name][0]["vocab_size"]
    ids = rand_ids(vocab, 255, 3)
    want = plain_logits(plain_models, name, ids)
    s = eng.acquire()
    rows = [eng.step([entry(s, ids[:5], range(5))]).clone()]
    rows += [eng.step([entry(s, [t], [0])]).clone() for t in ids[5:]]
    close(torch.cat(rows), want, dtype)
    windowed = [g for g in eng.cache.book.groups if g.window > 0]
    for g in windowed:
        dead = [p for p in g.table[s] if p < 0]
        assert len(dead) == (255 - g.window - 63) // 64 + 1 if 255 - g.window >= 63 else not dead
    eng.release(s)
    assert eng.cache.free_pages == eng.cache.num_pages


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_first_tokens_of_a_sequence(engines, plain_models, name, dtype):
    """A sequence that starts with a single token, and the first decoded tokens after
    prompts of one and two tokens."""
    eng = engines(name, dtype)
    vocab = plain_models[name][0]["vocab_size"]
    ids = rand_ids(vocab, 6, 11)
    want = plain_logits(plain_models, name, ids)
    for first in (1, 2):
        s = eng.acquire()
        rows = [eng.step([entry(s, ids[:first], range(first))]).clone()]
        rows += [eng.step([entry(s, [t], [0])]).clone() for t in ids[first:]]
        close(torch.cat(rows), want, dtype)
        eng.release(s)


@pytest.mark.parametrize("name", NAMES)
def test_cutting_batching_order_and_slots_change_no_bit_in_32_bit(engines, plain_models, name):
    eng = engines(name, "float32")
    vocab = plain_models[name][0]["vocab_size"]
    reqs = [rand_ids(vocab, n, 40 + n) for n in (70, 9, 33)]

    def run(order, chunks, burn):
        burned = [eng.acquire() for _ in range(burn)]              # shifts the slot numbers
        slots = {i: eng.acquire() for i in order}
        got = {i: [] for i in order}
        pos = {i: 0 for i in order}
        while any(pos[i] < len(reqs[i]) for i in order):
            live = [i for i in order if pos[i] < len(reqs[i])]
            ents = []
            for i in live:
                n = min(chunks, len(reqs[i]) - pos[i])
                ents.append(entry(slots[i], reqs[i][pos[i]:pos[i] + n], range(n)))
            logits = eng.step(ents)
            r = 0
            for i, e in zip(live, ents):
                got[i].append(logits[r:r + len(e.tokens)].clone())
                r += len(e.tokens)
                pos[i] += len(e.tokens)
        for s in list(slots.values()) + burned:
            eng.release(s)
        return {i: torch.cat(v) for i, v in got.items()}

    base = run([0, 1, 2], 1000, 0)
    for order, chunks, burn in (([2, 0, 1], 1000, 0), ([0, 1, 2], 7, 0), ([1, 2, 0], 64, 3), ([0, 1, 2], 1, 2)):
        other = run(order, chunks, burn)
        for i in range(3):
            assert torch.equal(other[i], base[i]), (order, chunks, burn, i)
    for i in range(3):
        close(base[i], plain_logits(plain_models, name, reqs[i]), "float32")


@pytest.mark.parametrize("dtype", DTYPES)
def test_chunked_prompts_equal_whole_prompts(engines, plain_models, dtype):
    eng = engines("C", dtype)
    vocab = plain_models["C"][0]["vocab_size"]
    ids = rand_ids(vocab, 230, 5)
    want = plain_logits(plain_models, "C", ids)
    s = eng.acquire()
    rows = []
    for a in range(0, 230, 50):
        chunk = ids[a:a + 50]
        rows.append(eng.step([entry(s, chunk, range(len(chunk)))]).clone())
    eng.release(s)
    close(torch.cat(rows), want, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "C"])
def test_graph_replay_and_padding_change_no_result(model_dirs, plain_models, name, dtype):
    """One-token steps of 3 sequences run in a bucket of 4 (one padding row) as a
    captured graph; the same steps run eagerly without padding. Same bits."""
    import hector_engine_amd as he
    vocab = plain_models[name][0]["vocab_size"]
    reqs = [rand_ids(vocab, n, 60 + n) for n in (40, 75, 12)]
    outs = []
    for graphs in (True, False):
        eng = he.Engine(model_dirs[name], dtype=dtype, max_tokens=2048, max_slots=4, max_seq_len=512, beyond_max_positions=True,
                        use_graphs=graphs)
        slots = [eng.acquire() for _ in reqs]
        eng.step([entry(s, r[:6], []) for s, r in zip(slots, reqs)])
        rows = []
        for t in range(6, 12):
            rows.append(eng.step([entry(s, [r[t]], [0]) for s, r in zip(slots, reqs)]).clone())
        outs.append(torch.stack(rows))                # [6 steps, 3, vocab]
        if graphs:
            assert eng.stats["graph_replays"] >= 4 and eng.stats["graph_captures"] == 1
        else:
            assert eng.stats["graph_replays"] == 0
    assert torch.equal(outs[0], outs[1])
    for i, r in enumerate(reqs):
        close(outs[0][:, i], plain_logits(plain_models, name, r[:12])[6:12], dtype)


def test_errors_leave_the_cache_untouched(engines, plain_models):
    from hector_engine_amd.cache import CacheError, CacheFull
    from hector_engine_amd.engine.engine import StepError
    eng = engines("A", "float32", max_tokens=256, max_slots=4)       # four pages
    s, t = eng.acquire(), eng.acquire()
    with pytest.raises(StepError, match="token ids"):
        eng.step([entry(s, [1, 999], [0])])
    with pytest.raises(StepError, match="twice"):
        eng.step([entry(s, [1], [0]), entry(s, [2], [0])])
    with pytest.raises(StepError, match="wanted place"):
        eng.step([entry(s, [1, 2], [2])])
    with pytest.raises(StepError, match="at least one token"):
        eng.step([entry(s, [], [])])
    with pytest.raises(CacheError, match="not held"):
        eng.step([entry(3, [1], [0])])
    with pytest.raises(CacheFull):
        eng.step([entry(s, [1] * 130, []), entry(t, [1] * 130, [])])     # 3 + 3 pages, 4 exist
    assert eng.length(s) == 0 and eng.length(t) == 0 and eng.cache.free_pages == 4
    eng.step([entry(s, [1] * 130, [])])
    with pytest.raises(StepError, match="longest sequence"):
        eng.step([entry(s, [1] * 127, [])])
    eng.release(s)
    eng.release(t)
    with pytest.raises(CacheError):
        eng.release(t)
    eng.cache.book.check_invariants()


def test_a_reused_slot_holds_nothing_of_its_past(engines, plain_models):
    """A long request fills pages; after release a short request gets the same slot and
    pages. Its logits equal those of a fresh engine bit for bit (32-bit)."""
    eng = engines("B", "float32", max_tokens=512, max_slots=2)
    vocab = plain_models["B"][0]["vocab_size"]
    long, short = rand_ids(vocab, 300, 1), rand_ids(vocab, 70, 2)
    s = eng.acquire()
    first = eng.step([entry(s, short, range(70))]).clone()
    eng.release(s)
    s = eng.acquire()
    eng.step([entry(s, long, [])])
    eng.release(s)
    s2 = eng.acquire()
    assert s2 == s
    again = eng.step([entry(s2, short, range(70))]).clone()
    eng.release(s2)
    assert torch.equal(first, again)
    close(again, plain_logits(plain_models, "B", short), "float32")


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_step_of_thousands_of_rows(model_dirs, plain_models, dtype):
    """24 prompts of 400 tokens in one step: more rows than the feed-forward holds at once (it
    then works in turns and gives their temporaries back), layers that take the activation
    arenas in turn, and the decode step after it."""
    import hector_engine_amd as he
    name = "C"
    vocab = plain_models[name][0]["vocab_size"]
    eng = he.Engine(model_dirs[name], dtype=dtype, max_tokens=24 * 448, max_slots=24, max_seq_len=448, beyond_max_positions=True)
    prompts = [rand_ids(vocab, 400 - (i % 3), 300 + i) for i in range(24)]
    slots = [eng.acquire() for _ in prompts]
    got = eng.step([entry(s, p, [0, len(p) - 1]) for s, p in zip(slots, prompts)])
    assert sum(len(p) for p in prompts) > 8192
    for i in (0, 7, 23):
        want = plain_logits(plain_models, name, prompts[i])
        close(got[2 * i:2 * i + 2], want[[0, len(prompts[i]) - 1]], dtype)
    nxt = [int(t) for t in got[1::2].argmax(-1).tolist()]
    got2 = eng.step([entry(s, [t], [0]) for s, t in zip(slots, nxt)])
    for i in (0, 23):
        want = plain_logits(plain_models, name, prompts[i] + [nxt[i]])
        close(got2[i:i + 1], want[-1:], dtype)
    for s in slots:
        eng.release(s)


def test_a_failed_capture_falls_back_to_eager_steps(model_dirs, plain_models, monkeypatch):
    """When capturing the one-token step of a batch size fails, the engine says so once, records why,
    and runs steps of that size without a graph (the reference falls back the same way:
    src/engine.cpp:233-261). The failure is made on the host: torch's capture context is replaced by
    one that raises. An error that is the step's own is not swallowed: it comes back from the eager
    run of the same step and reaches the caller."""
    import contextlib
    import warnings
    import hector_engine_amd as he
    from hector_engine_amd.engine import engine as engine_module

    @contextlib.contextmanager
    def broken(graph):
        raise RuntimeError("capture refused (made up by the test)")
        yield

    eng = he.Engine(model_dirs["D"], dtype="bfloat16", max_tokens=1024, max_slots=4)
    monkeypatch.setattr(engine_module.torch.cuda, "graph", broken)
    vocab = plain_models["D"][0]["vocab_size"]
    ids = rand_ids(vocab, 30, 5)
    want = plain_logits(plain_models, "D", ids)
    s = eng.acquire()
    eng.step([entry(s, ids[:10], [])])
    rows = []
    with warnings.catch_warnings(record=True) as seen:
        warnings.simplefilter("always")
        for t in ids[10:]:
            rows.append(eng.step([entry(s, [t], [0])]).clone())
    eng.release(s)
    assert len([w for w in seen if "HIP graph failed" in str(w.message)]) == 1       # said once
    assert eng.stats["graph_captures"] == 0 and eng.stats["graph_replays"] == 0
    assert eng.stats["eager_steps"] == 21
    close(torch.cat(rows), want[10:], "bfloat16")
    assert eng.stats["graph_capture_failures"] == 1 and "made up by the test" in eng.capture_failures[0]
    # the fallback is the bucket's own: another batch size tries its own capture
    monkeypatch.undo()
    a, b = eng.acquire(), eng.acquire()
    pair = [eng.step([entry(a, [t], [0]), entry(b, [t], [0])]).clone() for t in ids[:4]]
    assert eng.stats["graph_captures"] == 1 and eng.stats["graph_replays"] >= 2
    close(torch.cat([r[:1] for r in pair]), want[:4], "bfloat16")
    # an error of the step itself (here: of the model's forward) during the capture is raised
    forward, calls = eng.model.forward, []

    def failing(*args, **kw):
        calls.append(1)
        if len(calls) > 1:
            raise ValueError("a part's own bug (made up by the test)")
        return forward(*args, **kw)
    monkeypatch.setattr(eng.model, "forward", failing)
    c = eng.acquire()
    three = [entry(x, [ids[0]], [0]) for x in (a, b, c)]
    eng.step(three)                                   # the bucket of four rows: first use, eager
    with pytest.raises(ValueError, match="own bug"):
        eng.step([entry(x, [ids[1]], [0]) for x in (a, b, c)])
    for x in (a, b, c):
        eng.release(x)


def test_profile_mode_times_every_kernel(model_dirs):
    """Engine(profile=True): every launch between two events, steps without graphs; the table names
    the kernels with their calls, in the reference's columns."""
    import hector_engine_amd as he
    eng = he.Engine(model_dirs["D"], dtype="bfloat16", max_tokens=1024, max_slots=2, profile=True)
    assert not eng.use_graphs
    s = eng.acquire()
    ids = rand_ids(200, 40, 9)
    eng.step([entry(s, ids[:36], [35])])
    for t in ids[36:]:
        eng.step([entry(s, [t], [0])])
    eng.release(s)
    rows = {name: (calls, ms) for name, calls, ms, _, _ in eng.profiler.rows()}
    assert rows["embedding"][0] == 5 and rows["attention_prefill"][0] == 2        # two layers, one prompt step
    assert rows["attention_decode_fused"][0] == 8 and rows["gemm_blocksplit"][0] >= 4 * 2 * 4
    assert all(ms > 0 for _, ms in rows.values())
    text = eng.profile_summary()
    assert text.startswith("=== Engine Profile ===") and "TOTAL" in text and "Avg(ms)" in text
    assert eng.stats["graph_replays"] == 0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_a_request_joins_three_that_decode(engines, plain_models, name, dtype):
    """Three sequences decode through the replayed graph; in one step a fourth joins with a prompt
    of 37 tokens while the three bring one token each; then all four decode. Every logit of every
    request against the plain implementation."""
    eng = engines(name, dtype)
    vocab = plain_models[name][0]["vocab_size"]
    requests = [rand_ids(vocab, n, 700 + i) for i, n in enumerate((29, 42, 79, 41))]
    prompt = [20, 33, 70]
    slots = [eng.acquire() for _ in range(3)]
    out = [[] for _ in requests]
    replays = eng.stats["graph_replays"]
    logits = eng.step([entry(s, r[:n], range(n)) for s, r, n in zip(slots, requests, prompt)])
    for i, part in enumerate(logits.split(prompt)):
        out[i].append(part.clone())
    fed = list(prompt) + [0]
    for _ in range(4):                                   # eager, captured, replayed, replayed
        logits = eng.step([entry(s, [requests[i][fed[i]]], [0]) for i, s in enumerate(slots)])
        for i in range(3):
            out[i].append(logits[i:i + 1].clone())
            fed[i] += 1
    assert eng.stats["graph_replays"] >= replays + 2
    # the mixed step: one token each of the three, the fourth's whole prompt
    slots.append(eng.acquire())
    logits = eng.step([entry(slots[i], [requests[i][fed[i]]], [0]) for i in range(3)]
                      + [entry(slots[3], requests[3][:37], range(37))])
    for i in range(3):
        out[i].append(logits[i:i + 1].clone())
        fed[i] += 1
    out[3].append(logits[3:].clone())
    fed[3] = 37
    for _ in range(4):
        logits = eng.step([entry(s, [requests[i][fed[i]]], [0]) for i, s in enumerate(slots)])
        for i in range(4):
            out[i].append(logits[i:i + 1].clone())
            fed[i] += 1
    assert fed == [len(r) for r in requests]
    for s in slots:
        eng.release(s)
    for i, ids in enumerate(requests):
        close(torch.cat(out[i]), plain_logits(plain_models, name, ids), dtype)
    if dtype == "float32":
        s = eng.acquire()
        alone = eng.step([entry(s, requests[3], range(41))]).clone()
        eng.release(s)
        assert torch.equal(alone, torch.cat(out[3]))    # joining a running batch changed no bit


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_truncate_then_refeed_equals_a_fresh_run(engines, plain_models, name, dtype):
    """A turn that is taken back: 150 tokens are fed, the slot is cut back, other tokens follow.
    The logits are those of a sequence that never held the dropped tokens (bit for bit in 32-bit),
    the pages beyond the cut are free again, and a cut that a windowed layer can no longer serve
    (its older pages are gone) is refused and changes nothing."""
    from hector_engine_amd.cache import CacheError
    eng = engines(name, dtype)
    cfg = plain_models[name][0]
    vocab = cfg["vocab_size"]
    first, other = rand_ids(vocab, 150, 31), rand_ids(vocab, 40, 32)
    free = eng.cache.free_pages
    s = eng.acquire()
    eng.step([entry(s, first, [])])
    keep = 70
    if cfg.get("use_sliding_window"):
        # the windowed layers (8, 70 or 40 keys) have given back their first page or two: a query at
        # position 70 would read keys that are gone, one at 141 reads only what is still held
        with pytest.raises(CacheError, match="window"):
            eng.truncate(s, keep)
        assert eng.length(s) == 150 and eng.cache.free_pages == free - 3
        keep = 141
    eng.truncate(s, keep)
    assert eng.length(s) == keep and eng.cache.free_pages == free - (keep + 63) // 64
    cut = eng.step([entry(s, other, range(40))]).clone()
    eng.release(s)
    s = eng.acquire()
    eng.step([entry(s, first[:keep], [])])
    fresh = eng.step([entry(s, other, range(40))]).clone()
    eng.release(s)
    want = plain_logits(plain_models, name, first[:keep] + other)[keep:]
    close(cut, want, dtype)
    if dtype == "float32":
        assert torch.equal(cut, fresh)
    with pytest.raises(CacheError):
        eng.truncate(s, 0)                                # the slot is no longer held
    assert eng.cache.free_pages == free
    eng.cache.book.check_invariants()


def test_sync_each_launch_mode_gives_the_same_logits(model_dirs, plain_models):
    """The debugging mode (a wait after every launch, no graphs) changes no bit of the 32-bit path."""
    import hector_engine_amd as he
    ids = rand_ids(200, 40, 77)
    outs = []
    for mode in (False, True):
        eng = he.Engine(model_dirs["D"], dtype="float32", max_tokens=1024, max_slots=2, sync_each_launch=mode)
        s = eng.acquire()
        rows = [eng.step([entry(s, ids[:30], range(30))]).clone()]
        rows += [eng.step([entry(s, [t], [0])]).clone() for t in ids[30:]]
        outs.append(torch.cat(rows))
        assert eng.use_graphs is not mode
        if mode:
            assert eng.stats["graph_replays"] == 0
    assert torch.equal(outs[0], outs[1])
    close(outs[1], plain_logits(plain_models, "D", ids), "float32")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_short_prompt_and_mixed_steps_replay_a_graph(model_dirs, plain_models, name, dtype):
    """Prompt steps and mixed steps of up to a few hundred rows run as HIP graphs, one per bucket of
    their sizes: the first step of a bucket runs eagerly, the second is captured, later ones replay.
    Steps of different lengths that share a bucket (prompts of 37, 41 and 60 tokens; three one-token
    entries beside a prompt of 33 to 50) replay the same graph; every logit is the plain
    implementation's, and in 32-bit bit for bit what an engine without such graphs gives."""
    import hector_engine_amd as he
    opts = dict(max_tokens=4096, max_slots=8, max_seq_len=1024, beyond_max_positions=True)
    eng = he.Engine(model_dirs[name], dtype=dtype, **opts)
    plain_eng = he.Engine(model_dirs[name], dtype=dtype, graph_step_rows=0, **opts)
    vocab = plain_models[name][0]["vocab_size"]

    def both(make_entries):
        a = eng.step(make_entries(eng))
        b = plain_eng.step(make_entries(plain_eng))
        if dtype == "float32":
            assert torch.equal(a, b)
        return a.clone()

    # whole prompts of lengths that share the bucket of 64 rows, all positions wanted
    for i, n in enumerate((37, 41, 60, 33, 64)):
        ids = rand_ids(vocab, n, 800 + i)
        slots = {}

        def prompt(e, ids=ids, n=n):
            slots[e] = e.acquire()
            return [entry(slots[e], ids, range(n))]
        got = both(prompt)
        close(got, plain_logits(plain_models, name, ids), dtype)
        for e, s in slots.items():
            e.release(s)
    assert eng.stats["step_graph_captures"] == 1 and eng.stats["step_graph_replays"] == 4
    assert plain_eng.stats["step_graph_captures"] == 0
    # three sequences that decode, and a prompt that joins them: five mixed steps in a row, the
    # joining prompt of another length each time, only some places wanted
    requests = [rand_ids(vocab, n, 820 + i) for i, n in enumerate((30, 52, 75))]
    held = {e: [e.acquire() for _ in requests] for e in (eng, plain_eng)}
    fed = [20, 40, 60]
    both(lambda e: [entry(s, r[:n], [n - 1]) for s, r, n in zip(held[e], requests, fed)])
    rows = [[] for _ in requests]
    for step, n in enumerate((33, 50, 41, 36, 48)):
        joiner = rand_ids(vocab, n, 840 + step)
        extra = {}

        def mixed(e, joiner=joiner, n=n):
            extra[e] = e.acquire()
            return [entry(s, [r[k]], [0]) for s, r, k in zip(held[e], requests, fed)] \
                + [entry(extra[e], joiner, [0, n // 2, n - 1])]
        got = both(mixed)
        for i in range(3):
            rows[i].append(got[i:i + 1])
            fed[i] += 1
        close(got[3:], plain_logits(plain_models, name, joiner)[[0, n // 2, n - 1]], dtype)
        for e, s in extra.items():
            e.release(s)
    for i, r in enumerate(requests):
        close(torch.cat(rows[i]), plain_logits(plain_models, name, r[:fed[i]])[fed[i] - 5:], dtype)
    assert eng.stats["step_graph_captures"] >= 2 and eng.stats["step_graph_replays"] >= 4 + 3
    assert not eng.capture_failures
    for e, ss in held.items():
        for s in ss:
            e.release(s)
        assert e.cache.free_pages == e.cache.num_pages


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B"])
def test_whole_chunks_of_a_long_prompt_replay_a_graph(model_dirs, plain_models, name, dtype):
    """A step of more rows than the padded buckets take is captured as it is when its row count is a
    multiple of 256: a prompt of 768 tokens fed in three chunks of 256 (each chunk a bucket of its
    own, by the keys behind it), three requests in a row, so that every bucket runs eagerly, is
    captured and is replayed; two prompts of 128 tokens packed into one such step; a step of 300 rows
    runs eagerly, and so does a chunk of which every place is wanted. Every logit is the plain implementation's, and in 32-bit bit for bit what an engine
    without such graphs gives."""
    import hector_engine_amd as he
    opts = dict(max_tokens=4096, max_slots=4, max_seq_len=1024, beyond_max_positions=True)
    eng = he.Engine(model_dirs[name], dtype=dtype, graph_step_rows=64, **opts)
    plain_eng = he.Engine(model_dirs[name], dtype=dtype, graph_step_rows=0, **opts)
    vocab = plain_models[name][0]["vocab_size"]
    for r in range(3):
        ids = rand_ids(vocab, 768, 870 + r)
        want = plain_logits(plain_models, name, ids)
        slots = {e: e.acquire() for e in (eng, plain_eng)}
        for c in range(3):
            piece = ids[256 * c:256 * (c + 1)]
            a, b = (e.step([entry(slots[e], piece, [0, 100, 255])]).clone() for e in (eng, plain_eng))
            if dtype == "float32":
                assert torch.equal(a, b)
            close(a, want[[256 * c, 256 * c + 100, 256 * c + 255]], dtype)
        for e, s in slots.items():
            e.release(s)
    assert eng.stats["step_graph_captures"] == 3 and eng.stats["step_graph_replays"] == 6
    for r in range(3):
        pair = [rand_ids(vocab, 128, 880 + 2 * r), rand_ids(vocab, 128, 881 + 2 * r)]
        slots = {e: [e.acquire(), e.acquire()] for e in (eng, plain_eng)}
        a, b = (e.step([entry(s, p, [127]) for s, p in zip(slots[e], pair)]).clone() for e in (eng, plain_eng))
        if dtype == "float32":
            assert torch.equal(a, b)
        close(a, torch.cat([plain_logits(plain_models, name, p)[127:128] for p in pair]), dtype)
        for e, ss in slots.items():
            for s in ss:
                e.release(s)
    assert eng.stats["step_graph_captures"] == 4 and eng.stats["step_graph_replays"] == 8
    ids = rand_ids(vocab, 300, 890)
    slot = eng.acquire()
    assert eng._step_plan([entry(slot, ids, [299])], False) is None
    assert eng._step_plan([entry(slot, ids[:256], range(256))], False) is None     # a bucket would keep 256 rows of logits
    assert eng._step_plan([entry(slot, ids[:256], [255])], False) is not None
    close(eng.step([entry(slot, ids, [299])]), plain_logits(plain_models, name, ids)[299:300], dtype)
    eng.release(slot)
    assert eng.stats["step_graph_captures"] == 4 and not eng.capture_failures
    assert eng.cache.free_pages == eng.cache.num_pages


def test_step_graphs_are_kept_least_recently_used_first_out(model_dirs, plain_models):
    """No more graphs of prompt steps are kept than GRAPH_MAX_STEP_PLANS: the one used longest ago
    goes, and a bucket that comes again after that is captured anew, with the same logits."""
    import hector_engine_amd as he
    from hector_engine_amd.engine import engine as engine_module
    eng = he.Engine(model_dirs["A"], dtype="float32", max_tokens=4096, max_slots=8, max_seq_len=512,
                    beyond_max_positions=True)
    ids = rand_ids(256, 300, 860)
    want = plain_logits(plain_models, "A", ids[:20])

    def run(n_seqs, n, places):
        slots = [eng.acquire() for _ in range(n_seqs)]
        out = eng.step([entry(s, ids[:n], places) for s in slots]).clone()
        for s in slots:
            eng.release(s)
        return out
    first = [run(1, 20, [19]) for _ in range(3)]
    close(first[2], want[19:20], "float32")
    assert len(eng._plans) == 1
    # 24 other buckets: 1, 2, 4 or 8 sequences, runs of 2 to 64 new tokens, two places wanted of each
    for s in (1, 2, 3, 5):
        for n in (2, 3, 5, 9, 17, 33):
            run(s, n, [0, n - 1])
    assert len(eng._plans) == engine_module.GRAPH_MAX_STEP_PLANS == 24
    captures = eng.stats["step_graph_captures"]
    again = [run(1, 20, [19]) for _ in range(3)]
    assert eng.stats["step_graph_captures"] == captures + 1
    assert all(torch.equal(a, first[0]) for a in again + first)
