"""The attention and position-encoding kernels at the context lengths the benchmark runs at
(2,048 to 32,768 cached tokens; 28 query heads over 4 kv heads of 128), each against the
plain implementation in float64.

Among thousands of keys with random scores no single key matters, and a page that is skipped
or read twice would stay below any sensible bound. So the queries here are long (a standard
deviation of 4 in the scores): a handful of keys at random places carry each head's result.
Beside that, one key per sequence is made to take all the weight of its kv group's first
head, at a place chosen for what is special about it: the first key, a page's edge, the edge
of a slice of the keys, the oldest key of a window and the one before it."""
import math

import pytest
import torch

from tests.plain import qwen2_plain as P
from tests.test_kernels_gpu import PAGE, dev, page_maps, rnd

pytestmark = pytest.mark.gpu
H, KVH, HD = 28, 4, 128
G = H // KVH
TOL = 2 ** -6


@pytest.fixture(scope="module")
def ops():
    import hector_engine_amd  # noqa: F401
    from hector_engine_amd.kernels import lib, ops as _ops
    lib.load()
    return _ops


class Cache:
    """A paged cache on the device with scattered pages; block b of sequence s is left without
    a page (-1) where `dead(s, b)` says so."""

    def __init__(self, lengths, max_blocks, seed, dead=None, kvh=KVH, hd=HD, dtype=torch.bfloat16):
        g = torch.Generator().manual_seed(seed)
        self.kvh, self.hd = kvh, hd
        B = len(lengths)
        blocks = [(n + PAGE - 1) // PAGE for n in lengths]
        self.num_pages = sum(blocks) + 5
        perm = iter(torch.randperm(self.num_pages, generator=g).tolist())
        self.slots = list(range(B))[::-1]
        self.table = torch.full((B + 1, max_blocks), -1, dtype=torch.int32)
        for i, (s, nb) in enumerate(zip(self.slots, blocks)):
            for b in range(nb):
                page = next(perm)
                if dead is None or not dead(i, b):
                    self.table[s, b] = page
        km, vm = page_maps(hd)
        self.km, self.vm = km.reshape(-1).cuda(), vm.reshape(-1).cuda()
        # what a page holds beyond a sequence's end is someone else's old data: finite, and large
        self.kpool = torch.full((self.num_pages, kvh, km.numel()), 50.0, dtype=dtype, device="cuda")
        self.vpool = torch.full((self.num_pages, kvh, vm.numel()), 50.0, dtype=dtype, device="cuda")

    def fill(self, i, k, v):
        """k, v: [n, kvh, hd] of sequence i, into its pages (blocks without a page are skipped)."""
        n = k.shape[0]
        nb = (n + PAGE - 1) // PAGE
        pages = self.table[self.slots[i], :nb].long()
        live = (pages >= 0).nonzero().flatten()
        for pool, m, x in ((self.kpool, self.km, k), (self.vpool, self.vm, v)):
            padded = torch.full((nb * PAGE, self.kvh, self.hd), 50.0, dtype=x.dtype)
            padded[:n] = x
            rows = padded.reshape(nb, PAGE, self.kvh, self.hd).permute(0, 2, 1, 3).reshape(nb, self.kvh, -1)
            block = torch.empty((len(live), self.kvh, pool.shape[-1]), dtype=pool.dtype, device="cuda")
            block[:, :, m] = rows[live].cuda()
            pool[pages[live].cuda()] = block

    def key(self, i, pos):
        page = self.table[self.slots[i], pos // PAGE].item()
        return self.kpool[page][:, self.km.reshape(PAGE, self.hd)[pos % PAGE]]

    def value(self, i, pos):
        page = self.table[self.slots[i], pos // PAGE].item()
        return self.vpool[page][:, self.vm.reshape(PAGE, self.hd)[pos % PAGE]]


def marker_places(n, window):
    """Places of a sequence of n keys (the query is the last) where a mistake would show."""
    first = 0 if window <= 0 else max(0, n - window)
    places = [first, first + 1, n - 2, (first + n) // 2]
    for edge in (64, 2048, 4096, 8192, 16384):
        places += [edge - 1, edge]
    return [p for p in dict.fromkeys(places) if first <= p < n - 1]


def decode_batch(rows, long_lengths):
    """`rows` sequences: the long ones first, the rest between 70 and 2,100 keys."""
    rest = [70 + (1013 * i) % 2031 for i in range(rows - len(long_lengths))]
    return (list(long_lengths) + rest)[:rows]


CASES = [
    # rows, max_keys, lengths of the long sequences, window
    (1, 8192, [2100], 0), (1, 8192, [8192], 0), (1, 32768, [8193], 0), (1, 32768, [20000], 0),
    (8, 8192, [8191, 8192, 2100], 0), (8, 32768, [20000, 8193, 8192], 0),
    (64, 8192, [8192, 8191], 0), (64, 32768, [20000, 8193], 0),
    (1, 32768, [10000], 4096), (8, 32768, [10000, 4096, 4097, 12000], 4096), (64, 32768, [10000], 4096),
]


def case_id(c):
    return f"rows{c[0]}-max{c[1]}-{'_'.join(map(str, c[2]))}-w{c[3]}"


@pytest.mark.parametrize("case", CASES, ids=case_id)
@pytest.mark.parametrize("kind", ["split", "fused", "fused_spread"])
def test_one_token_attention_at_long_contexts(ops, kind, case):
    """The split one-token kernel (rotated q given) and the one-launch kernel (bias, rotation,
    cache write, attention) at 1, 8 and 64 rows, up to 20,000 keys, with max_keys below and above
    16,384 (the most slices a sequence is cut into differs), and through a window of 4,096 whose
    dead pages have been given back; the one-launch kernel also with the grid for a step whose
    sequences have very unequal lengths (more workgroups a sequence, most of them without keys
    for the short ones)."""
    rows, max_keys, long_lengths, window = case
    lengths = decode_batch(rows, long_lengths)
    B = len(lengths)
    theta = 1e6
    dead = None
    if window:
        # as the cache does after the step before: block b has gone once 64 b + 63 <= (n - 1) - window
        dead = lambda i, b: 64 * b + 63 <= lengths[i] - 1 - window   # noqa: E731
    cache = Cache(lengths, (max_keys + PAGE - 1) // PAGE, 300 + rows, dead)
    scale = 1.0 / math.sqrt(HD)
    width = (H + 2 * KVH) * HD
    qkv = rnd(B, width, seed=301, scale=1.0).to(torch.bfloat16)
    qkv[:, :H * HD] *= 4                                  # long queries: few keys carry a head's result
    bias = rnd(width, seed=302, scale=0.25).to(torch.bfloat16)
    fused, spread = kind.startswith("fused"), kind == "fused_spread"
    x = qkv.double() + (bias.double() if fused else 0)
    pos = torch.tensor([n - 1 for n in lengths])
    q = x[:, :H * HD].reshape(B, H, HD)
    if fused:
        q = torch.stack([P.rope(q[i:i + 1], pos[i:i + 1], theta, HD)[0] for i in range(B)])
    q = q.to(torch.bfloat16).double()
    ks, vs, marks = [], [], []
    for i, n in enumerate(lengths):
        old = n - 1 if fused else n
        k = rnd(old, KVH, HD, seed=310 + i).to(torch.bfloat16)
        v = rnd(old, KVH, HD, seed=410 + i).to(torch.bfloat16)
        places = marker_places(n, window)
        mark = places[(i + rows) % len(places)] if places else None
        if mark is not None:       # this key takes all the weight of each group's first head
            k[mark] = (q[i, ::G] * 0.25).to(torch.bfloat16)
        if window and n - 1 - window >= 0 and not dead(i, (n - 1 - window) // PAGE):
            # the youngest key outside the window, in a page that is still there: it would take
            # all the weight of each group's second head if it were seen
            k[n - 1 - window] = (q[i, 1::G] * 0.25).to(torch.bfloat16)
        cache.fill(i, k, v)
        ks.append(k), vs.append(v), marks.append(mark)
    positions = dev(pos.int())
    row_seq = dev(torch.arange(B, dtype=torch.int32))
    seq_slot = dev(torch.tensor(cache.slots, dtype=torch.int32))
    out = torch.full((B, H * HD), 7.0, dtype=torch.bfloat16, device="cuda")
    if fused:
        floats = ops.attention_decode_fused_workspace_floats(B, H, KVH, HD, max_keys, spread)
        assert not spread or floats >= B * H * 8 * (HD + 2)       # at least 8 workgroups a sequence and kv head
        ws = torch.empty(floats, device="cuda") if floats else None
        ops.attention_decode_fused(out, dev(qkv), dev(bias), cache.kpool, cache.vpool, positions, row_seq,
                                   seq_slot, dev(cache.table), dev(P.rope_inv_freq(HD, theta)), HD, B, H, KVH,
                                   HD, window, scale, max_keys, True, ws, spread=spread)
    else:
        ws = torch.empty(max(1, ops.attention_decode_workspace_floats(B, H, KVH, HD, max_keys)), device="cuda")
        ops.attention_decode(out, dev(q.to(torch.bfloat16).reshape(B, H * HD)), cache.kpool, cache.vpool,
                             positions, row_seq, seq_slot, dev(cache.table), B, H, KVH, HD, window, scale,
                             max_keys, ws)
    got = out.cpu().double().reshape(B, H, HD)
    for i, n in enumerate(lengths):
        k_all, v_all = ks[i].double(), vs[i].double()
        if fused:
            k_new = P.rope(x[i, H * HD:(H + KVH) * HD].reshape(1, KVH, HD), pos[i:i + 1], theta, HD)
            v_new = x[i, (H + KVH) * HD:].reshape(1, KVH, HD)
            k_new, v_new = k_new.to(torch.bfloat16).double(), v_new.to(torch.bfloat16).double()
            assert torch.allclose(cache.key(i, n - 1).cpu().double(), k_new[0], rtol=2 ** -7, atol=2 ** -7), i
            assert torch.allclose(cache.value(i, n - 1).cpu().double(), v_new[0], rtol=2 ** -7, atol=2 ** -7), i
            k_all, v_all = torch.cat([k_all, k_new]), torch.cat([v_all, v_new])
        want = P.attention(q[i:i + 1], k_all, v_all, pos[i:i + 1], torch.arange(n), window).reshape(H, HD)
        err = (got[i] - want).abs().max().item()
        assert torch.allclose(got[i], want, rtol=TOL, atol=TOL), (i, n, err)
        if marks[i] is not None:     # the marked key is what the first head of each group returns
            assert torch.allclose(want[::G], v_all[marks[i]], atol=0.05), (i, n, marks[i])


@pytest.mark.parametrize("total,new,window", [(4096, 4096, 0), (8192, 8192, 0), (8192, 2192, 0),
                                              (8192, 8192, 4096), (10000, 1500, 4096)])
def test_prompt_attention_at_long_contexts(ops, total, new, window):
    """Prompts of 4,096 and 8,192 tokens, a continuation of 2,192 tokens behind 6,000 cached
    ones, and a window of 4,096 with its edge inside the prompt, and behind pages that have been
    given back: a sample of the query rows (the first and last ones, those around a page's edge
    and around the window's edge, others at random) against the plain implementation."""
    start = total - new
    dead = None
    if window:
        dead = lambda i, b: i == 0 and 64 * b + 63 <= start - window   # noqa: E731  (as after the step before)
    cache = Cache([total, 300], (total + PAGE - 1) // PAGE + 1, 500 + total, dead)
    k = rnd(total, KVH, HD, seed=501).to(torch.bfloat16)
    v = rnd(total, KVH, HD, seed=502).to(torch.bfloat16)
    q = (rnd(new, H, HD, seed=503) * 4).to(torch.bfloat16)
    g = torch.Generator().manual_seed(504)
    sample = set(range(8)) | set(range(new - 8, new)) | set(torch.randint(0, new, (150,), generator=g).tolist())
    edge = [r for r in range(new) if (start + r) % PAGE in (0, 63)][:6]
    sample |= set(edge)
    marked = []
    if window:
        # rows whose oldest visible key (or the one before it) takes the weight of a head
        for j, r in enumerate(r for r in (new // 2, new // 2 + 37, new - 1, new - 64) if start + r - window >= 0):
            p = start + r
            seen = j % 2 == 0
            at = p - window + 1 if seen else p - window
            if dead is not None and dead(0, at // PAGE):
                continue
            k[at] = (q[r, (0 if seen else 1)::G].double() * 0.25).to(torch.bfloat16)
            marked.append((r, at, seen))
            sample.add(r)
    cache.fill(0, k, v)
    k2 = rnd(300, KVH, HD, seed=505).to(torch.bfloat16)
    v2 = rnd(300, KVH, HD, seed=506).to(torch.bfloat16)
    q2 = (rnd(300, H, HD, seed=507) * 4).to(torch.bfloat16)
    cache.fill(1, k2, v2)                       # a short prompt in the same launch
    rows = new + 300
    out = torch.full((rows, H * HD), 7.0, dtype=torch.bfloat16, device="cuda")
    ops.attention_prefill(out, dev(torch.cat([q, q2]).reshape(rows, H * HD)), cache.kpool, cache.vpool,
                          dev(torch.tensor([0, new, rows], dtype=torch.int32)),
                          dev(torch.tensor(cache.slots, dtype=torch.int32)),
                          dev(torch.tensor([start, 0], dtype=torch.int32)), dev(cache.table), 2, new, rows,
                          H, KVH, HD, window, 1.0 / math.sqrt(HD))
    got = out.cpu().double()
    sel = torch.tensor(sorted(sample))
    want = P.attention(q[sel].double(), k.double(), v.double(), start + sel, torch.arange(total), window)
    err = (got[sel] - want).abs().max().item()
    assert torch.allclose(got[sel], want, rtol=TOL, atol=TOL), err
    want2 = P.attention(q2.double(), k2.double(), v2.double(), torch.arange(300), torch.arange(300), window)
    assert torch.allclose(got[new:], want2, rtol=TOL, atol=TOL)
    where = {int(r): i for i, r in enumerate(sel.tolist())}
    for r, at, seen in marked:
        head = 0 if seen else 1
        near = torch.allclose(want[where[r]].reshape(H, HD)[head::G], v[at].double(), atol=0.05)
        assert near == seen, (r, at, seen)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("theta", [1e4, 1e6])
def test_position_encoding_at_far_positions(ops, dtype, theta):
    """Rotation and cache write at positions up to 32,767: angles of tens of thousands of radians
    (theta 1e4: the first pair turns by a radian a position) against sine and cosine in float64
    of the same float32 angle."""
    h, kvh, hd = 6, 2, 64
    starts = [32760, 16380, 0, 9999, 20479]
    new = [8, 11, 4, 1, 2]
    max_blocks = 512
    num_pages = 12
    table = torch.full((len(starts), max_blocks), -1, dtype=torch.int32)
    page = iter(range(num_pages))
    for s, (a, m) in enumerate(zip(starts, new)):
        for b in range(a // PAGE, (a + m - 1) // PAGE + 1):
            table[s, b] = next(page)
    km, vm = page_maps(hd)
    kpool = torch.zeros(num_pages, kvh, km.numel(), dtype=dtype, device="cuda")
    vpool = torch.zeros(num_pages, kvh, vm.numel(), dtype=dtype, device="cuda")
    rows = sum(new)
    width = (h + 2 * kvh) * hd
    qkv = rnd(rows, width, seed=601).to(dtype)
    bias = rnd(width, seed=602).to(dtype)
    positions = torch.cat([torch.arange(a, a + m) for a, m in zip(starts, new)]).int()
    row_seq = torch.cat([torch.full((m,), i) for i, m in enumerate(new)]).int()
    q_out = torch.zeros(rows, h * hd, dtype=dtype, device="cuda")
    ops.qkv_rope_cache(q_out, kpool, vpool, dev(qkv), h * hd, kvh * hd, dev(bias), dev(positions), dev(row_seq),
                       dev(torch.arange(len(starts), dtype=torch.int32)), dev(table),
                       dev(P.rope_inv_freq(hd, theta)), hd, rows, h, kvh, hd, True)
    x = qkv.double() + bias.double()
    q = P.rope(x[:, :h * hd].reshape(rows, h, hd), positions, theta, hd)
    k = P.rope(x[:, h * hd:(h + kvh) * hd].reshape(rows, kvh, hd), positions, theta, hd)
    v = x[:, (h + kvh) * hd:].reshape(rows, kvh, hd)
    tol = 3e-6 if dtype == torch.float32 else 2 ** -7
    assert torch.allclose(q_out.cpu().double().reshape(rows, h, hd), q, rtol=tol, atol=tol * 4)
    kp, vp = kpool.cpu(), vpool.cpu()
    for r in range(rows):
        p = positions[r].item()
        pg = table[row_seq[r], p // PAGE].item()
        assert torch.allclose(kp[pg][:, km[p % PAGE]].double(), k[r], rtol=tol, atol=tol * 4), (r, p)
        assert torch.allclose(vp[pg][:, vm[p % PAGE]].double(), v[r], rtol=tol, atol=tol * 4), (r, p)
    # the rotation is not the identity out there: a kernel that lost the position would fail above
    assert (q - x[:, :h * hd].reshape(rows, h, hd)).abs().max() > 0.5


def test_engine_through_a_window_of_4096_at_10000_tokens(tmp_path):
    """A tiny model whose second layer attends through a window of 4,096: 10,000 tokens in
    three steps, then eight one-token steps, against the plain implementation; the windowed
    group has given back the pages no later query can see."""
    import hector_engine_amd as he
    from hector_engine_amd.engine.engine import StepEntry
    from hector_engine_amd.registry import config_from_dict
    from tests.helpers import close, rand_ids
    cfg = {"architectures": ["Qwen2ForCausalLM"], "num_hidden_layers": 2, "hidden_size": 64,
           "num_attention_heads": 2, "num_key_value_heads": 1, "head_dim": 64, "intermediate_size": 96,
           "vocab_size": 211, "rope_theta": 1000000.0, "rms_norm_eps": 1e-6, "max_position_embeddings": 16384,
           "tie_word_embeddings": True, "use_sliding_window": True, "sliding_window": 4096,
           "max_window_layers": 1}
    folder = str(tmp_path)
    he.write_random_model(config_from_dict(dict(cfg)), 23, folder, "bfloat16")
    ids = rand_ids(211, 10008, 77)
    pcfg, w = P.read_model(folder)
    want = P.forward(pcfg, w, ids)[-9:]
    for dtype in ("float32", "bfloat16"):
        eng = he.Engine(folder, dtype=dtype, max_tokens=16384, max_slots=2)
        s = eng.acquire()
        assert eng.step([StepEntry(s, ids[:4000], [])]) is None
        assert eng.step([StepEntry(s, ids[4000:9000], [])]) is None
        rows = [eng.step([StepEntry(s, ids[9000:10000], [999])]).clone()]
        rows += [eng.step([StepEntry(s, [t], [0])]).clone() for t in ids[10000:]]
        close(torch.cat(rows), want, dtype)
        full, windowed = (g.pool for g in eng.cache.book.groups)
        assert len(full.held) == (10008 + 63) // 64
        assert len(windowed.held) <= 4096 // 64 + 2
        eng.release(s)
        assert eng.cache.free_pages == eng.cache.num_pages
        del eng


def test_engine_short_continuations_of_long_sequences(tmp_path):
    """A few new tokens behind thousands of cached ones, the step whose prompt attention cuts the keys
    into parts: 70 tokens after 3,000 and, in the same step, 130 after 2,100 and a whole prompt of 40;
    every position against the plain implementation."""
    import hector_engine_amd as he
    from hector_engine_amd.engine.engine import StepEntry
    from hector_engine_amd.kernels import ops
    from hector_engine_amd.registry import config_from_dict
    from tests.helpers import close, rand_ids
    cfg = {"architectures": ["Qwen2ForCausalLM"], "num_hidden_layers": 2, "hidden_size": 96,
           "num_attention_heads": 3, "num_key_value_heads": 1, "head_dim": 32, "intermediate_size": 80,
           "vocab_size": 157, "rope_theta": 10000.0, "rms_norm_eps": 1e-5, "max_position_embeddings": 4096,
           "tie_word_embeddings": False}
    assert ops.attention_prefill_parts(3, 130, 3, 32, 3070) > 1
    folder = str(tmp_path)
    he.write_random_model(config_from_dict(dict(cfg)), 29, folder, "bfloat16")
    reqs = [rand_ids(157, 3070, 81), rand_ids(157, 2230, 82), rand_ids(157, 40, 83)]
    fed = [3000, 2100, 0]
    pcfg, w = P.read_model(folder)
    want = [P.forward(pcfg, w, r)[f:] for r, f in zip(reqs, fed)]
    for dtype in ("float32", "bfloat16"):
        eng = he.Engine(folder, dtype=dtype, max_tokens=8192, max_slots=3)
        slots = [eng.acquire() for _ in reqs]
        assert eng.step([StepEntry(s, r[:f], []) for s, r, f in zip(slots[:2], reqs, fed)]) is None
        out = eng.step([StepEntry(s, r[f:], list(range(len(r) - f))) for s, r, f in zip(slots, reqs, fed)])
        r0 = 0
        for r, f, wnt in zip(reqs, fed, want):
            close(out[r0:r0 + len(r) - f], wnt, dtype)
            r0 += len(r) - f
        del eng


def test_engine_one_long_sequence_among_short_ones(tmp_path):
    """One-token steps of a batch in which one sequence has thousands of keys and the others a few dozen:
    the step is flagged (the attention grid spreads every sequence over more workgroups), has a graph of
    its own, and gives the plain implementation's logits; when the long sequence has ended the others go on
    in the ordinary graph."""
    import hector_engine_amd as he
    from hector_engine_amd.engine.engine import StepEntry
    from hector_engine_amd.registry import config_from_dict
    from tests.helpers import close, rand_ids
    cfg = {"architectures": ["Qwen2ForCausalLM"], "num_hidden_layers": 2, "hidden_size": 128,
           "num_attention_heads": 4, "num_key_value_heads": 2, "head_dim": 64, "intermediate_size": 88,
           "vocab_size": 173, "rope_theta": 1000000.0, "rms_norm_eps": 1e-6, "max_position_embeddings": 8192,
           "tie_word_embeddings": True}
    folder = str(tmp_path)
    he.write_random_model(config_from_dict(dict(cfg)), 31, folder, "bfloat16")
    reqs = [rand_ids(173, 4310, 91)] + [rand_ids(173, 30 + 3 * i, 92 + i) for i in range(5)]
    steps = 6
    pcfg, w = P.read_model(folder)
    want = [P.forward(pcfg, w, r) for r in reqs]
    for dtype in ("float32", "bfloat16"):
        eng = he.Engine(folder, dtype=dtype, max_tokens=8192, max_slots=8)
        slots = [eng.acquire() for _ in reqs]
        fed = [len(r) - steps - (3 if i else 0) for i, r in enumerate(reqs)]
        eng.step([StepEntry(s, r[:f], []) for s, r, f in zip(slots, reqs, fed)])
        entries = lambda live: [StepEntry(slots[i], [reqs[i][fed[i]]], [0]) for i in live]   # noqa: E731
        for t in range(steps):
            live = list(range(len(reqs)))
            assert eng._step_hints(entries(live)) == (True,)
            out = eng.step(entries(live))
            for j, i in enumerate(live):
                close(out[j:j + 1], want[i][fed[i]:fed[i] + 1], dtype)
                fed[i] += 1
        captured = eng.stats["graph_captures"]
        eng.release(slots[0])
        for t in range(3):
            live = list(range(1, len(reqs)))
            assert eng._step_hints(entries(live)) == (False,)
            out = eng.step(entries(live))
            for j, i in enumerate(live):
                close(out[j:j + 1], want[i][fed[i]:fed[i] + 1], dtype)
                fed[i] += 1
        if dtype == "bfloat16":
            assert captured == 1 and eng.stats["graph_captures"] == 2
        del eng
