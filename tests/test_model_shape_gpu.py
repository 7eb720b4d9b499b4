"""The benchmark model's layer sizes (Qwen2.5-7B: hidden 3584, 28 heads, 4 kv heads,
head_dim 128, intermediate 18944, vocabulary 152064) with two layers and random
weights: the MFMA kernels at the sizes they are tuned for. The 32-bit path is compared with
the plain implementation (float64, on the CPU, from a model folder both read; the reference
checks its engine against an independent 32-bit oracle the same way:
tools/quant_bench/ref_qwen3.py:76-129) and does not depend on the cut; the bfloat16 path is
compared with the 32-bit path by the metrics of the reference's
tools/quant_bench/compare_logits.py:9-23 (error, correlation, argmax, top-k overlap).

HECTOR_TEST_TUNE_LIBRARY=1 builds the bfloat16 engines with the library's tuner on, as the
benchmark runs them; the last test runs this file so in a process of its own."""
import os
import subprocess
import sys

import pytest
import torch

from tests.helpers import rand_ids

pytestmark = pytest.mark.gpu

SHAPE = dict(architectures=["Qwen2ForCausalLM"], num_hidden_layers=2, hidden_size=3584,
             num_attention_heads=28, num_key_value_heads=4, head_dim=128, intermediate_size=18944,
             vocab_size=152064, rope_theta=1000000.0, rms_norm_eps=1e-6, max_position_embeddings=32768,
             tie_word_embeddings=False)


TUNED = os.environ.get("HECTOR_TEST_TUNE_LIBRARY") == "1"


@pytest.fixture(scope="module")
def engines():
    import hector_engine_amd as he
    from hector_engine_amd.registry import config_from_dict
    cfg = config_from_dict(dict(SHAPE))
    made = {}

    def get(dtype, slots=8):
        if (dtype, slots) not in made:
            made[(dtype, slots)] = he.Engine(config=cfg, seed=3, dtype=dtype, max_tokens=max(4096, 128 * slots),
                                             max_slots=slots, max_seq_len=1024,
                                             tune_library=TUNED and dtype == "bfloat16")
        return made[(dtype, slots)]

    return get


def entry(slot, tokens, want):
    from hector_engine_amd.engine.engine import StepEntry
    return StepEntry(slot, list(tokens), list(want))


def run(eng, reqs, first):
    """Prompts (the first `first[i]` tokens) in one step, then one token each."""
    slots = [eng.acquire() for _ in reqs]
    rows = {i: [] for i in range(len(reqs))}
    fed = list(first)
    logits = eng.step([entry(s, r[:n], range(n)) for s, r, n in zip(slots, reqs, fed)])
    o = 0
    for i, n in enumerate(fed):
        rows[i].append(logits[o:o + n].clone())
        o += n
    live = [i for i in range(len(reqs)) if fed[i] < len(reqs[i])]
    while live:
        logits = eng.step([entry(slots[i], [reqs[i][fed[i]]], [0]) for i in live])
        for j, i in enumerate(live):
            rows[i].append(logits[j:j + 1].clone())
            fed[i] += 1
        live = [i for i in live if fed[i] < len(reqs[i])]
    for s in slots:
        eng.release(s)
    return [torch.cat(rows[i]) for i in range(len(reqs))]


def test_seven_b_layer_sizes(engines):
    reqs = [rand_ids(152064, n, 500 + n) for n in (300, 77, 130)]
    e32, e16 = engines("float32"), engines("bfloat16")
    whole32 = run(e32, reqs, [len(r) for r in reqs])
    cut32 = run(e32, reqs, [len(r) - 12 for r in reqs])
    for a, b in zip(whole32, cut32):
        assert torch.equal(a, b)                             # 32-bit: the cut changes no bit
    whole16 = run(e16, reqs, [len(r) for r in reqs])
    cut16 = run(e16, reqs, [len(r) - 12 for r in reqs])     # 12 one-token steps through the graph
    for ref, w, c in zip(whole32, whole16, cut16):
        ref = ref.double()
        for got in (w.double(), c.double()):
            d = got - ref
            scale = ref.abs().max().item()
            assert d.abs().max().item() < 0.03 * scale
            assert (d ** 2).mean().sqrt().item() < 0.005 * scale
            last = slice(-12, None)
            corr = torch.corrcoef(torch.stack([got[last].flatten(), ref[last].flatten()]))[0, 1].item()
            assert corr > 0.999
            top_ref = ref[last].topk(10, -1).indices
            top_got = got[last].topk(10, -1).indices
            overlap = sum(len(set(a.tolist()) & set(b.tolist())) for a, b in zip(top_ref, top_got)) / (10 * 12)
            assert overlap > 0.8
            # the first choice agrees wherever the 32-bit path's lead is clear
            t2 = ref.topk(2, -1).values
            clear = (t2[:, 0] - t2[:, 1]) > 0.03 * scale
            assert torch.equal(got.argmax(-1)[clear], ref.argmax(-1)[clear])
    assert e16.stats["graph_replays"] > 0


def test_queued_steps_at_seven_b_layer_sizes(engines):
    """Runs of 8 queued one-token steps (ids handed on the device, HIP graph replays back to back)
    give the tokens of one step at a time, greedy and sampled, at the sizes of the benchmark."""
    import hector_engine_amd as he
    eng = engines("bfloat16")
    prompts = [rand_ids(152064, n, 700 + n) for n in (40, 9, 21, 33, 5)]
    for sampling in (he.SamplingConfig.deterministic(), he.SamplingConfig(temperature=0.9, top_k=50, seed=11)):
        one = he.generate(eng, prompts, max_new_tokens=27, sampling=sampling, run_of_steps=1)
        many = he.generate(eng, prompts, max_new_tokens=27, sampling=sampling, run_of_steps=8)
        assert [r.tokens for r in one] == [r.tokens for r in many]
        assert all(len(r.tokens) == 27 for r in many)
    assert eng.cache.free_pages == eng.cache.num_pages


def test_larger_batches_at_seven_b_layer_sizes(engines):
    """Sixty-six requests of unequal lengths: as they end, the one-token steps run at 66 rows and then at every
    row range that has kernels of its own (the library's products above 16 rows, the wavefront kernel, the
    block-split kernel below), at the benchmark's layer sizes, against the 32-bit path."""
    reqs = [rand_ids(152064, 4 + (i * 7) % 23, 900 + i) for i in range(66)]
    first = [max(1, len(r) - 3 - i % 9) for i, r in enumerate(reqs)]
    ref = run(engines("float32", 66), reqs, first)
    got = run(engines("bfloat16", 66), reqs, first)
    for r, g in zip(ref, got):
        r, g = r.double(), g.double()
        scale = r.abs().max().item()
        assert (g - r).abs().max().item() < 0.03 * scale
        assert ((g - r) ** 2).mean().sqrt().item() < 0.005 * scale
        t2 = r.topk(2, -1).values
        clear = (t2[:, 0] - t2[:, 1]) > 0.03 * scale
        assert torch.equal(g.argmax(-1)[clear], r.argmax(-1)[clear])


LARGER = {
    "32b": dict(hidden_size=5120, num_attention_heads=40, num_key_value_heads=8, intermediate_size=27648),
    "72b": dict(hidden_size=8192, num_attention_heads=64, num_key_value_heads=8, intermediate_size=29568),
}


@pytest.mark.parametrize("name", sorted(LARGER))
def test_one_layer_at_the_larger_models_sizes(name):
    """One layer of the Qwen2.5-32B and Qwen2-72B sizes (K of 27648 and 29568, 55296 and 59136
    gate and up rows, 40 and 64 query heads over 8 kv heads) with a vocabulary that is no power of
    two: prompts of unequal lengths in one step, then one-token steps at 64, 32, 8 and 1 rows,
    bfloat16 against the 32-bit path."""
    import hector_engine_amd as he
    from hector_engine_amd.registry import config_from_dict
    cfg = config_from_dict(dict(SHAPE, **LARGER[name], num_hidden_layers=1, vocab_size=20011))
    # 32 requests take two one-token steps, 24 four, 7 six and one eight
    steps = [2] * 32 + [4] * 24 + [6] * 7 + [8]
    reqs = [rand_ids(20011, 3 + (i * 5) % 19 + steps[i], 1300 + i) for i in range(64)]
    first = [len(r) - steps[i] for i, r in enumerate(reqs)]
    outs = {}
    for dtype in ("float32", "bfloat16"):
        eng = he.Engine(config=cfg, seed=5, dtype=dtype, max_tokens=64 * 64, max_slots=64, max_seq_len=64,
                        tune_library=TUNED and dtype == "bfloat16")
        outs[dtype] = run(eng, reqs, first)
        if dtype == "bfloat16":
            assert eng.stats["graph_replays"] > 0
        del eng
        torch.cuda.empty_cache()
    for r, g in zip(outs["float32"], outs["bfloat16"]):
        r, g = r.double(), g.double()
        scale = r.abs().max().item()
        assert (g - r).abs().max().item() < 0.03 * scale
        assert ((g - r) ** 2).mean().sqrt().item() < 0.005 * scale
        t2 = r.topk(2, -1).values
        clear = (t2[:, 0] - t2[:, 1]) > 0.03 * scale
        assert torch.equal(g.argmax(-1)[clear], r.argmax(-1)[clear])


@pytest.fixture(scope="module")
def folder(tmp_path_factory):
    """A model folder of these sizes (config.json, model.safetensors: bfloat16 values, 3.1 GB)."""
    import hector_engine_amd as he
    from hector_engine_amd.registry import config_from_dict
    path = str(tmp_path_factory.mktemp("seven_b_two_layers"))
    he.write_random_model(config_from_dict(dict(SHAPE)), 17, path, "bfloat16")
    return path


def plain_logits_on_columns(folder, ids, cols):
    """The plain implementation's logits [len(ids), len(cols)] in float64. Only what it needs is
    kept in float64: the layers, the embedding rows of these ids (ids renumbered to them) and
    the head's rows `cols`; every other function of it runs as for a tiny model."""
    from tests.plain import qwen2_plain as P
    cfg, w = P.read_model(folder, torch.float32)
    used = sorted(set(ids))
    place = {t: i for i, t in enumerate(used)}
    small = {k: v.double() for k, v in w.items() if k.startswith("model.layers.") or k == "model.norm.weight"}
    small["model.embed_tokens.weight"] = w["model.embed_tokens.weight"][used].double()
    small["lm_head.weight"] = w["lm_head.weight"][cols].double()
    del w
    return P.forward(cfg, small, [place[t] for t in ids])


@pytest.mark.skipif(TUNED, reason="the 32-bit path has no library products")
def test_float32_equals_plain_at_seven_b_layer_sizes(folder):
    """A request of 300 tokens whole (all positions), and again with its last 12 tokens one by
    one, in true 32-bit against the plain implementation, on every 37th column of the
    vocabulary and on its last columns. The sums here are over 3584 to 18944 terms: the bound
    is the tiny configurations' (2e-5 of the largest logit) times sqrt(18944 / 160)."""
    import hector_engine_amd as he
    ids = rand_ids(152064, 300, 4242)
    cols = sorted(set(range(0, 152064, 37)) | set(range(152064 - 70, 152064)))
    want = plain_logits_on_columns(folder, ids, cols)
    eng = he.Engine(folder, dtype="float32", max_tokens=1024, max_slots=2, max_seq_len=512)
    s = eng.acquire()
    whole = eng.step([entry(s, ids, range(300))]).clone()
    eng.release(s)
    s = eng.acquire()
    assert eng.step([entry(s, ids[:288], [])]) is None
    tail = torch.cat([eng.step([entry(s, [t], [0])]).clone() for t in ids[288:]])
    eng.release(s)
    assert torch.equal(tail, whole[288:])
    got = whole[:, cols].cpu().double()
    scale = want.abs().max().item()
    err = (got - want).abs().max().item()
    assert err <= 2e-5 * (18944 / 160) ** 0.5 * scale, (err, scale)
    assert torch.equal(got.argmax(-1), want.argmax(-1))
    # and the bfloat16 path against the plain implementation, by the same measures as against
    # the 32-bit path above
    e16 = he.Engine(folder, dtype="bfloat16", max_tokens=1024, max_slots=2, max_seq_len=512)
    s = e16.acquire()
    parts = [e16.step([entry(s, ids[:288], range(288))]).clone()]
    parts += [e16.step([entry(s, [t], [0])]).clone() for t in ids[288:]]
    e16.release(s)
    got16 = torch.cat(parts)[:, cols].cpu().double()
    d = got16 - want
    assert d.abs().max().item() < 0.03 * scale
    assert (d ** 2).mean().sqrt().item() < 0.005 * scale
    t2 = want.topk(2, -1).values
    clear = (t2[:, 0] - t2[:, 1]) > 0.03 * scale
    assert torch.equal(got16.argmax(-1)[clear], want.argmax(-1)[clear])


@pytest.mark.skipif(TUNED, reason="the comparison with the plain implementation runs once")
def test_unequal_batch_equals_plain_at_seven_b_layer_sizes(folder):
    """Three requests of unequal lengths in one batch, their prompts in one step, then one token
    each, the shortest ending first: every position of every request against the plain
    implementation (on vocabulary columns), in true 32-bit and in bfloat16, and once more from the
    slots the first batch gave back."""
    import hector_engine_amd as he
    reqs = [rand_ids(152064, n, 900 + n) for n in (41, 23, 60)]
    first = [30, 19, 33]                    # the second request has 4 tokens left, the first 11, the third 27
    cols = sorted(set(range(5, 152064, 97)) | set(range(152064 - 40, 152064)))
    want = [plain_logits_on_columns(folder, ids, cols) for ids in reqs]
    for dtype in ("float32", "bfloat16"):
        eng = he.Engine(folder, dtype=dtype, max_tokens=1024, max_slots=3, max_seq_len=256)
        for batch in range(2):
            got = run(eng, reqs, first)
            assert eng.cache.free_pages == eng.cache.num_pages
            for g, w in zip(got, want):
                g = g[:, cols].cpu().double()
                scale = w.abs().max().item()
                d = g - w
                if dtype == "float32":
                    assert d.abs().max().item() <= 2e-5 * (18944 / 160) ** 0.5 * scale
                    assert torch.equal(g.argmax(-1), w.argmax(-1))
                else:
                    assert d.abs().max().item() < 0.03 * scale
                    assert (d ** 2).mean().sqrt().item() < 0.005 * scale
                    t2 = w.topk(2, -1).values
                    clear = (t2[:, 0] - t2[:, 1]) > 0.03 * scale
                    assert torch.equal(g.argmax(-1)[clear], w.argmax(-1)[clear])
        if dtype == "bfloat16":
            assert eng.stats["graph_replays"] > 0
        del eng
        torch.cuda.empty_cache()


@pytest.mark.skipif(TUNED, reason="this is the run it starts")
def test_the_same_with_the_library_tuner_on():
    """The benchmark runs with the library's tuner choosing the kernel of every product above 16
    rows: the comparisons of this file once more with such engines, in a process of their own
    (the tuner's state is the process's)."""
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, HECTOR_TEST_TUNE_LIBRARY="1")
    done = subprocess.run([sys.executable, "-u", "-m", "pytest", "-x", "-q", "--timeout", "300",
                           "--timeout-method", "thread", "-p", "no:cacheprovider", os.path.abspath(__file__),
                           "-k", "seven_b_layer_sizes and not plain or larger"],
                          cwd=root, env=env, capture_output=True, text=True, timeout=600)
    assert done.returncode == 0, done.stdout[-3000:] + done.stderr[-2000:]
    assert " passed" in done.stdout and "skipped" not in done.stdout.splitlines()[-1].split("passed")[0]
