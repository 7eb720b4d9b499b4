"""The benchmark model's layer sizes (Qwen2.5-7B: hidden 3584, 28 heads, 4 kv heads,
head_dim 128, intermediate 18944, vocabulary 152064) with two layers and random
weights: the MFMA kernels at the sizes they are tuned for. The 32-bit path does not
depend on the cut; the bfloat16 path is compared with the 32-bit path by the metrics of
the reference's tools/quant_bench/compare_logits.py:9-23 (error, correlation, argmax,
top-k overlap). Parity with the plain implementation at this size is not pinned (the
plain implementation runs on the CPU); it is pinned at the tiny configurations."""
import pytest
import torch

from tests.helpers import rand_ids

pytestmark = pytest.mark.gpu

SHAPE = dict(architectures=["Qwen2ForCausalLM"], num_hidden_layers=2, hidden_size=3584,
             num_attention_heads=28, num_key_value_heads=4, head_dim=128, intermediate_size=18944,
             vocab_size=152064, rope_theta=1000000.0, rms_norm_eps=1e-6, max_position_embeddings=32768,
             tie_word_embeddings=False)


@pytest.fixture(scope="module")
def engines():
    import hector_engine_amd as he
    from hector_engine_amd.registry import config_from_dict
    cfg = config_from_dict(dict(SHAPE))
    made = {}

    def get(dtype, slots=8):
        if (dtype, slots) not in made:
            made[(dtype, slots)] = he.Engine(config=cfg, seed=3, dtype=dtype, max_tokens=max(4096, 128 * slots),
                                             max_slots=slots, max_seq_len=1024)
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
