"""Pins of the plain implementation: what fixes each formula beside the
reference's text. Special cases that reduce to a library routine, invariants,
and the vectors the reference's own tests hold, each chosen so that a plausible
mistake (a wrong sign or pairing, a norm in the wrong place, an off-by-one
window) fails it."""
import math

import numpy as np
import torch

from tests.plain import qwen2_plain as P

torch.manual_seed(0)


def test_embedding_is_row_equality_and_bad_ids_give_zero():
    table = torch.randn(10, 8, dtype=torch.float64)
    out = P.embedding(torch.tensor([2, 9, -1, 10]), table)
    assert torch.equal(out[0], table[2])          # tests/test_kernels.cu:204-217 holds out == table[2]
    assert torch.equal(out[1], table[9])
    assert out[2].abs().max() == 0 and out[3].abs().max() == 0    # kernels/linear.cu:56-61


def test_rmsnorm_unit_weight_gives_unit_rms():
    x = torch.randn(5, 64, dtype=torch.float64) * 3
    y = P.rmsnorm(x, torch.ones(64, dtype=torch.float64), 1e-12)
    assert torch.allclose((y * y).mean(-1), torch.ones(5, dtype=torch.float64), atol=1e-9)   # tests/test_kernels.cu:163-173
    w = torch.randn(64, dtype=torch.float64)
    want = x / torch.sqrt((x * x).mean(-1, keepdim=True) + 1e-6) * w
    assert torch.allclose(P.rmsnorm(x, w, 1e-6), want)
    # the weight multiplies directly: zero weight gives zero (a 1 + w variant would not)
    assert P.rmsnorm(x, torch.zeros(64, dtype=torch.float64), 1e-6).abs().max() == 0
    # eps matters for tiny inputs
    tiny = torch.full((1, 64), 1e-4, dtype=torch.float64)
    a = P.rmsnorm(tiny, torch.ones(64, dtype=torch.float64), 1e-6)
    b = P.rmsnorm(tiny, torch.ones(64, dtype=torch.float64), 1e-5)
    assert (a - b).abs().max() > 0.01


def test_silu_and_swiglu():
    z = torch.linspace(-2, 2, 41, dtype=torch.float64)      # the reference checks [-2, 2]: tests/test_kernels.cu:116-122
    assert torch.allclose(P.silu(z), torch.nn.functional.silu(z))
    x = torch.randn(3, 8, dtype=torch.float64)
    wg, wu, wd = (torch.randn(*s, dtype=torch.float64) for s in ((12, 8), (12, 8), (8, 12)))
    want = (torch.nn.functional.silu(x @ wg.T) * (x @ wu.T)) @ wd.T
    assert torch.allclose(P.swiglu(x, wg, wu, wd), want)
    # gate and up are not interchangeable
    assert not torch.allclose(P.swiglu(x, wu, wg, wd), want)


def test_linear_weight_rows_are_outputs():
    x = torch.ones(2, 5, dtype=torch.float64)
    w = torch.ones(3, 5, dtype=torch.float64)
    assert torch.equal(P.linear(x, w), torch.full((2, 3), 5.0, dtype=torch.float64))   # ones give K: tests/test_kernels.cu:244-262
    b = torch.tensor([1.0, 2.0, 3.0], dtype=torch.float64)
    assert torch.equal(P.linear(torch.zeros(2, 5, dtype=torch.float64), w, b), b.expand(2, 3))   # bias only


def test_rope_position_zero_is_identity_and_norms_are_kept():
    x = torch.randn(4, 3, 32, dtype=torch.float64)
    assert torch.allclose(P.rope(x, torch.zeros(4, dtype=torch.int64), 1e4), x)
    y = P.rope(x, torch.tensor([1, 7, 100, 3000]), 1e6)
    half = 16
    assert torch.allclose(x[..., :half] ** 2 + x[..., half:] ** 2, y[..., :half] ** 2 + y[..., half:] ** 2)


def test_rope_is_complex_rotation_of_half_split_pairs():
    x = torch.randn(5, 2, 16, dtype=torch.float64)
    pos = torch.tensor([0, 1, 2, 50, 999])
    theta = 1e4
    f = 1.0 / theta ** (torch.arange(0, 16, 2, dtype=torch.float64) / 16)
    ang = (pos[:, None].to(torch.float32) * f.to(torch.float32)[None]).to(torch.float64)
    z = torch.complex(x[..., :8], x[..., 8:]) * torch.polar(torch.ones_like(ang), ang)[:, None, :]
    want = torch.cat([z.real, z.imag], -1)
    assert torch.allclose(P.rope(x, pos, theta), want, atol=1e-12)
    # the interleaved pairing (2i, 2i+1) is a different function: this vector tells them apart
    e = torch.zeros(1, 1, 16, dtype=torch.float64)
    e[..., 0] = 1.0
    out = P.rope(e, torch.tensor([1]), theta)
    assert abs(out[0, 0, 8].item() - math.sin(1.0)) < 1e-6 and abs(out[0, 0, 1].item()) < 1e-12


def test_rope_scores_depend_on_distance_only():
    q, k = torch.randn(1, 1, 32, dtype=torch.float64), torch.randn(1, 1, 32, dtype=torch.float64)
    def score(m, n):
        return (P.rope(q, torch.tensor([m]), 1e4) * P.rope(k, torch.tensor([n]), 1e4)).sum().item()
    assert abs(score(5, 3) - score(105, 103)) < 1e-4       # angles are formed in fp32, hence 1e-4
    assert abs(score(5, 3) - score(3, 5)) > 1e-3           # the sign of the distance matters


def test_partial_rotary_leaves_the_tail():
    x = torch.randn(2, 1, 16, dtype=torch.float64)
    y = P.rope(x, torch.tensor([3, 4]), 1e4, rotary_dim=8)
    assert torch.equal(y[..., 8:], x[..., 8:]) and not torch.allclose(y[..., :8], x[..., :8])


def test_attention_reduces_to_the_library_routine():
    S, H, hd = 7, 3, 16
    q, k, v = (torch.randn(S, H, hd, dtype=torch.float64) for _ in range(3))
    pos = torch.arange(S)
    got = P.attention(q, k, v, pos, pos)
    want = torch.nn.functional.scaled_dot_product_attention(
        q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1), is_causal=True).transpose(0, 1).reshape(S, H * hd)
    assert torch.allclose(got, want, atol=1e-12)
    # no mask at all: the last query sees everything
    full = torch.nn.functional.scaled_dot_product_attention(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1))
    assert torch.allclose(got[-1], full.transpose(0, 1).reshape(S, H * hd)[-1], atol=1e-12)


def test_attention_special_cases():
    hd = 8
    q = torch.randn(1, 2, hd, dtype=torch.float64)
    k = torch.randn(1, 2, hd, dtype=torch.float64)
    v = torch.randn(1, 2, hd, dtype=torch.float64)
    assert torch.allclose(P.attention(q, k, v, torch.tensor([0]), torch.tensor([0])), v.reshape(1, -1))   # single key
    S = 6
    ks = k.expand(S, 2, hd).clone()
    vs = torch.randn(S, 2, hd, dtype=torch.float64)
    out = P.attention(q, ks, vs, torch.tensor([S - 1]), torch.arange(S))
    assert torch.allclose(out, vs.mean(0).reshape(1, -1))                         # uniform keys: mean of v
    qs = torch.randn(S, 2, hd, dtype=torch.float64)
    pos = torch.arange(S)
    assert torch.allclose(P.attention(qs, ks, vs, pos, pos, window=S), P.attention(qs, ks, vs, pos, pos))
    assert torch.allclose(P.attention(qs, ks, vs, pos, pos, window=1), vs.reshape(S, -1))   # window 1: own value


def test_window_counts_the_querys_own_position():
    """Visible keys are (p - window, p] (kernels/attention.cu:60): with window 3 the
    query at 5 sees 3, 4, 5 and not 2."""
    S, hd = 8, 4
    q = torch.zeros(S, 1, hd, dtype=torch.float64)          # all scores equal: plain means
    k = torch.zeros(S, 1, hd, dtype=torch.float64)
    v = torch.arange(S, dtype=torch.float64)[:, None, None].expand(S, 1, hd).clone()
    out = P.attention(q, k, v, torch.arange(S), torch.arange(S), window=3)
    assert torch.allclose(out[5], torch.full((hd,), 4.0, dtype=torch.float64))    # mean of 3, 4, 5
    assert torch.allclose(out[1], torch.full((hd,), 0.5, dtype=torch.float64))    # mean of 0, 1


def test_gqa_group_mapping():
    """kv head = h // (H / KVH): heads of a group are contiguous (kernels/attention.cu:180)."""
    S, H, KVH, hd = 4, 6, 2, 8
    q = torch.randn(S, H, hd, dtype=torch.float64)
    k, v = torch.randn(S, KVH, hd, dtype=torch.float64), torch.randn(S, KVH, hd, dtype=torch.float64)
    pos = torch.arange(S)
    out = P.attention(q, k, v, pos, pos).reshape(S, H, hd)
    for h in range(H):
        one = P.attention(q[:, h:h + 1], k[:, h // 3:h // 3 + 1], v[:, h // 3:h // 3 + 1], pos, pos)
        assert torch.allclose(out[:, h], one)


def tiny_model(tied, window=None, layers=2, seed=0):
    g = torch.Generator().manual_seed(seed)
    D, H, KVH, hd, I, V = 24, 3, 1, 8, 40, 50
    cfg = {"num_hidden_layers": layers, "hidden_size": D, "num_attention_heads": H, "num_key_value_heads": KVH,
           "head_dim": hd, "intermediate_size": I, "vocab_size": V, "rope_theta": 1e4, "rms_norm_eps": 1e-6,
           "tie_word_embeddings": tied}
    if window:
        cfg.update(use_sliding_window=True, sliding_window=window, max_window_layers=1)
    r = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64) * 0.3
    w = {"model.embed_tokens.weight": r(V, D), "model.norm.weight": 1 + r(D)}
    if not tied:
        w["lm_head.weight"] = r(V, D)
    for l in range(layers):
        p = f"model.layers.{l}."
        w.update({p + "input_layernorm.weight": 1 + r(D), p + "post_attention_layernorm.weight": 1 + r(D),
                  p + "self_attn.q_proj.weight": r(H * hd, D), p + "self_attn.q_proj.bias": r(H * hd),
                  p + "self_attn.k_proj.weight": r(KVH * hd, D), p + "self_attn.k_proj.bias": r(KVH * hd),
                  p + "self_attn.v_proj.weight": r(KVH * hd, D), p + "self_attn.v_proj.bias": r(KVH * hd),
                  p + "self_attn.o_proj.weight": r(D, H * hd), p + "mlp.gate_proj.weight": r(I, D),
                  p + "mlp.up_proj.weight": r(I, D), p + "mlp.down_proj.weight": r(D, I)})
    return cfg, w


def test_model_is_causal_and_shift_invariant():
    cfg, w = tiny_model(tied=False)
    ids = [3, 14, 15, 9, 2, 6, 5]
    full = P.forward(cfg, w, ids)
    assert torch.allclose(P.forward(cfg, w, ids[:4]), full[:4], atol=1e-12)      # a prefix does not see the rest
    shifted = P.forward(cfg, w, ids, positions=torch.arange(len(ids)) + 37)
    assert torch.allclose(shifted, full, atol=1e-4)                              # only distances count
    assert not torch.allclose(P.forward(cfg, w, ids, positions=torch.arange(len(ids)) * 2), full, atol=1e-4)


def test_tied_and_untied_heads():
    cfg, w = tiny_model(tied=True)
    ids = [1, 2, 3]
    a = P.forward(cfg, w, ids)
    w2 = dict(w)
    w2["model.embed_tokens.weight"] = w["model.embed_tokens.weight"] * 1.0
    w2["model.embed_tokens.weight"][40] += 1.0          # a row no id uses: only the head sees it
    b = P.forward(cfg, w2, ids)
    assert not torch.allclose(a[:, 40], b[:, 40]) and torch.allclose(a[:, :40], b[:, :40])
    cfg, w = tiny_model(tied=False)
    a = P.forward(cfg, w, ids)
    w2 = dict(w)
    w2["model.embed_tokens.weight"] = w["model.embed_tokens.weight"].clone()
    w2["model.embed_tokens.weight"][40] += 1.0
    assert torch.allclose(P.forward(cfg, w2, ids), a)   # untied: the head has its own matrix


def test_a_zeroed_layer_is_the_identity_and_window_only_acts_where_configured():
    cfg, w = tiny_model(tied=False, layers=2)
    ids = list(range(12))
    w0 = dict(w)
    w0["model.layers.1.self_attn.o_proj.weight"] = torch.zeros_like(w["model.layers.1.self_attn.o_proj.weight"])
    w0["model.layers.1.mlp.down_proj.weight"] = torch.zeros_like(w["model.layers.1.mlp.down_proj.weight"])
    cfg1 = dict(cfg, num_hidden_layers=1)
    assert torch.allclose(P.forward(cfg, w0, ids), P.forward(cfg1, w, ids), atol=1e-12)   # residual passes through
    cfgw, _ = tiny_model(tied=False, window=4)
    a, b = P.forward(cfg, w, ids), P.forward(cfgw, w, ids)
    assert torch.allclose(a[:4], b[:4], atol=1e-12) and not torch.allclose(a[6:], b[6:], atol=1e-6)
    assert P.layer_window(cfgw, 0) == 0 and P.layer_window(cfgw, 1) == 4


def test_the_final_norm_stands_directly_before_the_head():
    """A zero gain of model.norm gives zero logits; twice the gain, twice the logits (the head is
    linear and nothing stands between): src/graph_builder.cpp:1014-1036."""
    for tied in (False, True):
        cfg, w = tiny_model(tied=tied)
        ids = [3, 14, 15, 9, 2]
        a = P.forward(cfg, w, ids)
        assert a.abs().max() > 0.1
        z = dict(w)
        z["model.norm.weight"] = torch.zeros_like(w["model.norm.weight"])
        assert P.forward(cfg, z, ids).abs().max() == 0
        d = dict(w)
        d["model.norm.weight"] = 2 * w["model.norm.weight"]
        assert torch.allclose(P.forward(cfg, d, ids), 2 * a, atol=1e-12)
        # it normalises: scaling the last layer's output barely moves the logits (eps aside)
        m = dict(w)
        m["model.layers.1.mlp.down_proj.weight"] = torch.zeros_like(w["model.layers.1.mlp.down_proj.weight"])
        m["model.layers.1.self_attn.o_proj.weight"] = torch.zeros_like(w["model.layers.1.self_attn.o_proj.weight"])
        head = w["model.embed_tokens.weight"] if tied else w["lm_head.weight"]
        x = P.forward(dict(cfg, num_hidden_layers=1), m, ids)        # the same model: layer 1 is the identity
        assert torch.allclose(P.forward(cfg, m, ids), x, atol=1e-12)
        assert x.shape == (5, head.shape[0])


def test_the_second_norm_stands_between_the_attention_residual_and_the_feed_forward():
    """One layer, put together by hand from the parts: x1 = x + attention(norm1(x)),
    x2 = x1 + mlp(norm2(x1)) (src/graph_builder.cpp:1195, :1366-1396, :1415-1443,
    kernels/fused_add_rmsnorm.cu:47-81). A zero gain of norm 2 removes the feed-forward alone; twice
    the gain is twice the feed-forward's input, which is not twice its output (a norm behind the
    feed-forward, or on the residual before the attention was added, fails one of these)."""
    cfg, w = tiny_model(tied=False, layers=1)
    ids = [7, 1, 30, 22, 5, 48]
    pos = torch.arange(len(ids))
    eps = cfg["rms_norm_eps"]
    p = "model.layers.0."
    x = P.embedding(torch.tensor(ids), w["model.embed_tokens.weight"])
    a, _ = P.attention_block(cfg, w, p + "self_attn.", P.rmsnorm(x, w[p + "input_layernorm.weight"], eps), pos, 0)
    x1 = x + a

    def by_hand(gain):
        n2 = P.rmsnorm(x1, gain, eps)
        x2 = x1 + P.swiglu(n2, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
        return P.linear(P.rmsnorm(x2, w["model.norm.weight"], eps), w["lm_head.weight"])

    g = w[p + "post_attention_layernorm.weight"]
    for gain in (g, torch.zeros_like(g), 2 * g):
        v = dict(w)
        v[p + "post_attention_layernorm.weight"] = gain
        assert torch.allclose(P.forward(cfg, v, ids), by_hand(gain), atol=1e-12)
    assert not torch.allclose(by_hand(2 * g), by_hand(g), atol=1e-3)
    no_ff = P.linear(P.rmsnorm(x1, w["model.norm.weight"], eps), w["lm_head.weight"])
    assert torch.allclose(by_hand(torch.zeros_like(g)), no_ff, atol=1e-12)
    # with the attention's output zeroed, x1 is the embedding itself
    v = dict(w)
    v[p + "self_attn.o_proj.weight"] = torch.zeros_like(w[p + "self_attn.o_proj.weight"])
    n2 = P.rmsnorm(x, g, eps)
    x2 = x + P.swiglu(n2, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
    want = P.linear(P.rmsnorm(x2, w["model.norm.weight"], eps), w["lm_head.weight"])
    assert torch.allclose(P.forward(cfg, v, ids), want, atol=1e-12)


def test_greedy_below_a_temperature_of_one_hundredth():
    """temperature < 0.01 is greedy (src/sampler.cpp:141): at 0.009 the seed does not matter, at
    0.01 the draw is made (and, that cold, still lands on the maximum unless two logits tie)."""
    cfg, w = tiny_model(tied=False)
    greedy = P.generate(cfg, w, [1, 2, 3], 6)
    assert P.generate(cfg, w, [1, 2, 3], 6, temperature=0.009, seed=5) == greedy
    logits = torch.tensor([1.0, 1.0, 0.0])           # a tie: greedy takes the first, a draw may take the second
    assert P.argmax_lowest(logits) == 0
    assert P.sample(logits, 0.01, 0, 1.0, 2 ** 32 - 1) == 1


def test_schedule_and_shared_cache_variants():
    cfg, w = tiny_model(tied=False, layers=2)
    ids = [4, 8, 15, 16, 23, 42]
    twice = P.forward(cfg, w, ids, schedule=[0, 1, 1])
    cfg3 = dict(cfg, num_hidden_layers=3)
    w3 = dict(w)
    for k, v in w.items():
        if k.startswith("model.layers.1."):
            w3[k.replace("layers.1.", "layers.2.")] = v
    assert torch.allclose(twice, P.forward(cfg3, w3, ids), atol=1e-12)    # naming a layer twice = a copy of it
    shared = P.forward(cfg, w, ids, schedule=[0, 1], kv_from={1: 0})
    assert not torch.allclose(shared, P.forward(cfg, w, ids), atol=1e-6)


def test_sampling_rules():
    logits = torch.tensor([1.0, 3.0, 3.0, -2.0, 0.5])
    assert P.argmax_lowest(logits) == 1                                   # first maximum
    assert P.sample(logits, 1.0, 1, 1.0, 4000000000) == 1                 # top_k 1 is greedy
    assert P.sample(logits, 0.01, 0, 1.0, 0) == 1                         # cold: the (first) maximum
    # u = 0 takes the first candidate in sorted order, u -> 1 the last kept one
    assert P.sample(logits, 1.0, 0, 1.0, 0) == 1
    assert P.sample(logits, 1.0, 0, 1.0, 2 ** 32 - 1) == 3
    assert P.sample(logits, 1.0, 3, 1.0, 2 ** 32 - 1) == 0                # top-3 = {1, 2, 0}
    p = torch.softmax(logits.double(), 0)
    assert P.sample(logits, 1.0, 0, float(p[1] + p[2] - 1e-3), 2 ** 32 - 1) == 2    # nucleus of two
    n = 20000
    draws = [P.sample(logits, 1.0, 0, 1.0, P.uniform_u32(3, 0, i)) for i in range(n)]
    freq = np.bincount(draws, minlength=5) / n
    assert np.abs(freq - p.numpy()).max() < 0.015


def test_penalties_rule():
    x = torch.tensor([2.0, -2.0, 1.0, 0.0])
    out = P.apply_penalties(x, [0, 1, 1, 9], 384, 2.0, 0.5, 0.25)
    assert abs(out[0].item() - (1.0 - 0.5 - 0.25)) < 1e-6                 # positive: divided
    assert abs(out[1].item() - (-4.0 - 1.0 - 0.25)) < 1e-6                # negative: multiplied; count 2
    assert out[2] == 1.0 and out[3] == 0.0
    out = P.apply_penalties(x, [0, 1, 1, 2], 1, 2.0, 0.0, 0.0)            # window of one: only the last token
    assert out[0] == 2.0 and out[1] == -2.0 and out[2] == 0.5
