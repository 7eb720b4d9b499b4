"""Each part alone against the plain function of the same name; and the
generality of the assembly: a toy mixer with state of its own, a toy position
encoding and toy schedules (a layer named twice, a layer that reads another
layer's cache) are registered here, built and stepped without a change to the
framework's files. The toys are test fixtures, not models."""
import dataclasses
import os

import pytest
import torch

from tests.helpers import close, rand_ids
from tests.plain import qwen2_plain as P

pytestmark = pytest.mark.gpu
PAGE = 64


@pytest.fixture(scope="module")
def fw():
    import hector_engine_amd  # noqa: F401
    from hector_engine_amd import parts
    from hector_engine_amd.cache.paged import PagedCache, RunPlan
    from hector_engine_amd.engine.scratch import ScratchPool

    class NS:
        pass

    ns = NS()
    ns.parts, ns.PagedCache, ns.RunPlan, ns.ScratchPool = parts, PagedCache, RunPlan, ScratchPool
    return ns


def env_for(fw, dtype, fast=True):
    return fw.parts.BuildEnv(torch.device("cuda:0"), dtype, fast)


def make_ctx(fw, env, q_lens, starts, slots):
    rows = sum(q_lens)
    positions = torch.cat([torch.arange(s, s + n) for s, n in zip(starts, q_lens)]).int().cuda()
    row_seq = torch.cat([torch.full((n,), i) for i, n in enumerate(q_lens)]).int().cuda()
    cu = torch.tensor([0] + list(torch.tensor(q_lens).cumsum(0)), dtype=torch.int32).cuda()
    return fw.parts.StepContext(
        rows=rows, num_seqs=len(q_lens), positions=positions, row_seq=row_seq,
        seq_slot=torch.tensor(slots, dtype=torch.int32).cuda(), cu_seqlens=cu,
        seq_start=torch.tensor(starts, dtype=torch.int32).cuda(), max_q_len=max(q_lens), max_keys=1024,
        all_single=all(n == 1 for n in q_lens), env=env, scratch=fw.ScratchPool(env.device),
        host={"q_lens": q_lens, "starts": starts, "slots": slots})


def rnd(*shape, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g) * scale


DT = [torch.float32, torch.bfloat16]


def tol(dtype):
    return dict(rtol=3e-6, atol=3e-6) if dtype == torch.float32 else dict(rtol=2 ** -6, atol=2 ** -6)


def near(got, want, dtype):
    """Error bound relative to the size of the result: a few fp32 ulp, or for bfloat16
    2^-6 of the largest value (two bf16 ulp there; several roundings are chained)."""
    scale = want.abs().max().item()
    err = (got - want).abs().max().item()
    bound = (1e-5 if dtype == torch.float32 else 2 ** -6) * max(scale, 1e-3)
    assert err <= bound, f"max error {err:.3g} above {bound:.3g} (scale {scale:.3g})"


@pytest.mark.parametrize("dtype", DT)
def test_rmsnorm_part(fw, dtype):
    env = env_for(fw, dtype)
    norm = fw.parts.build_part("norm", fw.parts.PartSpec("rmsnorm", {"size": 80, "eps": 3e-6}), "n.", env)
    assert list(norm.tensor_specs()) == ["n.weight"]
    w = (1 + 0.1 * rnd(80, seed=1)).to(dtype)
    norm.bind({"n.weight": w.cuda()})
    ctx = make_ctx(fw, env, [5], [0], [0])
    resid, delta = rnd(5, 80, seed=2), rnd(5, 80, seed=3).to(dtype)
    r = resid.clone().cuda()
    out = norm.add_norm(r, delta.cuda(), 5, ctx)
    assert out.dtype == dtype
    assert torch.allclose(r.cpu().double(), resid.double() + delta.double(), atol=1e-6)
    assert torch.allclose(out.cpu().double(), P.rmsnorm(r.cpu().double(), w.double(), 3e-6), **tol(dtype))


def test_rotary_part(fw):
    env = env_for(fw, torch.float32)
    rot = fw.parts.build_part("position", fw.parts.PartSpec("rotary", {"head_dim": 48, "theta": 50000.0}), "", env)
    inv, r = rot.rotary()
    assert r == 48 and torch.equal(inv.cpu(), P.rope_inv_freq(48, 50000.0))
    part = fw.parts.build_part("position", fw.parts.PartSpec(
        "rotary", {"head_dim": 64, "theta": 1e4, "partial_rotary_factor": 0.5}), "", env)
    assert part.rotary()[1] == 32 and not rot.custom and rot.tensor_specs() == {}


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("rows", [5, 100])
@pytest.mark.parametrize("inter", [136, 160, 37])
def test_gated_mlp_part(fw, dtype, rows, inter):
    env = env_for(fw, dtype)
    mlp = fw.parts.build_part("feed_forward", fw.parts.PartSpec(
        "gated_mlp", {"hidden_size": 80, "intermediate_size": inter}), "m.", env)
    specs = mlp.tensor_specs()
    assert {k: v.shape for k, v in specs.items()} == {
        "m.gate_proj.weight": (inter, 80), "m.up_proj.weight": (inter, 80), "m.down_proj.weight": (80, inter)}
    w = {k: rnd(*v.shape, seed=i, scale=0.1).to(dtype) for i, (k, v) in enumerate(specs.items())}
    mlp.bind({k: v.cuda() for k, v in w.items()})
    ctx = make_ctx(fw, env, [rows], [0], [0])
    x = rnd(rows, 80, seed=9).to(dtype)
    out = mlp.forward(x.cuda(), ctx)
    want = P.swiglu(x.double(), w["m.gate_proj.weight"].double(), w["m.up_proj.weight"].double(),
                    w["m.down_proj.weight"].double())
    assert torch.allclose(out.cpu().double(), want, **tol(dtype))


def attention_spec(fw, D, H, KVH, hd, window, bias=True, theta=1e4):
    return fw.parts.PartSpec("attention", {
        "hidden_size": D, "num_heads": H, "num_kv_heads": KVH, "head_dim": hd, "qkv_bias": bias,
        "window": window, "position": fw.parts.PartSpec("rotary", {"head_dim": hd, "theta": theta})})


def attention_weights(specs, dtype, seed=0):
    return {k: rnd(*v.shape, seed=seed + i, scale=0.08).to(dtype) for i, (k, v) in enumerate(specs.items())}


@pytest.mark.parametrize("dtype,fast", [(torch.float32, True), (torch.bfloat16, True), (torch.bfloat16, False)])
@pytest.mark.parametrize("window", [0, 9])
def test_attention_part_prompt_then_tokens(fw, dtype, fast, window):
    D, H, KVH, hd = 80, 6, 3, 32
    env = env_for(fw, dtype, fast)
    att = fw.parts.build_part("mixer", attention_spec(fw, D, H, KVH, hd, window), "a.", env)
    need = att.kv_need()
    assert (need.kv_heads, need.head_dim, need.window, need.v_dim) == (KVH, hd, window, hd) and att.state_bytes() == 0
    # its pages are as large as its kernels keep them: keys in steps of 32 dims, values in tiles of 16
    assert (need.k_elems, need.v_elems) == (64 * 32 * ((hd + 31) // 32), 64 * 16 * ((hd + 15) // 16))
    w = attention_weights(att.tensor_specs(), dtype)
    att.bind({k: v.cuda() for k, v in w.items()})
    cache = fw.PagedCache([fw.RunPlan(att.kv_need(), None)], max_tokens=1024, max_slots=4, max_seq_len=512,
                          dtype=dtype, device=env.device)
    lc = cache.layer_cache(0)
    lens = [70, 3]
    slots = [cache.acquire(), cache.acquire()]
    xs = [rnd(n + 4, D, seed=20 + i).to(dtype) for i, n in enumerate(lens)]
    cfg = {"num_attention_heads": H, "num_key_value_heads": KVH, "head_dim": hd, "rope_theta": 1e4}
    wd = {k: v.double() for k, v in w.items()}
    want = [P.attention_block(cfg, wd, "a.", x.double(), torch.arange(x.shape[0]), window)[0] for x in xs]
    # the prompts in one step
    cache.reserve(list(zip(slots, lens)))
    ctx = make_ctx(fw, env, lens, [0, 0], slots)
    out = att.forward(torch.cat([x[:n] for x, n in zip(xs, lens)]).cuda(), ctx, lc).cpu().double()
    cache.commit(list(zip(slots, lens)))
    near(out[:70], want[0][:70], dtype)
    near(out[70:], want[1][:3], dtype)
    # then four single-token steps of both sequences
    for t in range(4):
        new = [n + t + 1 for n in lens]
        cache.reserve(list(zip(slots, new)))
        ctx = make_ctx(fw, env, [1, 1], [n + t for n in lens], slots)
        x = torch.stack([xs[0][70 + t], xs[1][3 + t]])
        out = att.forward(x.cuda(), ctx, lc).cpu().double()
        cache.commit(list(zip(slots, new)))
        near(out[0], want[0][70 + t], dtype)
        near(out[1], want[1][3 + t], dtype)


@pytest.mark.parametrize("dtype", DT)
def test_pre_norm_block_part(fw, dtype):
    D, H, KVH, hd, I = 64, 4, 2, 16, 96
    env = env_for(fw, dtype)
    norm = fw.parts.PartSpec("rmsnorm", {"size": D, "eps": 1e-5})
    spec = fw.parts.PartSpec("pre_norm", {
        "mixer_norm": norm, "feed_forward_norm": norm, "mixer": attention_spec(fw, D, H, KVH, hd, 0),
        "feed_forward": fw.parts.PartSpec("gated_mlp", {"hidden_size": D, "intermediate_size": I}),
        "names": {"mixer_norm": "ln1", "mixer": "att", "feed_forward_norm": "ln2", "feed_forward": "ff"}})
    block = fw.parts.build_part("block", spec, "L.", env)
    specs = block.tensor_specs()
    assert "L.ln1.weight" in specs and "L.att.q_proj.bias" in specs and "L.ff.down_proj.weight" in specs
    w = {k: (1 + rnd(*v.shape, seed=i, scale=0.1) if "ln" in k else rnd(*v.shape, seed=i, scale=0.1)).to(dtype)
         for i, (k, v) in enumerate(specs.items())}
    block.bind({k: v.cuda() for k, v in w.items()})
    cache = fw.PagedCache([fw.RunPlan(block.mixer.kv_need(), None)], max_tokens=256, max_slots=2,
                          max_seq_len=128, dtype=dtype, device=env.device)
    slot = cache.acquire()
    cache.reserve([(slot, 20)])
    ctx = make_ctx(fw, env, [20], [0], [slot])
    x = rnd(20, D, seed=50)
    stream = fw.parts.ResidualStream(x.clone().cuda(), 20)
    block.forward(stream, ctx, cache.layer_cache(0))
    got = stream.materialize(ctx).cpu().double()
    wd = {k: v.double() for k, v in w.items()}
    cfg = {"num_attention_heads": H, "num_key_value_heads": KVH, "head_dim": hd, "rope_theta": 1e4}
    h = x.double()
    a, _ = P.attention_block(cfg, wd, "L.att.", P.rmsnorm(h, wd["L.ln1.weight"], 1e-5), torch.arange(20), 0)
    h = h + a
    h = h + P.swiglu(P.rmsnorm(h, wd["L.ln2.weight"], 1e-5), wd["L.ff.gate_proj.weight"],
                     wd["L.ff.up_proj.weight"], wd["L.ff.down_proj.weight"])
    near(got, h, dtype)


@pytest.mark.parametrize("dtype", DT)
def test_embedding_and_heads(fw, dtype):
    env = env_for(fw, dtype)
    emb = fw.parts.build_part("embedding", fw.parts.PartSpec("token_embedding", {"vocab_size": 301, "hidden_size": 80}), "e.", env)
    tied = fw.parts.build_part("head", fw.parts.PartSpec("linear_head", {"vocab_size": 301, "hidden_size": 80, "tied_to": "e.weight"}), "h.", env)
    own = fw.parts.build_part("head", fw.parts.PartSpec("linear_head", {"vocab_size": 301, "hidden_size": 80}), "h.", env)
    assert tied.tensor_specs() == {} and list(own.tensor_specs()) == ["h.weight"]
    table, hw = rnd(301, 80, seed=1).to(dtype), rnd(301, 80, seed=2).to(dtype)
    tensors = {"e.weight": table.cuda(), "h.weight": hw.cuda()}
    for p in (emb, tied, own):
        p.bind(tensors)
    assert tied.linear.weight.data_ptr() == emb.table.data_ptr()            # an alias, not a copy
    ctx = make_ctx(fw, env, [4], [0], [0])
    ids = torch.tensor([3, 300, 0, 17], dtype=torch.int32).cuda()
    h = emb.forward(ids, 4, ctx)
    assert h.dtype == torch.float32 and torch.equal(h.cpu(), table.float()[[3, 300, 0, 17]])
    x = rnd(4, 80, seed=3).to(dtype)
    for head, wt in ((tied, table), (own, hw)):
        out = head.forward(x.cuda(), 4, ctx)
        assert out.dtype == torch.float32
        assert torch.allclose(out.cpu().double(), x.double() @ wt.double().T, rtol=1e-4, atol=1e-4)
    # 100 wanted rows: more than the MFMA kernels take at once (under bfloat16 the library writes the fp32 results)
    ctx = make_ctx(fw, env, [100], [0], [0])
    x = rnd(100, 80, seed=4).to(dtype)
    out = own.forward(x.cuda(), 100, ctx)
    assert torch.allclose(out.cpu().double(), x.double() @ hw.double().T, rtol=1e-4, atol=1e-4)


def test_a_weight_stored_in_32_bit_stays_so_under_bfloat16(fw):
    from hector_engine_amd.parts.linear import Linear
    env = env_for(fw, torch.bfloat16)
    w, b = rnd(37, 48, seed=1, scale=0.1), rnd(37, seed=2)
    lin = Linear(w.cuda(), b.cuda())
    ctx = make_ctx(fw, env, [9], [0], [0])
    x = rnd(9, 48, seed=3).to(torch.bfloat16)
    out = lin(x.cuda(), 9, ctx)
    assert out.dtype == torch.bfloat16 and lin.weight.dtype == torch.float32
    want = x.double() @ w.double().T + b.double()
    assert torch.allclose(out.cpu().double(), want, rtol=2 ** -7, atol=2 ** -7)


def test_a_kernel_route_registered_from_outside_is_the_one_that_runs(fw):
    """Another kernel for a product is added by registering a route: here one in front of the
    others that takes three rows of a 40-wide weight, counts its calls and runs the plain kernel.
    The Linear part is not edited for it; other sizes keep their routes."""
    from hector_engine_amd.kernels import routes
    from hector_engine_amd.parts.linear import Linear
    env = env_for(fw, torch.bfloat16)
    calls = []

    def run(lin, x, rows, ctx, bias, out_dtype, out, sink):
        calls.append(rows)
        return Linear._run_plain(lin, x, rows, ctx, bias, out_dtype, out, sink)
    key = (torch.bfloat16, torch.bfloat16)
    routes.register_route("linear", key, "toy_three_rows", lambda c: c.rows == 3 and c.N == 40, run, before="mfma")
    try:
        w, b = rnd(40, 48, seed=1, scale=0.1).to(torch.bfloat16), rnd(40, seed=2).to(torch.bfloat16)
        lin = Linear(w.cuda(), b.cuda())
        for rows in (3, 5):
            ctx = make_ctx(fw, env, [rows], [0], [0])
            assert lin.route(rows, ctx, torch.bfloat16).name == ("toy_three_rows" if rows == 3 else "mfma")
            assert not lin.reads_pieces(3, ctx) and lin.reads_pieces(5, ctx)
            x = rnd(rows, 48, seed=3).to(torch.bfloat16)
            out = lin(x.cuda(), rows, ctx)
            want = x.double() @ w.double().T + b.double()
            assert torch.allclose(out.cpu().double(), want, rtol=2 ** -7, atol=2 ** -7)
        assert calls == [3]
    finally:
        routes.unregister_route("linear", key, "toy_three_rows")
    assert [r.name for r in routes.routes_of("linear", key)] == ["mfma", "plain", "library"]


@pytest.mark.parametrize("rows", [65, 200, 512, 513])
@pytest.mark.parametrize("N,K,bias", [(72, 8192, True), (300, 9024, False), (40, 8200, True)])
def test_a_long_k_product_in_slices_through_the_library(fw, rows, N, K, bias):
    """More than 64 rows against a weight with a long K and few output columns (a down projection):
    up to 512 rows the library runs it as a batched product over K slices whose fp32 results are added
    in slice order; above, or where K does not divide, as one product. Either way the double-precision
    result, within bfloat16's rounding of the output."""
    from hector_engine_amd.parts.linear import Linear
    env = env_for(fw, torch.bfloat16)
    w = rnd(N, K, seed=11, scale=0.05).to(torch.bfloat16)
    b = rnd(N, seed=12).to(torch.bfloat16) if bias else None
    lin = Linear(w.cuda(), b.cuda() if bias else None)
    slices = lin._library_slices(rows)
    want = 1 if rows > 512 else 8          # a handful of the library's tiles at these sizes
    while want > 1 and K % (8 * want):
        want //= 2
    assert slices == want
    ctx = make_ctx(fw, env, [rows], [0], [0])
    x = rnd(rows, K, seed=13).to(torch.bfloat16)
    out = lin(x.cuda(), rows, ctx)
    want = x.double() @ w.double().T + (b.double() if bias else 0)
    assert out.dtype == torch.bfloat16
    assert torch.allclose(out.cpu().double(), want, rtol=2 ** -7, atol=2 ** -6 * want.abs().max().item())


# ---------------------------------------------------------------------------
# toys: registered here, in the test, through the public registries only
# ---------------------------------------------------------------------------
@pytest.fixture(scope="module")
def toys(fw):
    import hector_engine_amd as he
    from hector_engine_amd.config.base import ModelConfig, architecture_name, read_field
    parts = fw.parts

    # initial values of a kind of the toys' own: a rule registered from here gives a TensorSpec's
    # ("toy_near", centre) its mean and spread in the random-weights mode
    he.register_init("toy_near", lambda init: (float(init[1]), 0.05))

    @parts.register_part("mixer", "toy_running_mean")
    class RunningMean(parts.Mixer):
        """out_t = Wo . mean_{j<=t} x_j. Its state, the running sum and the count, lives in the
        cache's per-sequence state area; it keeps no keys or values."""
        graph_safe = False

        def __init__(self, params, prefix, env):
            super().__init__(prefix, env)
            self.D = parts.param(params, "hidden_size", int)

        def state_bytes(self):
            return 4 * (self.D + 1)

        def tensor_specs(self):
            return {self.prefix + "out.weight": parts.TensorSpec((self.D, self.D))}

        def bind(self, tensors):
            self.w = tensors[self.prefix + "out.weight"].float()

        def forward(self, x, ctx, cache):
            assert cache.kpool is None and cache.state.shape[1] == self.state_bytes()
            out = ctx.alloc((ctx.rows, self.D))
            r = 0
            for n, slot in zip(ctx.host["q_lens"], ctx.host["slots"]):
                st = cache.state[slot].view(torch.float32)          # [D + 1], zeroed at acquire
                sums = st[:self.D] + x[r:r + n].float().cumsum(0)
                counts = st[self.D] + torch.arange(1, n + 1, device=x.device)
                out[r:r + n] = ((sums / counts[:, None]) @ self.w.T).to(out.dtype)
                st[:self.D] = sums[-1]
                st[self.D] = counts[-1]
                r += n
            return out

    @parts.register_part("mixer", "toy_running_mean_on_device")
    class RunningMeanOnDevice(parts.Mixer):
        """The same mixer, planned on the device: its state rows are found through ctx.seq_slot
        and updated by index there, so that one-token steps can be captured into HIP graphs.
        Padding rows (row_seq -1) add zeros to a row of the state. It also names a step hint of
        its own (whether a sequence of the step holds 30 tokens or more): the engine keys its
        one-token graphs by it and hands the value over."""
        seen_hints = set()

        @staticmethod
        def step_hint(lengths, before):
            return max(lengths) >= 30

        def __init__(self, params, prefix, env):
            super().__init__(prefix, env)
            self.D = parts.param(params, "hidden_size", int)

        def state_bytes(self):
            return 4 * (self.D + 1)

        def tensor_specs(self):
            return {self.prefix + "out.weight": parts.TensorSpec((self.D, self.D))}

        def bind(self, tensors):
            self.w = tensors[self.prefix + "out.weight"].float()

        def forward(self, x, ctx, cache):
            D, rows = self.D, ctx.rows
            if ctx.all_single:
                type(self).seen_hints.add(ctx.hints[type(self).step_hint])
            st = cache.state.view(torch.float32)                       # [slots, D + 1]
            seq = ctx.row_seq[:rows].long()
            valid = seq >= 0
            seq = seq.clamp(min=0)
            slot = ctx.seq_slot.long()[seq].clamp(min=0)
            xf = x[:rows].float() * valid[:, None]
            ones = valid.float()
            if ctx.all_single:
                within, place = xf, ones
            else:     # sums over the rows of each sequence up to each row, without a trip to the host
                c = xf.double().cumsum(0)
                start = ctx.cu_seqlens.long()[seq]
                before = torch.where((start > 0)[:, None], c[(start - 1).clamp(min=0)], torch.zeros_like(c))
                within = (c - before).float()
                place = (torch.arange(rows, device=x.device) - start + 1).float() * ones
            sums = st[slot, :D] + within
            counts = (st[slot, D] + place).clamp(min=1)
            out = ctx.alloc((rows, D))
            out.copy_(((sums / counts[:, None]) @ self.w.T).to(out.dtype))
            st.index_add_(0, slot, torch.cat([xf, ones[:, None]], 1))
            return out

    @parts.register_part("mixer", "toy_wide_values")
    class WideValues(parts.Mixer):
        """One head whose keys are 16 wide (kept with 4 more elements a token: a code of its own)
        and whose values are 32 wide, in cache pages of its own group and of its own sizes: 64 x 20
        and 64 x 32 elements, token by token. The cache hands out pages of the sizes the mixer
        names and never looks inside them."""
        graph_safe = False

        def __init__(self, params, prefix, env):
            super().__init__(prefix, env)
            self.D = parts.param(params, "hidden_size", int)

        def kv_need(self):
            return parts.KVNeed(1, 16, 0, value_dim=32, k_page_elems=64 * 20)     # v: the default, 64 x value_dim

        def tensor_specs(self):
            p = self.prefix
            return {p + "q.weight": parts.TensorSpec((16, self.D)), p + "k.weight": parts.TensorSpec((16, self.D)),
                    p + "v.weight": parts.TensorSpec((32, self.D)), p + "o.weight": parts.TensorSpec((self.D, 32))}

        def bind(self, tensors):
            self.t = {n: tensors[self.prefix + n + ".weight"].float() for n in "qkvo"}

        def forward(self, x, ctx, cache):
            assert cache.kpool.shape[-1] == 64 * 20 and cache.vpool.shape[-1] == 64 * 32   # the sizes it asked for
            ar = torch.arange(64, device=x.device)[:, None]
            km = ar * 20 + torch.arange(16, device=x.device)[None, :]       # token t: elements 20 t .. 20 t + 15, then its code
            vm = ar * 32 + torch.arange(32, device=x.device)[None, :]
            xf = x[:ctx.rows].float()
            q, k, v = xf @ self.t["q"].T, xf @ self.t["k"].T, xf @ self.t["v"].T
            out = ctx.alloc((ctx.rows, self.D))
            r = 0
            for n, start, slot in zip(ctx.host["q_lens"], ctx.host["starts"], ctx.host["slots"]):
                table = cache.page_table[slot]
                for j in range(n):
                    p = start + j
                    cache.kpool[table[p // 64], 0, km[p % 64]] = k[r + j].to(cache.kpool.dtype)
                    cache.kpool[table[p // 64], 0, 20 * (p % 64) + 16:20 * (p % 64) + 20] = float(p % 7)   # the code
                    cache.vpool[table[p // 64], 0, vm[p % 64]] = v[r + j].to(cache.vpool.dtype)
                total = start + n
                pos = torch.arange(total, device=x.device)
                pages = table[pos // 64].long()
                keys = cache.kpool[pages, 0][torch.arange(total, device=x.device)[:, None], km[pos % 64]].float()
                vals = cache.vpool[pages, 0][torch.arange(total, device=x.device)[:, None], vm[pos % 64]].float()
                codes = cache.kpool[pages, 0][torch.arange(total, device=x.device), 20 * (pos % 64) + 16].float()
                assert torch.equal(codes, (pos % 7).float())      # what it wrote beside the keys is still there
                scores = q[r:r + n] @ keys.T / 4.0
                seen = pos[None, :] <= (start + torch.arange(n, device=x.device))[:, None]
                w = torch.softmax(scores.masked_fill(~seen, float("-inf")), -1)
                out[r:r + n] = ((w @ vals) @ self.t["o"].T).to(out.dtype)
                r += n
            return out

    @parts.register_part("position", "toy_scale_by_position")
    class ScaleByPosition(parts.PositionEncoding):
        """q, k <- q, k * (1 + pos / 100): not a rotation, so it runs through apply()."""
        custom = True

        def __init__(self, params, prefix, env):
            super().__init__(prefix, env)

        def apply(self, q, k, ctx):
            f = (1 + ctx.positions[:ctx.rows].float() / 100)[:, None, None]
            q.copy_((q.float() * f).to(q.dtype))
            if k is not None:
                k.copy_((k.float() * f).to(k.dtype))

    @parts.register_part("feed_forward", "toy_top1_experts")
    class Top1Experts(parts.FeedForward):
        """A router picks one of E gated MLPs per token (fp32 logits, the lowest index on ties).
        Every expert runs on every row and a mask keeps the chosen one: slow and simple, and
        without a host decision, so one-token steps can still be captured."""

        def __init__(self, params, prefix, env):
            super().__init__(prefix, env)
            self.D = parts.param(params, "hidden_size", int)
            self.I = parts.param(params, "intermediate_size", int)
            self.E = parts.param(params, "experts", int)

        def tensor_specs(self):
            specs = {self.prefix + "router.weight": parts.TensorSpec((self.E, self.D))}
            for e in range(self.E):
                q = f"{self.prefix}experts.{e}."
                specs[q + "gate_proj.weight"] = parts.TensorSpec((self.I, self.D))
                specs[q + "up_proj.weight"] = parts.TensorSpec((self.I, self.D))
                specs[q + "down_proj.weight"] = parts.TensorSpec((self.D, self.I))
            return specs

        def bind(self, tensors):
            self.t = {k[len(self.prefix):]: v for k, v in tensors.items() if k.startswith(self.prefix)}

        def forward(self, x, ctx):
            rows = ctx.rows
            xs = x[:rows]
            chosen = (xs.float() @ self.t["router.weight"].float().T).argmax(-1)
            out = ctx.alloc((rows, self.D))
            out.zero_()
            for e in range(self.E):
                g = xs @ self.t[f"experts.{e}.gate_proj.weight"].T
                u = xs @ self.t[f"experts.{e}.up_proj.weight"].T
                y = (torch.nn.functional.silu(g.float()) * u.float()).to(xs.dtype) @ self.t[f"experts.{e}.down_proj.weight"].T
                out += y * (chosen == e)[:, None].to(y.dtype)
            return out

    @parts.register_part("norm", "toy_centered")
    class Centered(parts.Norm):
        """y = (x - mean x) / sqrt(var x + eps) * weight: not of the form a pair of products can
        carry, so every reader gets plain rows from add_norm."""

        def __init__(self, params, prefix, env):
            super().__init__(prefix, env)
            self.size = parts.param(params, "size", int)
            self.eps = parts.param(params, "eps", float)

        def tensor_specs(self):
            return {self.prefix + "weight": parts.TensorSpec((self.size,), ("toy_near", 0.9))}

        def bind(self, tensors):
            self.w = tensors[self.prefix + "weight"].float()
            assert 0.6 < self.w.mean().item() < 1.2 and self.w.std().item() > 0     # the registered rule made them

        def add_norm(self, resid, delta, rows, ctx, want_out=True):
            r = resid[:rows]
            if delta is not None:
                r += delta[:rows].float()
            if not want_out:
                return None
            c = r - r.mean(-1, keepdim=True)
            out = ctx.alloc((rows, self.size))
            out.copy_((c * torch.rsqrt((c * c).mean(-1, keepdim=True) + self.eps) * self.w).to(out.dtype))
            return out

    @parts.register_part("block", "toy_parallel")
    class Parallel(parts.Block):
        """x = x + mixer(norm(x)) + feed_forward(norm(x)): one norm, both branches read it."""

        def __init__(self, params, prefix, env):
            super().__init__(prefix, env)
            self.norm = parts.build_part("norm", parts.param(params, "norm", parts.PartSpec), prefix + "ln.", env)
            self.mixer = parts.build_part("mixer", parts.param(params, "mixer", parts.PartSpec), prefix + "mix.", env)
            self.feed_forward = parts.build_part("feed_forward", parts.param(params, "feed_forward", parts.PartSpec),
                                                 prefix + "ff.", env)

        def children(self):
            return [self.norm, self.mixer, self.feed_forward]

        def first_norm(self):
            return self.norm           # all it reads the stream through

        def tensor_specs(self):
            specs = {}
            for c in self.children():
                specs.update(c.tensor_specs())
            return specs

        def bind(self, tensors):
            for c in self.children():
                c.bind(tensors)

        def forward(self, stream, ctx, cache):
            n = stream.normed(self.norm, ctx)
            stream.add(self.mixer.forward(n, ctx, cache), ctx)
            stream.add(self.feed_forward.forward(n, ctx), ctx)

    @dataclasses.dataclass
    class ToyConfig(ModelConfig):
        vocab_size: int = 0
        hidden_size: int = 0
        kind: str = "state"

        @classmethod
        def from_dict(cls, d):
            return cls(architecture=architecture_name(d), vocab_size=read_field(d, "vocab_size", int),
                       hidden_size=read_field(d, "hidden_size", int), kind=read_field(d, "kind", str, "state"))

        def to_dict(self):
            return {"architectures": [self.architecture], "vocab_size": self.vocab_size,
                    "hidden_size": self.hidden_size, "kind": self.kind}

    def toy_spec(cfg):
        D, V = cfg.hidden_size, cfg.vocab_size
        norm = parts.PartSpec("rmsnorm", {"size": D, "eps": 1e-5})
        ff = parts.PartSpec("gated_mlp", {"hidden_size": D, "intermediate_size": 2 * D + 8})
        names = {"mixer_norm": "ln1", "mixer": "mix", "feed_forward_norm": "ln2", "feed_forward": "ff"}

        def attn(pos):
            return parts.PartSpec("attention", {"hidden_size": D, "num_heads": 4, "num_kv_heads": 2,
                                                "head_dim": 16, "qkv_bias": True, "position": pos})

        def block(mixer, feed_forward=ff, mixer_norm=norm):
            return parts.PartSpec("pre_norm", {"mixer_norm": mixer_norm, "feed_forward_norm": norm, "mixer": mixer,
                                               "feed_forward": feed_forward, "names": names})

        rotary = parts.PartSpec("rotary", {"head_dim": 16, "theta": 1e4})
        routed = parts.PartSpec("toy_top1_experts", {"hidden_size": D, "intermediate_size": D + 16, "experts": 3})
        if cfg.kind in ("state", "device_state", "wide_values"):
            middle = {"state": "toy_running_mean", "device_state": "toy_running_mean_on_device",
                      "wide_values": "toy_wide_values"}[cfg.kind]
            mixers = [attn(rotary), parts.PartSpec(middle, {"hidden_size": D}), attn(rotary)]
            schedule = [parts.ScheduleEntry(0), parts.ScheduleEntry(1), parts.ScheduleEntry(2)]
        elif cfg.kind == "position":
            mixers = [attn(parts.PartSpec("toy_scale_by_position")), attn(parts.PartSpec("none"))]
            schedule = [parts.ScheduleEntry(0), parts.ScheduleEntry(1)]
        elif cfg.kind == "twice":
            mixers = [attn(rotary), attn(rotary)]
            schedule = [parts.ScheduleEntry(0), parts.ScheduleEntry(1), parts.ScheduleEntry(1)]
        elif cfg.kind == "routed":   # the last layer's feed-forward routes each token to one of three experts
            mixers = [attn(rotary), attn(rotary)]
            schedule = [parts.ScheduleEntry(0), parts.ScheduleEntry(1)]
        else:   # "shared": the third run reads the keys and values the second run wrote
            mixers = [attn(rotary), attn(rotary)]
            schedule = [parts.ScheduleEntry(0), parts.ScheduleEntry(1), parts.ScheduleEntry(1, cache_from=1)]
        layers = [parts.LayerSpec(f"layers.{i}.", block(m, routed if cfg.kind == "routed" and i == 1 else ff))
                  for i, m in enumerate(mixers)]
        if cfg.kind in ("parallel", "parallel_rms"):   # another arrangement (and another norm) between pre-norm blocks
            centered = parts.PartSpec("toy_centered", {"size": D, "eps": 1e-4}) if cfg.kind == "parallel" else norm
            layers = [parts.LayerSpec("layers.0.", block(attn(rotary))),
                      parts.LayerSpec("layers.1.", parts.PartSpec("toy_parallel", {"norm": centered, "mixer": attn(rotary),
                                                                                   "feed_forward": ff})),
                      parts.LayerSpec("layers.2.", block(attn(rotary), mixer_norm=centered))]
            schedule = [parts.ScheduleEntry(0), parts.ScheduleEntry(1), parts.ScheduleEntry(2)]
        return parts.ModelSpec(
            hidden_size=D, vocab_size=V,
            embedding=parts.PartSpec("token_embedding", {"vocab_size": V, "hidden_size": D}),
            embedding_prefix="emb.",
            layers=layers,
            schedule=schedule, final_norm=norm, final_norm_prefix="norm.",
            head=parts.PartSpec("linear_head", {"vocab_size": V, "hidden_size": D}), head_prefix="head.",
            max_positions=512)

    he.register_architecture("ToyForCausalLM", ToyConfig, toy_spec)
    return ToyConfig


def toy_plain(w, kind, ids):
    """The toy models, whole sequences, from the plain implementation's functions."""
    S = len(ids)
    pos = torch.arange(S)
    cfg = {"num_attention_heads": 4, "num_key_value_heads": 2, "head_dim": 16, "rope_theta": 1e4}
    x = P.embedding(torch.tensor(ids), w["emb.weight"])
    H, KVH, hd = 4, 2, 16

    def attn(l, n, encode, kv=None):
        p = f"layers.{l}.mix."
        q = P.linear(n, w[p + "q_proj.weight"], w[p + "q_proj.bias"]).reshape(S, H, hd)
        q = encode(q)
        if kv is None:
            k = encode(P.linear(n, w[p + "k_proj.weight"], w[p + "k_proj.bias"]).reshape(S, KVH, hd))
            v = P.linear(n, w[p + "v_proj.weight"], w[p + "v_proj.bias"]).reshape(S, KVH, hd)
        else:
            k, v = kv
        return P.linear(P.attention(q, k, v, pos, pos), w[p + "o_proj.weight"]), (k, v)

    margins = []

    def ff(l, h):
        p = f"layers.{l}."
        n2 = P.rmsnorm(h, w[p + "ln2.weight"], 1e-5)
        if p + "ff.router.weight" in w:      # one expert per token
            logits = n2 @ w[p + "ff.router.weight"].T
            top = logits.topk(2, -1).values
            margins.append((top[:, 0] - top[:, 1]) / logits.abs().max())
            chosen = [P.argmax_lowest(r) for r in logits]
            rows = [P.swiglu(n2[i:i + 1], w[f"{p}ff.experts.{e}.gate_proj.weight"], w[f"{p}ff.experts.{e}.up_proj.weight"],
                             w[f"{p}ff.experts.{e}.down_proj.weight"]) for i, e in enumerate(chosen)]
            return h + torch.cat(rows)
        return h + P.swiglu(n2, w[p + "ff.gate_proj.weight"], w[p + "ff.up_proj.weight"], w[p + "ff.down_proj.weight"])

    rot = lambda t: P.rope(t, pos, 1e4)
    scale = lambda t: t * (1 + pos.double() / 100)[:, None, None]
    same = lambda t: t
    if kind in ("parallel", "parallel_rms"):
        def centered(h, g):
            if kind == "parallel_rms":
                return P.rmsnorm(h, g, 1e-5)
            c = h - h.mean(-1, keepdim=True)
            return c / torch.sqrt((c * c).mean(-1, keepdim=True) + 1e-4) * g

        def mlp(l, n):
            p = f"layers.{l}.ff."
            return P.swiglu(n, w[p + "gate_proj.weight"], w[p + "up_proj.weight"], w[p + "down_proj.weight"])
        x = ff(0, x + attn(0, P.rmsnorm(x, w["layers.0.ln1.weight"], 1e-5), rot)[0])
        n = centered(x, w["layers.1.ln.weight"])
        x = x + attn(1, n, rot)[0] + mlp(1, n)
        x = ff(2, x + attn(2, centered(x, w["layers.2.ln1.weight"]), rot)[0])
        return P.linear(P.rmsnorm(x, w["norm.weight"], 1e-5), w["head.weight"])
    if kind in ("state", "device_state"):
        runs = [(0, rot, None), (1, "mean", None), (2, rot, None)]
    elif kind == "wide_values":
        runs = [(0, rot, None), (1, "wide", None), (2, rot, None)]
    elif kind == "position":
        runs = [(0, scale, None), (1, same, None)]
    elif kind == "twice":
        runs = [(0, rot, None), (1, rot, None), (1, rot, None)]
    elif kind == "routed":
        runs = [(0, rot, None), (1, rot, None)]
    else:
        runs = [(0, rot, None), (1, rot, None), (1, rot, 1)]
    kvs = {}
    for e, (l, enc, src) in enumerate(runs):
        n = P.rmsnorm(x, w[f"layers.{l}.ln1.weight"], 1e-5)
        if enc == "mean":
            a = (n.cumsum(0) / torch.arange(1, S + 1)[:, None]) @ w[f"layers.{l}.mix.out.weight"].T
        elif enc == "wide":      # one head, keys of 16 and values of 32, scale 1/4, causal
            m = f"layers.{l}.mix."
            scores = (n @ w[m + "q.weight"].T) @ (n @ w[m + "k.weight"].T).T / 4.0
            scores = scores.masked_fill(pos[None, :] > pos[:, None], float("-inf"))
            a = (torch.softmax(scores, -1) @ (n @ w[m + "v.weight"].T)) @ w[m + "o.weight"].T
        else:
            a, kvs[e] = attn(l, n, enc, kvs[src] if src is not None else None)
        x = ff(l, x + a)
    out = P.linear(P.rmsnorm(x, w["norm.weight"], 1e-5), w["head.weight"])
    if margins:      # the routed toy: also how clear each token's choice of expert was
        return out, margins[-1]
    return out


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("kind", ["state", "position", "twice", "shared", "parallel", "parallel_rms", "wide_values"])
def test_toy_models_build_and_step(fw, toys, tmp_path, kind, dtype):
    import hector_engine_amd as he
    from hector_engine_amd.engine.engine import StepEntry
    cfg = toys(architecture="ToyForCausalLM", vocab_size=97, hidden_size=64, kind=kind)
    folder = str(tmp_path / kind)
    he.write_random_model(cfg, 5, folder)
    assert he.load_config(folder) == cfg
    w = {k: v.double() for k, v in P.read_safetensors(os.path.join(folder, "model.safetensors")).items()}
    eng = he.Engine(folder, dtype=dtype, max_tokens=1024, max_slots=2, max_seq_len=256)
    assert eng.use_graphs == (kind not in ("state", "wide_values"))     # the host-planning toys switch graphs off
    if kind == "wide_values":      # keys of 16 and values of 32: a cache group of its own, beside the attention layers'
        assert len(eng.cache.groups) == 2 and [len(g.runs) for g in eng.cache.groups] == [2, 1]
        need = eng.cache.groups[1].need
        assert (need.head_dim, need.v_dim) == (16, 32) and eng.cache.groups[0].need.v_dim == 16
        assert eng.cache.groups[1].vpool.shape[-1] == 64 * 32 and eng.cache.groups[0].vpool.shape[-1] == 64 * 16
    if kind.startswith("parallel"):
        assert eng.model.blocks[1].first_norm() is eng.model.blocks[1].norm
    if kind == "state":
        assert eng.cache.state_bytes_per_slot >= 4 * 65 and eng.model.run_plans()[1].kv is None
        assert len(eng.cache.groups) == 1 and len(eng.cache.groups[0].runs) == 2
    if kind == "twice":
        assert len(eng.cache.groups[0].runs) == 3          # a layer named twice has two caches
    if kind == "shared":
        assert len(eng.cache.groups[0].runs) == 2 and not eng.caches[2].writes
        assert eng.caches[2].kpool.data_ptr() == eng.caches[1].kpool.data_ptr()
    reqs = [rand_ids(97, n, 70 + n) for n in (70, 9, 33, 20)]
    want = [toy_plain(w, kind, r) for r in reqs]
    # whole, alone
    for r, t in zip(reqs, want):
        s = eng.acquire()
        close(eng.step([StepEntry(s, r, list(range(len(r))))]), t, dtype)
        eng.release(s)
    # two batches through two slots: prompts together, then one token each; shorter ones leave;
    # the second batch takes the slots (and their state rows) that the first gave back
    for batch in ([0, 1], [2, 3]):
        slots = {i: eng.acquire() for i in batch}
        fed = {i: len(reqs[i]) // 2 for i in batch}
        got = {i: [] for i in batch}
        logits = eng.step([StepEntry(slots[i], reqs[i][:fed[i]], list(range(fed[i]))) for i in batch])
        r0 = 0
        for i in batch:
            got[i].append(logits[r0:r0 + fed[i]].clone())
            r0 += fed[i]
        live = list(batch)
        while live:
            logits = eng.step([StepEntry(slots[i], [reqs[i][fed[i]]], [0]) for i in live])
            for j, i in enumerate(live):
                got[i].append(logits[j:j + 1].clone())
                fed[i] += 1
            for i in list(live):
                if fed[i] == len(reqs[i]):
                    eng.release(slots.pop(i))
                    live.remove(i)
        for i in batch:
            close(torch.cat(got[i]), want[i], dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_toy_feed_forward_with_routing(fw, toys, tmp_path, dtype):
    """A routed feed-forward registered in the test: built, stepped whole and token by token (captured
    one-token steps included), and fed with plain rows although the mixer before it left its result as
    rows for the norm (the part does not take those)."""
    import hector_engine_amd as he
    from hector_engine_amd.engine.engine import StepEntry
    cfg = toys(architecture="ToyForCausalLM", vocab_size=97, hidden_size=64, kind="routed")
    folder = str(tmp_path / "routed")
    he.write_random_model(cfg, 6, folder)
    w = {k: v.double() for k, v in P.read_safetensors(os.path.join(folder, "model.safetensors")).items()}
    eng = he.Engine(folder, dtype=dtype, max_tokens=1024, max_slots=2, max_seq_len=256)
    assert eng.use_graphs
    ids = rand_ids(97, 40, 91)
    want, margin = toy_plain(w, "routed", ids)
    clear = (margin > (0.0 if dtype == "float32" else 0.05)).nonzero().flatten().tolist()
    assert len(clear) >= 25
    s = eng.acquire()
    close(eng.step([StepEntry(s, ids, clear)]), want[clear], dtype)
    eng.release(s)
    s = eng.acquire()
    got = [eng.step([StepEntry(s, ids[:8], list(range(8)))])]
    for t in ids[8:]:
        got.append(eng.step([StepEntry(s, [t], [0])]).clone())
    close(torch.cat(got)[clear], want[clear], dtype)
    assert eng.stats["graph_replays"] > 20
    eng.release(s)


def test_bad_schedules_are_refused(fw, toys):
    import hector_engine_amd as he
    from hector_engine_amd.registry import model_spec
    from hector_engine_amd.engine.model import DecoderModel
    cfg = toys(architecture="ToyForCausalLM", vocab_size=50, hidden_size=64, kind="shared")
    env = env_for(fw, torch.float32)
    spec = model_spec(cfg)
    spec.schedule = [fw.parts.ScheduleEntry(0), fw.parts.ScheduleEntry(1, cache_from=1)]
    with pytest.raises(ValueError, match="earlier"):
        DecoderModel(spec, env)
    spec.schedule = [fw.parts.ScheduleEntry(0), fw.parts.ScheduleEntry(5)]
    with pytest.raises(ValueError, match="names layer 5"):
        DecoderModel(spec, env)
    with pytest.raises(KeyError, match="registered"):
        fw.parts.build_part("mixer", fw.parts.PartSpec("no_such_mixer"), "", env)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_state_of_fixed_size_under_graph_replay(fw, toys, tmp_path, dtype):
    """A mixer with state of its own that finds and updates its rows on the device through
    seq_slot: its one-token steps are captured and replayed (three sequences in a bucket of four:
    one padding row), every replay is compared with the plain implementation, and a second batch
    takes the slots, and the state rows, that the first gave back."""
    import hector_engine_amd as he
    from hector_engine_amd.engine.engine import StepEntry
    cfg = toys(architecture="ToyForCausalLM", vocab_size=97, hidden_size=64, kind="device_state")
    folder = str(tmp_path / "device_state")
    he.write_random_model(cfg, 8, folder)
    w = {k: v.double() for k, v in P.read_safetensors(os.path.join(folder, "model.safetensors")).items()}
    eng = he.Engine(folder, dtype=dtype, max_tokens=2048, max_slots=4, max_seq_len=256)
    assert eng.use_graphs and eng.cache.state_bytes_per_slot >= 4 * 65
    reqs = [rand_ids(97, n, 170 + n) for n in (40, 23, 31, 37, 18, 29)]
    want = [toy_plain(w, "device_state", r) for r in reqs]
    for batch in ([0, 1, 2], [3, 4, 5]):
        slots = {i: eng.acquire() for i in batch}
        fed = {i: 5 + i for i in batch}
        got = {i: [] for i in batch}
        logits = eng.step([StepEntry(slots[i], reqs[i][:fed[i]], list(range(fed[i]))) for i in batch])
        r0 = 0
        for i in batch:
            got[i].append(logits[r0:r0 + fed[i]].clone())
            r0 += fed[i]
        live = list(batch)
        while live:
            logits = eng.step([StepEntry(slots[i], [reqs[i][fed[i]]], [0]) for i in live])
            for j, i in enumerate(live):
                close(logits[j:j + 1], want[i][fed[i]:fed[i] + 1], dtype)     # each replay on its own
                got[i].append(logits[j:j + 1].clone())
                fed[i] += 1
            for i in list(live):
                if fed[i] == len(reqs[i]):
                    eng.release(slots.pop(i))
                    live.remove(i)
        for i in batch:
            close(torch.cat(got[i]), want[i], dtype)
    assert eng.stats["graph_replays"] > 40 and eng.stats["graph_captures"] >= 2
    # the toy's own step hint reached it, with both of its values, and each value has graphs of its own
    mixer = type(eng.model.blocks[1].mixer)
    assert mixer.seen_hints == {False, True}
    assert {hints[-1] for _, hints in eng._buckets} == {False, True}
