"""Host-side rules that choose how a step runs: the table of kernel routes, which library products
are cut along K, which one-token steps count as uneven."""
import torch

import hector_engine_amd  # noqa: F401


def test_kernel_routes_are_tried_in_order_and_say_what_is_registered():
    """The table keyed by (operation, dtypes): the first route that takes the case wins, `before`
    puts a narrower route in front, a name is registered once per key, unknown dtypes and a case
    nobody takes are errors that list what there is."""
    import pytest
    from hector_engine_amd.kernels import routes
    f16 = (torch.float16,)
    routes.register_route("toy_op", f16, "general", lambda c: c < 100, lambda: "general")
    try:
        routes.register_route("toy_op", f16, "small", lambda c: c < 10, lambda: "small", traits=("tiny",),
                              before="general")
        assert [r.name for r in routes.routes_of("toy_op", f16)] == ["small", "general"]
        assert routes.choose("toy_op", f16, 3).run() == "small" and "tiny" in routes.choose("toy_op", f16, 3).traits
        assert routes.choose("toy_op", f16, 30).run() == "general"
        assert routes.table()["toy_op (float16)"] == ["small", "general"]
        with pytest.raises(ValueError, match="registered already"):
            routes.register_route("toy_op", f16, "small", lambda c: True, lambda: None)
        with pytest.raises(ValueError, match="'nowhere'.*not registered"):
            routes.register_route("toy_op", f16, "other", lambda c: True, lambda: None, before="nowhere")
        with pytest.raises(ValueError, match="none of the routes .*small.*general.*takes 1000"):
            routes.choose("toy_op", f16, 1000)
        with pytest.raises(TypeError, match=r"toy_op: no kernel for \(float64\); registered: \(float16\)"):
            routes.choose("toy_op", (torch.float64,), 1)
    finally:
        for name in [r.name for r in routes.routes_of("toy_op", f16)]:
            routes.unregister_route("toy_op", f16, name)
    assert routes.routes_of("toy_op", f16) == []
    with pytest.raises(ValueError, match="not registered"):
        routes.unregister_route("toy_op", f16, "small")


def test_which_route_a_product_and_an_attention_step_take():
    """The routes the parts register: products by dtypes, row count, K and the environment;
    attention by the cache's dtype, the step's kind and what the fused kernel takes."""
    import pytest
    from hector_engine_amd.kernels import routes
    from hector_engine_amd.parts.attention import AttentionCase
    from hector_engine_amd.parts.linear import ProductCase
    bf, f32 = torch.bfloat16, torch.float32
    table = routes.table()
    assert table["linear (bfloat16, bfloat16)"] == ["mfma", "plain", "library"]
    assert table["linear (float32, float32)"] == ["plain"] and table["linear (float32, bfloat16)"] == ["plain_widened"]
    assert table["attention (bfloat16)"] == ["fused_one_token", "plain", "mfma_one_token", "mfma_prompt"]
    assert table["attention (float32)"] == ["plain"]

    def product(rows, K=3584, fast=True, dtypes=(bf, bf)):
        return routes.choose("linear", dtypes, ProductCase(rows, 512, K, fast)).name
    assert [product(r) for r in (0, 1, 16, 17, 64, 65, 2048)] == ["library"] + ["mfma"] * 4 + ["library"] * 2
    assert product(8, K=3580) == "plain" and product(300, K=3580) == "plain"     # K not in steps of 8
    assert product(8, fast=False) == "plain" and product(300, fast=False) == "plain"
    assert product(8, dtypes=(f32, f32)) == "plain" and product(8, dtypes=(f32, bf)) == "plain_widened"
    with pytest.raises(TypeError, match=r"linear: no kernel for \(float16, bfloat16\); registered: .*\(bfloat16, bfloat16\)"):
        product(8, dtypes=(torch.float16, bf))
    # what a part may ask a route for: piece-major rows, the gated epilogue, the K slices of a product
    traits = {r.name: set(r.traits) for r in routes.routes_of("linear", (bf, bf))}
    assert traits == {"mfma": {"pieces", "gated", "k_slices"}, "plain": set(), "library": set()}

    def attention(all_single, fast=True, fusable=True, dtype=bf):
        return routes.choose("attention", (dtype,), AttentionCase(all_single, fast, fusable)).name
    assert attention(True) == "fused_one_token" and attention(True, fusable=False) == "mfma_one_token"
    assert attention(False) == "mfma_prompt" and attention(False, fusable=False) == "mfma_prompt"
    assert attention(True, fast=False) == "plain" and attention(False, fast=False) == "plain"
    assert attention(True, fast=False, dtype=f32) == "plain"


def test_which_library_products_are_cut_along_k():
    """The rule that sends a long-K product of up to 512 rows to the library in K slices: the down projections of
    the Qwen2 shapes in 2 to 8 slices, nothing for short K, wide outputs, more than 512 rows, or a K that does not divide."""
    from hector_engine_amd.parts.linear import Linear

    def slices(N, K, rows):
        return Linear(torch.empty(N, K, dtype=torch.bfloat16, device="meta"))._library_slices(rows)
    assert [slices(3584, 18944, r) for r in (65, 200, 256, 512, 513, 2048)] == [8, 8, 8, 4, 1, 1]
    assert slices(5120, 27648, 128) == 8 and slices(5120, 27648, 300) == 4
    assert slices(8192, 29568, 128) == 4 and slices(8192, 29568, 300) == 2
    assert slices(4608, 3584, 200) == 1 and slices(37888, 3584, 200) == 1 and slices(3584, 3584, 128) == 1
    assert slices(152064, 3584, 100) == 1
    assert slices(64, 8200, 100) == 1 and slices(64, 8208, 100) == 2 and slices(64, 8224, 100) == 4


def test_which_one_token_steps_count_as_uneven():
    """The attention part's hint for a one-token step in which one sequence has several times the keys of the
    others: the longest has 4096 or more and at least four times the mean; a single sequence, equal lengths or
    short ones do not count."""
    from hector_engine_amd.parts.attention import Attention, keys_uneven
    assert Attention.step_hint is keys_uneven

    def uneven(lengths, was=False):
        return keys_uneven(lengths, was)
    assert uneven([30000] + [200] * 7) and uneven([30000, 30000] + [500] * 62) and uneven([4096, 10, 10, 10, 10])
    assert not uneven([30000]) and not uneven([8000] * 8) and not uneven([16000, 16000] + [1000] * 6)
    assert not uneven([4000, 10, 10, 10, 10]) and not uneven([5000, 4000, 3000])
    # once up, the flag stays up until the longest has fewer than three times the mean
    assert not uneven([9000, 1000, 1000, 1000]) and uneven([9000, 1000, 1000, 1000], was=True)
    assert not uneven([5000, 1000, 1000, 1000], was=True) and not uneven([4000, 10, 10], was=True)


def test_sync_each_launch_names_the_op(monkeypatch):
    """The debugging mode waits for the GPU after every launch and, when that wait reports an
    error, raises one that names the op; outside the mode a launcher is called as it is."""
    from hector_engine_amd.kernels import profiler
    calls = []

    @profiler.op("toy_op")
    def launch(x):
        calls.append(x)
        return x + 1

    waits = []
    monkeypatch.setattr(torch.cuda, "synchronize", lambda *a: waits.append(1))
    assert launch(1) == 2 and waits == []                  # no mode, no wait
    with profiler.sync_each_launch():
        assert launch(2) == 3 and waits == [1]

        def broken(*a):
            raise RuntimeError("HIP error: an illegal memory access was encountered")
        monkeypatch.setattr(torch.cuda, "synchronize", broken)
        try:
            launch(3)
        except profiler.LaunchFault as exc:
            assert "toy_op" in str(exc) and "illegal memory access" in str(exc)
        else:
            raise AssertionError("the fault was not reported")
        try:
            with profiler.span("library_gemm"):
                pass
        except profiler.LaunchFault as exc:
            assert "library_gemm" in str(exc)
        else:
            raise AssertionError("the fault was not reported")
    assert launch(4) == 5 and calls == [1, 2, 3, 4]         # the mode ends with its context


def test_profiler_reads_its_oldest_events_on_the_way(monkeypatch):
    """A long profiled run does not pile up events: once MAX_PENDING launches wait to be read,
    the older half is read into the totals."""
    from hector_engine_amd.kernels import profiler

    class FakeEvent:
        def __init__(self, enable_timing=False):
            pass

        def record(self):
            pass

        def synchronize(self):
            pass

        def elapsed_time(self, other):
            return 0.5
    monkeypatch.setattr(torch.cuda, "Event", FakeEvent)
    monkeypatch.setattr(profiler, "MAX_PENDING", 8)
    prof = profiler.OpProfiler()
    for i in range(30):
        with prof.span("a" if i % 2 else "b"):
            pass
        assert len(prof._pending) < 8
    rows = {name: (calls, ms) for name, calls, ms, _, _ in prof.rows()}
    assert rows == {"a": (15, 7.5), "b": (15, 7.5)} and prof._pending == []
