"""Sampling options, the counter-based uniforms, the penalty window and the
command line's argument rules, all on the CPU."""
import pytest

import hector_engine_amd  # noqa: F401
from hector_engine_amd.cli import (context_length, gather_prompts, is_plain_number, parse_args, parse_prompts,
                                   sampling_options)
from hector_engine_amd.sampling import SamplingConfig, uniform_u32, window_counts
from tests.plain import qwen2_plain as P


def test_presets_are_the_references():
    g, c, b, d = (SamplingConfig.greedy(), SamplingConfig.creative(), SamplingConfig.balanced(),
                  SamplingConfig.deterministic())
    assert g.temperature == 0.0 and g.repetition_penalty == 1.2 and g.is_greedy
    assert (c.temperature, c.top_k, c.top_p, c.repetition_penalty, c.frequency_penalty) == (0.8, 50, 0.9, 1.15, 0.1)
    assert (b.temperature, b.top_k, b.repetition_penalty) == (0.7, 40, 1.2)
    assert d.is_greedy and not d.has_penalties
    assert SamplingConfig().temperature == 1.0 and SamplingConfig().top_k == 0 and SamplingConfig().top_p == 1.0
    assert SamplingConfig(temperature=0.009).is_greedy and not SamplingConfig(temperature=0.01).is_greedy


@pytest.mark.parametrize("bad", [dict(temperature=-1), dict(top_k=-2), dict(top_p=0.0), dict(top_p=1.5),
                                 dict(repetition_penalty=0.0)])
def test_validation(bad):
    with pytest.raises(ValueError):
        SamplingConfig(**bad).validate()


def test_uniforms_are_keyed_by_seed_sequence_and_step():
    seen = set()
    for seed in (0, 7):
        for seq in range(5):
            for step in range(20):
                u = uniform_u32(seed, seq, step)
                assert 0 <= u < 2 ** 32
                assert u == P.uniform_u32(seed, seq, step)        # the plain implementation's own copy
                seen.add(u)
    assert len(seen) == 200
    mean = sum(uniform_u32(1, 0, i) for i in range(4000)) / 4000 / 2 ** 32
    assert abs(mean - 0.5) < 0.02


def test_window_counts():
    assert window_counts([5, 5, 9, 5, 3], 3, 10) == ([9, 5, 3], [1, 1, 1])
    assert window_counts([5, 5, 9, 5, 3], 100, 10) == ([5, 9, 3], [3, 1, 1])
    assert window_counts([5, 11, -1], 100, 10) == ([5], [1])
    assert window_counts([], 4, 10) == ([], [])


def test_cli_argument_rules():
    assert is_plain_number("12") and is_plain_number("-3") and not is_plain_number("5,17") and not is_plain_number("1.5")
    ns, model, prompt, max_tokens, temp = parse_args(["m"])
    assert (model, prompt, max_tokens, temp) == ("m", None, 100, 0.0)
    _, model, prompt, max_tokens, temp = parse_args(["m", "5,17,3", "20", "0.8"])
    assert (model, prompt, max_tokens, temp) == ("m", "5,17,3", 20, 0.8)
    _, model, prompt, max_tokens, temp = parse_args(["m", "20", "0.5"])          # no prompt: a plain number is max_tokens
    assert (prompt, max_tokens, temp) == (None, 20, 0.5)
    ns, model, prompt, max_tokens, temp = parse_args(["--model", "m", "--ctx", "512", "--temp", "0.7"])
    assert (model, ns.ctx, temp) == ("m", 512, 0.7)
    assert parse_prompts("5,17,3;9 2") == [[5, 17, 3], [9, 2]]
    assert parse_prompts("raw:1,2") == [[1, 2]]


def test_cli_flags(tmp_path, monkeypatch):
    """Every flag of the command line: random weights from a configuration file and a seed,
    prompts from --tokens (repeated) and from a file, sampling options (a flag wins over the
    reference's HELIOS_* variable, which wins over the default), context and slots, profiling."""
    ns, model, prompt, max_tokens, temp = parse_args(
        ["--random", "cfg.json", "--seed", "9", "--tokens", "1,2,3", "--tokens", "4 5", "--max-new-tokens", "7",
         "--temperature", "0.8", "--top-k", "20", "--top-p", "0.5", "--sampler-seed", "3", "--max-seq", "256",
         "--slots", "2", "--profile", "--dtype", "float32", "--stop-ids", "5,6", "--no-graph"])
    assert (model, ns.random, ns.seed, prompt, max_tokens, temp) == (None, "cfg.json", 9, None, 7, 0.8)
    assert (ns.ctx, ns.slots, ns.profile, ns.dtype, ns.stop_ids, ns.no_graph) == (256, 2, True, "float32", "5,6", True)
    f = tmp_path / "prompts.txt"
    f.write_text("7,8,9\n\n# a comment\n10 11  # two ids\n")
    ns.tokens_file = str(f)
    assert gather_prompts(ns, "12;13,14") == [[1, 2, 3], [4, 5], [7, 8, 9], [10, 11], [12], [13, 14]]
    opts = sampling_options(ns, temp)
    assert (opts["top_k"], opts["top_p"], opts["seed"], opts["temperature"]) == (20, 0.5, 3, 0.8)
    # variables of the reference's session stand in for absent flags; flags win
    for k, v in (("HELIOS_TOPK", "11"), ("HELIOS_TOPP", "0.7"), ("HELIOS_SEED", "5"), ("HELIOS_REP", "1.3"),
                 ("HELIOS_FREQ", "0.2"), ("HELIOS_WINDOW", "64"), ("HELIOS_CTX", "1000")):
        monkeypatch.setenv(k, v)
    assert sampling_options(ns, temp)["top_k"] == 20
    ns2, *_ = parse_args(["m", "1,2", "5", "0.9"])
    o2 = sampling_options(ns2, 0.9)
    assert (o2["top_k"], o2["top_p"], o2["seed"], o2["repetition_penalty"], o2["frequency_penalty"],
            o2["penalty_window"]) == (11, 0.7, 5, 1.3, 0.2, 64)
    greedy = sampling_options(ns2, 0.0)
    assert (greedy["top_k"], greedy["top_p"]) == (0, 1.0)            # no truncation without sampling
    # the context: the flag as given; else HELIOS_CTX or 4096, never beyond what the model allows
    assert context_length(ns, 128) == 256 and context_length(ns2, 128) == 128 and context_length(ns2, 32768) == 1000
    monkeypatch.delenv("HELIOS_CTX")
    assert context_length(ns2, 32768) == 4096
    with pytest.raises(SystemExit):
        parse_args(["--model", "m", "--random", "c.json"])
    with pytest.raises(SystemExit):
        parse_args([])


def test_profile_table_has_the_references_columns():
    """Calls, total, average and share per op, largest total first, and a total line
    (src/engine.cpp:393-434)."""
    from hector_engine_amd.kernels.profiler import format_table, summarize
    rows = summarize({"gemm_blocksplit": (112, 5.6), "attention_decode_fused": (28, 0.7), "never": (0, 0.0)}, 6.3)
    assert [r[0] for r in rows] == ["gemm_blocksplit", "attention_decode_fused"]
    assert rows[0][1:] == (112, 5.6, pytest.approx(0.05), pytest.approx(100 * 5.6 / 6.3))
    text = format_table(rows).splitlines()
    assert text[0] == "=== Engine Profile ===" and text[1].split() == ["Op", "Calls", "Total(ms)", "Avg(ms)", "%"]
    assert text[3].split() == ["gemm_blocksplit", "112", "5.60", "0.050", "88.9%"]
    assert text[-1].split() == ["TOTAL", "6.30"]
    assert format_table([]) == "No profiling data"


def test_bench_refuses_more_than_one_gpu_and_what_does_not_fit():
    """bench.py keeps its contract at one GPU: any other count is one line and exit status 2
    (before anything touches a GPU), and so is a prompt that does not fit the context."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    for args, needle in ((["--gpus", "2"], "one GPU"), (["--prompt", "9000"], "do not fit")):
        r = subprocess.run([sys.executable, os.path.join(root, "bench.py")] + args, capture_output=True, text=True,
                           timeout=120)
        assert r.returncode == 2, r.stderr
        assert needle in r.stdout and len(r.stdout.strip().splitlines()) == 1


def test_bench_byte_and_flop_counts():
    """The roofline's figures for the benchmark shape: 7.6 billion parameters' worth of bytes a step
    and the prompt's flops (products and causal attention), as counted by hand."""
    import importlib.util
    import os
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    spec = importlib.util.spec_from_file_location("bench_module", os.path.join(root, "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    shape = bench.SHAPES["7b"][-1]
    D, I, V, L = 3584, 18944, 152064, 28
    per_layer = D * 4608 + 4608 + 3584 * D + 3 * D * I + 2 * D
    assert bench.weight_bytes(shape, L) == 2 * (L * per_layer + D + V * D)
    assert 14.1e9 < bench.weight_bytes(shape, L) < 14.3e9
    assert bench.kv_bytes_per_token(shape, L) == 57344
    T = 2048
    flops = bench.prefill_flops(shape, L, T)
    assert flops == L * (2 * T * (D * 4608 + 3584 * D + 3 * D * I) + 4 * 28 * 128 * T * (T + 1) // 2) + 2 * D * V
    assert 27.4e12 < flops < 27.7e12
