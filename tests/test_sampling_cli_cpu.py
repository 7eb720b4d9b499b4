"""Sampling options, the counter-based uniforms, the penalty window and the
command line's argument rules, all on the CPU."""
import pytest

import hector_engine_amd  # noqa: F401
from hector_engine_amd.cli import is_plain_number, parse_args, parse_prompts
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
