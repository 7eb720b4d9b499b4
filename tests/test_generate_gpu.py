"""Generation through the entry points on the GPU: greedy generation equals the
plain implementation's, sampled generation equals it given the same uniforms,
stop tokens, early finishers, batches in a row, penalties, and the command line."""
import os
import subprocess
import sys

import pytest
import torch

from tests.conftest import ROOT, TINY
from tests.helpers import rand_ids
from tests.plain import qwen2_plain as P

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def he():
    import hector_engine_amd
    return hector_engine_amd


def prompts_for(cfg, lengths, seed):
    return [rand_ids(cfg["vocab_size"], n, seed + i) for i, n in enumerate(lengths)]


@pytest.mark.parametrize("name,lengths,steps", [("A", [5, 9, 13], 8), ("B", [3, 7, 17, 30], 12), ("C", [60, 2, 31], 10)])
def test_greedy_generation_equals_plain(he, model_dirs, plain_models, name, lengths, steps):
    cfg, w = plain_models[name]
    prompts = prompts_for(cfg, lengths, 100)
    want = [P.generate(cfg, w, p, steps) for p in prompts]
    eng = he.Engine(model_dirs[name], dtype="float32", max_tokens=2048, max_seq_len=512, beyond_max_positions=True)
    got = he.generate(eng, prompts, max_new_tokens=steps)
    assert [r.tokens for r in got] == want
    assert all(r.finish_reason == "max_tokens" and r.prompt_tokens == len(p) for r, p in zip(got, prompts))
    # alone, in another order, and with two slots only (batches in a row): same tokens
    for p, t in zip(prompts, want):
        assert he.generate(eng, [p], max_new_tokens=steps)[0].tokens == t
    assert [r.tokens for r in he.generate(eng, prompts[::-1], max_new_tokens=steps)] == want[::-1]
    small = he.Engine(model_dirs[name], dtype="float32", max_tokens=2048, max_slots=2, max_seq_len=512, beyond_max_positions=True)
    assert [r.tokens for r in he.generate(small, prompts, max_new_tokens=steps)] == want
    assert small.cache.free_pages == small.cache.num_pages
    # bfloat16: the same tokens wherever the oracle's choice is clear
    eng16 = he.Engine(model_dirs[name], dtype="bfloat16", max_tokens=2048, max_seq_len=512, beyond_max_positions=True)
    got16 = he.generate(eng16, prompts, max_new_tokens=steps)
    for p, r, t in zip(prompts, got16, want):
        seq = list(p)
        for a, b in zip(r.tokens, t):
            if a != b:
                top = P.forward(cfg, w, seq)[-1].topk(2).values
                assert (top[0] - top[1]).item() < 0.02 * top[0].abs().item() + 1e-3     # a near tie
                break
            seq.append(a)


@pytest.mark.parametrize("name", ["A", "B"])
@pytest.mark.parametrize("kw", [dict(temperature=0.8, seed=7), dict(temperature=1.0, top_k=5, seed=1),
                                dict(temperature=0.7, top_k=40, top_p=0.9, seed=3)])
def test_sampled_generation_equals_plain(he, model_dirs, plain_models, name, kw):
    cfg, w = plain_models[name]
    prompts = prompts_for(cfg, [3, 7, 17, 30], 200)
    eng = he.Engine(model_dirs[name], dtype="float32", max_tokens=2048, max_seq_len=512, beyond_max_positions=True)
    got = he.generate(eng, prompts, max_new_tokens=12, sampling=he.SamplingConfig(**kw))
    for i, (p, r) in enumerate(zip(prompts, got)):
        want = P.generate(cfg, w, p, 12, temperature=kw["temperature"], top_k=kw.get("top_k", 0),
                          top_p=kw.get("top_p", 1.0), seed=kw["seed"], sequence=i)
        assert r.tokens == want
    # the draw is keyed by the request's index, not by the batch: one slot at a time, same tokens
    one = he.Engine(model_dirs[name], dtype="float32", max_tokens=2048, max_slots=1, max_seq_len=512, beyond_max_positions=True)
    again = he.generate(one, prompts, max_new_tokens=12, sampling=he.SamplingConfig(**kw))
    assert [r.tokens for r in again] == [r.tokens for r in got]


def test_random_generations(he, model_dirs, plain_models):
    """Sixty generations with random prompts, budgets, sampling options (greedy, temperature, top-k, top-p,
    penalties with short and long windows), stop tokens, runs of queued steps and fewer slots than prompts:
    the tokens of the plain implementation, request by request."""
    import random
    rng = random.Random(2)
    engines = {}
    for _ in range(60):
        name = rng.choice(list(TINY))
        cfg, w = plain_models[name]
        slots = rng.choice([1, 2, 3, 8])
        if (name, slots) not in engines:
            engines[(name, slots)] = he.Engine(model_dirs[name], dtype="float32", max_tokens=8 * 128, max_slots=slots,
                                               max_seq_len=128)
        eng = engines[(name, slots)]
        prompts = [[rng.randrange(cfg["vocab_size"]) for _ in range(rng.randint(1, 40))] for _ in range(rng.randint(1, 6))]
        steps = rng.randint(1, 24)
        T, top_k = rng.choice([0.0, 0.0, 0.5, 0.8, 1.0, 1.5]), rng.choice([0, 0, 1, 5, 40])
        top_p, seed = rng.choice([1.0, 1.0, 0.9, 0.5]), rng.randint(0, 1000)
        rep, freq, pres, win = 1.0, 0.0, 0.0, 384
        if rng.random() < 0.3:
            rep, freq, pres, win = rng.choice([1.0, 1.2]), rng.choice([0.0, 0.1]), rng.choice([0.0, 0.1]), rng.choice([4, 384])
        stop = set()
        if rng.random() < 0.4:
            free = P.generate(cfg, w, prompts[0], steps, T, top_k, top_p, seed, 0, (), rep, freq, pres, win)
            if free:
                stop = {free[rng.randrange(len(free))]}
        sampling = he.SamplingConfig(temperature=T, top_k=top_k, top_p=top_p, seed=seed, repetition_penalty=rep,
                                     frequency_penalty=freq, presence_penalty=pres, penalty_window=win)
        got = he.generate(eng, prompts, max_new_tokens=steps, sampling=sampling, stop_ids=sorted(stop),
                          run_of_steps=rng.choice([1, 2, 8, 32]))
        for i, (p, r) in enumerate(zip(prompts, got)):
            want = P.generate(cfg, w, p, steps, T, top_k, top_p, seed, i, stop, rep, freq, pres, win)
            assert r.tokens == want, (name, i, T, top_k, top_p, seed, (rep, freq, pres, win), stop)
        assert eng.cache.free_pages == eng.cache.num_pages


def test_stop_tokens_and_early_finishers(he, model_dirs, plain_models):
    cfg, w = plain_models["B"]
    prompts = prompts_for(cfg, [3, 7, 17, 30], 300)
    free = [P.generate(cfg, w, p, 12) for p in prompts]
    stop = {free[1][4], free[3][0]}                    # request 1 stops at its fifth token, request 3 at once
    want = [P.generate(cfg, w, p, 12, stop_ids=stop) for p in prompts]
    eng = he.Engine(model_dirs["B"], dtype="float32", max_tokens=2048, max_seq_len=512, beyond_max_positions=True)
    got = he.generate(eng, prompts, max_new_tokens=12, stop_ids=stop)
    assert [r.tokens for r in got] == want
    assert got[3].finish_reason == "eos" and got[3].tokens == []
    assert got[1].finish_reason == "eos" and len(got[1].tokens) <= 4
    assert all(t not in stop for r in got for t in r.tokens)
    assert eng.cache.free_pages == eng.cache.num_pages and eng.cache.book.slots.available == eng.cache.max_slots


@pytest.mark.parametrize("kw", [dict(), dict(temperature=0.9, top_k=20, seed=5)])
def test_runs_of_queued_steps_give_the_same_tokens(he, model_dirs, plain_models, kw):
    """Steps queued several at a time (ids handed from step to step on the device) against one
    step at a time: budgets that are no multiple of the run, a stop token inside a run, a
    sequence whose cache room ends inside one."""
    cfg, w = plain_models["B"]
    prompts = prompts_for(cfg, [3, 7, 17, 30, 50], 500)
    sampling = he.SamplingConfig(temperature=0.0, **kw) if not kw else he.SamplingConfig(**kw)
    eng = he.Engine(model_dirs["B"], dtype="float32", max_tokens=2048, max_seq_len=64)
    one = he.generate(eng, prompts, max_new_tokens=21, sampling=sampling, run_of_steps=1)
    stop = {one[1].tokens[9], one[2].tokens[2]}
    for budget, stops in ((21, ()), (13, stop), (40, stop)):
        a = he.generate(eng, prompts, max_new_tokens=budget, sampling=sampling, stop_ids=stops, run_of_steps=1)
        for run in (2, 8, 32):
            b = he.generate(eng, prompts, max_new_tokens=budget, sampling=sampling, stop_ids=stops, run_of_steps=run)
            assert [(r.tokens, r.finish_reason) for r in a] == [(r.tokens, r.finish_reason) for r in b]
        assert eng.cache.free_pages == eng.cache.num_pages
    assert {r.finish_reason for r in a} >= {"eos", "stop"}          # budget 40: the long prompts fill their room


def test_a_step_takes_its_tokens_from_the_device(he, model_dirs):
    from hector_engine_amd.engine.engine import StepEntry, StepError
    eng = he.Engine(model_dirs["A"], dtype="bfloat16", max_tokens=1024, max_seq_len=128)
    slots = [eng.acquire() for _ in range(3)]
    eng.step([StepEntry(s, [5, 6, 7 + s], [2]) for s in slots])
    toks = [11, 12, 13]
    for use_graph in (False, True, True):       # the first one-token step of a batch size runs eagerly
        want = eng.step([StepEntry(s, [t], [0]) for s, t in zip(slots, toks)]).clone()
        for s in slots:                          # the same step again, its tokens given on the device
            eng.cache.book.length[s] -= 1
        ids = torch.tensor(toks, dtype=torch.int32, device=eng.device)
        got = eng.step([StepEntry(s, [0], [0]) for s in slots], device_tokens=ids)
        assert torch.equal(got, want)
    with pytest.raises(StepError, match="device_tokens"):
        eng.step([StepEntry(slots[0], [1, 2], [1])], device_tokens=ids[:1])


def test_penalties(he, model_dirs, plain_models):
    cfg, w = plain_models["A"]
    p = prompts_for(cfg, [9], 400)[0]
    eng = he.Engine(model_dirs["A"], dtype="float32", max_tokens=1024, max_seq_len=512, beyond_max_positions=True)
    plainly = he.generate(eng, [p], max_new_tokens=16)[0].tokens
    cfg_s = he.SamplingConfig(temperature=0.0, repetition_penalty=1.3, frequency_penalty=0.2,
                              presence_penalty=0.1, penalty_window=6)
    got = he.generate(eng, [p], max_new_tokens=16, sampling=cfg_s)[0].tokens
    want = P.generate(cfg, w, p, 16, rep=1.3, freq=0.2, pres=0.1, penalty_window=6)
    assert got == want and got != plainly


def test_one_long_run_of_queued_steps_with_draws_and_penalties(he, model_dirs, plain_models):
    """Without stop ids the whole generation is one run of queued steps: 150 of them here, far
    more than the host keeps reads in flight, with random draws that go up eight steps at a time,
    a penalty window on the device that wraps round many times. Token for token what the plain loop
    gives, handed out in order."""
    cfg, w = plain_models["A"]
    prompts = prompts_for(cfg, [5, 21], 500)
    eng = he.Engine(model_dirs["A"], dtype="float32", max_tokens=1024, max_seq_len=512, beyond_max_positions=True)
    sampling = he.SamplingConfig(temperature=0.9, top_k=12, top_p=0.95, seed=11, repetition_penalty=1.2,
                                 frequency_penalty=0.1, presence_penalty=0.1, penalty_window=7)
    seen = {0: [], 1: []}
    got = he.generate(eng, prompts, max_new_tokens=150, sampling=sampling, stop_ids=(),
                      on_token=lambda i, tok: seen[i].append(tok))
    for i, (p, r) in enumerate(zip(prompts, got)):
        want = P.generate(cfg, w, p, 150, 0.9, 12, 0.95, 11, i, (), 1.2, 0.1, 0.1, 7)
        assert r.tokens == want and r.finish_reason == "max_tokens" and seen[i] == want
    assert eng.stats["graph_replays"] >= 140
    assert eng.cache.free_pages == eng.cache.num_pages


def test_cache_room_ends_a_sequence(he, model_dirs):
    eng = he.Engine(model_dirs["A"], dtype="bfloat16", max_tokens=128, max_slots=2, max_seq_len=64)
    r = he.generate(eng, [[1] * 60, [2] * 64], max_new_tokens=20)
    assert r[0].finish_reason == "stop" and len(r[0].tokens) == 5      # 60 + 4 fed fill 64 positions
    assert r[1].finish_reason == "context_full" and r[1].tokens == []


def test_command_line(model_dirs, plain_models):
    cfg, w = plain_models["A"]
    exe = os.path.join(ROOT, "bin", "hector_generate")
    out = subprocess.run([sys.executable, exe, model_dirs["A"], "5,17,3;9,2,77,13", "6", "--dtype", "float32"],
                         capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stderr
    want = [P.generate(cfg, w, p, 6) for p in ([5, 17, 3], [9, 2, 77, 13])]
    for i, t in enumerate(want):
        assert f"[{i}] prompt" in out.stdout and ",".join(map(str, t)) in out.stdout
    assert "Speed:" in out.stdout and "tok/s" in out.stdout and "Prompt: 7 tokens" in out.stdout
    env = dict(os.environ, HELIOS_SEED="7", HELIOS_TOPK="0", HELIOS_TOPP="1.0")
    out = subprocess.run([sys.executable, exe, "--model", model_dirs["A"], "--temp", "0.8", "5,17,3", "6",
                          "--dtype", "float32"], capture_output=True, text=True, timeout=120, env=env)
    assert out.returncode == 0, out.stderr
    t = P.generate(cfg, w, [5, 17, 3], 6, temperature=0.8, seed=7)
    assert ",".join(map(str, t)) in out.stdout


def test_command_line_flags(model_dirs, plain_models, tmp_path):
    """--random CONFIG.json --seed (the model write_random_model writes from the same configuration
    and seed), prompts from --tokens and --tokens-file, fewer slots than prompts, sampling flags in
    place of the variables, the kernel table of --profile, and the context bound."""
    import json
    import hector_engine_amd as he
    from hector_engine_amd.registry import config_from_dict
    from tests.conftest import TINY_B
    exe = os.path.join(ROOT, "bin", "hector_generate")
    cfg_file = tmp_path / "config.json"
    cfg_file.write_text(json.dumps(TINY_B))
    folder = str(tmp_path / "model")
    he.write_random_model(config_from_dict(dict(TINY_B)), 21, folder, "bfloat16")
    cfg, w = P.read_model(folder)
    prompts = [[5, 17, 3], [9, 2, 77, 13], [100, 200, 300, 1, 2]]
    tokens_file = tmp_path / "prompts.txt"
    tokens_file.write_text("9,2,77,13\n100 200 300 1 2\n")
    out = subprocess.run([sys.executable, exe, "--random", str(cfg_file), "--seed", "21", "--tokens", "5,17,3",
                          "--tokens-file", str(tokens_file), "--max-new-tokens", "7", "--temperature", "0.8",
                          "--top-k", "0", "--top-p", "1.0", "--sampler-seed", "7", "--slots", "2", "--dtype", "float32",
                          "--profile"], capture_output=True, text=True, timeout=180)
    assert out.returncode == 0, out.stderr
    for i, p in enumerate(prompts):
        t = P.generate(cfg, w, p, 7, temperature=0.8, seed=7, sequence=i)
        assert f"[{i}] prompt {len(p)} tokens -> 7 tokens (max_tokens): " + ",".join(map(str, t)) in out.stdout
    assert "=== Engine Profile ===" in out.stdout and "attention_plain" in out.stdout and "TOTAL" in out.stdout
    assert "random weights for" in out.stdout and "seed 21" in out.stdout
    # more context than the configuration's positions is refused by name; within them --max-seq holds
    out = subprocess.run([sys.executable, exe, folder, "5,17,3", "2", "--max-seq", "1000"], capture_output=True,
                         text=True, timeout=120)
    assert out.returncode != 0 and "256 positions" in out.stderr
    out = subprocess.run([sys.executable, exe, folder, "5,17,3", "40", "--max-seq", "16", "--dtype", "float32",
                          "--stream"], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0 and "-> 14 tokens (stop)" in out.stdout, out.stdout + out.stderr
    # --stream: every id on a line of its own as it comes, the same ids as the closing report's
    streamed = [line.split("+ ")[1] for line in out.stdout.splitlines() if line.startswith("[0] + ")]
    assert len(streamed) == 14 and "(stop): " + ",".join(streamed) in out.stdout


def test_command_line_chat(model_dirs, plain_models):
    """--chat: the prompt of the command line is the first turn, every line of standard input a
    further one; each answer continues the whole context."""
    cfg, w = plain_models["A"]
    exe = os.path.join(ROOT, "bin", "hector_generate")
    out = subprocess.run([sys.executable, exe, model_dirs["A"], "5,17,3", "6", "--dtype", "float32", "--chat",
                          "--stop-ids", ""], input="9,2,77\n4 4\n\n8,8\n", capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stderr
    t0 = P.generate(cfg, w, [5, 17, 3], 6)
    t1 = P.generate(cfg, w, [5, 17, 3] + t0 + [9, 2, 77], 6)
    t2 = P.generate(cfg, w, [5, 17, 3] + t0 + [9, 2, 77] + t1 + [4, 4], 6)
    for n, (fed, t) in enumerate([(3, t0), (4, t1), (3, t2)]):
        assert f"[turn {n}] {fed} tokens in" in out.stdout and "(max_tokens, " in out.stdout
        assert "): " + ",".join(map(str, t)) in out.stdout
    assert "[turn 3]" not in out.stdout           # the empty line ended the conversation


def test_command_line_with_the_library_tuner(model_dirs, tmp_path):
    """--tune-gemm: tall bfloat16 products go through the library's tuner (its own process, since the
    tuner is process-wide); the same tokens as without it where the decision is clear."""
    exe = os.path.join(ROOT, "bin", "hector_generate")
    prompt = ",".join(str(7 + (i * 37) % 290) for i in range(256))         # 256 rows: a library product
    env = dict(os.environ, TMPDIR=str(tmp_path))
    runs = []
    for extra in ([], ["--tune-gemm"]):
        out = subprocess.run([sys.executable, exe, model_dirs["C"], prompt, "4", "--dtype", "bfloat16"] + extra,
                             capture_output=True, text=True, timeout=300, env=env)
        assert out.returncode == 0, out.stderr
        runs.append([l for l in out.stdout.splitlines() if l.startswith("[0]")])
    assert runs[0] and runs[1]
    first = lambda lines: lines[0].rsplit(": ", 1)[-1].split(",")[0]       # "...(max_tokens): 12,7,..."
    assert first(runs[0]).isdigit() and first(runs[0]) == first(runs[1])
    # a row count that will hardly come again (77: above the hand-written kernels' 64, no multiple of 256)
    # runs without the tuner's trials; the file of results holds the 256-row products only
    odd = ",".join(str(3 + (i * 29) % 290) for i in range(77))
    out = subprocess.run([sys.executable, exe, model_dirs["C"], odd, "2", "--dtype", "bfloat16", "--tune-gemm"],
                         capture_output=True, text=True, timeout=300, env=env)
    assert out.returncode == 0, out.stderr
    results = [os.path.join(d, f) for d, _, fs in os.walk(str(tmp_path)) for f in fs if f.endswith(".csv")]
    assert results
    text = "".join(open(f).read() for f in results)
    assert "_256_" in text and "_77_" not in text


def test_tuning_policy_and_nested_blocks():
    from hector_engine_amd.kernels import library_tuning
    assert all(library_tuning.worth_tuning(r) for r in (256, 2048, 16384))
    assert not any(library_tuning.worth_tuning(r) for r in (1, 17, 64, 65, 77, 1937, 2049))


def test_smoke_entry():
    sys.path.insert(0, ROOT)
    import __graft_entry__
    __graft_entry__.smoke()


def test_default_stop_ids_are_the_model_folders_own(he, model_dirs, plain_models, tmp_path):
    """Without stop ids from the caller a sequence ends at the ids the model folder names: those of
    its generation_config.json (here: a list of two, as instruction-tuned checkpoints have), else
    those of its config.json; stop_ids=() switches them off."""
    import json
    import shutil
    cfg, w = plain_models["A"]
    prompts = prompts_for(cfg, [5, 9], 900)
    free = [P.generate(cfg, w, p, 10) for p in prompts]
    stop = [free[0][3], free[1][6]]
    want = [P.generate(cfg, w, p, 10, stop_ids=set(stop)) for p in prompts]
    assert len(want[0]) <= 3 and len(want[1]) <= 6
    folder = str(tmp_path / "with_generation_config")
    shutil.copytree(model_dirs["A"], folder)
    with open(os.path.join(folder, "generation_config.json"), "w") as f:
        json.dump({"eos_token_id": stop, "do_sample": True}, f)
    eng = he.Engine(folder, dtype="float32", max_tokens=1024, max_seq_len=128)
    assert eng.stop_ids == stop
    got = he.generate(eng, prompts, max_new_tokens=10)
    assert [r.tokens for r in got] == want and got[0].finish_reason == "eos"
    assert [r.tokens for r in he.generate(eng, prompts, max_new_tokens=10, stop_ids=())] == free
    # config.json's id counts when generation_config.json is absent
    os.remove(os.path.join(folder, "generation_config.json"))
    data = json.load(open(os.path.join(folder, "config.json")))
    data["eos_token_id"] = stop[0]
    json.dump(data, open(os.path.join(folder, "config.json"), "w"))
    eng = he.Engine(folder, dtype="float32", max_tokens=1024, max_seq_len=128)
    assert eng.stop_ids == [stop[0]]
    assert he.generate(eng, prompts[:1], max_new_tokens=10)[0].tokens == want[0]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_two_sessions_on_one_engine_share_the_weights_and_nothing_else(he, model_dirs, plain_models, name, dtype):
    """Several sessions over one loaded model, as the reference attaches sessions to one Model
    (src/inference_session.hpp:126-144): each has its slot, its sampler and its turn count, and
    turns that alternate between them give what each conversation gives alone. The second
    session samples, the first is greedy; a closed session's slot is taken by a third."""
    cfg, w = plain_models[name]
    V = cfg["vocab_size"]
    a1, a2, b1, b2, c1 = (rand_ids(V, n, 40 + i) for i, n in enumerate((9, 5, 66, 3, 12)))
    eng = he.Engine(model_dirs[name], dtype=dtype, max_tokens=1024, max_slots=2, max_seq_len=512,
                    beyond_max_positions=True)
    exact = dtype == "float32"
    hot = he.SamplingConfig(temperature=0.8, seed=3)
    sa, sb = he.Session(eng, stop_ids=()), he.Session(eng, hot, stop_ids=())
    assert sa.slot != sb.slot
    ra1 = sa.turn(a1, 7)
    rb1 = sb.turn(b1, 6)
    ra2 = sa.turn(a2, 8)
    rb2 = sb.turn(b2, 5)
    if exact:
        assert ra1.tokens == P.generate(cfg, w, a1, 7)
        assert rb1.tokens == P.generate(cfg, w, b1, 6, temperature=0.8, seed=3)
        assert ra2.tokens == P.generate(cfg, w, a1 + ra1.tokens + a2, 8)
        assert rb2.tokens == P.generate(cfg, w, b1 + rb1.tokens + b2, 5, temperature=0.8, seed=4)
    else:   # bfloat16: each conversation alone in a fresh engine gives the same tokens
        alone = he.Engine(model_dirs[name], dtype=dtype, max_tokens=1024, max_slots=1, max_seq_len=512,
                          beyond_max_positions=True)
        with he.Session(alone, stop_ids=()) as s:
            assert [s.turn(a1, 7).tokens, s.turn(a2, 8).tokens] == [ra1.tokens, ra2.tokens]
        with he.Session(alone, hot, stop_ids=()) as s:
            assert [s.turn(b1, 6).tokens, s.turn(b2, 5).tokens] == [rb1.tokens, rb2.tokens]
    assert sa.position == len(a1) + 7 + len(a2) + 8 - 1 and sb.position == len(b1) + 6 + len(b2) + 5 - 1
    freed = sa.slot
    sa.close()
    with he.Session(eng, stop_ids=()) as sc:      # the freed slot, used again beside the running one
        assert sc.slot == freed
        rc = sc.turn(c1, 6)
        if exact:
            assert rc.tokens == P.generate(cfg, w, c1, 6)
        rb3 = sb.turn(a2, 4)
        if exact:
            assert rb3.tokens == P.generate(cfg, w, b1 + rb1.tokens + b2 + rb2.tokens + a2, 4, temperature=0.8, seed=5)
    sb.close()
    assert eng.cache.free_pages == eng.cache.num_pages


@pytest.mark.parametrize("name", ["A", "B", "D"])
def test_a_session_of_turns_equals_plain_on_the_whole_context(he, model_dirs, plain_models, name):
    """A session keeps its slot: the second turn's tokens continue the first turn's context, the
    token that ended the first turn under its budget goes in front of them, every turn samples
    with numbers of its own (seed + turn), a stop token is neither given out nor left in the
    cache, and a rewind to the first turn's end followed by the same turn gives the same tokens.
    Configuration B keeps a window in some layers (a session then steps one token at a time where
    a stop token could come)."""
    cfg, w = plain_models[name]
    V = cfg["vocab_size"]
    p1, p2, p3 = rand_ids(V, 11, 1), rand_ids(V, 4, 2), rand_ids(V, 70, 3)
    eng = he.Engine(model_dirs[name], dtype="float32", max_tokens=1024, max_slots=2, max_seq_len=512,
                    beyond_max_positions=True)
    with he.Session(eng, stop_ids=()) as ses:
        assert ses.feed(p1[:4]) and ses.position == 4        # context without an answer, then the turn's rest
        r1 = ses.turn(p1[4:], 9)
        assert r1.tokens == P.generate(cfg, w, p1, 9) and r1.finish_reason == "max_tokens"
        ctx = p1 + r1.tokens
        assert ses.position == len(ctx) - 1
        sampling = he.SamplingConfig(temperature=0.8, seed=7)
        r2 = ses.turn(p2, 10, sampling=sampling)
        assert r2.tokens == P.generate(cfg, w, ctx + p2, 10, temperature=0.8, seed=7 + 1)
        at = ses.position
        ctx2 = ctx + p2 + r2.tokens
        # a long third turn (a prompt step of 70 tokens behind a context), then taken back and run again
        want3 = P.generate(cfg, w, ctx2 + p3, 6)
        assert ses.turn(p3, 6).tokens == want3
        if any(g.window for g in eng.cache.book.groups):
            # layers that keep a window have given pages back that the shorter sequence would read
            from hector_engine_amd.cache import CacheError
            with pytest.raises(CacheError, match="keeps a window"):
                ses.rewind(at)
        else:
            ses.rewind(at)
            ses.turns -= 1
            assert ses.turn([r2.tokens[-1]] + p3, 6).tokens == want3
    assert eng.cache.free_pages == eng.cache.num_pages
    # a stop token: the turn ends before it, the next turn continues behind the tokens given out
    stop = {P.generate(cfg, w, p1, 9)[4]}
    with he.Session(eng, stop_ids=stop) as ses:
        r = ses.turn(p1, 9)
        want = P.generate(cfg, w, p1, 9, stop_ids=stop)
        assert r.tokens == want and r.finish_reason == "eos" and ses.position == len(p1) + len(want)
        assert ses.turn(p2, 5).tokens == P.generate(cfg, w, p1 + want + p2, 5, stop_ids=stop)
    assert eng.cache.free_pages == eng.cache.num_pages
