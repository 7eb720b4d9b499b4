"""Command line in the manner of the reference's generation tools.

    hector_generate <model_dir> [prompt] [max_tokens=100] [temperature=0.0]

as test_generate_kv takes its arguments (test_generate_kv.cpp:43-65): the second
argument is the prompt unless it is a plain number, in which case it is
max_tokens. This library works on token ids, so the prompt is a list of ids
"5,17,3"; several prompts separated by ';' run as one batch. The flags of
tools/helios_runtime.cpp:261-263 are accepted too: --model, --ctx, --temp. The
sampling environment variables of the reference's session are read
(src/inference_session.cpp:380-385): HELIOS_REP, HELIOS_FREQ, HELIOS_WINDOW,
HELIOS_TOPK, HELIOS_TOPP, HELIOS_SEED, and HELIOS_CTX (helios_chat.cpp:549); a
flag wins over its variable. Options of this library's own: --random CONFIG.json
--seed N (random weights instead of a folder), --tokens / --tokens-file,
--max-new-tokens, --temperature, --top-k, --top-p, --sampler-seed, --max-seq,
--slots, --dtype, --stop-ids, --no-graph, --tune-gemm, --profile, --sync-each-launch,
--stream (print each sequence's ids as they come), --chat (one conversation: every line of
standard input is a turn of token ids, answered with the generated ids, the context staying in
the cache as in the reference's helios_chat; prompts given on the command line are the first turns).
Without --stop-ids a sequence ends at the model's own end-of-sequence ids: `eos_token_id` of
the folder's generation_config.json, else of its config.json.
It prints the generated ids and the reference's closing report
(test_generate_kv.cpp:294-300).
"""
from __future__ import annotations

import argparse
import os
import sys
import time


def _env(name: str, kind, default):
    v = os.environ.get(name)
    return default if v is None or v == "" else kind(v)


def parse_prompts(text: str) -> list[list[int]]:
    prompts = []
    for part in text.split(";"):
        part = part.strip()
        if part.startswith("raw:"):
            part = part[4:]
        if not part:
            continue
        prompts.append([int(t) for t in part.replace(" ", ",").split(",") if t != ""])
    return prompts


def is_plain_number(text: str) -> bool:
    """strtol consumes the whole string (test_generate_kv.cpp:55-61)."""
    try:
        int(text, 10)
        return True
    except ValueError:
        return False


def parse_args(argv: list[str]):
    ap = argparse.ArgumentParser(
        prog="hector_generate",
        usage="%(prog)s <model_dir> [prompt] [max_tokens] [temperature]\n"
              "   or: %(prog)s --model <model_dir> | --random <config.json> --seed N  [options] [prompt] [max_tokens]")
    ap.add_argument("--model", default=None, help="folder with config.json and model.safetensors")
    ap.add_argument("--random", default=None, metavar="CONFIG.json",
                    help="random weights for this configuration file instead of a model folder")
    ap.add_argument("--seed", type=int, default=0, help="seed of the random weights")
    ap.add_argument("--ctx", "--max-seq", dest="ctx", type=int, default=None,
                    help="longest sequence (HELIOS_CTX, else 4096, at most what the configuration allows)")
    ap.add_argument("--slots", type=int, default=None,
                    help="sequences that run together; more prompts than slots run batch after batch")
    ap.add_argument("--temp", "--temperature", dest="temp", type=float, default=None)
    ap.add_argument("--top-k", type=int, default=None, help="HELIOS_TOPK, else 50 when sampling")
    ap.add_argument("--top-p", type=float, default=None, help="HELIOS_TOPP, else 0.9 when sampling")
    ap.add_argument("--sampler-seed", type=int, default=None, help="HELIOS_SEED, else 0")
    ap.add_argument("--max-new-tokens", type=int, default=None)
    ap.add_argument("--tokens", action="append", default=[], metavar="ID,ID,...",
                    help="a prompt as token ids; repeat for a batch")
    ap.add_argument("--tokens-file", default=None, help="a file with one prompt of token ids a line")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--stop-ids", default=None, help="comma-separated stop token ids")
    ap.add_argument("--no-graph", action="store_true", help="run one-token steps without HIP graphs")
    ap.add_argument("--tune-gemm", action="store_true",
                    help="let the library's autotuner choose the kernels of tall matrix products (a second or so "
                         "per new shape)")
    ap.add_argument("--profile", action="store_true",
                    help="time every kernel with a pair of events (no HIP graphs) and print the table")
    ap.add_argument("--sync-each-launch", action="store_true",
                    help="debugging: wait for the GPU after every launch and name the op in an error")
    ap.add_argument("--stream", action="store_true",
                    help="print every token id as it comes ([sequence] + id), before the closing report")
    ap.add_argument("--chat", action="store_true",
                    help="one conversation in one slot: each prompt, then each line of standard input, is a turn")
    ap.add_argument("rest", nargs="*")
    ns = ap.parse_args(argv)
    rest = list(ns.rest)
    model = ns.model
    if model is None and ns.random is None:
        model = rest.pop(0) if rest else None
    if model is None and ns.random is None:
        ap.error("a model folder (or --random CONFIG.json) is needed")
    if model is not None and ns.random is not None:
        ap.error("--model and --random exclude each other")
    prompt = None
    if rest and not is_plain_number(rest[0]):
        prompt = rest.pop(0)
    max_tokens = int(rest.pop(0)) if rest else (ns.max_new_tokens if ns.max_new_tokens is not None else 100)
    temperature = float(rest.pop(0)) if rest else (ns.temp if ns.temp is not None else 0.0)
    return ns, model, prompt, max_tokens, temperature


def gather_prompts(ns, prompt: str | None) -> list[list[int]]:
    """The prompts of --tokens (each one), of --tokens-file (one a line) and of the positional
    argument (';' between prompts), in that order."""
    prompts: list[list[int]] = []
    for text in ns.tokens:
        prompts += parse_prompts(text)
    if ns.tokens_file is not None:
        with open(ns.tokens_file) as f:
            for line in f:
                line = line.split("#", 1)[0].strip()
                if line:
                    prompts += parse_prompts(line)
    if prompt is not None:
        prompts += parse_prompts(prompt)
    return prompts


def sampling_options(ns, temperature: float) -> dict:
    """Options of the sampler: flags first, then the reference session's HELIOS_* variables
    (src/inference_session.cpp:380-385), then its defaults."""
    sampled = temperature >= 0.01
    top_k = ns.top_k if ns.top_k is not None else _env("HELIOS_TOPK", int, 50)
    top_p = ns.top_p if ns.top_p is not None else _env("HELIOS_TOPP", float, 0.9)
    return dict(
        temperature=temperature,
        top_k=top_k if sampled else 0,
        top_p=top_p if sampled else 1.0,
        repetition_penalty=_env("HELIOS_REP", float, 1.0),
        frequency_penalty=_env("HELIOS_FREQ", float, 0.0),
        seed=ns.sampler_seed if ns.sampler_seed is not None else _env("HELIOS_SEED", int, 0),
        penalty_window=_env("HELIOS_WINDOW", int, 384),
    )


def context_length(ns, allowed: int) -> int:
    """--ctx / --max-seq as given (the engine refuses more than the configuration allows);
    else HELIOS_CTX or 4096, bounded by what the configuration allows."""
    if ns.ctx is not None:
        return ns.ctx
    return min(_env("HELIOS_CTX", int, 4096), allowed)


def main(argv: list[str] | None = None) -> int:
    ns, model, prompt, max_tokens, temperature = parse_args(sys.argv[1:] if argv is None else argv)
    import hector_engine_amd as he
    from hector_engine_amd.registry import config_from_dict, model_spec

    print("============================================")
    print("Hector engine (AMD) text generation (with KV cache)")
    print("============================================")
    if ns.random is not None:
        import json
        with open(ns.random) as f:
            config = config_from_dict(json.load(f))
    else:
        config = he.load_config(model)
    prompts = gather_prompts(ns, prompt)
    if not prompts and not ns.chat:
        first = config.bos_token_id if getattr(config, "bos_token_id", None) is not None else 0
        prompts = [[first]]
    ctx = context_length(ns, model_spec(config).max_positions)
    sampling = he.SamplingConfig(**sampling_options(ns, temperature))
    # None: the model's own end-of-sequence ids (generation_config.json, else config.json)
    stop_ids = [int(t) for t in ns.stop_ids.split(",") if t] if ns.stop_ids is not None else None
    slots = 1 if ns.chat else max(1, min(len(prompts), ns.slots or len(prompts)))
    pages = slots * ((ctx + 63) // 64)
    start = time.perf_counter()
    source = dict(config=config, seed=ns.seed) if ns.random is not None else dict(model_dir=model)
    engine = he.Engine(dtype=ns.dtype, max_tokens=pages * 64, max_slots=slots, max_seq_len=ctx,
                       use_graphs=not ns.no_graph, tune_library=ns.tune_gemm, profile=ns.profile,
                       sync_each_launch=ns.sync_each_launch, **source)
    what = f"random weights for {ns.random}, seed {ns.seed}" if ns.random is not None else model
    print(f"Model: {what}  ({config.architecture}, {ns.dtype})  loaded in "
          f"{(time.perf_counter() - start) * 1e3:.0f} ms")
    if ns.chat:
        return chat(he, engine, ns, prompts, sampling, stop_ids, max_tokens)
    t0 = time.perf_counter()
    on_token = None
    if ns.stream:
        def on_token(i, tok):
            print(f"[{i}] + {tok}", flush=True)
    results = he.generate(engine, prompts, max_new_tokens=max_tokens, sampling=sampling,
                          stop_ids=stop_ids, batch_size=slots, on_token=on_token)
    total_ms = (time.perf_counter() - t0) * 1e3
    for i, r in enumerate(results):
        print(f"[{i}] prompt {r.prompt_tokens} tokens -> {len(r.tokens)} tokens ({r.finish_reason}): "
              + ",".join(str(t) for t in r.tokens))
    gen = sum(len(r.tokens) for r in results)
    prefill_ms = max((r.prefill_ms for r in results), default=0.0)
    decode_ms = max((r.decode_ms for r in results), default=0.0)
    print("============================================")
    print(f"Prompt: {sum(r.prompt_tokens for r in results)} tokens ({prefill_ms:.0f} ms)")
    print(f"Tokens: {gen}")
    print(f"Time: {total_ms:.0f} ms")
    print(f"Speed: {gen * 1000.0 / decode_ms if decode_ms > 0 else 0.0:.1f} tok/s")
    print("============================================")
    if ns.profile:
        print(engine.profile_summary())
    return 0


def chat(he, engine, ns, first_turns, sampling, stop_ids, max_tokens) -> int:
    """Turn after turn in one session: the prompts of the command line, then every line of standard
    input (token ids; an empty line or the end of the input ends the conversation)."""
    def turns():
        yield from first_turns
        for line in sys.stdin:
            ids = parse_prompts(line.split("#", 1)[0])
            if not ids:
                return
            yield ids[0]
    with he.Session(engine, sampling, stop_ids) as session:
        for n, ids in enumerate(turns()):
            on_token = (lambda tok: print(f"[turn {n}] + {tok}", flush=True)) if ns.stream else None
            r = session.turn(ids, max_tokens, on_token=on_token)
            speed = len(r.tokens) * 1000.0 / r.decode_ms if r.decode_ms > 0 else 0.0
            print(f"[turn {n}] {r.prompt_tokens} tokens in ({r.prefill_ms:.0f} ms) -> {len(r.tokens)} tokens "
                  f"({r.finish_reason}, {speed:.1f} tok/s, context {session.position}): "
                  + ",".join(str(t) for t in r.tokens), flush=True)
    if ns.profile:
        print(engine.profile_summary())
    return 0


if __name__ == "__main__":
    sys.exit(main())
