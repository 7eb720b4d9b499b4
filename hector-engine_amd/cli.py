"""Command line in the manner of the reference's generation tools.

    hector_generate <model_dir> [prompt] [max_tokens=100] [temperature=0.0]

as test_generate_kv takes its arguments (test_generate_kv.cpp:43-65): the second
argument is the prompt unless it is a plain number, in which case it is
max_tokens. This library works on token ids, so the prompt is a list of ids
"5,17,3"; several prompts separated by ';' run as one batch. The flags of
tools/helios_runtime.cpp:261-263 are accepted too: --model, --ctx, --temp. The
sampling environment variables of the reference's session are read
(src/inference_session.cpp:380-385): HELIOS_REP, HELIOS_FREQ, HELIOS_WINDOW,
HELIOS_TOPK, HELIOS_TOPP, HELIOS_SEED, and HELIOS_CTX (helios_chat.cpp:549).
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
              "   or: %(prog)s --model <model_dir> [--ctx N] [--temp T] [prompt] [max_tokens]")
    ap.add_argument("--model", default=None)
    ap.add_argument("--ctx", type=int, default=None, help="context length (HELIOS_CTX, else 4096)")
    ap.add_argument("--temp", type=float, default=None)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--stop-ids", default=None, help="comma-separated stop token ids")
    ap.add_argument("--no-graph", action="store_true", help="run one-token steps without HIP graphs")
    ap.add_argument("--tune-gemm", action="store_true",
                    help="let the library's autotuner choose the kernels of tall matrix products (a second or so "
                         "per new shape)")
    ap.add_argument("rest", nargs="*")
    ns = ap.parse_args(argv)
    rest = list(ns.rest)
    model = ns.model or (rest.pop(0) if rest else None)
    if model is None:
        ap.error("a model folder is needed")
    prompt = None
    if rest and not is_plain_number(rest[0]):
        prompt = rest.pop(0)
    max_tokens = int(rest.pop(0)) if rest else 100
    temperature = float(rest.pop(0)) if rest else (ns.temp if ns.temp is not None else 0.0)
    return ns, model, prompt, max_tokens, temperature


def main(argv: list[str] | None = None) -> int:
    ns, model, prompt, max_tokens, temperature = parse_args(sys.argv[1:] if argv is None else argv)
    import hector_engine_amd as he

    print("============================================")
    print("Hector engine (AMD) text generation (with KV cache)")
    print("============================================")
    config = he.load_config(model)
    if prompt is None:
        first = config.bos_token_id if getattr(config, "bos_token_id", None) is not None else 0
        prompts = [[first]]
    else:
        prompts = parse_prompts(prompt)
    ctx = ns.ctx or _env("HELIOS_CTX", int, 4096)
    sampling = he.SamplingConfig(
        temperature=temperature,
        top_k=_env("HELIOS_TOPK", int, 50) if temperature >= 0.01 else 0,
        top_p=_env("HELIOS_TOPP", float, 0.9) if temperature >= 0.01 else 1.0,
        repetition_penalty=_env("HELIOS_REP", float, 1.0),
        frequency_penalty=_env("HELIOS_FREQ", float, 0.0),
        seed=_env("HELIOS_SEED", int, 0),
        penalty_window=_env("HELIOS_WINDOW", int, 384),
    )
    if ns.stop_ids is not None:
        stop_ids = [int(t) for t in ns.stop_ids.split(",") if t]
    else:
        stop_ids = list(getattr(config, "eos_token_id", None) or [])
    pages = max(1, len(prompts)) * ((ctx + 63) // 64)
    start = time.perf_counter()
    engine = he.Engine(model, dtype=ns.dtype, max_tokens=pages * 64, max_slots=max(1, len(prompts)),
                       max_seq_len=ctx, use_graphs=not ns.no_graph, tune_library=ns.tune_gemm)
    print(f"Model: {model}  ({config.architecture}, {ns.dtype})  loaded in "
          f"{(time.perf_counter() - start) * 1e3:.0f} ms")
    t0 = time.perf_counter()
    results = he.generate(engine, prompts, max_new_tokens=max_tokens, sampling=sampling,
                          stop_ids=stop_ids)
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
    return 0


if __name__ == "__main__":
    sys.exit(main())
