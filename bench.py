#!/usr/bin/env python3
"""Decode throughput of the Qwen2.5-7B shape (bf16, random weights, synthetic
token ids) on one MI355X, with prefill and roofline figures on the same line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--layers L] [--shape 7b|32b|72b]
                    [--context C] [--prompt P]

The default is the 7B shape; --shape runs the same measurement at the layer sizes of
Qwen2.5-32B (context 8192, prompts of 512 to 2048 tokens, batches 1 / 8 / 64) or
Qwen2-72B (context 4096, prompts of 2048 tokens, batches 1 / 8 / 32).

Beside the points at batch 1 and at the large batch the default run adds three more (--no-extra
leaves them out), each with its share of the HBM peak in `points_roofline_frac`:
  decode_b64_t7800   the large batch behind prompts of 7,800 tokens (30 GB of keys and values a step:
                     the one-token attention is then the kernel most of the time goes to)
  decode_b8_32b      batch 8 at the Qwen2.5-32B layer sizes (all 64 layers), prompts of 512 to 2,048 tokens
  decode_b1_fp32     batch 1 of the 7B shape in true 32-bit (28.3 GB of weights a step), and with it
                     `prefill_fp32`, the 2,048-token prompt in 32-bit against the fp32 peak

A step is one decode step of the whole batch: the engine's step function (HIP
graph replay) plus greedy sampling. As in the library's generation loop, steps are
queued ahead of the host: the chosen ids go into the next step on the device, and the host
reads a step's ids when 7 further steps are queued behind it.

The default warm-up of 64 steps is most of the first half second after the prompt step, during which
the machine runs every kernel of the one-token step 4 to 6 % slower than afterwards (the reference
leaves its first run and its thermal-low samples out: OPTIMIZATION_NOTES.md:114-117); `repeats` holds
every timed run, the earlier ones still show it.

Procedure (the reference quotes medians with their range over repeated runs:
tools/HQS_DECODE_OPTIMIZATION_PLAN.md:54-65): after the warm-up steps, `--repeats` (5) runs of
exactly `--steps` steps each are timed, each bracketed by a device synchronisation; `value` and
`ms_per_step` are the median run's, `repeats` holds all of them. The same holds for the points at
batch 1 and at the large batch. The prefill figure is the median of three whole-prompt steps of
one 2,048-token prompt (a step of that size replays a HIP graph from its third use on, as in the engine's
default configuration); `prefill_packed` is one step of `--batch` such prompts packed together.
"""
from __future__ import annotations

import argparse
import contextlib
import json
import sys
import time

import numpy as np

# layer sizes; the benchmark is quoted on the first (Qwen2.5-7B)
_COMMON = dict(head_dim=128, vocab_size=152064, rope_theta=1000000.0, rms_norm_eps=1e-6,
               max_position_embeddings=32768, tie_word_embeddings=False)
SHAPES = {
    # name, context per sequence, prompt lengths of the decode batches (lowest, highest), the large batch, sizes
    "7b": ("Qwen2.5-7B shape", 8192, (2048, 2048), 64, dict(_COMMON, num_hidden_layers=28, hidden_size=3584, num_attention_heads=28,
                                          num_key_value_heads=4, intermediate_size=18944)),
    "32b": ("Qwen2.5-32B shape", 8192, (512, 2048), 64, dict(_COMMON, num_hidden_layers=64, hidden_size=5120, num_attention_heads=40,
                                            num_key_value_heads=8, intermediate_size=27648)),
    "72b": ("Qwen2-72B shape", 4096, (2048, 2048), 32, dict(_COMMON, num_hidden_layers=80, hidden_size=8192, num_attention_heads=64,
                                          num_key_value_heads=8, intermediate_size=29568)),
}
PROMPT = 2048
RUN = 8          # one-token steps queued at a time
HBM_PEAK_GBS = 8000.0
BF16_PEAK_FLOPS = 2.5e15
FP32_PEAK_FLOPS = 157.3e12
LONG_PROMPT = 7800   # the long-context point: prompts of so many tokens in the shape's context


def weight_bytes(c, layers, itemsize=2):
    D, H, KVH, hd, I, V = (c["hidden_size"], c["num_attention_heads"], c["num_key_value_heads"],
                           c["head_dim"], c["intermediate_size"], c["vocab_size"])
    per_layer = D * (H + 2 * KVH) * hd + (H + 2 * KVH) * hd + H * hd * D + 3 * D * I + 2 * D
    return itemsize * (layers * per_layer + D + V * D)      # lm_head read once; embedding rows are negligible


def kv_bytes_per_token(c, layers, itemsize=2):
    return 2 * layers * c["num_key_value_heads"] * c["head_dim"] * itemsize


def prefill_flops(c, layers, T):
    D, H, KVH, hd, I, V = (c["hidden_size"], c["num_attention_heads"], c["num_key_value_heads"],
                           c["head_dim"], c["intermediate_size"], c["vocab_size"])
    gemm = 2 * T * (D * (H + 2 * KVH) * hd + H * hd * D + 3 * D * I)
    attn = 4 * H * hd * T * (T + 1) // 2
    return layers * (gemm + attn) + 2 * D * V


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=64)
    ap.add_argument("--repeats", type=int, default=5, help="timed runs of --steps steps each; the median counts")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the shape has (0 = all)")
    ap.add_argument("--shape", choices=sorted(SHAPES), default="7b")
    ap.add_argument("--context", type=int, default=0, help="another context length per sequence than the shape's")
    ap.add_argument("--prompt", type=int, default=0,
                    help="another prompt length of the decode batches (the prefill figure stays at 2048 tokens)")
    ap.add_argument("--no-points", action="store_true", help="skip the points at batch 1 and at the large batch")
    ap.add_argument("--no-extra", action="store_true",
                    help="skip the long-context point, the Qwen2.5-32B point and the 32-bit point")
    ap.add_argument("--continuation", default="", metavar="AFTER:NEW",
                    help="also time a step of NEW tokens of a sequence that holds AFTER tokens already "
                         "(a new turn of a conversation); reported as \"continuation\"")
    ap.add_argument("--short-steps", action="store_true",
                    help="also time prompt steps of 16, 64 and 256 tokens and a step of 8 one-token entries plus a "
                         "64-token prompt, as replayed graphs and issued launch by launch; reported as \"short_steps\"")
    ap.add_argument("--generation", action="store_true",
                    help="also time the generation loop (generate(): 72 new tokens after the decode batches' prompts, "
                         "steps queued ahead of the host) at batch 1, --batch and the large batch, greedy and with "
                         "the sampling presets; reported as \"generation\", decoded tokens a second")
    ap.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16",
                    help="float32: the whole measurement in true 32-bit (no library products, no extra points)")
    ap.add_argument("--no-tune", action="store_true",
                    help="leave the library's default kernels for the tall matrix products")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this library runs on one GPU; --gpus {args.gpus} is not supported")
        return 2
    MODEL, CONTEXT, (PROMPT_LO, PROMPT_HI), BIG_BATCH, SHAPE = SHAPES[args.shape]
    CONTEXT = args.context or CONTEXT
    if args.prompt:
        PROMPT_LO = PROMPT_HI = args.prompt
    if args.repeats < 1 or args.steps < 1:
        print("bench.py: --steps and --repeats must be at least 1")
        return 2
    if max(PROMPT, PROMPT_HI) + args.warmup + args.repeats * args.steps > CONTEXT:
        print(f"bench.py: prompts of {max(PROMPT, PROMPT_HI)} tokens and {args.warmup + args.repeats * args.steps} "
              f"steps do not fit a context of {CONTEXT}")
        return 2
    cont = None
    if args.continuation:
        try:
            cont = tuple(int(v) for v in args.continuation.split(":"))
            assert len(cont) == 2 and cont[0] >= 0 and cont[1] >= 1
        except (ValueError, AssertionError):
            print("bench.py: --continuation takes AFTER:NEW, two token counts")
            return 2
        if sum(cont) > CONTEXT:
            print(f"bench.py: a continuation of {cont[1]} tokens after {cont[0]} does not fit a context of {CONTEXT}")
            return 2
    FULL_LAYERS = SHAPE["num_hidden_layers"]
    args.layers = args.layers or FULL_LAYERS

    import torch
    import hector_engine_amd as he
    from hector_engine_amd.config.qwen2 import Qwen2Config
    from hector_engine_amd.engine.engine import StepEntry
    from hector_engine_amd.kernels import library_tuning

    t_start = time.perf_counter()

    def progress(what):
        print(f"[bench {time.perf_counter() - t_start:6.1f}s] {what}", file=sys.stderr, flush=True)

    rng = np.random.default_rng(0)

    class Model:
        """An engine of one shape and precision with what the measurements need of it."""

        def __init__(self, shape, layers, dtype, max_batch, context, tune):
            self.shape, self.layers, self.context = shape, layers, context
            self.itemsize = 2 if dtype == "bfloat16" else 4
            config = Qwen2Config.from_dict(dict(shape, num_hidden_layers=layers, architectures=["Qwen2ForCausalLM"]))
            t0 = time.perf_counter()
            self.engine = he.Engine(config=config, seed=0, dtype=dtype, max_tokens=max_batch * context,
                                    max_slots=max_batch, max_seq_len=context, tune_library=tune)
            self.sampler = he.Sampler(he.SamplingConfig.deterministic(), self.engine.device)
            torch.cuda.synchronize()
            self.load_s = time.perf_counter() - t0
            self.wbytes = weight_bytes(shape, layers, self.itemsize)
            self.packed = {}

        def prompts(self, n, lo, hi):
            return [rng.integers(0, self.shape["vocab_size"], int(rng.integers(lo, hi + 1))).tolist() for _ in range(n)]

        def prefill(self, ps, slots, fixed_length):
            """Prompts in groups of 8 sequences a step; returns the first sampled tokens."""
            toks = []
            # prompts of random lengths give row counts that never come again: not worth the tuner's trials
            tuning = contextlib.nullcontext() if fixed_length else library_tuning.no_new_tuning()
            with tuning:
                for g in range(0, len(ps), 8):
                    entries = [StepEntry(s, p, [len(p) - 1]) for s, p in zip(slots[g:g + 8], ps[g:g + 8])]
                    logits = self.engine.step(entries)
                    toks += self.sampler.sample(logits, list(range(len(entries))), [0] * len(entries))
            return toks

        def prompt_step(self, tokens):
            """Seconds of one whole-prompt step of `tokens` tokens: a first run warms the library's
            products, a second one is captured as a HIP graph where the engine keeps one for such a
            step, then the median of three."""
            p = self.prompts(1, tokens, tokens)[0]
            times = []
            for run in range(5):
                slot = self.engine.acquire()
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                self.engine.step([StepEntry(slot, p, [tokens - 1])])
                torch.cuda.synchronize()
                if run > 1:
                    times.append(time.perf_counter() - t0)
                self.engine.release(slot)
            return sorted(times)[1]

        def decode_run(self, batch, lo, hi, steps, warmup, repeats, time_prefill=False):
            """Prompts of lo to hi tokens, warm-up steps, then `repeats` timed runs of `steps` steps.
            Returns per run (seconds a step, bytes a step has to read)."""
            engine, sampler = self.engine, self.sampler
            slots = [engine.acquire() for _ in range(batch)]
            ps = self.prompts(batch, lo, hi)
            if time_prefill:      # the packed prompt step of the headline batch, timed
                warm = [engine.acquire() for _ in range(batch)]     # once untimed: the library's first call of a shape
                self.prefill(ps, warm, lo == hi)
                for s in warm:
                    engine.release(s)
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                toks = self.prefill(ps, slots, lo == hi)
                torch.cuda.synchronize()
                self.packed.update(tokens=sum(len(p) for p in ps), seconds=time.perf_counter() - t0,
                                   flops=sum(prefill_flops(self.shape, self.layers, len(p)) for p in ps))
            else:
                toks = self.prefill(ps, slots, lo == hi)
            seqs = list(range(batch))

            def many(toks, count):
                """`count` steps queued back to back: each step's ids go into the next on the device,
                the host reads the ids of a step when RUN - 1 further steps are queued behind it (as
                the generation loop does when nothing but the token budget ends a sequence)."""
                ids, reads = None, []
                for j in range(count):
                    logits = engine.step([StepEntry(s, [t], [0]) for s, t in zip(slots, toks)], device_tokens=ids)
                    ids = sampler.sample_device(logits, seqs, [0] * batch)
                    reads.append(sampler.read_later(ids))
                    if j >= RUN - 1:
                        reads[j - (RUN - 1)].wait()
                return reads[-1].wait() if reads else toks

            toks = many(toks, warmup)
            runs = []
            done = warmup
            kv = kv_bytes_per_token(self.shape, self.layers, self.itemsize)
            for _ in range(repeats):
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                toks = many(toks, steps)
                torch.cuda.synchronize()
                dt = time.perf_counter() - t0
                avg_len = sum(len(p) for p in ps) / batch + done + steps / 2
                done += steps
                runs.append((dt / steps, self.wbytes + batch * avg_len * kv))
            for s in slots:
                engine.release(s)
            if engine.capture_failures:
                # a step that fell back from its HIP graph would pass as a (slower) number
                raise RuntimeError(f"bench.py: one-token steps ran without their graph: {engine.capture_failures}")
            return runs

        def close(self):
            del self.engine, self.sampler
            torch.cuda.empty_cache()

    def median_run(runs):
        return sorted(runs)[len(runs) // 2]

    points, points_frac, points_ms = {}, {}, {}

    def point(name, model, batch, lo, hi, steps, warmup, repeats):
        progress(name)
        s, nbytes = median_run(model.decode_run(batch, lo, hi, steps, warmup, repeats))
        points[name] = round(batch / s, 1)
        points_ms[name] = round(s * 1e3, 4)
        points_frac[name] = round(nbytes / s / 1e9 / HBM_PEAK_GBS, 4)

    progress(f"{MODEL}: random weights, {args.layers} layers")
    max_batch = 2 * args.batch if args.no_points and not args.generation else max(2 * args.batch, BIG_BATCH)
    fp32 = args.dtype == "float32"
    if fp32:
        args.no_tune = True
    model = Model(SHAPE, args.layers, args.dtype, max_batch, CONTEXT, not args.no_tune)
    engine, load_s = model.engine, model.load_s

    # ---- prefill of one 2,048-token prompt
    progress(f"weights ready; prefill of {PROMPT} tokens")
    prefill_s = model.prompt_step(PROMPT)
    flops = prefill_flops(SHAPE, args.layers, PROMPT)

    # ---- a step of a few new tokens behind a long sequence: the median of three
    continuation = None
    if cont is not None:
        progress(f"{cont[1]} tokens after {cont[0]}")
        before, fresh = model.prompts(1, cont[0], cont[0])[0], model.prompts(1, cont[1], cont[1])[0]
        times = []
        for run in range(4):
            slot = engine.acquire()
            if before:
                engine.step([StepEntry(slot, before, [])])
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            engine.step([StepEntry(slot, fresh, [len(fresh) - 1])])
            torch.cuda.synchronize()
            if run > 0:
                times.append(time.perf_counter() - t0)
            engine.release(slot)
        continuation = {"after": cont[0], "tokens": cont[1], "ms": round(sorted(times)[1] * 1e3, 3)}

    # ---- short prompt steps and a mixed step: the replayed graph of their bucket against launches from the host
    short_steps = None
    if args.short_steps:
        progress("short steps")
        short_steps = {}

        def timed(step, reset):
            """(wall ms, ms between two events around the step on the GPU's own clock), medians."""
            times, spans = [], []
            for run in range(7):
                reset()
                before, after = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                before.record()
                step()
                after.record()
                torch.cuda.synchronize()
                if run > 2:               # the bucket's first step runs eagerly, its second is captured
                    times.append(time.perf_counter() - t0)
                    spans.append(before.elapsed_time(after))
            return round(sorted(times)[len(times) // 2] * 1e3, 3), round(sorted(spans)[len(spans) // 2], 3)

        for label, n_decoding, n_prompt in (("prompt16", 0, 16), ("prompt64", 0, 64), ("prompt256", 0, 256),
                                            ("decode8_prompt64", 8, 64)):
            slots = [engine.acquire() for _ in range(n_decoding + 1)]
            if n_decoding:
                engine.step([StepEntry(s, p, []) for s, p in zip(slots, model.prompts(n_decoding, 300, 300))])
            new = model.prompts(1, n_prompt, n_prompt)[0]

            def step():
                engine.step([StepEntry(s, [7], [0]) for s in slots[:-1]] + [StepEntry(slots[-1], new, [n_prompt - 1])])

            def reset():
                engine.truncate(slots[-1], 0)
                for s in slots[:-1]:
                    engine.truncate(s, 300)
            rows_allowed = engine.graph_step_rows
            graph_ms, graph_gpu_ms = timed(step, reset)
            engine.graph_step_rows = 0
            eager_ms, _ = timed(step, reset)
            engine.graph_step_rows = rows_allowed
            short_steps[label] = {"graph_ms": graph_ms, "graph_gpu_ms": graph_gpu_ms, "eager_ms": eager_ms}
            for s in slots:
                engine.release(s)

    # ---- decode at the headline batch
    progress(f"decode at batch {args.batch}")
    runs = model.decode_run(args.batch, PROMPT_LO, PROMPT_HI, args.steps, args.warmup, args.repeats,
                            time_prefill=args.batch <= 8)
    step_s, step_bytes = median_run(runs)
    achieved = step_bytes / step_s / 1e9
    packed = model.packed

    if not args.no_points:
        for b in (1, BIG_BATCH):
            point(f"decode_b{b}", model, b, PROMPT_LO, PROMPT_HI, args.steps, max(3, args.warmup // 2), args.repeats)

    # ---- the generation loop: what a caller of generate() gets, sampling included
    generation = None
    if args.generation:
        generation = {}
        settings = {"greedy": he.SamplingConfig.deterministic(),
                    "t0.8_k40_p0.9": he.SamplingConfig(temperature=0.8, top_k=40, top_p=0.9, seed=3),
                    "t0.8": he.SamplingConfig(temperature=0.8, seed=3),
                    "balanced": he.SamplingConfig.balanced(), "creative": he.SamplingConfig.creative()}
        for b in sorted({1, args.batch, BIG_BATCH}):
            progress(f"generation at batch {b}")
            ps = model.prompts(b, PROMPT_LO, PROMPT_HI)
            for name, sampling in settings.items():
                he.generate(engine, ps, max_new_tokens=8, sampling=sampling)           # warm: graphs, buffers
                results = he.generate(engine, ps, max_new_tokens=72, sampling=sampling)
                torch.cuda.synchronize()
                decode_ms = max(r.decode_ms for r in results)
                tokens = sum(len(r.tokens) for r in results)
                generation[f"b{b}_{name}"] = round((tokens - b) * 1e3 / decode_ms, 1)
    extra = not args.no_extra and not args.no_points and args.shape == "7b" and args.layers == FULL_LAYERS and not fp32
    prefill_fp32 = None
    if extra:
        # the large batch behind long prompts: 32 steps a run keep the sequences inside the context
        long_prompt = min(LONG_PROMPT, CONTEXT - 8 - 3 * 32 - 8)
        point(f"decode_b{BIG_BATCH}_t{LONG_PROMPT}", model, BIG_BATCH, long_prompt, long_prompt, 32, 8, 3)
    model.close()
    if extra:
        name32, ctx32, (lo32, hi32), _, shape32 = SHAPES["32b"]
        progress(f"{name32}: random weights, {shape32['num_hidden_layers']} layers")
        other = Model(shape32, shape32["num_hidden_layers"], "bfloat16", 8, ctx32, not args.no_tune)
        point("decode_b8_32b", other, 8, lo32, hi32, 32, 8, 3)
        other.close()
        progress(f"{MODEL} in 32-bit")
        other = Model(SHAPE, args.layers, "float32", 1, CONTEXT, False)
        fp32_s = other.prompt_step(PROMPT)
        prefill_fp32 = {"value": round(PROMPT / fp32_s, 1), "tokens": PROMPT, "ms": round(fp32_s * 1e3, 3),
                        "frac": round(flops / fp32_s / FP32_PEAK_FLOPS, 4)}
        point("decode_b1_fp32", other, 1, PROMPT_LO, PROMPT_HI, 16, 4, 3)
        other.close()

    PROMPTS = PROMPT_LO if PROMPT_LO == PROMPT_HI else f"{PROMPT_LO}-{PROMPT_HI}"
    line = {
        "metric": f"decode tok/s @ bs {args.batch}, {MODEL} {'fp32' if fp32 else 'bf16'}, context {CONTEXT}, prompts {PROMPTS}",
        "value": round(args.batch / step_s, 1),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(step_s * 1e3, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "fp32" if fp32 else "bf16",
        "data": "synthetic token ids (uniform), random N(0, 0.02) weights",
        "config": {
            "model": MODEL, "layers": args.layers, "layers_full": FULL_LAYERS,
            "hidden_size": SHAPE["hidden_size"], "heads": SHAPE["num_attention_heads"],
            "kv_heads": SHAPE["num_key_value_heads"], "head_dim": SHAPE["head_dim"],
            "intermediate_size": SHAPE["intermediate_size"], "vocab_size": SHAPE["vocab_size"],
            "rope_theta": SHAPE["rope_theta"], "rms_norm_eps": SHAPE["rms_norm_eps"],
            "global_batch": args.batch, "seq_len": CONTEXT, "prompt_len": PROMPTS,
            "parallelism": "single GPU", "sampling": "greedy, ids read 7 steps behind", "load_s": round(load_s, 1),
            "library_gemm_autotuned": not args.no_tune,
            "points_of_other_shapes": "decode_b8_32b: Qwen2.5-32B layer sizes, 64 layers, prompts 512-2048; "
                                      "decode_b1_fp32 and prefill_fp32: this shape in true 32-bit" if extra else "none",
        },
        "prefill": {"value": round(PROMPT / prefill_s, 1), "tokens": PROMPT,
                    "ms": round(prefill_s * 1e3, 3),
                    "frac": round(flops / prefill_s / (FP32_PEAK_FLOPS if fp32 else BF16_PEAK_FLOPS), 4)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4)},
        "points": points,
        "points_ms_per_step": points_ms,
        "points_roofline_frac": points_frac,
        "repeats": {"n": args.repeats, "steps_each": args.steps,
                    "ms_per_step": [round(t * 1e3, 4) for t, _ in runs],
                    "min": round(min(t for t, _ in runs) * 1e3, 4),
                    "median": round(step_s * 1e3, 4),
                    "max": round(max(t for t, _ in runs) * 1e3, 4)},
    }
    if prefill_fp32:
        line["prefill_fp32"] = prefill_fp32
    if short_steps:
        line["short_steps"] = short_steps
    if continuation:
        line["continuation"] = continuation
    if generation:
        line["generation"] = generation
    if packed:
        line["prefill_packed"] = {"value": round(packed["tokens"] / packed["seconds"], 1), "tokens": packed["tokens"],
                                  "ms": round(packed["seconds"] * 1e3, 3),
                                  "frac": round(packed["flops"] / packed["seconds"]
                                                / (FP32_PEAK_FLOPS if fp32 else BF16_PEAK_FLOPS), 4)}
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
