"""Plain, slow implementation of the Qwen2 dense decoder as the reference engine
computes it, written from the reference's formulas for use as the tests' oracle.

Whole sequences, no cache, one function per part, torch on the CPU only. It
shares no code with the package under test: it reads config.json and the
safetensors file with its own few lines. File:line citations point into the
reference repository (andresgv-beep/Hector-engine).
"""
from __future__ import annotations

import json
import math
import os
import struct

import numpy as np
import torch

DT = torch.float64


# --------------------------------------------------------------------------
# reading a model folder (layout as read by tools/quant_bench/ref_qwen3.py:45-62)
# --------------------------------------------------------------------------
_NP = {"F32": np.float32, "F16": np.float16, "BF16": np.uint16, "I32": np.int32, "I64": np.int64}


def read_safetensors(path: str) -> dict[str, torch.Tensor]:
    with open(path, "rb") as f:
        raw = f.read()
    (n,) = struct.unpack("<Q", raw[:8])
    header = json.loads(raw[8:8 + n])
    header.pop("__metadata__", None)
    out = {}
    for name, e in header.items():
        a, b = e["data_offsets"]
        arr = np.frombuffer(raw[8 + n + a:8 + n + b], dtype=_NP[e["dtype"]]).reshape(e["shape"])
        if e["dtype"] == "BF16":  # bf16 -> f32 is a 16-bit shift (ref_qwen3.py:60)
            arr = (arr.astype(np.uint32) << 16).view(np.float32)
        out[name] = torch.from_numpy(np.array(arr))
    return out


def read_model(folder: str, dtype=DT):
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    weights = {}
    for fn in sorted(os.listdir(folder)):
        if fn.endswith(".safetensors"):
            weights.update(read_safetensors(os.path.join(folder, fn)))
    weights = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    return cfg, weights


# --------------------------------------------------------------------------
# parts
# --------------------------------------------------------------------------
def embedding(ids: torch.Tensor, table: torch.Tensor) -> torch.Tensor:
    """h[t] = E[id_t]; an id outside [0, V) gives a zero row, no scaling
    (kernels/linear.cu:36-69, src/graph_builder.cpp:998)."""
    V = table.shape[0]
    ok = (ids >= 0) & (ids < V)
    rows = table[ids.clamp(0, V - 1)]
    return rows * ok[:, None].to(rows.dtype)


def rmsnorm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """y = x * rsqrt(mean(x^2) + eps) * w, the weight multiplies directly
    (kernels/normalization.cu:36-63)."""
    ms = (x * x).mean(-1, keepdim=True)
    return x * torch.rsqrt(ms + eps) * w


def linear(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor | None = None) -> torch.Tensor:
    """C[M,N] = A[M,K] . W[N,K]^T, weight rows are outputs
    (kernels/register_kernels.cpp:373-386); bias added after (kernels/elementwise.cu:307-323)."""
    y = x @ w.T
    return y if b is None else y + b


def rope_inv_freq(rotary_dim: int, theta: float) -> torch.Tensor:
    """f_i = 1 / theta^(2i/r), i in [0, r/2) (kernels/attention.cu:538-539;
    the same vector in tools/quant_bench/ref_qwen3.py:94, kept in float32 there)."""
    i = torch.arange(0, rotary_dim, 2, dtype=torch.float64)
    return (1.0 / (theta ** (i / rotary_dim))).to(torch.float32)


def rope(x: torch.Tensor, positions: torch.Tensor, theta: float, rotary_dim: int | None = None,
         scaling: float = 1.0) -> torch.Tensor:
    """x: [S, heads, hd]. Half-split pairing (i, i + r/2):
    y_i = x_i cos a - x_{i+r/2} sin a ; y_{i+r/2} = x_i sin a + x_{i+r/2} cos a,
    a = (pos / scaling) * f_i; dims >= r untouched (kernels/attention.cu:516-558).
    The angle is formed in float32 like the reference (float pos times float freq)."""
    hd = x.shape[-1]
    r = hd if rotary_dim is None else rotary_dim
    half = r // 2
    f = rope_inv_freq(r, theta)
    pos = positions.to(torch.float32) / np.float32(scaling)
    ang = (pos[:, None] * f[None, :]).to(torch.float32)  # fp32 product
    cos = torch.cos(ang.to(torch.float64)).to(x.dtype)[:, None, :]
    sin = torch.sin(ang.to(torch.float64)).to(x.dtype)[:, None, :]
    x0, x1, rest = x[..., :half], x[..., half:r], x[..., r:]
    return torch.cat([x0 * cos - x1 * sin, x0 * sin + x1 * cos, rest], -1)


def attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, q_pos: torch.Tensor,
              k_pos: torch.Tensor, window: int = 0, scale: float | None = None) -> torch.Tensor:
    """q: [Sq, H, hd], k/v: [Sk, KVH, hd]. kv head = h // (H // KVH)
    (kernels/attention.cu:180). The query at position p sees the keys j with
    j <= p and, with a window, j + window > p, i.e. (p - window, p]
    (kernels/attention.cu:60). s = (q . k) * scale, scale = 1/sqrt(hd)
    (src/graph_builder.cpp:1328); softmax over the visible keys; out = P V."""
    Sq, H, hd = q.shape
    KVH = k.shape[1]
    g = H // KVH
    scale = 1.0 / math.sqrt(hd) if scale is None else scale
    kk = k.repeat_interleave(g, dim=1)
    vv = v.repeat_interleave(g, dim=1)
    s = torch.einsum("qhd,khd->hqk", q, kk) * scale
    visible = k_pos[None, :] <= q_pos[:, None]
    if window > 0:
        visible &= (k_pos[None, :] + window) > q_pos[:, None]
    s = s.masked_fill(~visible[None], float("-inf"))
    p = torch.softmax(s, -1)
    return torch.einsum("hqk,khd->qhd", p, vv).reshape(Sq, H * hd)


def silu(z: torch.Tensor) -> torch.Tensor:
    """silu(z) = z / (1 + e^-z) (kernels/activations.cu:19-21)."""
    return z / (1.0 + torch.exp(-z))


def swiglu(x, w_gate, w_up, w_down):
    """d = (silu(x Wg^T) * (x Wu^T)) Wd^T, no biases (src/graph_builder.cpp:1415-1428)."""
    return linear(silu(linear(x, w_gate)) * linear(x, w_up), w_down)


# --------------------------------------------------------------------------
# configuration as the model folder gives it
# --------------------------------------------------------------------------
def layer_window(cfg: dict, layer: int) -> int:
    """Layers with index >= max_window_layers attend through the window when
    use_sliding_window is true; the others, and every layer otherwise, see all
    keys. (The reference passes no window on this path; the per-key rule is
    kernels/attention.cu:60.)"""
    if not cfg.get("use_sliding_window", False) or cfg.get("sliding_window") is None:
        return 0
    mwl = cfg.get("max_window_layers", cfg["num_hidden_layers"])
    return int(cfg["sliding_window"]) if layer >= mwl else 0


def head_dim(cfg: dict) -> int:
    return cfg.get("head_dim") or cfg["hidden_size"] // cfg["num_attention_heads"]


# --------------------------------------------------------------------------
# the decoder
# --------------------------------------------------------------------------
def attention_block(cfg, w, prefix, x, positions, window, kv_source=None):
    """norm -> q,k,v (+bias) -> rope(q,k) -> attention -> o_proj
    (src/graph_builder.cpp:1195-1374). Returns (output, (k, v)); with kv_source
    the keys and values of another layer are attended instead of this layer's."""
    H, KVH, hd = cfg["num_attention_heads"], cfg.get("num_key_value_heads") or cfg["num_attention_heads"], head_dim(cfg)
    S = x.shape[0]
    theta = cfg.get("rope_theta", 10000.0)
    q = linear(x, w[prefix + "q_proj.weight"], w.get(prefix + "q_proj.bias")).reshape(S, H, hd)
    q = rope(q, positions, theta)
    if kv_source is None:
        k = linear(x, w[prefix + "k_proj.weight"], w.get(prefix + "k_proj.bias")).reshape(S, KVH, hd)
        v = linear(x, w[prefix + "v_proj.weight"], w.get(prefix + "v_proj.bias")).reshape(S, KVH, hd)
        k = rope(k, positions, theta)
    else:
        k, v = kv_source
    a = attention(q, k, v, positions, positions, window)
    return linear(a, w[prefix + "o_proj.weight"], w.get(prefix + "o_proj.bias")), (k, v)


def forward(cfg: dict, w: dict, ids, positions=None, schedule=None, kv_from=None) -> torch.Tensor:
    """Logits [S, V] for one whole sequence.

    Layer l (src/graph_builder.cpp:968-1039, :1138-1444):
        x = x + attn(norm1(x));  x = x + mlp(norm2(x))
    then the final norm and the output head, lm_head.weight if the tensor exists
    and the embedding matrix otherwise (src/graph_builder.cpp:1019-1036).

    schedule: order in which layers run (default 0..L-1; an index may repeat);
    kv_from: {schedule entry -> earlier schedule entry} whose keys/values it reads.
    """
    ids = torch.as_tensor(ids, dtype=torch.int64)
    S = ids.shape[0]
    dtype = w["model.embed_tokens.weight"].dtype
    positions = torch.arange(S) if positions is None else torch.as_tensor(positions)
    eps = cfg.get("rms_norm_eps", 1e-6)
    L = cfg["num_hidden_layers"]
    schedule = list(range(L)) if schedule is None else schedule
    kv_from = kv_from or {}
    x = embedding(ids, w["model.embed_tokens.weight"]).to(dtype)
    kvs = {}
    for e, l in enumerate(schedule):
        p = f"model.layers.{l}."
        n = rmsnorm(x, w[p + "input_layernorm.weight"], eps)
        src = kvs[kv_from[e]] if e in kv_from else None
        a, kvs[e] = attention_block(cfg, w, p + "self_attn.", n, positions, layer_window(cfg, l), src)
        x = x + a
        n = rmsnorm(x, w[p + "post_attention_layernorm.weight"], eps)
        x = x + swiglu(n, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"],
                       w[p + "mlp.down_proj.weight"])
    x = rmsnorm(x, w["model.norm.weight"], eps)
    head = w["lm_head.weight"] if "lm_head.weight" in w and not cfg.get("tie_word_embeddings", False) \
        else w["model.embed_tokens.weight"]
    return linear(x, head)


# --------------------------------------------------------------------------
# sampling (src/sampler.cpp:112-195, kernels/sampling.cu:24-67, :411-451, :542-565)
# --------------------------------------------------------------------------
def argmax_lowest(logits: torch.Tensor) -> int:
    """First maximum: strict '>' keeps the lowest index (kernels/sampling.cu:24-67)."""
    best, bi = -math.inf, 0
    vals = logits.tolist()
    for i, v in enumerate(vals):
        if v > best:
            best, bi = v, i
    return bi


def apply_penalties(logits: torch.Tensor, context: list[int], window: int, rep: float, freq: float,
                    pres: float) -> torch.Tensor:
    """Last `window` context tokens, deduplicated with counts; per id:
    logit > 0 ? logit / rep : logit * rep; minus freq * count; minus presence
    (src/sampler.cpp:41-91, kernels/sampling.cu:542-565)."""
    out = logits.clone().to(torch.float32)
    counts: dict[int, int] = {}
    for t in context[max(0, len(context) - window):]:
        if 0 <= t < out.shape[0]:
            counts[t] = counts.get(t, 0) + 1
    for t, c in counts.items():
        v = np.float32(out[t].item())
        if rep != 1.0:
            v = np.float32(v / np.float32(rep)) if v > 0 else np.float32(v * np.float32(rep))
        if freq != 0.0:
            v = np.float32(v - np.float32(freq) * np.float32(c))
        if pres != 0.0:
            v = np.float32(v - np.float32(pres))
        out[t] = float(v)
    return out


def uniform_u32(seed: int, sequence: int, step: int) -> int:
    """The engine's own counter-based uniform (the reference draws from a host
    mt19937_64, src/sampler.hpp:129-130; one uniform per token either way)."""
    M = (1 << 64) - 1
    z = (seed * 0x9E3779B97F4A7C15 + sequence * 0xBF58476D1CE4E5B9 + step * 0x94D049BB133111EB + 0x2545F4914F6CDD1D) & M
    z ^= z >> 30
    z = (z * 0xBF58476D1CE4E5B9) & M
    z ^= z >> 27
    z = (z * 0x94D049BB133111EB) & M
    z ^= z >> 31
    return z >> 32


def sample(logits: torch.Tensor, temperature: float, top_k: int, top_p: float, u32: int) -> int:
    """Sorted candidates (value descending, index ascending on ties), first top_k,
    p_i = exp((v_i - v_0) / T), shortest prefix with mass >= top_p of the kept
    mass, r = u * mass of that prefix, first i with r < cum_i
    (kernels/sampling.cu:411-451). Masses are 40-bit fixed point as in the
    engine, so the rule is exact in integers; the reference uses floats."""
    x = logits.to(torch.float32).numpy().copy()
    x[np.isnan(x)] = -np.inf
    V = x.shape[0]
    order = np.lexsort((np.arange(V), -x.astype(np.float64)))  # value desc, index asc
    if 0 < top_k < V:
        order = order[:top_k]
    m = np.float32(x.max())
    inv_t = np.float32(1.0) / np.float32(temperature)
    wts = np.exp(((x[order] - m) * inv_t).astype(np.float32)).astype(np.float32)
    q = [int(np.float32(wi) * np.float32(2.0 ** 40)) for wi in wts]
    Z = sum(q)
    n = len(q)
    if 0.0 < top_p < 1.0:
        target = min(max(int(math.ceil(float(np.float32(top_p)) * float(Z))), 1), Z)
        cum = 0
        for i, qi in enumerate(q):
            cum += qi
            if cum >= target:
                n = i + 1
                break
    Zn = sum(q[:n])
    r = (u32 * Zn) >> 32
    cum = 0
    for i in range(n):
        cum += q[i]
        if r < cum:
            return int(order[i])
    return int(order[n - 1])


def generate(cfg, w, prompt: list[int], max_new_tokens: int, temperature: float = 0.0,
             top_k: int = 0, top_p: float = 1.0, seed: int = 0, sequence: int = 0,
             stop_ids=(), rep: float = 1.0, freq: float = 0.0, pres: float = 0.0,
             penalty_window: int = 384) -> list[int]:
    """Prefill, then one token at a time, recomputing the whole sequence each step.
    The penalty context holds generated tokens only (src/inference_session.cpp:651).
    Stop tokens end the sequence and are neither emitted nor fed back
    (src/inference_session.cpp:597-660); temperature < 0.01 is greedy
    (src/sampler.cpp:141)."""
    seq = list(prompt)
    out: list[int] = []
    for step in range(max_new_tokens):
        logits = forward(cfg, w, seq)[-1].to(torch.float32)
        if rep != 1.0 or freq != 0.0 or pres != 0.0:
            logits = apply_penalties(logits, out, penalty_window, rep, freq, pres)
        if temperature < 0.01:
            tok = argmax_lowest(logits)
        else:
            tok = sample(logits, temperature, top_k, top_p, uniform_u32(seed, sequence, step))
        if tok in stop_ids:
            break
        out.append(tok)
        seq.append(tok)
    return out
