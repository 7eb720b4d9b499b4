"""Grouped-query attention over the paged cache.

q = n Wq^T + bq, k = n Wk^T + bk, v = n Wv^T + bv (one product over q||k||v, the
reference's optional fusion: src/graph_builder.cpp:1543-1670); q and k are
encoded by the position part after the bias and before the cache write, v is
not (src/graph_builder.cpp:1213-1326); the new keys and values are written
before attention so that a query sees its own key (:1318-1326); the query at
position p attends the keys (p - window, p], all of [0, p] without a window
(kernels/attention.cu:60, :196, :696); kv head = h // (H / KVH) (:180);
scale 1/sqrt(head_dim) (src/graph_builder.cpp:1328); then o = a Wo^T.
"""
from __future__ import annotations

import math
from dataclasses import dataclass

import torch

from ..kernels import kv_layout, ops, routes
from .base import (BuildEnv, KVNeed, LayerCache, Mixer, PartSpec, PieceRows, StepContext, TensorSpec,
                   build_part, param, register_part)
from .linear import Linear


@dataclass(frozen=True)
class AttentionCase:
    """What a route of "attention" decides by."""
    all_single: bool    # every sequence of the step brings one token
    fast: bool          # sizes and environment allow the MFMA kernels
    fusable: bool       # head size and position encoding are ones the fused one-token kernel takes


def keys_uneven(lengths: list[int], before=None) -> bool:
    """Whether one sequence of a one-token step has several times the keys of the others (and
    thousands of them): the one-token attention then cuts every sequence's keys across more
    workgroups, or the long sequence would be left to a few of them. Once up (`before`), the flag
    stays up until the longest sequence has fewer than three times the mean (four to raise it), so
    that a batch at the edge does not go back and forth between two graphs."""
    longest = max(lengths)
    return longest >= 4096 and longest * len(lengths) >= (3 if before else 4) * sum(lengths)


@register_part("mixer", "attention")
class Attention(Mixer):
    accepts_normed_rows = True
    step_hint = staticmethod(keys_uneven)

    def __init__(self, params: dict, prefix: str, env: BuildEnv):
        super().__init__(prefix, env)
        self.hidden = param(params, "hidden_size", int)
        self.H = param(params, "num_heads", int)
        self.KVH = param(params, "num_kv_heads", int)
        self.hd = param(params, "head_dim", int)
        self.qkv_bias = param(params, "qkv_bias", bool, False)
        self.out_bias = param(params, "out_bias", bool, False)
        self.window = param(params, "window", int, 0)
        self.kv_projection = param(params, "kv_projection", bool, True)
        self.scale = param(params, "scale", float, 1.0 / math.sqrt(self.hd))
        if self.H % self.KVH:
            raise ValueError(f"attention: {self.H} heads are not a multiple of {self.KVH} kv heads")
        self.position = build_part("position", param(params, "position", PartSpec, PartSpec("none")),
                                   prefix, env)
        self.qkv: Linear | None = None
        self.q_only: Linear | None = None
        self.o_proj: Linear | None = None
        self._chosen: dict[tuple, routes.Route] = {}      # (all one-token, dtype) -> route, for one version of the table
        self._chosen_version = -1
        self.fast = env.dtype == torch.bfloat16 and getattr(env, "fast_kernels", True) \
            and self.hd % 16 == 0 and self.hd <= 256 and self.scale > 0   # else the plain kernel

    def children(self):
        return [self.position]

    def kv_need(self):
        # pages in the order the attention kernels read their operands
        return KVNeed(self.KVH, self.hd, self.window, k_page_elems=kv_layout.k_page_elems(self.hd),
                      v_page_elems=kv_layout.v_page_elems(self.hd))

    def tensor_specs(self):
        p, hd = self.prefix, self.hd
        specs = {p + "q_proj.weight": TensorSpec((self.H * hd, self.hidden)),
                 p + "o_proj.weight": TensorSpec((self.hidden, self.H * hd))}
        if self.kv_projection:
            specs[p + "k_proj.weight"] = TensorSpec((self.KVH * hd, self.hidden))
            specs[p + "v_proj.weight"] = TensorSpec((self.KVH * hd, self.hidden))
        if self.qkv_bias:
            specs[p + "q_proj.bias"] = TensorSpec((self.H * hd,))
            if self.kv_projection:
                specs[p + "k_proj.bias"] = TensorSpec((self.KVH * hd,))
                specs[p + "v_proj.bias"] = TensorSpec((self.KVH * hd,))
        if self.out_bias:
            specs[p + "o_proj.bias"] = TensorSpec((self.hidden,))
        specs.update(self.position.tensor_specs())
        return specs

    def bind(self, tensors):
        p = self.prefix
        names = ["q_proj"] + (["k_proj", "v_proj"] if self.kv_projection else [])
        ws = [tensors.pop(p + n + ".weight") for n in names]
        if len({w.dtype for w in ws}) != 1:
            raise TypeError(f"{p}q/k/v projections are stored in different dtypes")
        w = torch.cat(ws, 0).contiguous() if len(ws) > 1 else ws[0]
        b = None
        if self.qkv_bias:
            bs = [tensors.pop(p + n + ".bias") for n in names]
            if len({x.dtype for x in bs}) != 1:
                raise TypeError(f"{p}q/k/v biases are stored in different dtypes")
            b = torch.cat(bs, 0).contiguous() if len(bs) > 1 else bs[0]
        del ws
        self.qkv = Linear(w, b)
        q_rows = self.H * self.hd
        self.q_only = Linear(w[:q_rows], None if b is None else b[:q_rows])
        self.o_proj = Linear(tensors[p + "o_proj.weight"], tensors.get(p + "o_proj.bias"))
        self.position.bind(tensors)

    def forward(self, x, ctx: StepContext, cache: LayerCache):
        if cache.writes and not self.kv_projection:
            raise RuntimeError(f"{self.prefix}: a mixer without k/v projections must read another run's cache")
        if self._chosen_version != routes.version():
            self._chosen.clear()
            self._chosen_version = routes.version()
        key = (ctx.all_single, ctx.env.dtype)
        route = self._chosen.get(key)
        if route is None:
            rot = self.position.rotary()
            case = AttentionCase(
                all_single=ctx.all_single, fast=self.fast,
                fusable=not self.position.custom and rot is not None
                and ops.attention_decode_fused_ok(self.H, self.KVH, self.hd, rot[1]))
            route = self._chosen[key] = routes.choose("attention", (ctx.env.dtype,), case)
        return route.run(self, x, ctx, cache)

    # ---- the routes' bodies ----

    def _run_fused_one_token(self, x, ctx: StepContext, cache: LayerCache):
        """One-token steps: bias, rotation, cache write and attention in one launch."""
        rows, H, KVH, hd = ctx.rows, self.H, self.KVH, self.hd
        proj = self.qkv if cache.writes else self.q_only
        rot = self.position.rotary()
        # where the projection is cut along K (17 to 64 rows), the kernel below adds the slices
        # itself: the same bits, and the launch that would add them is not needed
        qkv = proj.k_slices(x, rows, ctx)
        if qkv is None:
            qkv = proj(x, rows, ctx, use_bias=False)
        pieces = self.o_proj.reads_pieces(rows, ctx)       # the layout the output product reads best
        out = ctx.alloc(ops.pieces_shape(rows, H * hd) if pieces else (rows, H * hd))
        uneven = bool(ctx.hints.get(keys_uneven, False))
        floats = ops.attention_decode_fused_workspace_floats(rows, H, KVH, hd, ctx.max_keys, uneven)
        ws = ctx.alloc((floats,), torch.float32) if floats else None
        # the page numbers of the step's rows, where the host has put them beside the step's metadata
        by_row = ctx.row_tables.get(cache.page_table.data_ptr())
        ops.attention_decode_fused(out, qkv, proj.bias, cache.kpool, cache.vpool, ctx.positions,
                                   ctx.row_seq, None if by_row is not None else ctx.seq_slot,
                                   by_row if by_row is not None else cache.page_table, rot[0], rot[1],
                                   rows, H, KVH, hd, self.window, self.scale, ctx.max_keys,
                                   cache.writes, ws, out_pieces=pieces, spread=uneven)
        return self.o_proj(PieceRows(out) if pieces else out, rows, ctx, sink=ctx.take_sink())

    def _encoded_q(self, x, ctx: StepContext, cache: LayerCache):
        """q with bias and position encoding, after the new keys and values went into the cache."""
        rows, H, KVH, hd = ctx.rows, self.H, self.KVH, self.hd
        writes = cache.writes
        proj = self.qkv if writes else self.q_only
        rot = self.position.rotary()
        # With a rotation (or no encoding) the bias is added inside the fused kernel;
        # any other encoding sees q and k with their bias already added.
        fused_bias = not self.position.custom
        qkv = proj(x, rows, ctx, use_bias=not fused_bias)
        if not fused_bias:
            q_cols, kv_cols = H * hd, KVH * hd
            qv = qkv[:, :q_cols].unflatten(1, (H, hd))
            kv = qkv[:, q_cols:q_cols + kv_cols].unflatten(1, (KVH, hd)) if writes else None
            self.position.apply(qv, kv, ctx)
        q = ctx.alloc((rows, H * hd))
        inv_freq, r = rot if rot is not None else (None, 0)
        ops.qkv_rope_cache(q, cache.kpool, cache.vpool, qkv, H * hd, KVH * hd,
                           proj.bias if fused_bias else None, ctx.positions, ctx.row_seq,
                           ctx.seq_slot, cache.page_table, inv_freq, r, rows, H, KVH, hd, writes)
        return q

    def _run_plain(self, x, ctx: StepContext, cache: LayerCache):
        """The plain kernel: one fixed order per (query, head), in the precision of the cache."""
        rows, H, KVH, hd = ctx.rows, self.H, self.KVH, self.hd
        q = self._encoded_q(x, ctx, cache)
        out = ctx.alloc((rows, H * hd))
        floats = ops.attention_plain_workspace_floats(rows, H, hd, ctx.most_keys, self.window)
        ws = ctx.alloc((floats,), torch.float32) if floats else None
        ops.attention_plain(out, q, cache.kpool, cache.vpool, ctx.positions, ctx.row_seq,
                            ctx.seq_slot, cache.page_table, rows, H, KVH, hd, self.window,
                            self.scale, ctx.most_keys, ws)
        return self.o_proj(out, rows, ctx, sink=ctx.take_sink())

    def _run_mfma_one_token(self, x, ctx: StepContext, cache: LayerCache):
        """One-token steps of the head sizes and encodings the fused kernel does not take."""
        rows, H, KVH, hd = ctx.rows, self.H, self.KVH, self.hd
        q = self._encoded_q(x, ctx, cache)
        out = ctx.alloc((rows, H * hd))
        floats = ops.attention_decode_workspace_floats(rows, H, KVH, hd, ctx.max_keys)
        ws = ctx.alloc((max(floats, 1),), torch.float32)
        ops.attention_decode(out, q, cache.kpool, cache.vpool, ctx.positions, ctx.row_seq,
                             ctx.seq_slot, cache.page_table, rows, H, KVH, hd, self.window,
                             self.scale, ctx.max_keys, ws)
        return self.o_proj(out, rows, ctx, sink=ctx.take_sink())

    def _run_mfma_prompt(self, x, ctx: StepContext, cache: LayerCache):
        """Prompt steps and mixed steps."""
        rows, H, KVH, hd = ctx.rows, self.H, self.KVH, self.hd
        q = self._encoded_q(x, ctx, cache)
        out = ctx.alloc((rows, H * hd))
        # few queries against many keys (a continuation of a long sequence): the keys in parts
        most = ctx.most_keys
        if self.window > 0:
            most = min(most, self.window + ctx.max_q_len)
        parts = ops.attention_prefill_parts(ctx.num_seqs, ctx.max_q_len, H, hd, most)
        ws = ctx.alloc((ops.attention_prefill_workspace_floats(rows, H, hd, parts),), torch.float32) \
            if parts > 1 else None
        if ctx.padded:
            # the prompt kernels write the rows of sequences only: padding rows hold zeros (their
            # parts too, whose join then gives zeros), never what the buffer held before
            (ws if ws is not None else out).zero_()
        ops.attention_prefill(out, q, cache.kpool, cache.vpool, ctx.cu_seqlens, ctx.seq_slot,
                              ctx.seq_start, cache.page_table, ctx.num_seqs, ctx.max_q_len,
                              rows, H, KVH, hd, self.window, self.scale, parts=parts, workspace=ws)
        return self.o_proj(out, rows, ctx, sink=ctx.take_sink())


_BF16 = (torch.bfloat16,)
routes.register_route("attention", _BF16, "fused_one_token",
                      lambda c: c.fast and c.all_single and c.fusable, Attention._run_fused_one_token)
routes.register_route("attention", _BF16, "plain", lambda c: not c.fast, Attention._run_plain)
routes.register_route("attention", _BF16, "mfma_one_token", lambda c: c.all_single, Attention._run_mfma_one_token)
routes.register_route("attention", _BF16, "mfma_prompt", lambda c: True, Attention._run_mfma_prompt)
routes.register_route("attention", (torch.float32,), "plain", lambda c: True, Attention._run_plain)
