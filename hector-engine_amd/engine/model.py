"""The decoder assembled from a :class:`ModelSpec`: embedding, the layers'
blocks run in the order the schedule gives, final norm, output head. It knows
no architecture; everything it does follows from the data."""
from __future__ import annotations

import torch

from ..cache.paged import RunPlan
from ..kernels import ops
from ..parts.base import BuildEnv, LayerCache, ModelSpec, ResidualStream, StepContext, build_part


class DecoderModel:
    def __init__(self, spec: ModelSpec, env: BuildEnv):
        self.spec = spec
        self.env = env
        self.embedding = build_part("embedding", spec.embedding, spec.embedding_prefix, env)
        self.blocks = [build_part("block", ls.block, ls.prefix, env) for ls in spec.layers]
        self.final_norm = build_part("norm", spec.final_norm, spec.final_norm_prefix, env)
        self.head = build_part("head", spec.head, spec.head_prefix, env)
        self.schedule = list(spec.schedule)
        for e, entry in enumerate(self.schedule):
            if not 0 <= entry.layer < len(self.blocks):
                raise ValueError(f"schedule entry {e} names layer {entry.layer}, "
                                 f"the model has {len(self.blocks)}")
            if entry.cache_from is not None:
                src = entry.cache_from
                if not 0 <= src < e or self.schedule[src].cache_from is not None:
                    raise ValueError(f"schedule entry {e}: cache_from {src} must be an earlier "
                                     "entry with a cache of its own")
                a = self.blocks[entry.layer].mixer.kv_need()
                b = self.blocks[self.schedule[src].layer].mixer.kv_need()
                if a != b:
                    raise ValueError(f"schedule entry {e} reads the cache of entry {src}, whose "
                                     f"keys/values {b} differ from its own {a}")

    # -- tensors ------------------------------------------------------------
    def parts(self):
        return [self.embedding, *self.blocks, self.final_norm, self.head]

    def graph_safe(self) -> bool:
        """True when every part works from the device-side batch alone."""
        todo = list(self.parts())
        while todo:
            p = todo.pop()
            if not p.graph_safe:
                return False
            todo += p.children()
        return True

    def step_hints(self) -> list:
        """The distinct step_hint functions of the model's parts, in a fixed order."""
        found, todo = [], list(self.parts())
        while todo:
            p = todo.pop(0)
            fn = getattr(p, "step_hint", None)
            if fn is not None and fn not in found:
                found.append(fn)
            todo += p.children()
        return found

    def tensor_specs(self):
        specs = {}
        for p in self.parts():
            specs.update(p.tensor_specs())
        return specs

    def bind(self, tensors: dict[str, torch.Tensor]) -> None:
        for p in self.parts():
            p.bind(tensors)

    # -- cache ----------------------------------------------------------------
    def run_plans(self) -> list[RunPlan]:
        plans = []
        for entry in self.schedule:
            mixer = self.blocks[entry.layer].mixer
            kv = mixer.kv_need() if entry.cache_from is None else None
            plans.append(RunPlan(kv, entry.cache_from, mixer.state_bytes()))
        return plans

    # -- one step -----------------------------------------------------------
    def forward(self, ids: torch.Tensor, ctx: StepContext, caches: list[LayerCache],
                want_rows: torch.Tensor | None, n_want: int) -> torch.Tensor | None:
        """ids: int32 [rows]. Returns fp32 logits [n_want, vocab] of the rows
        named by want_rows (int32 [n_want]), or None when nothing is wanted."""
        rows = ctx.rows
        resid = self.embedding.forward(ids, rows, ctx)
        stream = ResidualStream(resid, rows)
        last = len(self.schedule) - 1
        for e, entry in enumerate(self.schedule):
            # the norm that reads the stream after this block: the next block's first, or the
            # final norm when every row's logits are wanted (no gather in between)
            if e < last:
                ctx.next_norm = self.blocks[self.schedule[e + 1].layer].first_norm()
            else:
                ctx.next_norm = self.final_norm if (ctx.want_all and n_want == rows) else None
            ctx.scratch.begin_layer()
            self.blocks[entry.layer].forward(stream, ctx, caches[e])
        ctx.scratch.end_layers()
        ctx.next_norm = None
        if n_want == 0:
            stream.materialize(ctx)
            return None
        if ctx.want_all and n_want == rows:
            normed = stream.normed(self.final_norm, ctx, getattr(self.head, "accepts_normed_rows", False))
            return self.head.forward(normed, n_want, ctx)
        stream.materialize(ctx)
        sel = ctx.alloc((n_want, self.spec.hidden_size), torch.float32)
        ops.gather_rows_f32(sel, resid, want_rows, n_want, rows)
        normed = self.final_norm.add_norm(sel, None, n_want, ctx)
        return self.head.forward(normed, n_want, ctx)
