"""Arrangement of a layer: pre-norm residual block
    x = x + mixer(norm1(x));  x = x + feed_forward(norm2(x))
(reference: src/graph_builder.cpp:1195, :1366-1374, :1396, :1443). Each
residual add is carried as pending and fused into the next norm, or, with few
rows, done by the last product of the mixer / feed-forward, which then also prepares
the rows of the norm that follows (parts.base.ResidualSink)."""
from __future__ import annotations

from .base import (Block, BuildEnv, LayerCache, PartSpec, ResidualStream, StepContext,
                   build_part, param, register_part)


@register_part("block", "pre_norm")
class PreNormBlock(Block):
    def __init__(self, params: dict, prefix: str, env: BuildEnv):
        super().__init__(prefix, env)
        names = param(params, "names", dict)
        self.mixer_norm = build_part("norm", param(params, "mixer_norm", PartSpec),
                                     prefix + names["mixer_norm"] + ".", env)
        self.mixer = build_part("mixer", param(params, "mixer", PartSpec),
                                prefix + names["mixer"] + ".", env)
        self.ff_norm = build_part("norm", param(params, "feed_forward_norm", PartSpec),
                                  prefix + names["feed_forward_norm"] + ".", env)
        self.feed_forward = build_part("feed_forward", param(params, "feed_forward", PartSpec),
                                       prefix + names["feed_forward"] + ".", env)

    def children(self):
        return [self.mixer_norm, self.mixer, self.ff_norm, self.feed_forward]

    def first_norm(self):
        return self.mixer_norm

    def tensor_specs(self):
        specs = {}
        for c in self.children():
            specs.update(c.tensor_specs())
        return specs

    def bind(self, tensors):
        for c in self.children():
            c.bind(tensors)

    def forward(self, stream: ResidualStream, ctx: StepContext, cache: LayerCache) -> None:
        after = ctx.next_norm                  # reads the stream once this block is done
        n = stream.normed(self.mixer_norm, ctx, self.mixer.accepts_normed_rows)
        ctx.sink = stream.sink_for(self.ff_norm, ctx)
        delta = self.mixer.forward(n, ctx, cache)
        ctx.sink = None
        stream.add(delta, ctx)
        n = stream.normed(self.ff_norm, ctx, self.feed_forward.accepts_normed_rows)
        ctx.sink = stream.sink_for(after, ctx)
        delta = self.feed_forward.forward(n, ctx)
        ctx.sink = None
        stream.add(delta, ctx)
