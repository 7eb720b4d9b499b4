"""Token embedding and output head.

Embedding: h[t] = E[id_t], no scaling, written straight into the fp32 residual
stream (reference: src/graph_builder.cpp:998, kernels/linear.cu:36-69).
Head: logits = n W^T with W the head's own matrix, or the embedding matrix when
tied (src/graph_builder.cpp:1019-1036); only the wanted rows are computed and
the logits are fp32 in both precisions.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import BuildEnv, Part, StepContext, TensorSpec, param, register_part
from .linear import Linear


@register_part("embedding", "token_embedding")
class TokenEmbedding(Part):
    def __init__(self, params: dict, prefix: str, env: BuildEnv):
        super().__init__(prefix, env)
        self.vocab = param(params, "vocab_size", int)
        self.hidden = param(params, "hidden_size", int)
        self.table: torch.Tensor | None = None

    def tensor_specs(self):
        return {self.prefix + "weight": TensorSpec((self.vocab, self.hidden))}

    def bind(self, tensors):
        self.table = tensors[self.prefix + "weight"]

    def forward(self, ids: torch.Tensor, rows: int, ctx: StepContext) -> torch.Tensor:
        out = ctx.alloc((rows, self.hidden), torch.float32)
        ops.embedding(out, self.table, ids, rows)
        return out


@register_part("head", "linear_head")
class LinearHead(Part):
    accepts_normed_rows = True

    def __init__(self, params: dict, prefix: str, env: BuildEnv):
        super().__init__(prefix, env)
        self.vocab = param(params, "vocab_size", int)
        self.hidden = param(params, "hidden_size", int)
        self.tied_to = param(params, "tied_to", str, "")   # full name of the tensor it shares
        self.linear: Linear | None = None

    def tensor_specs(self):
        if self.tied_to:
            return {}
        return {self.prefix + "weight": TensorSpec((self.vocab, self.hidden))}

    def bind(self, tensors):
        name = self.tied_to or self.prefix + "weight"
        self.linear = Linear(tensors[name])

    def forward(self, x: torch.Tensor, rows: int, ctx: StepContext) -> torch.Tensor:
        return self.linear(x, rows, ctx, out_dtype=torch.float32)
