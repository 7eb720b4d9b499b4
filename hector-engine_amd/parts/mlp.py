"""Dense gated feed-forward: d = (act(x Wg^T) * (x Wu^T)) Wd^T with act = SiLU,
no biases (reference: src/graph_builder.cpp:1415-1428,
kernels/activations.cu:183-198). Gate and up are one product over the
row-concatenated weight gate||up (the reference's optional fusion:
src/graph_builder.cpp:1400-1414)."""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import BuildEnv, FeedForward, StepContext, TensorSpec, param, register_part
from .linear import Linear

# rows of the intermediate activations held at once in a long prompt step
_ROW_CHUNK = 8192


@register_part("feed_forward", "gated_mlp")
class GatedMLP(FeedForward):
    def __init__(self, params: dict, prefix: str, env: BuildEnv):
        super().__init__(prefix, env)
        self.hidden = param(params, "hidden_size", int)
        self.inter = param(params, "intermediate_size", int)
        act = param(params, "activation", str, "silu")
        if act not in ("silu", "swish"):
            raise ValueError(f"gated_mlp: unsupported activation '{act}'")
        self.gate_up: Linear | None = None
        self.down: Linear | None = None

    def tensor_specs(self):
        p = self.prefix
        return {
            p + "gate_proj.weight": TensorSpec((self.inter, self.hidden)),
            p + "up_proj.weight": TensorSpec((self.inter, self.hidden)),
            p + "down_proj.weight": TensorSpec((self.hidden, self.inter)),
        }

    def bind(self, tensors):
        p = self.prefix
        g, u = tensors.pop(p + "gate_proj.weight"), tensors.pop(p + "up_proj.weight")
        if g.dtype != u.dtype:
            raise TypeError(f"{p}gate_proj and up_proj are stored in different dtypes")
        self.gate_up = Linear(torch.cat([g, u], 0).contiguous())
        del g, u
        self.down = Linear(tensors[p + "down_proj.weight"])

    def forward(self, x, ctx: StepContext):
        rows = ctx.rows
        out = ctx.alloc((rows, self.hidden))
        for r0 in range(0, rows, _ROW_CHUNK):
            n = min(_ROW_CHUNK, rows - r0)
            gu = self.gate_up(x[r0:r0 + n], n, ctx)
            h = ctx.alloc((n, self.inter))
            ops.silu_mul(h, gu, n)
            self.down(h, n, ctx, out=out[r0:r0 + n])
        return out
