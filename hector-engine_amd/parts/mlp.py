"""Dense gated feed-forward: d = (act(x Wg^T) * (x Wu^T)) Wd^T with act = SiLU,
no biases (reference: src/graph_builder.cpp:1415-1428,
kernels/activations.cu:183-198). Gate and up are one product over the
row-concatenated weight gate||up (the reference's optional fusion:
src/graph_builder.cpp:1400-1414)."""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import BuildEnv, FeedForward, NormedRows, PieceRows, StepContext, TensorSpec, param, register_part
from .linear import Linear

# rows of the intermediate activations held at once in a long prompt step
_ROW_CHUNK = 8192


@register_part("feed_forward", "gated_mlp")
class GatedMLP(FeedForward):
    accepts_normed_rows = True

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
        # gate and up rows alternate (gate i at row 2i, its up at 2i + 1): the four neighbouring
        # rows whose sums a thread of the MFMA product holds are then two (gate, up) pairs, and
        # the gated activation is that product's epilogue
        w = torch.stack([g, u], 1).reshape(2 * g.shape[0], g.shape[1])
        self.gate_up = Linear(w.contiguous())
        del g, u, w
        self.down = Linear(tensors[p + "down_proj.weight"])

    def forward(self, x, ctx: StepContext):
        rows = ctx.rows
        if rows <= _ROW_CHUNK:
            act = x.scaled.dtype if isinstance(x, NormedRows) else x.dtype
            if self.gate_up.gated_silu_rows(rows, ctx, act):
                # up to 64 rows: the activation is the product's epilogue, and its result goes to the
                # down projection piece-major where that reads it so
                pieces = self.inter % 8 == 0 and self.down.reads_pieces(rows, ctx) and self.gate_up.gated_pieces(rows)
                h = ctx.alloc(ops.pieces_shape(rows, self.inter) if pieces else (rows, self.inter))
                self.gate_up.gated_silu(x, rows, ctx, h, out_pieces=pieces)
                return self.down(PieceRows(h) if pieces else h, rows, ctx, sink=ctx.take_sink())
            h = ctx.alloc((rows, self.inter))
            gu = self.gate_up(x, rows, ctx)
            ops.silu_mul(h, gu, rows, True)
            return self.down(h, rows, ctx, sink=ctx.take_sink())
        if not isinstance(x, torch.Tensor):
            x = x.tensor(ctx)
        out = ctx.alloc((rows, self.hidden))
        for r0 in range(0, rows, _ROW_CHUNK):
            n = min(_ROW_CHUNK, rows - r0)
            turn = ctx.scratch.mark()
            h = ctx.alloc((n, self.inter))
            gu = self.gate_up(x[r0:r0 + n], n, ctx)
            ops.silu_mul(h, gu, n, True)
            self.down(h, n, ctx, out=out[r0:r0 + n])
            ctx.scratch.release(turn)       # the next turn reuses h and gate||up
        return out
