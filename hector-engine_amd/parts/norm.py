"""RMS normalisation: y = x * rsqrt(mean(x^2) + eps) * weight, the weight
multiplying directly (reference: kernels/normalization.cu:36-63). Applied to the
fp32 residual stream, fused with the pending residual add
(kernels/fused_add_rmsnorm.cu:47-81)."""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import BuildEnv, Norm, StepContext, TensorSpec, param, register_part


@register_part("norm", "rmsnorm")
class RMSNorm(Norm):
    def __init__(self, params: dict, prefix: str, env: BuildEnv):
        super().__init__(prefix, env)
        self.size = param(params, "size", int)
        self.eps = param(params, "eps", float)
        self.weight: torch.Tensor | None = None

    def tensor_specs(self):
        return {self.prefix + "weight": TensorSpec((self.size,), ("gain", 1.0, 0.1))}

    def bind(self, tensors):
        self.weight = tensors[self.prefix + "weight"]

    def carried(self):
        return self.weight, self.eps

    def add_norm(self, resid, delta, rows, ctx: StepContext, want_out: bool = True):
        out = ctx.alloc((rows, self.size)) if want_out else None
        ops.add_rmsnorm(resid, delta, self.weight, out, rows, self.eps)
        return out
