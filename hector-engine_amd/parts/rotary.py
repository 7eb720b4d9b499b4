"""Rotary position encoding with half-split pairing (i, i + r/2):
a = pos * theta^(-2i/r); (y_i, y_{i+r/2}) = (x_i cos a - x_{i+r/2} sin a,
x_i sin a + x_{i+r/2} cos a); dims >= r pass through
(reference: kernels/attention.cu:516-558; r = 2*floor(hd*partial/2),
kernels/register_kernels.cpp:702-704). The frequencies are computed once in
float64 and held in float32; the angle and its sine/cosine are formed in fp32
inside the fused q/k kernel from each row's own position."""
from __future__ import annotations

import torch

from .base import BuildEnv, PositionEncoding, param, register_part


@register_part("position", "rotary")
class Rotary(PositionEncoding):
    def __init__(self, params: dict, prefix: str, env: BuildEnv):
        super().__init__(prefix, env)
        self.head_dim = param(params, "head_dim", int)
        self.theta = param(params, "theta", float)
        partial = param(params, "partial_rotary_factor", float, 1.0)
        r = 2 * int(self.head_dim * partial / 2)
        self.rotary_dim = self.head_dim if r <= 0 else r
        if self.rotary_dim % 2 or self.rotary_dim > self.head_dim:
            raise ValueError(f"rotary: rotary_dim {self.rotary_dim} must be even and at most head_dim")
        i = torch.arange(0, self.rotary_dim, 2, dtype=torch.float64)
        inv = 1.0 / (torch.tensor(self.theta, dtype=torch.float64) ** (i / self.rotary_dim))
        self.inv_freq = inv.to(torch.float32).to(env.device).contiguous()

    def rotary(self):
        return self.inv_freq, self.rotary_dim


@register_part("position", "none")
class NoPosition(PositionEncoding):
    """No encoding of positions at this place."""

    def __init__(self, params: dict, prefix: str, env: BuildEnv):
        super().__init__(prefix, env)
