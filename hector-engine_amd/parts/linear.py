"""The linear layer all parts share: y[M,N] = x[M,K] . W[N,K]^T (+ bias).

Which kernel runs is decided by precision and row count:
  float32                 -> the plain FMA kernel (fixed summation order per element)
  bfloat16, M <= 64       -> the hand-written MFMA kernel that streams each weight once
  bfloat16, M  > 64       -> the library matrix product (the reference calls its
                             BLAS library here: kernels/matmul_cublas.cu:240-277)
A weight that was stored in 32-bit stays 32-bit; under bfloat16 activations it
runs through the float32 kernel.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import StepContext


class Linear:
    def __init__(self, weight: torch.Tensor, bias: torch.Tensor | None = None):
        if weight.dim() != 2:
            raise ValueError("Linear weight must be [out, in]")
        self.weight = weight
        self.bias = bias
        self.out_features, self.in_features = weight.shape

    def __call__(self, x: torch.Tensor, rows: int, ctx: StepContext, *, use_bias: bool = True,
                 out_dtype: torch.dtype | None = None, out: torch.Tensor | None = None) -> torch.Tensor:
        w = self.weight
        N, K = w.shape
        bias = self.bias if use_bias else None
        act = x.dtype
        out_dtype = out_dtype or act
        if out is None:
            out = ctx.alloc((rows, N), out_dtype)
        if rows == 0:
            return out
        if w.dtype == torch.float32:
            if act == torch.float32:
                if out_dtype != torch.float32:
                    raise TypeError("float32 activations give float32 outputs")
                ops.gemm_plain(out, x, w, bias, rows)
                return out
            # weight kept in 32-bit under bfloat16 activations
            x32 = ctx.alloc((rows, K), torch.float32)
            x32.copy_(x[:rows])
            y32 = out if out_dtype == torch.float32 else ctx.alloc((rows, N), torch.float32)
            ops.gemm_plain(y32, x32, w, bias, rows)
            if y32 is not out:
                out[:rows].copy_(y32)
            return out
        if w.dtype != torch.bfloat16 or act != torch.bfloat16:
            raise TypeError(f"Linear: weight {w.dtype} with activations {act} is not supported")
        if not ctx.env.fast_kernels:
            ops.gemm_plain(out, x, w, bias, rows)   # the plain kernel also under bfloat16
            return out
        if rows <= ops.SKINNY_MAX_M:
            self._skinny(out, x, bias, rows, ctx)
            return out
        if out_dtype == torch.float32:
            # fp32 results of a tall product: 64 rows at a time through the MFMA kernel
            for r0 in range(0, rows, ops.SKINNY_MAX_M):
                r1 = min(rows, r0 + ops.SKINNY_MAX_M)
                self._skinny(out[r0:r1], x[r0:r1], bias, r1 - r0, ctx)
            return out
        if bias is not None:
            torch.addmm(bias, x[:rows], w.t(), out=out[:rows])
        else:
            torch.mm(x[:rows], w.t(), out=out[:rows])
        return out

    def _skinny(self, out, x, bias, rows, ctx):
        N, K = self.weight.shape
        floats = ops.gemm_skinny_workspace_floats(rows, N, K)
        ws = ctx.alloc((max(floats, 1),), torch.float32)
        ops.gemm_skinny(out, x, self.weight, bias, rows, ws)
