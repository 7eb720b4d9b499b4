"""The linear layer all parts share: y[M,N] = x[M,K] . W[N,K]^T (+ bias).

Which kernel runs is decided by precision and row count:
  float32 weights          -> the plain FMA kernel (fixed summation order per element);
                              a weight that was stored in 32-bit stays 32-bit and runs
                              through it also under bfloat16 activations
  bfloat16, M <= 16        -> the block-split MFMA kernel: K is cut inside the workgroup,
                              one launch gives the finished result
  bfloat16, 17 <= M <= 64  -> the library, except for long K (>= 8192) while the library's
                              tuner is off (its default kernels do not cut K): then the
                              block-split kernel up to 32 rows and, up to 64, the wavefront
                              kernel with K cut across workgroups
  bfloat16, M > 64         -> the library matrix product (the reference calls its BLAS
                              library for every product: kernels/matmul_cublas.cu:240-277)
  fp32 results (logits)    -> the MFMA kernels up to 32 rows, above that the library,
                              which writes fp32 from bf16 operands
The wavefront kernel's fp32 partial sums are added by a small kernel, or, when a caller
says `allow_split` and SPLIT_TO_CONSUMER is on, handed over as a :class:`SplitSum` to a
kernel that adds the slices while it reads (the fused norm, the q/k/v kernel). That
hand-over is off: with few rows the reading kernel has one workgroup per row and adding
the slices there is slower than the small kernel.

The block-split kernel also carries an RMS norm across a pair of products, so that a
step of few rows has no norm kernels: given a :class:`ResidualSink` it adds its result
to the residual rows itself and leaves r * gain and the sums of r^2 for the norm that
follows (:class:`NormedRows`); given NormedRows as input it applies the owed row scale
to its sums. Any other path turns NormedRows into a tensor first and ignores the sink.

Between block-split products of up to 16 rows the bf16 rows travel piece-major
(kernels.ops.pieces_shape): the product's operand loads then touch two cache lines instead
of sixteen (at the Qwen2.5-7B shapes 2 us a layer at 8 rows, 10 us at 16). The rows it
leaves for the next norm are written so; a producer of its input (attention, the gated
product) writes so after asking reads_pieces().
"""
from __future__ import annotations

import torch

from ..kernels import library_tuning, ops, profiler
from .base import NormedRows, PieceRows, ResidualSink, StepContext


class SplitSum:
    """fp32 partial sums [slices, rows, N] of one product (+ a bias not yet added)."""

    def __init__(self, partial: torch.Tensor, bias: torch.Tensor | None, rows: int):
        self.partial = partial
        self.bias = bias
        self.rows = rows
        self.splits = partial.shape[0]

    def materialize(self, ctx: StepContext, dtype: torch.dtype | None = None,
                    out: torch.Tensor | None = None) -> torch.Tensor:
        if out is None:
            out = ctx.alloc((self.rows, self.partial.shape[-1]), dtype or ctx.env.dtype)
        ops.splitk_reduce(out, self.partial, self.bias, self.rows, self.splits)
        return out


def as_tensor(x, ctx: StepContext) -> torch.Tensor:
    """A tensor, whether x is one or the split sums of one."""
    return x.materialize(ctx) if isinstance(x, SplitSum) else x


SPLIT_TO_CONSUMER = False
LONG_K = 8192


def _library_is_faster(rows: int, N: int, K: int) -> bool:
    """Measured on MI355X at the Qwen2.5-7B shapes: above 16 rows the library's product
    is faster than the MFMA kernels here unless K is long (its default kernels do not cut
    K; the ones its tuner finds do: the down projection at 32 rows 39 us against 53 us
    here, at 64 rows 46 us against 51 us)."""
    return rows > 16 and (K < LONG_K or library_tuning.enabled())


def _operand(x):
    """(activation dtype, the tensor a kernel reads, the owed row scale or None, whether
    that tensor lies piece-major) of a tensor, NormedRows or PieceRows."""
    if isinstance(x, NormedRows):
        return x.scaled.dtype, x.scaled, (x.partials, x.eps), x.pieces
    if isinstance(x, PieceRows):
        return x.pieces.dtype, x.pieces, None, True
    return x.dtype, x, None, False


class Linear:
    def __init__(self, weight: torch.Tensor, bias: torch.Tensor | None = None):
        if weight.dim() != 2:
            raise ValueError("Linear weight must be [out, in]")
        self.weight = weight
        self.bias = bias
        self.out_features, self.in_features = weight.shape
        self._splits: dict[int, int] = {}

    def _blocksplit_rows(self, rows: int, ctx: StepContext, act: torch.dtype) -> bool:
        """Whether the block-split kernel runs this product."""
        N, K = self.weight.shape
        return (self.weight.dtype == torch.bfloat16 and act == torch.bfloat16
                and ctx.env.fast_kernels and K % 8 == 0
                and 0 < rows <= (16 if _library_is_faster(ops.BLOCKSPLIT_MAX_M, N, K) else ops.BLOCKSPLIT_MAX_M))

    def reads_pieces(self, rows: int, ctx: StepContext) -> bool:
        """Whether bf16 input rows may come piece-major (PieceRows)."""
        return rows <= ops.PIECES_MAX_M and self._blocksplit_rows(rows, ctx, torch.bfloat16)

    def __call__(self, x, rows: int, ctx: StepContext, *, use_bias: bool = True,
                 out_dtype: torch.dtype | None = None, out: torch.Tensor | None = None,
                 allow_split: bool = False, sink: ResidualSink | None = None):
        """x: a tensor, NormedRows or PieceRows. With a sink the result may go into the
        residual stream directly; the call then returns None."""
        w = self.weight
        N, K = w.shape
        bias = self.bias if use_bias else None
        act, a, scale, pieces = _operand(x)
        out_dtype = out_dtype or act
        if self._blocksplit_rows(rows, ctx, act):
            if sink is not None and out is None and out_dtype == act and rows <= 16 \
                    and sink.stream.rows == rows and sink.stream.resid.shape[-1] == N:
                return self._into_residual(x, bias, rows, ctx, sink)
            if out is None:
                out = ctx.alloc((rows, N), out_dtype)
            ops.gemm_blocksplit(out, a, w, bias, rows, row_scale=scale, x_pieces=pieces)
            return out
        if isinstance(x, PieceRows):
            raise TypeError("Linear: piece-major rows for a product that does not read them (ask reads_pieces)")
        if isinstance(x, NormedRows):
            x = x.tensor(ctx)
        if rows == 0:
            return out if out is not None else ctx.alloc((0, N), out_dtype)
        if w.dtype == torch.float32:
            if out is None:
                out = ctx.alloc((rows, N), out_dtype)
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
        if not ctx.env.fast_kernels or K % 8 != 0:
            # the plain kernel also under bfloat16; the MFMA kernels take K in steps of 8
            if out is None:
                out = ctx.alloc((rows, N), out_dtype)
            ops.gemm_plain(out, x, w, bias, rows)
            return out
        # fp32 results of bf16 operands (the logits): the library writes them too. The head of the
        # Qwen2.5-7B shape at 64 rows: 221 us against 337 us for the MFMA kernel here.
        library_f32 = out_dtype == torch.float32 and bias is None and rows > ops.BLOCKSPLIT_MAX_M
        if rows <= ops.SKINNY_MAX_M and not library_f32 \
                and not (out_dtype == torch.bfloat16 and _library_is_faster(rows, N, K)):
            return self._skinny(x, bias, rows, ctx, out, out_dtype, allow_split)
        if out is None:
            out = ctx.alloc((rows, N), out_dtype)
        if library_tuning.enabled() and not library_tuning.worth_tuning(rows):
            with library_tuning.no_new_tuning():
                return self._library(x, bias, rows, out, out_dtype, library_f32, ctx)
        return self._library(x, bias, rows, out, out_dtype, library_f32, ctx)

    def _library(self, x, bias, rows, out, out_dtype, library_f32, ctx):
        w = self.weight
        if library_f32:
            with profiler.span("library_gemm"):
                torch.mm(x[:rows], w.t(), out_dtype=torch.float32, out=out[:rows])
            return out
        if out_dtype == torch.float32:
            # fp32 results of a tall product: 64 rows at a time through the MFMA kernel
            for r0 in range(0, rows, ops.SKINNY_MAX_M):
                r1 = min(rows, r0 + ops.SKINNY_MAX_M)
                self._skinny(x[r0:r1], bias, r1 - r0, ctx, out[r0:r1], out_dtype, False)
            return out
        with profiler.span("library_gemm"):
            if bias is not None:
                torch.addmm(bias, x[:rows], w.t(), out=out[:rows])
            else:
                torch.mm(x[:rows], w.t(), out=out[:rows])
        return out

    def _into_residual(self, x, bias, rows, ctx, sink: ResidualSink):
        N, K = self.weight.shape
        gain, eps = sink.norm.carried()
        out_pieces = N % 8 == 0 and rows <= ops.PIECES_MAX_M
        xg = ctx.alloc(ops.pieces_shape(rows, N) if out_pieces else (rows, N), torch.bfloat16)
        sq = ctx.alloc((rows, ops.gemm_blocksplit_blocks(rows, N, K)), torch.float32)
        _, a, scale, pieces = _operand(x)
        ops.gemm_blocksplit(None, a, self.weight, bias, rows, row_scale=scale,
                            residual=(sink.stream.resid, gain, xg, sq), x_pieces=pieces,
                            out_pieces=out_pieces)
        sink.stream.prepared = (sink.norm, NormedRows(xg, sq, eps, rows, out_pieces))
        return None

    def _skinny(self, x, bias, rows, ctx, out, out_dtype, allow_split):
        N, K = self.weight.shape
        if rows <= ops.BLOCKSPLIT_MAX_M and (rows <= 16 or K >= LONG_K):
            if out is None:
                out = ctx.alloc((rows, N), out_dtype)
            ops.gemm_blocksplit(out, x, self.weight, bias, rows)
            return out
        splits = self._splits.get(rows)
        if splits is None:
            splits = self._splits[rows] = ops.gemm_skinny_splits(rows, N, K)
        if splits == 1:
            if out is None:
                out = ctx.alloc((rows, N), out_dtype)
            ops.gemm_skinny(out, None, x, self.weight, bias, rows)
            return out
        partial = ctx.alloc((splits, rows, N), torch.float32)
        used = ops.gemm_skinny(None, partial, x, self.weight, None, rows, out_dtype=out_dtype)
        if used != splits:
            raise RuntimeError(f"Linear: planned {splits} K slices, the kernel used {used}")
        s = SplitSum(partial, bias, rows)
        if allow_split and SPLIT_TO_CONSUMER and out is None:
            return s
        return s.materialize(ctx, out_dtype, out)

    def gated_silu_rows(self, rows: int, ctx: StepContext, act: torch.dtype) -> bool:
        """Whether gated_silu applies to this many rows of this dtype."""
        w = self.weight
        return (ctx.env.fast_kernels and w.dtype == torch.bfloat16 and act == torch.bfloat16
                and 0 < rows <= 16 and w.shape[1] % 8 == 0 and w.shape[0] % 2 == 0)

    def gated_silu(self, x, rows: int, ctx: StepContext, out: torch.Tensor,
                   out_pieces: bool = False) -> None:
        """out[rows, N/2] = silu(gate) * up in one kernel, for a weight whose rows alternate gate
        and up (gate i at row 2i, its up at 2i + 1), where gated_silu_rows() says so. x: a tensor,
        NormedRows or PieceRows; out_pieces: out is shaped and written piece-major."""
        act, a, scale, pieces = _operand(x)
        if not self.gated_silu_rows(rows, ctx, act):
            raise ValueError("Linear.gated_silu: not for these rows (ask gated_silu_rows)")
        ops.gemm_blocksplit(out, a, self.weight, None, rows, gated=True, row_scale=scale,
                            x_pieces=pieces, out_pieces=out_pieces)
