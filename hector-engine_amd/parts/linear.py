"""The linear layer all parts share: y[M,N] = x[M,K] . W[N,K]^T (+ bias).

Which kernel runs is looked up in the table of kernel routes (kernels.routes) under
("linear", (weight dtype, activation dtype)) with the step's row count; the routes this file
registers:
  float32 weights          -> the plain FMA kernel (fixed summation order per element);
                              a weight that was stored in 32-bit stays 32-bit and runs
                              through it also under bfloat16 activations
  bfloat16, M <= 16        -> the block-split MFMA kernel: K is cut inside the workgroup,
                              one launch gives the finished result
  bfloat16, 17 <= M <= 64  -> the MFMA kernel that shares the activation rows of a workgroup
                              through LDS (kernels.ops.gemm_rows); products with few weight rows
                              are cut along K across workgroups and leave fp32 slices, which a
                              small kernel adds (into the result, or straight into the residual)
  bfloat16, M > 64         -> the library matrix product (the reference calls its BLAS
                              library for every product: kernels/matmul_cublas.cu:240-277)
  fp32 results (logits)    -> the MFMA kernels up to 64 rows, above that the library,
                              which writes fp32 from bf16 operands

Both MFMA kernels carry an RMS norm across a pair of products, so that a step of up to 64
rows has no norm kernels: given a :class:`ResidualSink` the product adds its result
to the residual rows itself and leaves r * gain and the sums of r^2 for the norm that
follows (:class:`NormedRows`); given NormedRows as input it applies the owed row scale
to its sums. Any other path turns NormedRows into a tensor first and ignores the sink.

Between such products the bf16 rows travel piece-major (kernels.ops.pieces_shape): an
operand load then touches two cache lines instead of sixteen (at the Qwen2.5-7B shapes 2 us a
layer at 8 rows, 10 us at 16; at 64 rows the gated product takes 61 us against 97 us). The
rows a product leaves for the next norm are written so; a producer of its input (attention,
the gated product) writes so after asking reads_pieces().
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

from ..kernels import library_tuning, ops, profiler, routes
from .base import NormedRows, PieceRows, ResidualSink, StepContext

BF16, F32 = torch.bfloat16, torch.float32


@dataclass(frozen=True)
class ProductCase:
    """What a route of "linear" decides by."""
    rows: int
    N: int
    K: int
    fast: bool          # the environment allows the MFMA kernels and the library


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
        self._plans: dict[bool, tuple[int, int]] = {}
        self._chosen: dict[tuple, routes.Route] = {}     # (rows, activations, fast) -> route, for one version of the table
        self._chosen_version = -1

    def route(self, rows: int, ctx: StepContext, act: torch.dtype) -> routes.Route:
        """The kernel route of this product at this many rows of this activation dtype (remembered
        per row count while the table of routes does not change: a step asks a hundred times)."""
        if self._chosen_version != routes.version() or len(self._chosen) > 256:
            self._chosen.clear()
            self._chosen_version = routes.version()
        key = (rows, act, ctx.env.fast_kernels)
        route = self._chosen.get(key)
        if route is None:
            N, K = self.weight.shape
            route = routes.choose("linear", (self.weight.dtype, act), ProductCase(rows, N, K, ctx.env.fast_kernels))
            self._chosen[key] = route
        return route

    def _has(self, trait: str, rows: int, ctx: StepContext, act: torch.dtype) -> bool:
        if not routes.routes_of("linear", (self.weight.dtype, act)):
            return False
        return trait in self.route(rows, ctx, act).traits

    def reads_pieces(self, rows: int, ctx: StepContext) -> bool:
        """Whether bf16 input rows may come piece-major (PieceRows)."""
        return self._has("pieces", rows, ctx, BF16)

    def k_slices(self, x, rows: int, ctx: StepContext):
        """The product without bias as the fp32 sums of its K slices, [slices, rows, N], where the
        kernel of this step cuts it along K across workgroups (17 to 64 rows of a weight with few
        rows); None where it does not, and the caller calls the layer as usual. A reader that adds
        the slices itself, in their order, and rounds to the activation dtype has the bits the
        layer's own sum would have written, and saves that launch."""
        act, a, scale, pieces = _operand(x)
        if rows <= ops.BLOCKSPLIT_PIECES_MAX_M or not self._has("k_slices", rows, ctx, act):
            return None
        splits = self._plan(rows)[1]
        if splits == 1:
            return None
        partial = ctx.alloc((splits, rows, self.weight.shape[0]), torch.float32)
        ops.gemm_rows(None, partial, a, self.weight, None, rows, row_scale=scale, x_pieces=pieces)
        return partial

    def _plan(self, rows: int) -> tuple[int, int]:
        """(workgroups along N, K slices) of the 17-to-64-row kernel for this weight."""
        key = rows <= 32
        if key not in self._plans:
            self._plans[key] = ops.gemm_rows_plan(rows, *self.weight.shape)
        return self._plans[key]

    def __call__(self, x, rows: int, ctx: StepContext, *, use_bias: bool = True,
                 out_dtype: torch.dtype | None = None, out: torch.Tensor | None = None,
                 sink: ResidualSink | None = None):
        """x: a tensor, NormedRows or PieceRows. With a sink the result may go into the
        residual stream directly; the call then returns None."""
        bias = self.bias if use_bias else None
        act = _operand(x)[0]
        return self.route(rows, ctx, act).run(self, x, rows, ctx, bias, out_dtype or act, out, sink)

    # ---- the routes' bodies ----

    def _run_mfma(self, x, rows, ctx, bias, out_dtype, out, sink):
        """Up to 64 rows of bf16: the block-split kernel (up to 16 rows) or the rows kernel."""
        w = self.weight
        N = w.shape[0]
        act, a, scale, pieces = _operand(x)
        if sink is not None and out is None and out_dtype == act \
                and sink.stream.rows == rows and sink.stream.resid.shape[-1] == N:
            return self._into_residual(x, bias, rows, ctx, sink)
        if out is None:
            out = ctx.alloc((rows, N), out_dtype)
        if rows <= ops.BLOCKSPLIT_PIECES_MAX_M:
            ops.gemm_blocksplit(out, a, w, bias, rows, row_scale=scale, x_pieces=pieces)
            return out
        splits = self._plan(rows)[1]
        if splits == 1:
            ops.gemm_rows(out, None, a, w, bias, rows, row_scale=scale, x_pieces=pieces)
            return out
        partial = ctx.alloc((splits, rows, N), torch.float32)
        ops.gemm_rows(None, partial, a, w, None, rows, row_scale=scale, x_pieces=pieces)
        ops.splitk_reduce(out, partial, bias, rows, splits)
        return out

    def _dense(self, x, rows, ctx, out_dtype, out):
        """(x as a plain tensor, the result buffer) for the routes that read row-major rows."""
        if isinstance(x, PieceRows):
            raise TypeError("Linear: piece-major rows for a product that does not read them (ask reads_pieces)")
        if isinstance(x, NormedRows):
            x = x.tensor(ctx)
        if out is None:
            out = ctx.alloc((rows, self.weight.shape[0]), out_dtype)
        return x, out

    def _run_plain(self, x, rows, ctx, bias, out_dtype, out, sink):
        """The plain kernel (fixed summation order) in the precision of its operands."""
        x, out = self._dense(x, rows, ctx, out_dtype, out)
        if rows == 0:
            return out
        if x.dtype == torch.float32 and out_dtype != torch.float32:
            raise TypeError("float32 activations give float32 outputs")
        self._plain(out, x, bias, rows, ctx)
        return out

    def _run_plain_widened(self, x, rows, ctx, bias, out_dtype, out, sink):
        """A weight kept in 32-bit under bfloat16 activations: the rows widened, the plain kernel."""
        x, out = self._dense(x, rows, ctx, out_dtype, out)
        if rows == 0:
            return out
        N, K = self.weight.shape
        x32 = ctx.alloc((rows, K), torch.float32)
        x32.copy_(x[:rows])
        y32 = out if out_dtype == torch.float32 else ctx.alloc((rows, N), torch.float32)
        self._plain(y32, x32, bias, rows, ctx)
        if y32 is not out:
            out[:rows].copy_(y32)
        return out

    def _run_library(self, x, rows, ctx, bias, out_dtype, out, sink):
        x, out = self._dense(x, rows, ctx, out_dtype, out)
        if rows == 0:
            return out
        if library_tuning.enabled() and not library_tuning.worth_tuning(rows):
            with library_tuning.no_new_tuning():
                return self._library(x, bias, rows, out, out_dtype, ctx)
        return self._library(x, bias, rows, out, out_dtype, ctx)

    def _plain(self, out, x, bias, rows: int, ctx: StepContext) -> None:
        """The plain product (fixed summation order); with few rows through its kernels for them,
        which want a workspace for their segment sums."""
        floats = ops.gemm_plain_workspace_floats(rows, *self.weight.shape)
        ws = ctx.alloc((floats,), torch.float32) if floats else None
        ops.gemm_plain(out, x, self.weight, bias, rows, workspace=ws)

    def _library_slices(self, rows: int) -> int:
        """K slices for the library's product of a long-K weight with few output columns at up to
        512 rows (the down projection in a step of a few hundred tokens): the library's tiles of
        256 x 256 outputs would be a dozen or two for a chip of 256 compute units, each walking all
        of K. As a batched product over K slices with fp32 results, which he_splitk_reduce adds
        in slice order, the Qwen2.5-7B down projection takes 58 us instead of 99 at 128 rows, 50
        instead of 122 at 200, 54 instead of 126 at 256, 80 instead of 197 at 512 (four slices); the
        Qwen2.5-32B one 68 instead of 180 at 128 rows, the Qwen2-72B one (four slices) 142 instead of 226. Products with
        K below 8192 gain nothing (q||k||v, o, gate||up: measured)."""
        N, K = self.weight.shape
        if rows > 512 or K < 8192 or K < 3 * N:
            return 1
        tiles = -(-rows // 256) * -(-N // 256)
        slices = 8 if tiles <= 20 else 4 if tiles <= 40 else 2 if tiles <= 64 else 1
        while slices > 1 and K % (8 * slices):
            slices //= 2
        return slices

    def _library(self, x, bias, rows, out, out_dtype, ctx):
        """More than 64 rows: the library's product; it also writes fp32 results (the logits) from
        bf16 operands (the head of the Qwen2.5-7B shape at 64 rows: 217 us)."""
        w = self.weight
        slices = self._library_slices(rows) if out_dtype == torch.bfloat16 and x.is_contiguous() else 1
        if slices > 1:
            N, K = w.shape
            partial = ctx.alloc((slices, rows, N), torch.float32)
            with profiler.span("library_gemm"):
                # views, no copies: slice s of x is [rows, K / slices] at row stride K, of w likewise
                torch.bmm(x[:rows].view(rows, slices, K // slices).transpose(0, 1),
                          w.view(N, slices, K // slices).permute(1, 2, 0),
                          out_dtype=torch.float32, out=partial)
            ops.splitk_reduce(out, partial, bias, rows, slices)
            return out
        with profiler.span("library_gemm"):
            if out_dtype == torch.float32:
                torch.mm(x[:rows], w.t(), out_dtype=torch.float32, out=out[:rows])
                if bias is not None:
                    out[:rows] += bias
            elif bias is not None:
                torch.addmm(bias, x[:rows], w.t(), out=out[:rows])
            else:
                torch.mm(x[:rows], w.t(), out=out[:rows])
        return out

    def _into_residual(self, x, bias, rows, ctx, sink: ResidualSink):
        """The product added into the residual rows, and the rows of the norm that follows left as
        NormedRows: by the product's own epilogue, or, where it is cut along K, by the kernel
        that adds the slices."""
        N, K = self.weight.shape
        gain, eps = sink.norm.carried()
        out_pieces = N % 8 == 0
        xg = ctx.alloc(ops.pieces_shape(rows, N) if out_pieces else (rows, N), torch.bfloat16)
        _, a, scale, pieces = _operand(x)
        if rows <= ops.BLOCKSPLIT_PIECES_MAX_M:
            sq = ctx.alloc((rows, ops.gemm_blocksplit_blocks(rows, N, K)), torch.float32)
            ops.gemm_blocksplit(None, a, self.weight, bias, rows, row_scale=scale,
                                residual=(sink.stream.resid, gain, xg, sq), x_pieces=pieces,
                                out_pieces=out_pieces)
        else:
            groups, splits = self._plan(rows)
            if splits == 1:
                sq = ctx.alloc((rows, groups), torch.float32)
                ops.gemm_rows(None, None, a, self.weight, bias, rows, row_scale=scale,
                              residual=(sink.stream.resid, gain, xg, sq), x_pieces=pieces, out_pieces=out_pieces)
            else:
                partial = ctx.alloc((splits, rows, N), torch.float32)
                ops.gemm_rows(None, partial, a, self.weight, None, rows, row_scale=scale, x_pieces=pieces)
                sq = ctx.alloc((rows, ops.splitk_reduce_residual_blocks(N)), torch.float32)
                ops.splitk_reduce_residual(sink.stream.resid, partial, bias, gain, xg, sq, rows, splits,
                                           out_pieces=out_pieces)
        sink.stream.prepared = (sink.norm, NormedRows(xg, sq, eps, rows, out_pieces))
        return None

    def gated_silu_rows(self, rows: int, ctx: StepContext, act: torch.dtype) -> bool:
        """Whether gated_silu applies to this many rows of this dtype."""
        return self._has("gated", rows, ctx, act) and self.weight.shape[0] % 2 == 0

    def gated_silu(self, x, rows: int, ctx: StepContext, out: torch.Tensor,
                   out_pieces: bool = False) -> None:
        """out[rows, N/2] = silu(gate) * up in one kernel, for a weight whose rows alternate gate
        and up (gate i at row 2i, its up at 2i + 1), where gated_silu_rows() says so. x: a tensor,
        NormedRows or PieceRows; out_pieces: out is shaped and written piece-major."""
        act, a, scale, pieces = _operand(x)
        if not self.gated_silu_rows(rows, ctx, act):
            raise ValueError("Linear.gated_silu: not for these rows (ask gated_silu_rows)")
        if rows <= ops.BLOCKSPLIT_PIECES_MAX_M:
            ops.gemm_blocksplit(out, a, self.weight, None, rows, gated=True, row_scale=scale,
                                x_pieces=pieces, out_pieces=out_pieces)
            return
        splits = self._plan(rows)[1]
        if splits == 1:
            ops.gemm_rows(out, None, a, self.weight, None, rows, gated=True, row_scale=scale,
                          x_pieces=pieces, out_pieces=out_pieces)
            return
        # few weight rows, cut along K: the activation kernel adds the slices while it reads them
        if out_pieces:
            raise ValueError("Linear.gated_silu: a product cut along K writes row-major (ask gated_pieces)")
        partial = ctx.alloc((splits, rows, self.weight.shape[0]), torch.float32)
        ops.gemm_rows(None, partial, a, self.weight, None, rows, row_scale=scale, x_pieces=pieces)
        ops.silu_mul(out, partial, rows, True, splits)

    def gated_pieces(self, rows: int) -> bool:
        """Whether gated_silu can write its result piece-major at this many rows."""
        return rows <= ops.BLOCKSPLIT_PIECES_MAX_M or self._plan(rows)[1] == 1


def _mfma_takes(case: ProductCase) -> bool:
    # the MFMA kernels take K in steps of 8
    return case.fast and case.K % 8 == 0 and 0 < case.rows <= ops.ROWS_MAX_M


routes.register_route("linear", (BF16, BF16), "mfma", _mfma_takes, Linear._run_mfma,
                      traits=("pieces", "gated", "k_slices"))
routes.register_route("linear", (BF16, BF16), "plain", lambda c: not c.fast or c.K % 8 != 0, Linear._run_plain)
routes.register_route("linear", (BF16, BF16), "library", lambda c: True, Linear._run_library)
routes.register_route("linear", (F32, F32), "plain", lambda c: True, Linear._run_plain)
routes.register_route("linear", (F32, BF16), "plain_widened", lambda c: True, Linear._run_plain_widened)
