"""Python faces of the HIP kernels: they check shapes, dtypes and contiguity on
the host, then launch on torch's current stream. Tensors are torch tensors on
the GPU; nothing here computes in torch."""
from __future__ import annotations

import torch

from . import kv_layout as layout
from . import lib as _lib
from .profiler import op as _op

F32, BF16, F16 = 0, 1, 2
PAGE_TOKENS = 64

_CODES = {torch.float32: F32, torch.bfloat16: BF16}


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _CODES[dtype]
    except KeyError:
        raise TypeError(f"kernels take float32 or bfloat16 tensors, not {dtype}") from None


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _need(t: torch.Tensor, name: str, dtype=None, shape=None) -> None:
    if not t.is_cuda:
        raise ValueError(f"{name}: expected a GPU tensor")
    if not t.is_contiguous():
        raise ValueError(f"{name}: expected a contiguous tensor")
    if dtype is not None and t.dtype != dtype:
        raise TypeError(f"{name}: expected {dtype}, got {t.dtype}")
    if shape is not None:
        if len(shape) != t.dim() or any(s is not None and s != d for s, d in zip(shape, t.shape)):
            raise ValueError(f"{name}: expected shape {tuple(shape)}, got {tuple(t.shape)}")


def _ptr(t: torch.Tensor | None) -> int | None:
    return None if t is None else t.data_ptr()


@_op("fill_random")
def fill_random(out, key: int, quantiles, mean: float, std: float) -> None:
    """out (float32 or bfloat16, any shape, contiguous) = seeded normal values, element by
    element what weights.random_init.normal_values gives on the host for the same key."""
    _need(out, "out")
    _need(quantiles, "quantiles", torch.float32, (65536,))
    L = _lib.load()
    _lib.check(L.he_fill_random(out.data_ptr(), out.numel(), dtype_code(out.dtype), key & ((1 << 64) - 1),
                                quantiles.data_ptr(), float(mean), float(std), _stream()))


@_op("fill_random")
def fill_random_integers(out_i32, key: int, high: int) -> None:
    _need(out_i32, "out", torch.int32)
    L = _lib.load()
    _lib.check(L.he_fill_random_integers(out_i32.data_ptr(), out_i32.numel(), key & ((1 << 64) - 1), int(high),
                                         _stream()))


@_op("cast")
def cast(out, src) -> None:
    """out (float32 or bfloat16) = src (float32, bfloat16 or float16) converted, same element count."""
    _need(out, "out")
    _need(src, "src")
    if out.numel() != src.numel():
        raise ValueError("cast: out and src differ in size")
    code = F16 if src.dtype == torch.float16 else dtype_code(src.dtype)
    L = _lib.load()
    _lib.check(L.he_cast(out.data_ptr(), src.data_ptr(), src.numel(), code, dtype_code(out.dtype), _stream()))


@_op("embedding")
def embedding(out_f32, table, ids, rows: int) -> None:
    V, D = table.shape
    _need(table, "table")
    _need(out_f32, "out", torch.float32)
    _need(ids, "ids", torch.int32)
    if out_f32.numel() < rows * D or ids.numel() < rows:
        raise ValueError("embedding: buffers smaller than the row count")
    L = _lib.load()
    _lib.check(L.he_embedding(out_f32.data_ptr(), table.data_ptr(), ids.data_ptr(), rows, D, V,
                              dtype_code(table.dtype), _stream()))


@_op("gather_rows")
def gather_rows_f32(out, src, rows_idx, n_out: int, n_src: int) -> None:
    D = src.shape[-1]
    _need(src, "src", torch.float32)
    _need(out, "out", torch.float32)
    _need(rows_idx, "rows", torch.int32)
    if out.numel() < n_out * D or rows_idx.numel() < n_out or src.numel() < n_src * D:
        raise ValueError("gather_rows: buffers smaller than the row counts")
    L = _lib.load()
    _lib.check(L.he_gather_rows_f32(out.data_ptr(), src.data_ptr(), rows_idx.data_ptr(), n_out, D,
                                    n_src, _stream()))


@_op("residual_add")
def residual_add(resid_f32, delta, rows: int) -> None:
    D = resid_f32.shape[-1]
    _need(resid_f32, "resid", torch.float32)
    _need(delta, "delta")
    if delta.shape[-1] != D or resid_f32.numel() < rows * D or delta.numel() < rows * D:
        raise ValueError("residual_add: shape mismatch")
    L = _lib.load()
    _lib.check(L.he_residual_add(resid_f32.data_ptr(), delta.data_ptr(), rows * D,
                                 dtype_code(delta.dtype), _stream()))


@_op("silu_mul")
def silu_mul(out, gate_up, rows: int, interleaved: bool = False, splits: int = 0) -> None:
    """out[rows, I] = silu(gate) * up. gate_up: [rows, 2I] in out's dtype, or with
    splits > 0 the fp32 K slices [splits, rows, 2I] of the product. Its columns are all
    gates then all ups, or, interleaved, gate i in column 2i and its up in 2i + 1."""
    I = out.shape[-1]
    _need(out, "out")
    _need(gate_up, "gate_up", torch.float32 if splits > 0 else out.dtype)
    if gate_up.shape[-1] != 2 * I or out.numel() < rows * I or \
            gate_up.numel() < max(splits, 1) * rows * 2 * I:
        raise ValueError("silu_mul: gate_up must be [rows, 2*I] for out [rows, I]")
    if splits > 0 and tuple(gate_up.shape) != (splits, rows, 2 * I):
        raise ValueError("silu_mul: split sums must be [splits, rows, 2*I]")
    L = _lib.load()
    _lib.check(L.he_silu_mul(out.data_ptr(), gate_up.data_ptr(), rows, I, int(interleaved), splits,
                             dtype_code(out.dtype), _stream()))


@_op("add_rmsnorm")
def add_rmsnorm(resid_f32, delta, weight, out, rows: int, eps: float) -> None:
    """resid += delta (if given); out = rmsnorm(resid) * weight (if out given)."""
    D = resid_f32.shape[-1]
    _need(resid_f32, "resid", torch.float32)
    _need(weight, "weight", shape=(D,))
    if resid_f32.numel() < rows * D:
        raise ValueError("add_rmsnorm: resid smaller than the row count")
    act = None
    if out is not None:
        _need(out, "out")
        if out.shape[-1] != D or out.numel() < rows * D:
            raise ValueError(f"add_rmsnorm: out does not match [rows, {D}]")
        act = out.dtype
    if delta is not None:
        _need(delta, "delta")
        if delta.shape[-1] != D or delta.numel() < rows * D:
            raise ValueError(f"add_rmsnorm: delta does not match [rows, {D}]")
        if act is not None and delta.dtype != act:
            raise TypeError("add_rmsnorm: delta and out must share a dtype")
        act = delta.dtype
    L = _lib.load()
    _lib.check(L.he_add_rmsnorm(resid_f32.data_ptr(), _ptr(delta), weight.data_ptr(), _ptr(out), rows, D,
                                float(eps), dtype_code(act or torch.float32), dtype_code(weight.dtype),
                                _stream()))


@_op("rmsnorm_rows")
def rmsnorm_rows(out, x, weight, rows: int, D: int, x_stride: int, out_stride: int,
                 eps: float) -> None:
    if out.dtype != x.dtype:
        raise TypeError("rmsnorm_rows: out and x must share a dtype")
    if weight is not None:
        _need(weight, "weight", shape=(D,))
    if rows > 0 and (x.numel() < (rows - 1) * x_stride + D or out.numel() < (rows - 1) * out_stride + D):
        raise ValueError("rmsnorm_rows: buffers smaller than rows and strides need")
    L = _lib.load()
    _lib.check(L.he_rmsnorm_rows(out.data_ptr(), x.data_ptr(), _ptr(weight), rows, D, x_stride,
                                 out_stride, float(eps), dtype_code(x.dtype),
                                 dtype_code(weight.dtype) if weight is not None else F32, _stream()))


def gemm_plain_workspace_floats(M: int, N: int, K: int) -> int:
    """Floats of workspace with which gemm_plain runs a product of few rows through the kernels made
    for it (0: none needed)."""
    return int(_lib.load().he_gemm_plain_workspace_floats(M, N, K))


@_op("gemm_plain")
def gemm_plain(out, a, w, bias, M: int, workspace=None) -> None:
    """out[M,N] = a[M,K] . w[N,K]^T (+ bias), fixed summation order. workspace: fp32, of
    gemm_plain_workspace_floats(M, N, K) elements or more, for a product of few rows (the result
    is the same bit for bit without it, and slower)."""
    N, K = w.shape
    _need(a, "a")
    _need(w, "w", a.dtype)
    _need(out, "out")
    if a.shape[-1] != K or out.shape[-1] != N or a.numel() < M * K or out.numel() < M * N:
        raise ValueError(f"gemm_plain: shapes a{tuple(a.shape)} w{tuple(w.shape)} out{tuple(out.shape)} M={M}")
    if bias is not None:
        _need(bias, "bias", shape=(N,))
    L = _lib.load()
    if workspace is not None:
        _need(workspace, "workspace", torch.float32)
    _lib.check(L.he_gemm_plain(out.data_ptr(), a.data_ptr(), w.data_ptr(), _ptr(bias), M, N, K, K,
                               K, N, dtype_code(a.dtype), dtype_code(out.dtype),
                               dtype_code(bias.dtype) if bias is not None else F32,
                               _ptr(workspace), workspace.numel() if workspace is not None else 0, _stream()))


BLOCKSPLIT_MAX_M = 32


PIECES_MAX_M = 64
BLOCKSPLIT_PIECES_MAX_M = 16   # the block-split product reads and writes pieces up to 16 rows
ROWS_MAX_M = 64


def pieces_shape(M: int, D: int) -> tuple[int, int, int]:
    """Shape of a piece-major [M, D] bf16 tensor: 16-byte pieces of 8 columns, the M pieces of
    one column group next to each other: element (m, d) at [d // 8, m, d % 8]. The block-split
    product reads its rows best this way (a wavefront's load of 16 rows x 16 bytes touches two
    cache lines, not sixteen), and writes them so for the next one; at most PIECES_MAX_M rows."""
    if D % 8 != 0 or not 0 < M <= PIECES_MAX_M:
        raise ValueError(f"piece-major rows: D={D} must be a multiple of 8 and 0 < M={M} <= {PIECES_MAX_M}")
    return (D // 8, M, 8)


def gemm_blocksplit_blocks(M: int, N: int, K: int) -> int:
    """Partial sums of squares per row that the residual epilogue of this product gives."""
    return int(_lib.load().he_gemm_blocksplit_blocks(M, N, K))


@_op("gemm_blocksplit")
def gemm_blocksplit(out, a, w, bias, M: int, gated: bool = False, plan=(0, 0, 0), *,
                    row_scale=None, residual=None, x_pieces: bool = False, out_pieces: bool = False) -> None:
    """bf16 MFMA product for M <= 32 with K cut inside the workgroup; one launch, complete
    result (bf16 or fp32), with bias or, gated, as [M, N/2] = silu(gate) * up for a weight
    that alternates gate and up rows (gate i at row 2i, its up at 2i + 1). plan = (R, U, NW),
    zeros = heuristic.

    row_scale = (partials fp32 [M, count], eps): the rows of `a` are r * gain of an RMS norm
    whose 1/sqrt(mean(r^2) + eps) is applied to the sums here (mean over K).
    residual = (resid fp32 [M, N], gain [N], xg bf16 [M, N], sq fp32 [M, blocks]): instead of
    writing `out` (None), resid += result in place, xg = resid * gain, sq = the sums of resid^2
    per workgroup (blocks = gemm_blocksplit_blocks(M, N, K)).
    x_pieces: `a` is piece-major, shaped pieces_shape(M, K). out_pieces: the bf16 output (`out`,
    or xg of the residual epilogue) is written piece-major, shaped pieces_shape(M, its width)."""
    N, K = w.shape
    NO = N // 2 if gated else N
    _need(a, "a", torch.bfloat16)
    _need(w, "w", torch.bfloat16)
    if M > BLOCKSPLIT_MAX_M:
        raise ValueError(f"gemm_blocksplit: M={M} above {BLOCKSPLIT_MAX_M}")
    if (x_pieces or out_pieces) and M > BLOCKSPLIT_PIECES_MAX_M:
        raise ValueError(f"gemm_blocksplit: piece-major rows are for up to {BLOCKSPLIT_PIECES_MAX_M} rows, not {M}")
    if x_pieces:
        _need(a, "a", shape=pieces_shape(M, K))
    elif a.shape[-1] != K or a.numel() < M * K:
        raise ValueError(f"gemm_blocksplit: shapes a{tuple(a.shape)} w{tuple(w.shape)} M={M}")
    if residual is None:
        _need(out, "out")
        if out_pieces:
            _need(out, "out", torch.bfloat16, pieces_shape(M, NO))
        elif out.shape[-1] != NO or out.numel() < M * NO:
            raise ValueError(f"gemm_blocksplit: out{tuple(out.shape)} for M={M} N={NO}")
    elif out is not None or gated or plan != (0, 0, 0):
        raise ValueError("gemm_blocksplit: the residual epilogue writes no `out`, is not gated and plans itself")
    if bias is not None:
        _need(bias, "bias", shape=(N,))
    sp, sc, se = None, 0, 0.0
    if row_scale is not None:
        partials, se = row_scale
        _need(partials, "row_scale partials", torch.float32)
        if partials.dim() != 2 or partials.shape[0] < M:
            raise ValueError("gemm_blocksplit: row_scale partials must be [M, count]")
        sp, sc = partials.data_ptr(), partials.shape[1]
    rp = gp = xp = qp = None
    gdt, qc = F32, 0
    if residual is not None:
        resid, gain, xg, sq = residual
        _need(resid, "resid", torch.float32)
        _need(gain, "gain", shape=(N,))
        _need(xg, "xg", torch.bfloat16)
        _need(sq, "sq", torch.float32)
        if out_pieces:
            _need(xg, "xg", shape=pieces_shape(M, N))
        if resid.shape[-1] != N or resid.numel() < M * N or xg.numel() < M * N \
                or (not out_pieces and xg.shape[-1] != N) or sq.dim() != 2 or sq.shape[0] < M:
            raise ValueError("gemm_blocksplit: residual buffers do not match [M, N]")
        rp, gp, xp, qp = resid.data_ptr(), gain.data_ptr(), xg.data_ptr(), sq.data_ptr()
        gdt, qc = dtype_code(gain.dtype), sq.shape[1]
    L = _lib.load()
    _lib.check(L.he_gemm_blocksplit_fused_bf16(
        _ptr(out), a.data_ptr(), w.data_ptr(), _ptr(bias), M, N, K,
        dtype_code(out.dtype) if out is not None else BF16,
        dtype_code(bias.dtype) if bias is not None else F32, int(gated),
        int(plan[0]), int(plan[1]), int(plan[2]), sp, sc, float(se), rp, gp, gdt, xp, qp, qc,
        int(x_pieces), int(out_pieces), _stream()))


def gemm_rows_plan(M: int, N: int, K: int) -> tuple[int, int]:
    """(workgroups along N, K slices) of gemm_rows for this product: the count of partial sums of
    squares its residual epilogue gives, and whether it leaves plain sums or partial sums."""
    import ctypes
    g, s = ctypes.c_int(0), ctypes.c_int(0)
    _lib.check(_lib.load().he_gemm_rows_plan(M, N, K, ctypes.byref(g), ctypes.byref(s)))
    return g.value, s.value


@_op("gemm_rows")
def gemm_rows(out, partial, a, w, bias, M: int, gated: bool = False, plan=(0, 0, 0), *, row_scale=None,
              residual=None, x_pieces: bool = False, out_pieces: bool = False) -> int:
    """bf16 MFMA product for M <= 64 whose activation rows go through LDS once per workgroup; the
    epilogues of gemm_blocksplit (see there: bias, gated, row_scale, residual, x_pieces, out_pieces).
    plan = (R, NWV, splits), zeros = heuristic. A product cut into several K slices writes its fp32
    sums into `partial` ([slices, M, N], each already scaled by row_scale) and takes no other
    epilogue. Returns the number of slices."""
    import ctypes
    N, K = w.shape
    NO = N // 2 if gated else N
    _need(a, "a", torch.bfloat16)
    _need(w, "w", torch.bfloat16)
    if not 0 < M <= ROWS_MAX_M:
        raise ValueError(f"gemm_rows: M={M} outside [1, {ROWS_MAX_M}]")
    if x_pieces:
        _need(a, "a", shape=pieces_shape(M, K))
    elif a.shape[-1] != K or a.numel() < M * K:
        raise ValueError(f"gemm_rows: shapes a{tuple(a.shape)} w{tuple(w.shape)} M={M}")
    if out is not None:
        _need(out, "out")
        if out_pieces:
            _need(out, "out", torch.bfloat16, pieces_shape(M, NO))
        elif out.shape[-1] != NO or out.numel() < M * NO:
            raise ValueError(f"gemm_rows: out{tuple(out.shape)} for M={M} N={NO}")
    pf = 0
    if partial is not None:
        _need(partial, "partial", torch.float32)
        pf = partial.numel()
    if bias is not None:
        _need(bias, "bias", shape=(N,))
    sp, sc, se = None, 0, 0.0
    if row_scale is not None:
        partials, se = row_scale
        _need(partials, "row_scale partials", torch.float32)
        if partials.dim() != 2 or partials.shape[0] < M:
            raise ValueError("gemm_rows: row_scale partials must be [M, count]")
        sp, sc = partials.data_ptr(), partials.shape[1]
    rp = gp = xp = qp = None
    gdt, qc = F32, 0
    if residual is not None:
        resid, gain, xg, sq = residual
        _need(resid, "resid", torch.float32)
        _need(gain, "gain", shape=(N,))
        _need(xg, "xg", torch.bfloat16)
        _need(sq, "sq", torch.float32)
        if out_pieces:
            _need(xg, "xg", shape=pieces_shape(M, N))
        if resid.shape[-1] != N or resid.numel() < M * N or xg.numel() < M * N \
                or (not out_pieces and xg.shape[-1] != N) or sq.dim() != 2 or sq.shape[0] < M:
            raise ValueError("gemm_rows: residual buffers do not match [M, N]")
        rp, gp, xp, qp = resid.data_ptr(), gain.data_ptr(), xg.data_ptr(), sq.data_ptr()
        gdt, qc = dtype_code(gain.dtype), sq.shape[1]
    used = ctypes.c_int(0)
    L = _lib.load()
    _lib.check(L.he_gemm_rows_bf16(
        _ptr(out), _ptr(partial), pf, a.data_ptr(), w.data_ptr(), _ptr(bias), M, N, K,
        dtype_code(out.dtype) if out is not None else BF16,
        dtype_code(bias.dtype) if bias is not None else F32, int(gated),
        int(plan[0]), int(plan[1]), int(plan[2]), sp, sc, float(se), rp, gp, gdt, xp, qp, qc,
        int(x_pieces), int(out_pieces), ctypes.byref(used), _stream()))
    return used.value


def splitk_reduce_residual_blocks(N: int) -> int:
    return int(_lib.load().he_splitk_reduce_residual_blocks(N))


@_op("splitk_reduce_residual")
def splitk_reduce_residual(resid, partial, bias, gain, xg, sq, M: int, splits: int,
                           out_pieces: bool = False) -> None:
    """resid [M, N] (fp32, in place) += the K slices partial [splits, M, N] in index order (+ bias);
    xg = bf16(resid * gain), piece-major with out_pieces; sq [M, blocks] = sums of resid^2 per block
    of columns (blocks = splitk_reduce_residual_blocks(N))."""
    N = resid.shape[-1]
    _need(resid, "resid", torch.float32)
    _need(partial, "partial", torch.float32)
    _need(gain, "gain", shape=(N,))
    _need(xg, "xg", torch.bfloat16)
    _need(sq, "sq", torch.float32)
    if out_pieces:
        _need(xg, "xg", shape=pieces_shape(M, N))
    if resid.numel() < M * N or partial.numel() < splits * M * N or xg.numel() < M * N \
            or sq.dim() != 2 or sq.shape[0] < M or (not out_pieces and xg.shape[-1] != N):
        raise ValueError("splitk_reduce_residual: buffers do not match [splits, M, N]")
    if bias is not None:
        _need(bias, "bias", shape=(N,))
    L = _lib.load()
    _lib.check(L.he_splitk_reduce_residual(
        resid.data_ptr(), partial.data_ptr(), _ptr(bias), dtype_code(bias.dtype) if bias is not None else F32,
        gain.data_ptr(), dtype_code(gain.dtype), xg.data_ptr(), sq.data_ptr(), sq.shape[1], M, N, splits,
        int(out_pieces), _stream()))


@_op("scale_rows")
def scale_rows(out, x, partials, eps: float, rows: int, x_pieces: bool = False) -> None:
    """out = x / sqrt(sum(partials of the row) / D + eps) for rows x = r * gain (bf16). out is
    row-major; x_pieces: x is piece-major, shaped pieces_shape(rows, D)."""
    D = out.shape[-1]
    _need(out, "out", torch.bfloat16)
    _need(x, "x", torch.bfloat16)
    _need(partials, "partials", torch.float32)
    if x_pieces:
        _need(x, "x", shape=pieces_shape(rows, D))
    if out.numel() < rows * D or x.numel() < rows * D or (not x_pieces and x.shape[-1] != D) \
            or partials.dim() != 2 or partials.shape[0] < rows:
        raise ValueError("scale_rows: buffers do not match [rows, D]")
    _lib.check(_lib.load().he_scale_rows_bf16(out.data_ptr(), x.data_ptr(), partials.data_ptr(),
                                              partials.shape[1], rows, D, float(eps), int(x_pieces),
                                              _stream()))


@_op("splitk_reduce")
def splitk_reduce(out, partial, bias, M: int, splits: int) -> None:
    """out[M, N] = sum of partial[s] over the slices in index order (+ bias)."""
    N = out.shape[-1]
    _need(out, "out")
    _need(partial, "partial", torch.float32)
    if partial.numel() < splits * M * N or out.numel() < M * N:
        raise ValueError("splitk_reduce: buffers smaller than [splits, M, N]")
    if bias is not None:
        _need(bias, "bias", shape=(N,))
    L = _lib.load()
    _lib.check(L.he_splitk_reduce(out.data_ptr(), partial.data_ptr(), _ptr(bias), M, N, splits,
                                  dtype_code(out.dtype),
                                  dtype_code(bias.dtype) if bias is not None else F32, _stream()))


@_op("qkv_rope_cache")
def qkv_rope_cache(q_out, kpool, vpool, qkv, q_cols: int, kv_cols: int, bias, positions, row_seq,
                   seq_slot, page_table, inv_freq, rotary_dim: int, rows: int, H: int, KVH: int,
                   hd: int, write_kv: bool) -> None:
    """qkv: [rows, q_cols (+ 2 kv_cols)] projected rows without bias; bias (optional) has the same
    column layout. Rotated q goes to q_out [rows, H*hd]; k, v go into the pools at
    (slot, position) when write_kv."""
    _need(qkv, "qkv")
    _need(q_out, "q_out")
    if qkv.dtype != q_out.dtype:
        raise TypeError("qkv_rope_cache: qkv and q_out must share a dtype")
    width = qkv.shape[-1]
    if q_cols != H * hd or (write_kv and (kv_cols != KVH * hd or width != q_cols + 2 * kv_cols)):
        raise ValueError("qkv_rope_cache: column layout does not match the head sizes")
    if not write_kv and width < q_cols:
        raise ValueError("qkv_rope_cache: qkv narrower than the query columns")
    if qkv.numel() < rows * width or q_out.numel() < rows * q_cols:
        raise ValueError("qkv_rope_cache: buffers smaller than the row count")
    _need(positions, "positions", torch.int32)
    _need(row_seq, "row_seq", torch.int32)
    _need(seq_slot, "seq_slot", torch.int32)
    if positions.numel() < rows or row_seq.numel() < rows:
        raise ValueError("qkv_rope_cache: metadata shorter than the row count")
    es = qkv.element_size()
    base = qkv.data_ptr()
    k_in = v_in = None
    max_blocks = num_pages = 0
    if write_kv:
        _need(kpool, "kpool", q_out.dtype, (None, KVH, layout.k_page_elems(hd)))
        _need(vpool, "vpool", q_out.dtype, (None, KVH, layout.v_page_elems(hd)))
        _need(page_table, "page_table", torch.int32)
        num_pages = kpool.shape[0]
        max_blocks = page_table.shape[1]
        k_in = base + q_cols * es
        v_in = base + (q_cols + kv_cols) * es
    qb = kb = vb = None
    bias_code = F32
    if bias is not None:
        _need(bias, "bias", shape=(width,))
        bias_code = dtype_code(bias.dtype)
        bes = bias.element_size()
        qb = bias.data_ptr()
        if write_kv:
            kb = qb + q_cols * bes
            vb = qb + (q_cols + kv_cols) * bes
    if rotary_dim:
        _need(inv_freq, "inv_freq", torch.float32, (rotary_dim // 2,))
    L = _lib.load()
    _lib.check(L.he_qkv_rope_cache(
        q_out.data_ptr(), _ptr(kpool) if write_kv else None, _ptr(vpool) if write_kv else None,
        base, k_in, v_in, width, qb, kb, vb, bias_code, positions.data_ptr(), row_seq.data_ptr(),
        seq_slot.data_ptr(), _ptr(page_table) if write_kv else None, max_blocks, num_pages,
        _ptr(inv_freq) if rotary_dim else None, rotary_dim, rows, H, KVH if write_kv else 0, hd,
        dtype_code(q_out.dtype), _stream()))


def _check_attention(out, q, kpool, vpool, page_table, rows, H, KVH, hd):
    _need(q, "q")
    _need(out, "out", q.dtype)
    _need(kpool, "kpool", q.dtype, (None, KVH, layout.k_page_elems(hd)))
    _need(vpool, "vpool", q.dtype, (None, KVH, layout.v_page_elems(hd)))
    _need(page_table, "page_table", torch.int32)
    if page_table.dim() != 2:
        raise ValueError("attention: page_table must be [slots, blocks]")
    if q.numel() < rows * H * hd or out.numel() < rows * H * hd:
        raise ValueError("attention: q/out smaller than the row count")


@_op("attention_plain")
def attention_plain(out, q, kpool, vpool, positions, row_seq, seq_slot, page_table, rows: int,
                    H: int, KVH: int, hd: int, window: int, scale: float, most_keys: int = 0,
                    workspace=None) -> None:
    """most_keys: a bound on the keys any sequence holds after the step, and workspace: fp32, of
    attention_plain_workspace_floats elements or more: the pages of a query then run in parallel
    (a step of few queries over many keys); the result is the same bit for bit without them."""
    _check_attention(out, q, kpool, vpool, page_table, rows, H, KVH, hd)
    if workspace is not None:
        _need(workspace, "workspace", torch.float32)
    for name, t in (("positions", positions), ("row_seq", row_seq), ("seq_slot", seq_slot)):
        _need(t, name, torch.int32)
    if positions.numel() < rows or row_seq.numel() < rows:
        raise ValueError("attention: metadata shorter than the row count")
    L = _lib.load()
    _lib.check(L.he_attention_plain(
        out.data_ptr(), q.data_ptr(), kpool.data_ptr(), vpool.data_ptr(), positions.data_ptr(),
        row_seq.data_ptr(), seq_slot.data_ptr(), page_table.data_ptr(), page_table.shape[1],
        kpool.shape[0], rows, H, KVH, hd, window, float(scale), dtype_code(q.dtype), int(most_keys),
        _ptr(workspace), workspace.numel() if workspace is not None else 0, _stream()))


def attention_plain_workspace_floats(rows: int, H: int, hd: int, most_keys: int, window: int) -> int:
    return int(_lib.load().he_attention_plain_workspace_floats(rows, H, hd, most_keys, window))


def attention_decode_workspace_floats(rows: int, H: int, KVH: int, hd: int, max_keys: int) -> int:
    return int(_lib.load().he_attention_decode_workspace_floats(rows, H, KVH, hd, max_keys))


@_op("attention_decode")
def attention_decode(out, q, kpool, vpool, positions, row_seq, seq_slot, page_table, rows: int,
                     H: int, KVH: int, hd: int, window: int, scale: float, max_keys: int,
                     workspace) -> None:
    _check_attention(out, q, kpool, vpool, page_table, rows, H, KVH, hd)
    _need(q, "q", torch.bfloat16)
    for name, t in (("positions", positions), ("row_seq", row_seq), ("seq_slot", seq_slot)):
        _need(t, name, torch.int32)
    if positions.numel() < rows or row_seq.numel() < rows:
        raise ValueError("attention: metadata shorter than the row count")
    _need(workspace, "workspace", torch.float32)
    L = _lib.load()
    _lib.check(L.he_attention_decode_bf16(
        out.data_ptr(), q.data_ptr(), kpool.data_ptr(), vpool.data_ptr(), positions.data_ptr(),
        row_seq.data_ptr(), seq_slot.data_ptr(), page_table.data_ptr(), page_table.shape[1],
        kpool.shape[0], rows, H, KVH, hd, window, float(scale), max_keys, workspace.data_ptr(),
        workspace.numel(), _stream()))


def attention_decode_fused_ok(H: int, KVH: int, hd: int, rotary_dim: int) -> bool:
    return int(_lib.load().he_attention_decode_fused_ok(H, KVH, hd, rotary_dim)) > 0


def attention_decode_fused_workspace_floats(rows: int, H: int, KVH: int, hd: int, max_keys: int,
                                           spread: bool = False) -> int:
    return int(_lib.load().he_attention_decode_fused_workspace_floats(rows, H, KVH, hd, max_keys, int(spread)))


@_op("attention_decode_fused")
def attention_decode_fused(out, qkv, bias, kpool, vpool, positions, row_seq, seq_slot, page_table,
                           inv_freq, rotary_dim: int, rows: int, H: int, KVH: int, hd: int,
                           window: int, scale: float, max_keys: int, write_kv: bool,
                           workspace, out_pieces: bool = False, spread: bool = False) -> None:
    """One-token steps in one launch: bias, rotation of q and of the new key, cache write,
    attention over the cache, merge. spread: one sequence has several times the keys of the
    others (every sequence's keys are then cut across more workgroups; the workspace is asked for
    with the same flag). qkv: bf16 [rows, (H + 2 KVH) hd] without bias, or fp32 [slices, rows, width]:
    the sums of the projection's K slices as gemm_rows leaves them; q columns
    alone where the run reads another run's cache (write_kv False). out_pieces: out is written
    piece-major for exactly `rows` rows (see :func:`to_pieces`). seq_slot None: page_table has a row
    per row of the step ([rows or more, blocks]: the page numbers of the row's sequence), not a
    row per slot; the kernel then asks for them at its start, without the chain through the slot."""
    width = (H + 2 * KVH) * hd if write_kv else H * hd
    _need(out, "out", torch.bfloat16)
    slices, slice_stride = 0, 0
    if qkv.dtype == torch.float32:
        # the fp32 sums of the projection's K slices, [slices, rows of the product, width] (gemm_rows):
        # the kernel adds them itself, in slice order, and rounds as splitk_reduce would have
        _need(qkv, "qkv (K slices)", torch.float32)
        if qkv.dim() != 3 or qkv.shape[2] != width or qkv.shape[1] < rows:
            raise ValueError("attention_decode_fused: K slices [slices, rows, width] do not match the head sizes and row count")
        slices, slice_stride = qkv.shape[0], qkv.shape[1] * width
    else:
        _need(qkv, "qkv", torch.bfloat16)
        if qkv.dim() != 2 or qkv.shape[1] != width or qkv.shape[0] < rows:
            raise ValueError("attention_decode_fused: qkv does not match the head sizes and row count")
    if out.numel() < rows * H * hd:
        raise ValueError("attention_decode_fused: out does not match the head sizes and row count")
    if out_pieces:
        _need(out, "out", shape=pieces_shape(rows, H * hd))
    _need(kpool, "kpool", torch.bfloat16, (None, KVH, layout.k_page_elems(hd)))
    _need(vpool, "vpool", torch.bfloat16, (None, KVH, layout.v_page_elems(hd)))
    _need(page_table, "page_table", torch.int32)
    for name, t in (("positions", positions), ("row_seq", row_seq)) + ((("seq_slot", seq_slot),) if seq_slot is not None else ()):
        _need(t, name, torch.int32)
    if positions.numel() < rows or row_seq.numel() < rows or page_table.dim() != 2:
        raise ValueError("attention_decode_fused: metadata shorter than the row count")
    if seq_slot is None and page_table.shape[0] < rows:
        raise ValueError("attention_decode_fused: a page table by rows needs a row per row of the step")
    if bias is not None:
        _need(bias, "bias", shape=(width,))
    _need(inv_freq, "inv_freq", torch.float32, (rotary_dim // 2,))
    if workspace is not None:
        _need(workspace, "workspace", torch.float32)
    L = _lib.load()
    _lib.check(L.he_attention_decode_fused_bf16(
        out.data_ptr(), qkv.data_ptr() if not slices else None, qkv.data_ptr() if slices else None, slices,
        slice_stride, width, _ptr(bias),
        dtype_code(bias.dtype) if bias is not None else F32, kpool.data_ptr(), vpool.data_ptr(),
        positions.data_ptr(), row_seq.data_ptr(), _ptr(seq_slot), page_table.data_ptr(),
        page_table.shape[1], kpool.shape[0], inv_freq.data_ptr(), rotary_dim, rows, H, KVH, hd,
        window, float(scale), max_keys, int(spread), int(write_kv), int(out_pieces), _ptr(workspace),
        workspace.numel() if workspace is not None else 0, _stream()))


def attention_prefill_parts(num_seqs: int, max_q_len: int, H: int, hd: int, most_keys: int) -> int:
    """Parts the library would cut the keys of this prompt step into (1: none): more than one
    for a step of few queries against many keys, which would otherwise leave most of the chip idle."""
    return int(_lib.load().he_attention_prefill_parts(num_seqs, max_q_len, H, hd, most_keys))


def attention_prefill_workspace_floats(total_rows: int, H: int, hd: int, parts: int) -> int:
    return int(_lib.load().he_attention_prefill_workspace_floats(total_rows, H, hd, parts))


@_op("attention_prefill")
def attention_prefill(out, q, kpool, vpool, cu_seqlens, seq_slot, seq_start, page_table,
                      num_seqs: int, max_q_len: int, total_rows: int, H: int, KVH: int, hd: int,
                      window: int, scale: float, kernel: int = 0, parts: int = 1, workspace=None) -> None:
    """kernel: 0 leaves the choice to the library (by head size and prompt length); 1 or 2
    name it: 16 queries a wavefront with operands from global memory, or 32 queries a
    wavefront with the pages shared through LDS (head sizes up to 128). parts > 1 (kernel 2):
    the keys in that many parts side by side, joined by a second launch; the workspace holds
    attention_prefill_workspace_floats() floats."""
    _check_attention(out, q, kpool, vpool, page_table, total_rows, H, KVH, hd)
    _need(q, "q", torch.bfloat16)
    for name, t in (("cu_seqlens", cu_seqlens), ("seq_slot", seq_slot), ("seq_start", seq_start)):
        _need(t, name, torch.int32)
    if cu_seqlens.numel() < num_seqs + 1 or seq_slot.numel() < num_seqs or seq_start.numel() < num_seqs:
        raise ValueError("attention_prefill: metadata shorter than the sequence count")
    if workspace is not None:
        _need(workspace, "workspace", torch.float32)
    L = _lib.load()
    _lib.check(L.he_attention_prefill_bf16(
        out.data_ptr(), q.data_ptr(), kpool.data_ptr(), vpool.data_ptr(), cu_seqlens.data_ptr(),
        seq_slot.data_ptr(), seq_start.data_ptr(), page_table.data_ptr(), page_table.shape[1],
        kpool.shape[0], num_seqs, max_q_len, H, KVH, hd, window, float(scale), int(kernel),
        total_rows, int(parts), _ptr(workspace), workspace.numel() if workspace is not None else 0,
        _stream()))


@_op("argmax_rows")
def argmax_rows(out_i32, logits, rows: int) -> None:
    _need(logits, "logits", torch.float32)
    _need(out_i32, "out", torch.int32)
    V = logits.shape[-1]
    if logits.numel() < rows * V or out_i32.numel() < rows:
        raise ValueError("argmax_rows: buffers smaller than the row count")
    L = _lib.load()
    need = int(L.he_argmax_workspace_bytes(rows, V))
    ws = torch.empty(need, dtype=torch.uint8, device=logits.device) if need else None
    _lib.check(L.he_argmax_rows(out_i32.data_ptr(), logits.data_ptr(), rows, V, V, _ptr(ws), need, _stream()))


@_op("apply_penalties")
def apply_penalties(logits, rows: int, ids, counts, offsets, rep: float, freq: float,
                    pres: float) -> None:
    _need(logits, "logits", torch.float32)
    for name, t in (("ids", ids), ("counts", counts), ("offsets", offsets)):
        _need(t, name, torch.int32)
    V = logits.shape[-1]
    if logits.numel() < rows * V or offsets.numel() < rows + 1 or ids.numel() != counts.numel():
        raise ValueError("apply_penalties: buffers do not match the row count")
    L = _lib.load()
    _lib.check(L.he_apply_penalties(logits.data_ptr(), rows, V, V, ids.data_ptr(),
                                    counts.data_ptr(), offsets.data_ptr(), float(rep), float(freq),
                                    float(pres), _stream()))


PENALTY_WINDOW_MAX = 4096


@_op("apply_penalties_window")
def apply_penalties_window(logits, rows: int, window, appended, last_ids, rep: float, freq: float,
                           pres: float) -> None:
    """The penalties of apply_penalties from a ring of recent tokens on the device: window int32
    [rows, W] (token number n at n % W), appended int32 [rows] (tokens ever appended). last_ids
    (int32 [rows] or None) are appended first. Changes logits in place."""
    _need(logits, "logits", torch.float32)
    _need(window, "window", torch.int32)
    _need(appended, "appended", torch.int32)
    V = logits.shape[-1]
    if window.dim() != 2 or window.shape[0] < rows or appended.numel() < rows or logits.numel() < rows * V:
        raise ValueError("apply_penalties_window: buffers smaller than the row count")
    if last_ids is not None:
        _need(last_ids, "last_ids", torch.int32)
        if last_ids.numel() < rows:
            raise ValueError("apply_penalties_window: fewer ids than rows")
    L = _lib.load()
    _lib.check(L.he_apply_penalties_window(logits.data_ptr(), rows, V, V, window.data_ptr(),
                                           appended.data_ptr(), window.shape[1], _ptr(last_ids),
                                           float(rep), float(freq), float(pres), _stream()))


@_op("sample_rows")
def sample_rows(out_i32, logits, rows: int, uniforms_u32, temperature: float, top_k: int,
                top_p: float) -> None:
    _need(logits, "logits", torch.float32)
    _need(out_i32, "out", torch.int32)
    _need(uniforms_u32, "uniforms")
    if uniforms_u32.element_size() != 4 or uniforms_u32.numel() < rows:
        raise ValueError("sample_rows: uniforms must be one 32-bit word per row")
    V = logits.shape[-1]
    if logits.numel() < rows * V or out_i32.numel() < rows:
        raise ValueError("sample_rows: buffers smaller than the row count")
    L = _lib.load()
    _lib.check(L.he_sample_rows(out_i32.data_ptr(), logits.data_ptr(), rows, V, V,
                                uniforms_u32.data_ptr(), float(temperature), int(top_k),
                                float(top_p), _stream()))
