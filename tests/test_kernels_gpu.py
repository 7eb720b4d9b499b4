"""Each HIP kernel alone against a plain fp32/fp64 torch reference of the same
op, at sizes other than the engine's tiny models (widths that are no power of
two, head sizes in steps of 16, odd row counts, scattered cache pages)."""
import math

import numpy as np
import pytest
import torch

from tests.plain import qwen2_plain as P

pytestmark = pytest.mark.gpu
PAGE = 64


@pytest.fixture(scope="module")
def ops():
    import hector_engine_amd  # noqa: F401
    from hector_engine_amd.kernels import lib, ops as _ops
    lib.load()
    assert lib.loaded_path().endswith(".so")
    return _ops


def dev(t):
    return t.to("cuda")


def rnd(*shape, seed=0, scale=1.0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype)


# ------------------------------------------------------------------ row-wise
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embedding_rows_and_bad_ids(ops, dtype):
    V, D = 301, 80
    table = rnd(V, D, seed=1).to(dtype)
    ids = torch.tensor([2, 300, 0, -1, 301, 17], dtype=torch.int32)
    out = torch.empty(len(ids), D, device="cuda")
    ops.embedding(out, dev(table), dev(ids), len(ids))
    ref = P.embedding(ids.long(), table.float())
    assert torch.equal(out.cpu(), ref)           # a copy: exact
    assert torch.equal(out.cpu()[0], table[2].float())   # the reference's own row check
    assert out.cpu()[3].abs().max() == 0 and out.cpu()[4].abs().max() == 0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_silu_mul(ops, dtype):
    rows, I = 7, 136
    x = rnd(rows, 2 * I, seed=2, scale=2.0).to(dtype)
    out = torch.empty(rows, I, dtype=dtype, device="cuda")
    ops.silu_mul(out, dev(x), rows)
    xf = x.double()
    ref = P.silu(xf[:, :I]) * xf[:, I:]
    tol = 1e-6 if dtype == torch.float32 else 2 ** -7
    assert torch.allclose(out.cpu().double(), ref, rtol=tol, atol=tol)


def test_gather_rows(ops):
    src = rnd(9, 50, seed=3)
    idx = torch.tensor([8, 0, 3, 3], dtype=torch.int32)
    out = torch.empty(4, 50, device="cuda")
    ops.gather_rows_f32(out, dev(src), dev(idx), 4, 9)
    assert torch.equal(out.cpu(), src[idx.long()])


@pytest.mark.parametrize("dtype,wdtype", [(torch.float32, torch.float32), (torch.bfloat16, torch.bfloat16),
                                          (torch.bfloat16, torch.float32)])
@pytest.mark.parametrize("D,eps", [(80, 3e-6), (3584, 1e-6), (100, 1e-5)])
def test_add_rmsnorm(ops, dtype, wdtype, D, eps):
    rows = 5
    resid = rnd(rows, D, seed=4)
    delta = rnd(rows, D, seed=5).to(dtype)
    w = (1 + 0.1 * rnd(D, seed=6)).to(wdtype)
    r = dev(resid.clone())
    out = torch.empty(rows, D, dtype=dtype, device="cuda")
    ops.add_rmsnorm(r, dev(delta), dev(w), out, rows, eps)
    want_r = resid.double() + delta.double()
    assert torch.allclose(r.cpu().double(), want_r, rtol=1e-6, atol=1e-6)       # residual output
    ref = P.rmsnorm(r.cpu().double(), w.double(), eps)                           # norm of the stored sum
    tol = 2e-6 if dtype == torch.float32 else 2 ** -7
    assert torch.allclose(out.cpu().double(), ref, rtol=tol, atol=tol)
    # without delta: plain norm, residual untouched
    r2 = dev(resid.clone())
    ops.add_rmsnorm(r2, None, dev(w), out, rows, eps)
    assert torch.equal(r2.cpu(), resid)
    assert torch.allclose(out.cpu().double(), P.rmsnorm(resid.double(), w.double(), eps), rtol=tol, atol=tol)


def test_rmsnorm_rows_strided(ops):
    rows, D, stride = 6, 48, 100
    x = rnd(rows, stride, seed=7)
    w = 1 + 0.1 * rnd(D, seed=8)
    out = torch.zeros(rows, stride, device="cuda")
    ops.rmsnorm_rows(out, dev(x), dev(w), rows, D, stride, stride, 1e-5)
    ref = P.rmsnorm(x[:, :D].double(), w.double(), 1e-5)
    assert torch.allclose(out.cpu()[:, :D].double(), ref, rtol=2e-6, atol=2e-6)
    assert out.cpu()[:, D:].abs().max() == 0


# ------------------------------------------------------------------ matrix products
@pytest.mark.parametrize("M,N,K", [(1, 33, 100), (7, 130, 65), (64, 64, 16), (70, 301, 136)])
def test_gemm_plain_f32(ops, M, N, K):
    a, w, b = rnd(M, K, seed=9), rnd(N, K, seed=10), rnd(N, seed=11)
    out = torch.empty(M, N, device="cuda")
    ops.gemm_plain(out, dev(a), dev(w), dev(b), M)
    ref = a.double() @ w.double().T + b.double()
    assert torch.allclose(out.cpu().double(), ref, rtol=1e-5, atol=1e-5)
    # all-ones gives K (the reference's own matmul check, tests/test_kernels.cu:244-262)
    ones = torch.ones(M, K), torch.ones(N, K)
    ops.gemm_plain(out, dev(ones[0]), dev(ones[1]), None, M)
    assert torch.equal(out.cpu(), torch.full((M, N), float(K)))


def test_gemm_plain_rows_do_not_depend_on_the_batch(ops):
    a, w = rnd(70, 136, seed=12), rnd(301, 136, seed=13)
    full = torch.empty(70, 301, device="cuda")
    ops.gemm_plain(full, dev(a), dev(w), None, 70)
    one = torch.empty(1, 301, device="cuda")
    for r in (0, 37, 69):
        ops.gemm_plain(one, dev(a[r:r + 1].contiguous()), dev(w), None, 1)
        assert torch.equal(one.cpu()[0], full.cpu()[r])      # bit-equal


@pytest.mark.parametrize("N,K", [(33, 100), (301, 136), (64, 256), (130, 257), (70, 1000), (5, 3), (200, 515),
                                 (301, 384), (130, 128), (70, 1024), (7, 640)])   # K in whole segments: the kernel that turns the tile round
def test_gemm_plain_for_few_rows_gives_the_bits_of_the_tile_kernel(ops, N, K):
    """The plain product has one summation order (segments of 128 k, each a chain in ascending k, added
    in segment order): its kernels for up to 8 rows, which take a workspace, and its tile kernel
    give the same bits, with a bias or without, for widths that are no multiple of anything; a row of
    a product of 70 rows equals the same row alone; and a workspace that is too small is not used."""
    w, b = rnd(N, K, seed=13), rnd(N, seed=14)
    a = rnd(70, K, seed=12)
    full = torch.empty(70, N, device="cuda")
    ops.gemm_plain(full, dev(a), dev(w), dev(b), 70)
    ref = a.double() @ w.double().T + b.double()
    assert torch.allclose(full.cpu().double(), ref, rtol=1e-5, atol=1e-6 * K)      # sums of K products of size one
    # a step of 128 rows or more runs in tiles of 128 x 128: the same bits for the rows both hold
    more = torch.cat([a, rnd(133, K, seed=15)])
    wide = torch.empty(203, N, device="cuda")
    ops.gemm_plain(wide, dev(more), dev(w), dev(b), 203)
    assert torch.equal(wide[:70], full)
    assert torch.allclose(wide.cpu().double(), more.double() @ w.double().T + b.double(), rtol=1e-5, atol=1e-6 * K)
    for M in (1, 2, 3, 4, 5, 8):
        floats = ops.gemm_plain_workspace_floats(M, N, K)
        assert floats == -(-K // 128) * M * N
        rows = dev(a[7:7 + M].contiguous())
        tiled = torch.empty(M, N, device="cuda")
        ops.gemm_plain(tiled, rows, dev(w), dev(b), M)
        few = torch.full((M, N), 7.0, device="cuda")
        ops.gemm_plain(few, rows, dev(w), dev(b), M, workspace=torch.empty(floats + 5, device="cuda"))
        assert torch.equal(few, tiled) and torch.equal(few.cpu(), full.cpu()[7:7 + M])
        ops.gemm_plain(few, rows, dev(w), None, M, workspace=torch.empty(floats, device="cuda"))
        ops.gemm_plain(tiled, rows, dev(w), None, M, workspace=torch.empty(max(floats - 1, 1), device="cuda"))
        assert torch.equal(few, tiled)
    assert ops.gemm_plain_workspace_floats(9, N, K) == 0
    # bfloat16 operands through the same kernels (the plain path of a bfloat16 model)
    a16, w16 = a[:4].bfloat16().contiguous(), w.bfloat16()
    tiled = torch.empty(4, N, dtype=torch.bfloat16, device="cuda")
    few = torch.empty(4, N, dtype=torch.bfloat16, device="cuda")
    ops.gemm_plain(tiled, dev(a16), dev(w16), None, 4)
    ops.gemm_plain(few, dev(a16), dev(w16), None, 4, workspace=torch.empty(ops.gemm_plain_workspace_floats(4, N, K), device="cuda"))
    assert torch.equal(few, tiled)


def test_splitk_reduce_and_the_gated_activation_add_slices_in_order(ops):
    """K slices of a product are added in index order (+ bias) by splitk_reduce, and by the gated
    activation while it reads them."""
    rows, D, S = 5, 96, 3
    parts = rnd(S, rows, D, seed=76)
    bias = rnd(D, seed=77)
    summed = torch.empty(rows, D, device="cuda")
    ops.splitk_reduce(summed, dev(parts), dev(bias), rows, S)
    want = ((parts[0] + parts[1]) + parts[2]) + bias
    assert torch.equal(summed.cpu(), want)
    h = torch.empty(rows, D // 2, dtype=torch.bfloat16, device="cuda")
    ops.silu_mul(h, dev(parts), rows, True, S)
    x = parts.double().sum(0)
    ref = P.silu(x[:, 0::2]) * x[:, 1::2]
    assert torch.allclose(h.cpu().double(), ref, rtol=2 ** -7, atol=2 ** -7)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("M,I", [(1, 160), (33, 1008), (5, 37)])
def test_silu_mul_of_alternating_columns(ops, dtype, M, I):
    """The layout the fused gate||up weight gives: gate i in column 2i, its up in 2i + 1."""
    gu = rnd(M, 2 * I, seed=73, scale=2.0).to(dtype)
    out = torch.empty(M, I, dtype=dtype, device="cuda")
    ops.silu_mul(out, dev(gu), M, True)
    ref = P.silu(gu.double()[:, 0::2]) * gu.double()[:, 1::2]
    t = 1e-6 if dtype == torch.float32 else 2 ** -7
    assert torch.allclose(out.cpu().double(), ref, rtol=t, atol=1e-6)


def alternate_rows(g, u):
    """gate i at row 2i, its up at row 2i + 1"""
    return torch.stack([g, u], 1).reshape(2 * g.shape[0], g.shape[1]).contiguous()


@pytest.mark.parametrize("M", [1, 8, 16, 20, 32])
@pytest.mark.parametrize("N,K", [(301, 136), (1000, 1544), (37, 4104), (4608, 3584), (2051, 264)])
@pytest.mark.parametrize("plan", [(0, 0, 0), (1, 1, 1), (2, 2, 4), (1, 2, 16), (2, 1, 8)])
def test_gemm_blocksplit(ops, M, N, K, plan):
    """K cut inside the workgroup: every tiling gives the product, twice the same bits."""
    if (N, K) == (4608, 3584) and (M not in (1, 32) or plan[2] not in (0, 16)):
        pytest.skip("large shape at two row counts and two tilings only")
    if M > 16 and plan[1] == 4:
        pytest.skip("not instantiated")
    a = rnd(M, K, seed=90).to(torch.bfloat16)
    w = rnd(N, K, seed=91, scale=0.05).to(torch.bfloat16)
    b = rnd(N, seed=92).to(torch.bfloat16)
    ref = a.double() @ w.double().T + b.double()
    outs = []
    for _ in range(2):
        out = torch.empty(M, N, dtype=torch.float32, device="cuda")
        ops.gemm_blocksplit(out, dev(a), dev(w), dev(b), M, plan=plan)
        outs.append(out.cpu())
    assert torch.equal(outs[0], outs[1])
    assert (outs[0].double() - ref).abs().max().item() <= 1e-4 * ref.abs().max().item()
    out16 = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
    ops.gemm_blocksplit(out16, dev(a), dev(w), None, M, plan=plan)
    ref0 = a.double() @ w.double().T
    assert (out16.cpu().double() - ref0).abs().max().item() <= 2 ** -8 * ref0.abs().max().item() + 1e-6


@pytest.mark.parametrize("M", [1, 8, 20, 32])
@pytest.mark.parametrize("I,K", [(160, 64), (1008, 520), (37, 136), (1515, 264)])
@pytest.mark.parametrize("plan", [(0, 0, 0), (1, 0, 1), (2, 0, 8)])
def test_gemm_blocksplit_gated_epilogue(ops, M, I, K, plan):
    """Widths that are no multiple of a tile, one so wide (3030 rows) that the rows are dealt out
    evenly to the workgroups, 12 each."""
    x = rnd(M, K, seed=93).to(torch.bfloat16)
    g = rnd(I, K, seed=94, scale=0.1).to(torch.bfloat16)
    u = rnd(I, K, seed=95, scale=0.1).to(torch.bfloat16)
    w = alternate_rows(g, u)
    out = torch.empty(M, I, dtype=torch.bfloat16, device="cuda")
    ops.gemm_blocksplit(out, dev(x), dev(w), None, M, gated=True, plan=plan)
    ref = P.silu(x.double() @ g.double().T) * (x.double() @ u.double().T)
    assert (out.cpu().double() - ref).abs().max().item() <= 2 ** -8 * ref.abs().max().item() + 1e-6


@pytest.mark.parametrize("M", [1, 8, 16])
@pytest.mark.parametrize("D,K,N2,eps", [(80, 136, 301, 3e-6), (3584, 520, 160, 1e-6), (1000, 18944, 64, 1e-5),
                                        (2312, 264, 64, 1e-6)])
@pytest.mark.parametrize("gain_dtype", [torch.bfloat16, torch.float32])
def test_gemm_blocksplit_carries_the_norm(ops, M, D, K, N2, eps, gain_dtype):
    """A product adds its result to the residual rows and leaves r * gain and the sums of
    r^2; the next product (plain, gated) applies the owed scale: together they equal
    add + RMS norm + product of the plain implementation, without a norm kernel."""
    if K == 18944 and (M == 8 or gain_dtype == torch.float32):
        pytest.skip("long K at two row counts, one gain dtype")
    x = rnd(M, K, seed=100).to(torch.bfloat16)
    w1 = rnd(D, K, seed=101, scale=0.05).to(torch.bfloat16)
    b1 = rnd(D, seed=102).to(torch.bfloat16)
    r0 = rnd(M + 1, D, seed=103, scale=3.0)
    gain = (1 + 0.1 * rnd(D, seed=104)).to(gain_dtype)
    blocks = ops.gemm_blocksplit_blocks(M, D, K)
    assert blocks >= (D + 31) // 32
    resid = dev(r0.clone())
    xg = torch.zeros(M, D, dtype=torch.bfloat16, device="cuda")
    sq = torch.full((M, blocks), float("nan"), device="cuda")
    ops.gemm_blocksplit(None, dev(x), dev(w1), dev(b1), M, residual=(resid, dev(gain), xg, sq))
    r1 = r0[:M].double() + x.double() @ w1.double().T + b1.double()
    got_r = resid.cpu()
    assert torch.equal(got_r[M], r0[M])                                   # the row after the last is untouched
    assert (got_r[:M].double() - r1).abs().max().item() <= 1e-4 * r1.abs().max().item()
    want_xg = (got_r[:M] * gain.float()).to(torch.bfloat16)
    assert (xg.cpu().float() - want_xg.float()).abs().max().item() <= 2 ** -7 * want_xg.float().abs().max().item()
    assert torch.allclose(sq.cpu().double().sum(1), (got_r[:M].double() ** 2).sum(1), rtol=1e-5)
    # the consumer: scale applied to the sums, then bias
    normed = P.rmsnorm(got_r[:M].double(), gain.double(), eps)
    w2 = rnd(N2, D, seed=105, scale=0.05).to(torch.bfloat16)
    b2 = rnd(N2, seed=106).to(torch.bfloat16)
    out = torch.empty(M, N2, dtype=torch.float32, device="cuda")
    ops.gemm_blocksplit(out, xg, dev(w2), dev(b2), M, row_scale=(sq, eps))
    ref = normed @ w2.double().T + b2.double()
    assert (out.cpu().double() - ref).abs().max().item() <= 2 ** -7 * ref.abs().max().item()
    # gated consumer
    I = N2 // 2
    if I:
        g, u = w2[:I], rnd(I, D, seed=107, scale=0.05).to(torch.bfloat16)
        wi = alternate_rows(g, u)
        h = torch.empty(M, I, dtype=torch.bfloat16, device="cuda")
        ops.gemm_blocksplit(h, xg, dev(wi), None, M, gated=True, row_scale=(sq, eps))
        ref = P.silu(normed @ g.double().T) * (normed @ u.double().T)
        assert (h.cpu().double() - ref).abs().max().item() <= 2 ** -6 * ref.abs().max().item() + 1e-6
    # and as a tensor for anything that is not such a product
    t = torch.empty(M, D, dtype=torch.bfloat16, device="cuda")
    ops.scale_rows(t, xg, sq, eps, M)
    assert (t.cpu().double() - normed).abs().max().item() <= 2 ** -6 * normed.abs().max().item()
    # a chain: the consumer is itself a producer (row scale and residual epilogue together)
    resid2 = dev(r0.clone())
    w3 = rnd(D, D, seed=108, scale=0.05).to(torch.bfloat16)
    blocks3 = ops.gemm_blocksplit_blocks(M, D, D)
    xg2 = torch.zeros(M, D, dtype=torch.bfloat16, device="cuda")
    sq2 = torch.zeros(M, blocks3, device="cuda")
    ops.gemm_blocksplit(None, xg, dev(w3), None, M, row_scale=(sq, eps), residual=(resid2, dev(gain), xg2, sq2))
    r2 = r0[:M].double() + normed @ w3.double().T
    assert (resid2.cpu()[:M].double() - r2).abs().max().item() <= 2 ** -7 * r2.abs().max().item()
    assert torch.allclose(sq2.cpu().double().sum(1), (resid2.cpu()[:M].double() ** 2).sum(1), rtol=1e-5)


def to_pieces(x):
    """[M, D] -> piece-major [D / 8, M, 8]: 16-byte pieces, the M pieces of a column group together."""
    M, D = x.shape
    return x.reshape(M, D // 8, 8).permute(1, 0, 2).contiguous()


def from_pieces(p):
    return p.permute(1, 0, 2).reshape(p.shape[1], -1).contiguous()


@pytest.mark.parametrize("M", [1, 3, 8, 16])
@pytest.mark.parametrize("N,K", [(264, 136), (3584, 520), (1000, 18944), (2312, 264), (4608, 3584)])
def test_gemm_blocksplit_piece_major(ops, M, N, K):
    """Operand rows and bf16 results in the piece-major layout: the same sums in the same
    order as row-major, so equal bit for bit: plain, gated, with the residual epilogue and
    the owed row scale, and back to a tensor."""
    if K == 18944 and M in (3, 8):
        pytest.skip("long K at two row counts")
    x = dev(rnd(M, K, seed=110).to(torch.bfloat16))
    w = dev(rnd(N, K, seed=111, scale=0.05).to(torch.bfloat16))
    b = dev(rnd(N, seed=112).to(torch.bfloat16))
    xp = to_pieces(x)
    assert tuple(xp.shape) == ops.pieces_shape(M, K)
    want = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
    ops.gemm_blocksplit(want, x, w, b, M)
    ref = x.cpu().double() @ w.cpu().double().T + b.cpu().double()
    assert (want.cpu().double() - ref).abs().max().item() <= 2 ** -7 * ref.abs().max().item()
    for xin, op in ((True, False), (False, True), (True, True)):
        out = torch.full(ops.pieces_shape(M, N) if op else (M, N), 7.0, dtype=torch.bfloat16, device="cuda")
        ops.gemm_blocksplit(out, xp if xin else x, w, b, M, x_pieces=xin, out_pieces=op)
        assert torch.equal(from_pieces(out) if op else out, want), (xin, op)
    out32, want32 = (torch.empty(M, N, device="cuda") for _ in range(2))          # fp32 results stay row-major
    ops.gemm_blocksplit(want32, x, w, b, M)
    ops.gemm_blocksplit(out32, xp, w, b, M, x_pieces=True)
    assert torch.equal(out32, want32)
    # gated: [M, N / 2]
    if (N // 2) % 8 == 0:
        wh, oh = torch.empty(M, N // 2, dtype=torch.bfloat16, device="cuda"), \
            torch.empty(ops.pieces_shape(M, N // 2), dtype=torch.bfloat16, device="cuda")
        ops.gemm_blocksplit(wh, x, w, None, M, gated=True)
        ops.gemm_blocksplit(oh, xp, w, None, M, gated=True, x_pieces=True, out_pieces=True)
        assert torch.equal(from_pieces(oh), wh)
    # residual epilogue leaving piece-major rows, read by a product with the owed scale
    r0 = dev(rnd(M, N, seed=113, scale=3.0))
    gain = dev((1 + 0.1 * rnd(N, seed=114)).to(torch.bfloat16))
    blocks = ops.gemm_blocksplit_blocks(M, N, K)
    res_a, res_b = r0.clone(), r0.clone()
    xg_a = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
    xg_b = torch.empty(ops.pieces_shape(M, N), dtype=torch.bfloat16, device="cuda")
    sq_a, sq_b = (torch.empty(M, blocks, device="cuda") for _ in range(2))
    ops.gemm_blocksplit(None, x, w, b, M, residual=(res_a, gain, xg_a, sq_a))
    ops.gemm_blocksplit(None, xp, w, b, M, residual=(res_b, gain, xg_b, sq_b), x_pieces=True, out_pieces=True)
    assert torch.equal(res_a, res_b) and torch.equal(sq_a, sq_b) and torch.equal(from_pieces(xg_b), xg_a)
    w2 = dev(rnd(72, N, seed=115, scale=0.05).to(torch.bfloat16))
    y_a, y_b = (torch.empty(M, 72, dtype=torch.bfloat16, device="cuda") for _ in range(2))
    ops.gemm_blocksplit(y_a, xg_a, w2, None, M, row_scale=(sq_a, 1e-6))
    ops.gemm_blocksplit(y_b, xg_b, w2, None, M, row_scale=(sq_b, 1e-6), x_pieces=True)
    assert torch.equal(y_a, y_b)
    t_a, t_b = (torch.empty(M, N, dtype=torch.bfloat16, device="cuda") for _ in range(2))
    ops.scale_rows(t_a, xg_a, sq_a, 1e-6, M)
    ops.scale_rows(t_b, xg_b, sq_b, 1e-6, M, x_pieces=True)
    assert torch.equal(t_a, t_b)


def test_piece_major_rows_are_refused_beyond_their_sizes(ops):
    from hector_engine_amd.kernels.lib import KernelLibraryError
    with pytest.raises(ValueError, match="piece-major"):
        ops.pieces_shape(65, 64)
    with pytest.raises(ValueError, match="piece-major"):
        ops.pieces_shape(4, 60)
    with pytest.raises(ValueError, match="up to 16 rows"):      # the block-split product's own limit
        ops.gemm_blocksplit(torch.empty(ops.pieces_shape(17, 64), dtype=torch.bfloat16, device="cuda"),
                            torch.zeros(17, 64, dtype=torch.bfloat16, device="cuda"),
                            torch.zeros(64, 64, dtype=torch.bfloat16, device="cuda"), None, 17, out_pieces=True)
    M, N, K = 4, 64, 64
    x = torch.zeros(ops.pieces_shape(M, K), dtype=torch.bfloat16, device="cuda")
    w = torch.zeros(N, K, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ValueError, match="shape"):       # row-major operand where pieces are announced
        ops.gemm_blocksplit(torch.empty(M, N, dtype=torch.bfloat16, device="cuda"),
                            torch.zeros(M, K, dtype=torch.bfloat16, device="cuda"), w, None, M, x_pieces=True)
    with pytest.raises(TypeError):                         # fp32 results are not written piece-major
        ops.gemm_blocksplit(torch.empty(ops.pieces_shape(M, N), device="cuda"), x, w, None, M,
                            x_pieces=True, out_pieces=True)
    w20 = torch.zeros(20, K, dtype=torch.bfloat16, device="cuda")  # gated width 10: no whole pieces
    with pytest.raises((ValueError, KernelLibraryError)):
        ops.gemm_blocksplit(torch.empty(M, 10, dtype=torch.bfloat16, device="cuda"), x, w20, None, M,
                            gated=True, x_pieces=True, out_pieces=True)


def test_gemm_blocksplit_residual_epilogue_checks_its_buffers(ops):
    from hector_engine_amd.kernels.lib import KernelLibraryError
    M, D, K = 4, 64, 64
    x = torch.zeros(M, K, dtype=torch.bfloat16, device="cuda")
    w = torch.zeros(D, K, dtype=torch.bfloat16, device="cuda")
    resid = torch.zeros(M, D, device="cuda")
    gain = torch.ones(D, device="cuda")
    xg = torch.zeros(M, D, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(KernelLibraryError, match="partial sums per row"):
        ops.gemm_blocksplit(None, x, w, None, M, residual=(resid, gain, xg, torch.zeros(M, 1, device="cuda")))
    with pytest.raises(ValueError):
        ops.gemm_blocksplit(None, x, w, None, M, gated=True, residual=(resid, gain, xg, torch.zeros(M, 4, device="cuda")))


# ------------------------------------------------------------------ rope + cache + attention
def paged_setup(lengths, KVH, hd, dtype, seed, extra_pages=3):
    """Scattered pages: a random permutation of page ids, slots in reverse order."""
    g = torch.Generator().manual_seed(seed)
    B = len(lengths)
    blocks = [(n + PAGE - 1) // PAGE for n in lengths]
    num_pages = sum(blocks) + extra_pages
    perm = torch.randperm(num_pages, generator=g).tolist()
    max_blocks = max(blocks) + 1
    slots = list(range(B))[::-1]
    table = torch.full((B + 1, max_blocks), -1, dtype=torch.int32)
    it = iter(perm)
    for s, nb in zip(slots, blocks):
        for b in range(nb):
            table[s, b] = next(it)
    kpool = torch.zeros(num_pages, KVH, 64 * 32 * ((hd + 31) // 32), dtype=dtype)
    vpool = torch.zeros(num_pages, KVH, 64 * 16 * ((hd + 15) // 16), dtype=dtype)
    return slots, table, kpool, vpool


_maps = {}


def page_maps(hd):
    """Where element (token, dim) of a page lies, written out from the layout's description
    (operand order): K [half][key tile][k step][lane][8], V [half][dim tile][lane][8] with
    lane = 16 lg + lr; K: key = 32 h + 8 (lr // 4) + 4 t + lr % 4, dim = 32 ks + 8 lg + e;
    V: dim = 16 dt + lr, key = 32 h + 8 lg + e. Returns index tensors [64, hd]."""
    if hd not in _maps:
        KS, NT = (hd + 31) // 32, (hd + 15) // 16
        km = torch.full((PAGE, hd), -1, dtype=torch.long)
        vm = torch.full((PAGE, hd), -1, dtype=torch.long)
        for h in range(2):
            for lane in range(64):
                lr, lg = lane % 16, lane // 16
                for e in range(8):
                    for t in range(2):
                        for ks in range(KS):
                            key, dim = 32 * h + 8 * (lr // 4) + 4 * t + lr % 4, 32 * ks + 8 * lg + e
                            if dim < hd:
                                km[key, dim] = ((((h * 2 + t) * KS + ks) * 64) + lane) * 8 + e
                    for dt in range(NT):
                        key, dim = 32 * h + 8 * lg + e, 16 * dt + lr
                        if dim < hd:
                            vm[key, dim] = ((h * NT + dt) * 64 + lane) * 8 + e
        assert (km >= 0).all() and (vm >= 0).all() and km.unique().numel() == PAGE * hd
        _maps[hd] = (km, vm)
    return _maps[hd]


def cached_k(kpool, page, token, hd):
    """[KVH, hd] of one token of a page."""
    return kpool[page][:, page_maps(hd)[0][token]]


def cached_v(vpool, page, token, hd):
    return vpool[page][:, page_maps(hd)[1][token]]


def fill_cache(table, slots, kpool, vpool, ks, vs):
    for s, k, v in zip(slots, ks, vs):
        for b in range((k.shape[0] + PAGE - 1) // PAGE):
            page = table[s, b].item()
            kb, vb = k[b * PAGE:(b + 1) * PAGE], v[b * PAGE:(b + 1) * PAGE]
            km, vm = page_maps(kb.shape[-1])
            n = kb.shape[0]
            kpool[page][:, km[:n].reshape(-1)] = kb.transpose(0, 1).reshape(kb.shape[1], -1)
            vpool[page][:, vm[:n].reshape(-1)] = vb.transpose(0, 1).reshape(vb.shape[1], -1)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,KVH,hd,rot", [(6, 3, 48, 48), (4, 1, 64, 32), (5, 5, 16, 0)])
def test_qkv_rope_cache(ops, dtype, H, KVH, hd, rot):
    lengths = [70, 5, 130]           # new tokens start at these offsets
    new = [3, 64, 1]
    theta = 50000.0
    slots, table, kpool, vpool = paged_setup([a + b for a, b in zip(lengths, new)], KVH, hd, dtype, 20)
    rows = sum(new)
    width = (H + 2 * KVH) * hd
    qkv = rnd(rows, width, seed=21).to(dtype)
    bias = rnd(width, seed=22).to(dtype)
    positions = torch.cat([torch.arange(a, a + b) for a, b in zip(lengths, new)]).int()
    row_seq = torch.cat([torch.full((b,), i) for i, b in enumerate(new)]).int()
    # a padding row at the end must be left alone
    qkv = torch.cat([qkv, torch.zeros(1, width, dtype=dtype)])
    positions = torch.cat([positions, torch.zeros(1, dtype=torch.int32)])
    row_seq = torch.cat([row_seq, torch.full((1,), -1, dtype=torch.int32)])
    seq_slot = torch.tensor(slots, dtype=torch.int32)
    inv = P.rope_inv_freq(rot, theta) if rot else None
    q_out = torch.zeros(rows + 1, H * hd, dtype=dtype, device="cuda")
    kp, vp = dev(kpool), dev(vpool)
    ops.qkv_rope_cache(q_out, kp, vp, dev(qkv), H * hd, KVH * hd, dev(bias), dev(positions),
                       dev(row_seq), dev(seq_slot), dev(table), dev(inv) if rot else None, rot,
                       rows + 1, H, KVH, hd, True)
    x = (qkv[:rows].double() + bias.double())
    q = x[:, :H * hd].reshape(rows, H, hd)
    k = x[:, H * hd:(H + KVH) * hd].reshape(rows, KVH, hd)
    v = x[:, (H + KVH) * hd:].reshape(rows, KVH, hd)
    pos = positions[:rows]
    if rot:
        q, k = P.rope(q, pos, theta, rot), P.rope(k, pos, theta, rot)
    tol = 3e-6 if dtype == torch.float32 else 2 ** -7
    assert torch.allclose(q_out.cpu()[:rows].double().reshape(rows, H, hd), q, rtol=tol, atol=tol * 4)
    kp, vp = kp.cpu(), vp.cpu()
    for r in range(rows):
        s = slots[row_seq[r]]
        page = table[s, pos[r] // PAGE].item()
        assert torch.allclose(cached_k(kp, page, pos[r] % PAGE, hd).double(), k[r], rtol=tol, atol=tol * 4)
        assert torch.allclose(cached_v(vp, page, pos[r] % PAGE, hd).double(), v[r], rtol=tol, atol=tol * 4)
    # nothing else in the pools was touched
    assert (kp != 0).sum().item() <= rows * KVH * hd


def attention_case(ops, kind, dtype, H, KVH, hd, window, lengths, q_lens, seed, pad=0, tiles=0, plant=None, parts=1):
    """Runs one attention kernel over a crafted cache; returns (got, want) lists per sequence.
    plant(ks, vs) may change keys and values before they go into the cache."""
    B = len(lengths)
    slots, table, kpool, vpool = paged_setup(lengths, KVH, hd, dtype, seed)
    ks = [rnd(n, KVH, hd, seed=seed + 10 + i).to(dtype) for i, n in enumerate(lengths)]
    vs = [rnd(n, KVH, hd, seed=seed + 20 + i).to(dtype) for i, n in enumerate(lengths)]
    if plant is not None:
        plant(ks, vs)
    fill_cache(table, slots, kpool, vpool, ks, vs)
    qs = [rnd(m, H, hd, seed=seed + 30 + i, scale=2.0).to(dtype) for i, m in enumerate(q_lens)]
    rows = sum(q_lens)
    q = torch.cat(qs + [torch.zeros(pad, H, hd, dtype=dtype)]).reshape(rows + pad, H * hd)
    positions = torch.cat([torch.arange(n - m, n) for n, m in zip(lengths, q_lens)] +
                          [torch.zeros(pad, dtype=torch.int64)]).int()
    row_seq = torch.cat([torch.full((m,), i) for i, m in enumerate(q_lens)] +
                        [torch.full((pad,), -1)]).int()
    cu = torch.tensor([0] + list(np.cumsum(q_lens)), dtype=torch.int32)
    seq_start = torch.tensor([n - m for n, m in zip(lengths, q_lens)], dtype=torch.int32)
    seq_slot = torch.tensor(slots, dtype=torch.int32)
    out = torch.full((rows + pad, H * hd), 7.0, dtype=dtype, device="cuda")
    scale = 1.0 / math.sqrt(hd)
    args = (dev(kpool), dev(vpool))
    if kind == "plain":
        ops.attention_plain(out, dev(q), *args, dev(positions), dev(row_seq), dev(seq_slot),
                            dev(table), rows + pad, H, KVH, hd, window, scale)
        # page by page in parallel (a bound on the keys and a workspace): the same bits
        most = max(lengths) + 3
        floats = ops.attention_plain_workspace_floats(rows + pad, H, hd, most, window)
        if floats:
            again = torch.full((rows + pad, H * hd), 7.0, dtype=dtype, device="cuda")
            ops.attention_plain(again, dev(q), *args, dev(positions), dev(row_seq), dev(seq_slot), dev(table),
                                rows + pad, H, KVH, hd, window, scale, most, torch.empty(floats, device="cuda"))
            assert torch.equal(again, out)
    elif kind == "decode":
        max_keys = 4096
        ws = torch.empty(ops.attention_decode_workspace_floats(rows + pad, H, KVH, hd, max_keys), device="cuda")
        ops.attention_decode(out, dev(q), *args, dev(positions), dev(row_seq), dev(seq_slot),
                             dev(table), rows + pad, H, KVH, hd, window, scale, max_keys, ws)
    else:
        ws = torch.empty(ops.attention_prefill_workspace_floats(rows, H, hd, parts), device="cuda") if parts > 1 else None
        ops.attention_prefill(out, dev(q), *args, dev(cu), dev(seq_slot), dev(seq_start), dev(table),
                              B, max(q_lens), rows, H, KVH, hd, window, scale, kernel=tiles, parts=parts, workspace=ws)
    got, want = [], []
    r = 0
    for i, (n, m) in enumerate(zip(lengths, q_lens)):
        got.append(out.cpu()[r:r + m].double())
        want.append(P.attention(qs[i].double(), ks[i].double(), vs[i].double(),
                                torch.arange(n - m, n), torch.arange(n), window))
        r += m
    if pad and kind != "prefill":
        assert out.cpu()[rows:].abs().max() == 0     # padding rows give zeros
    return got, want


ATT_SHAPES = [(6, 3, 48), (4, 1, 64), (28, 4, 128), (5, 5, 16), (2, 1, 80), (4, 2, 192), (2, 1, 256)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,KVH,hd", ATT_SHAPES)
@pytest.mark.parametrize("window", [0, 70])
def test_attention_plain(ops, dtype, H, KVH, hd, window):
    got, want = attention_case(ops, "plain", dtype, H, KVH, hd, window, [200, 3, 65], [5, 3, 1], 40, pad=2)
    tol = 3e-6 if dtype == torch.float32 else 2 ** -6
    for g, w in zip(got, want):
        assert torch.allclose(g, w, rtol=tol, atol=tol)
    assert ops.attention_plain_workspace_floats(11, H, hd, 203, window) == \
        11 * H * (hd + 2) * (min(4, 3) if window else 4)       # 203 keys lie in 4 pages, a window of 70 in 3 at most
    assert ops.attention_plain_workspace_floats(100000, H, hd, 203, window) == 0      # many queries: one wavefront each
    # a bound on the keys that is too low must not pass for a result
    if dtype == torch.float32 and not window:
        slots, table, kpool, vpool = paged_setup([200], KVH, hd, dtype, 3)
        q = rnd(1, H * hd, seed=5)
        out = torch.zeros(1, H * hd, device="cuda")
        ops.attention_plain(out, dev(q), dev(kpool), dev(vpool), dev(torch.tensor([199], dtype=torch.int32)),
                            dev(torch.zeros(1, dtype=torch.int32)), dev(torch.tensor(slots, dtype=torch.int32)), dev(table),
                            1, H, KVH, hd, 0, 0.1, 128, torch.empty(ops.attention_plain_workspace_floats(1, H, hd, 128, 0),
                                                                   device="cuda"))
        assert torch.isnan(out).all()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,KVH,hd", [(6, 3, 48), (28, 4, 128), (2, 1, 256), (3, 1, 320)])
@pytest.mark.parametrize("window", [0, 70])
def test_attention_plain_of_many_queries_gives_the_bits_of_one_at_a_time(ops, dtype, H, KVH, hd, window):
    """A step of 64 rows or more takes four neighbouring queries of a sequence in one wavefront (they
    share the keys they fetch); a step of fewer rows takes them one by one: the same rows, cut into
    steps of at most 40, give the same bits. Sequences that end inside a group of four, a
    continuation (70 new tokens behind 130) and a single token are among them."""
    lengths, q_lens = [150, 200, 67, 1, 90], [150, 70, 67, 1, 3]
    slots, table, kpool, vpool = paged_setup(lengths, KVH, hd, dtype, 50)
    ks = [rnd(n, KVH, hd, seed=60 + i).to(dtype) for i, n in enumerate(lengths)]
    vs = [rnd(n, KVH, hd, seed=70 + i).to(dtype) for i, n in enumerate(lengths)]
    fill_cache(table, slots, kpool, vpool, ks, vs)
    qs = [rnd(m, H, hd, seed=80 + i, scale=2.0).to(dtype) for i, m in enumerate(q_lens)]
    rows = sum(q_lens)
    q = torch.cat(qs).reshape(rows, H * hd)
    positions = torch.cat([torch.arange(n - m, n) for n, m in zip(lengths, q_lens)]).int()
    row_seq = torch.cat([torch.full((m,), i) for i, m in enumerate(q_lens)]).int()
    seq_slot = torch.tensor(slots, dtype=torch.int32)
    scale = 1.0 / math.sqrt(hd)
    whole = torch.full((rows, H * hd), 7.0, dtype=dtype, device="cuda")
    ops.attention_plain(whole, dev(q), dev(kpool), dev(vpool), dev(positions), dev(row_seq), dev(seq_slot),
                        dev(table), rows, H, KVH, hd, window, scale)
    r = 0
    for i, (n, m) in enumerate(zip(lengths, q_lens)):
        want = P.attention(qs[i].double(), ks[i].double(), vs[i].double(), torch.arange(n - m, n), torch.arange(n), window)
        tol = 3e-6 if dtype == torch.float32 else 2 ** -6
        assert torch.allclose(whole.cpu()[r:r + m].double().reshape(want.shape), want, rtol=tol, atol=tol)
        r += m
    for lo in range(0, rows, 37):
        hi = min(rows, lo + 37)
        part = torch.full((hi - lo, H * hd), 7.0, dtype=dtype, device="cuda")
        ops.attention_plain(part, dev(q[lo:hi].contiguous()), dev(kpool), dev(vpool), dev(positions[lo:hi].contiguous()),
                            dev(row_seq[lo:hi].contiguous()), dev(seq_slot), dev(table), hi - lo, H, KVH, hd, window, scale)
        assert torch.equal(part, whole[lo:hi])


@pytest.mark.parametrize("H,KVH,hd", ATT_SHAPES + [(40, 2, 32)])
@pytest.mark.parametrize("window", [0, 70])
def test_attention_decode(ops, H, KVH, hd, window):
    got, want = attention_case(ops, "decode", torch.bfloat16, H, KVH, hd, window,
                               [700, 1, 64, 65, 300], [1, 1, 1, 1, 1], 41, pad=3)
    for g, w in zip(got, want):
        assert torch.allclose(g, w, rtol=2 ** -6, atol=2 ** -6)


@pytest.mark.parametrize("H,KVH,hd", ATT_SHAPES)
@pytest.mark.parametrize("window", [0, 70])
@pytest.mark.parametrize("tiles", [0, 1, 2])
def test_attention_prefill(ops, H, KVH, hd, window, tiles):
    """Each of the prompt kernels (1: 16 queries a wavefront without LDS, 2: 32 queries a wavefront
    with the pages shared through LDS; 0 = the library's choice): whole prompts, a continuation
    (200 cached + 37 new) and a single token."""
    if tiles >= 2 and hd > 128:
        from hector_engine_amd.kernels.lib import KernelLibraryError
        with pytest.raises(KernelLibraryError, match="head_dim"):
            attention_case(ops, "prefill", torch.bfloat16, H, KVH, hd, window, [150], [150], 42, tiles=tiles)
        return
    got, want = attention_case(ops, "prefill", torch.bfloat16, H, KVH, hd, window,
                               [150, 237, 3, 66], [150, 37, 3, 1], 42, tiles=tiles)
    for g, w in zip(got, want):
        assert torch.allclose(g, w, rtol=2 ** -6, atol=2 ** -6)


@pytest.mark.parametrize("H,KVH,hd", [(4, 1, 64), (7, 1, 128), (3, 3, 48)])
@pytest.mark.parametrize("window", [0, 70, 300])
@pytest.mark.parametrize("tiles", [1, 2])
def test_attention_prefill_of_many_tiles(ops, H, KVH, hd, window, tiles):
    """Prompts of several workgroups' worth of query tiles: an even and an odd number of tiles, a
    last tile that is not full, a continuation whose first position is no multiple of 32 (its tiles'
    diagonals then fall into different steps of 32 keys), and short prompts."""
    got, want = attention_case(ops, "prefill", torch.bfloat16, H, KVH, hd, window,
                               [1024, 713, 530, 48, 272], [1024, 713, 330, 48, 17], 43, tiles=tiles)
    for g, w in zip(got, want):
        assert torch.allclose(g, w, rtol=2 ** -6, atol=2 ** -6)


@pytest.mark.parametrize("H,KVH,hd,window", [(7, 1, 128, 0), (4, 2, 64, 0), (3, 1, 80, 0), (4, 1, 128, 200)])
def test_attention_prefill_shared_pages_edges(ops, H, KVH, hd, window):
    """The kernel that shares pages through LDS, where its loops change over. Continuations whose
    first new position is 31 or 63 past a multiple of 64 (the first query of a tile is then the last
    key of a step, and of a page), a last tile of one query, one new token behind 700 cached ones, a
    prompt of exactly one page, and 129 queries (a second workgroup for one query)."""
    lengths = [64 * 5 + 31 + 97, 64 * 3 + 63 + 160, 64 * 4 + 33, 701, 64, 129]
    q_lens = [97, 160, 33, 1, 64, 129]
    got, want = attention_case(ops, "prefill", torch.bfloat16, H, KVH, hd, window, lengths, q_lens, 47, tiles=2)
    for g, w in zip(got, want):
        assert torch.allclose(g, w, rtol=2 ** -6, atol=2 ** -6)


@pytest.mark.parametrize("H,KVH,hd,window", [(7, 1, 128, 0), (4, 2, 64, 0), (3, 1, 80, 70), (4, 1, 128, 300), (2, 1, 16, 0)])
@pytest.mark.parametrize("parts", [2, 3, 5, 16])
def test_attention_prefill_keys_in_parts(ops, H, KVH, hd, window, parts):
    """The keys of a block of queries cut into parts that run side by side and are joined: short
    continuations of long sequences (what the parts are for), whole prompts whose first blocks have
    fewer pages than there are parts (parts without pages), a window (parts before its start hold
    nothing), one new token, a block of one query, starts that are no multiple of 32."""
    lengths = [1500 + 40, 64 * 9 + 31 + 97, 700, 701, 129, 64 * 4 + 33]
    q_lens = [40, 97, 700, 1, 129, 33]
    got, want = attention_case(ops, "prefill", torch.bfloat16, H, KVH, hd, window, lengths, q_lens, 51, tiles=2,
                               parts=parts)
    for g, w in zip(got, want):
        assert torch.allclose(g, w, rtol=2 ** -6, atol=2 ** -6)


def test_attention_prefill_keys_in_parts_reference_points(ops):
    """Parts whose reference points lie far apart: one key in the first part and one in the last
    are made large, so the join weighs parts by 2^(hundreds) against each other."""
    def plant(ks, vs):
        ks[0][100] *= 60
        ks[0][1900] *= 200
    got, want = attention_case(ops, "prefill", torch.bfloat16, 7, 1, 128, 0, [2000], [90], 52, tiles=2,
                               plant=plant, parts=4)
    assert torch.allclose(got[0], want[0], rtol=2 ** -6, atol=2 ** -6)


def test_attention_prefill_parts_rule_and_errors(ops):
    """The library's own choice: none for a whole prompt that fills the chip or for a short context, several
    for a short continuation of a long sequence; parts are refused for the kernel that cannot run them and
    without room for them."""
    from hector_engine_amd.kernels.lib import KernelLibraryError
    assert ops.attention_prefill_parts(1, 2048, 28, 128, 2048) == 1
    assert ops.attention_prefill_parts(1, 300, 28, 128, 300) == 1
    assert ops.attention_prefill_parts(1, 1024, 28, 128, 2048) == 1     # fewer than four keys a query
    assert ops.attention_prefill_parts(1, 200, 28, 128, 8200) == 9
    assert ops.attention_prefill_parts(1, 64, 28, 128, 8064) == 16
    assert ops.attention_prefill_parts(1, 8, 28, 128, 508) == 2
    assert ops.attention_prefill_parts(1, 16, 28, 128, 2016) == 8
    assert ops.attention_prefill_parts(4, 8, 28, 128, 3008) == 4
    assert ops.attention_prefill_parts(1, 200, 28, 256, 8200) == 1      # head size of the other kernel
    with pytest.raises(KernelLibraryError, match="kernel 2"):
        attention_case(ops, "prefill", torch.bfloat16, 4, 1, 64, 0, [300], [100], 53, tiles=1, parts=2)
    q = torch.zeros(100, 4 * 64, dtype=torch.bfloat16, device="cuda")
    pool = torch.zeros(8, 1, 64 * 64, dtype=torch.bfloat16, device="cuda")
    i32 = lambda *v: torch.tensor(v, dtype=torch.int32, device="cuda")
    with pytest.raises(KernelLibraryError, match="workspace"):
        ops.attention_prefill(torch.empty_like(q), q, pool, pool, i32(0, 100), i32(0), i32(200),
                              torch.arange(8, dtype=torch.int32, device="cuda").reshape(1, 8), 1, 100, 100, 4, 1, 64,
                              0, 0.125, kernel=2, parts=2, workspace=torch.empty(10, device="cuda"))


@pytest.mark.parametrize("tiles", [1, 2])
def test_attention_prefill_reference_point_moves(ops, tiles):
    """Random scores never make the softmax's reference point move after the first step, so the
    branch that rescales the accumulators would go untested: two keys far before the diagonal are
    made large (scores of several hundred for about half of the queries, first at key 300, larger
    still at key 700), and one inside the last page."""
    def plant(ks, vs):
        ks[0][300] *= 40
        ks[0][700] *= 160
        ks[0][1000] *= 300
    got, want = attention_case(ops, "prefill", torch.bfloat16, 7, 1, 128, 0, [1024], [1024], 48, tiles=tiles,
                               plant=plant)
    assert torch.allclose(got[0], want[0], rtol=2 ** -6, atol=2 ** -6)


@pytest.mark.parametrize("H,KVH,hd", [(4, 1, 64), (28, 4, 128), (6, 3, 64), (40, 2, 128)])
@pytest.mark.parametrize("window", [0, 70])
@pytest.mark.parametrize("write_kv", [True, False])
@pytest.mark.parametrize("copies", [1, 24])
def test_attention_decode_fused(ops, H, KVH, hd, window, write_kv, copies):
    """Bias, rotation, cache write, attention and merge in one launch against the plain parts.
    Lengths sit at page and slice edges; a padding row stands between the sequences. With few
    sequences the keys are cut across workgroups and joined by a second launch; with many
    (copies > 1) one workgroup serves a sequence and kv head."""
    theta = 50000.0
    lengths = [700, 1, 64, 65, 300, 129] * copies
    if copies > 1:
        lengths = [min(n, 200) for n in lengths]
    B = len(lengths)
    assert ops.attention_decode_fused_ok(H, KVH, hd, hd)
    floats = ops.attention_decode_fused_workspace_floats(B + 1, H, KVH, hd, 4096)
    assert (floats == 0) == ((B + 1) * KVH * ((H // KVH + 15) // 16) >= 256)
    ws = torch.empty(floats, device="cuda") if floats else None
    slots, table, kpool, vpool = paged_setup(lengths, KVH, hd, torch.bfloat16, 60)
    old = [n if not write_kv else n - 1 for n in lengths]
    ks = [rnd(n, KVH, hd, seed=61 + i).to(torch.bfloat16) for i, n in enumerate(old)]
    vs = [rnd(n, KVH, hd, seed=71 + i).to(torch.bfloat16) for i, n in enumerate(old)]
    fill_cache(table, slots, kpool, vpool, ks, vs)
    width = (H + 2 * KVH) * hd if write_kv else H * hd
    qkv = rnd(B, width, seed=81, scale=1.5).to(torch.bfloat16)
    bias = rnd(width, seed=82).to(torch.bfloat16)
    pad_at = 2
    order = list(range(pad_at)) + [-1] + list(range(pad_at, B))          # row -> sequence
    rows = len(order)
    qkv_rows = torch.stack([qkv[s] if s >= 0 else torch.zeros(width, dtype=torch.bfloat16) for s in order])
    positions = torch.tensor([lengths[s] - 1 if s >= 0 else 0 for s in order], dtype=torch.int32)
    row_seq = torch.tensor(order, dtype=torch.int32)
    seq_slot = torch.tensor(slots, dtype=torch.int32)
    inv = P.rope_inv_freq(hd, theta)
    out = torch.full((rows, H * hd), 7.0, dtype=torch.bfloat16, device="cuda")
    kp, vp = dev(kpool), dev(vpool)
    ops.attention_decode_fused(out, dev(qkv_rows), dev(bias), kp, vp, dev(positions), dev(row_seq),
                               dev(seq_slot), dev(table), dev(inv), hd, rows, H, KVH, hd, window,
                               1.0 / math.sqrt(hd), 4096, write_kv, ws)
    got = out.cpu().double()
    kp, vp = kp.cpu(), vp.cpu()
    assert got[pad_at].abs().max() == 0
    x = qkv.double() + bias.double()
    for r, s in enumerate(order):
        if s < 0:
            continue
        n = lengths[s]
        pos = torch.tensor([n - 1])
        q = P.rope(x[s, :H * hd].reshape(1, H, hd), pos, theta, hd).to(torch.bfloat16).double()
        k_all, v_all = ks[s].double(), vs[s].double()
        if write_kv:
            k_new = P.rope(x[s, H * hd:(H + KVH) * hd].reshape(1, KVH, hd), pos, theta, hd)
            v_new = x[s, (H + KVH) * hd:].reshape(1, KVH, hd)
            k_new, v_new = k_new.to(torch.bfloat16), v_new.to(torch.bfloat16)
            page = table[slots[s], (n - 1) // PAGE].item()
            assert torch.allclose(cached_k(kp, page, (n - 1) % PAGE, hd).double(), k_new[0].double(),
                                  rtol=2 ** -7, atol=2 ** -7), s
            assert torch.allclose(cached_v(vp, page, (n - 1) % PAGE, hd).double(), v_new[0].double(),
                                  rtol=2 ** -7, atol=2 ** -7), s
            k_all, v_all = torch.cat([k_all, k_new.double()]), torch.cat([v_all, v_new.double()])
        want = P.attention(q, k_all, v_all, pos, torch.arange(n), window).reshape(-1)
        assert torch.allclose(got[r], want, rtol=2 ** -6, atol=2 ** -6), (s, (got[r] - want).abs().max())
    if write_kv:   # nothing but the new rows was written
        before = dev(kpool).cpu()
        assert (kp != before).sum().item() <= B * KVH * hd
    if rows <= ops.PIECES_MAX_M:   # the same result piece-major, as the output product reads it
        out2 = torch.full(ops.pieces_shape(rows, H * hd), 7.0, dtype=torch.bfloat16, device="cuda")
        ops.attention_decode_fused(out2, dev(qkv_rows), dev(bias), dev(kp), dev(vp), dev(positions),
                                   dev(row_seq), dev(seq_slot), dev(table), dev(inv), hd, rows, H, KVH,
                                   hd, window, 1.0 / math.sqrt(hd), 4096, write_kv, ws, out_pieces=True)
        assert torch.equal(from_pieces(out2).cpu(), out.cpu())
    # the page numbers handed over row by row (a padding row's are -1) instead of through the slots
    by_row = torch.stack([table[slots[s]] if s >= 0 else torch.full_like(table[0], -1) for s in order])
    out3 = torch.full((rows, H * hd), 7.0, dtype=torch.bfloat16, device="cuda")
    ops.attention_decode_fused(out3, dev(qkv_rows), dev(bias), dev(kp), dev(vp), dev(positions), dev(row_seq),
                               None, dev(by_row), dev(inv), hd, rows, H, KVH, hd, window,
                               1.0 / math.sqrt(hd), 4096, write_kv, ws)
    assert torch.equal(out3.cpu(), out.cpu())
    # the projection rows as the fp32 sums of K slices (what the rows kernel leaves at 17 to 64 rows):
    # the kernel adds them in slice order and rounds as the kernel that sums them would have
    S = 7 if copies == 1 else 3
    parts = rnd(S, rows, width, seed=83, scale=0.6).cuda()
    summed = torch.empty(rows, width, dtype=torch.bfloat16, device="cuda")
    ops.splitk_reduce(summed, parts, None, rows, S)
    outs, pools = [], []
    for given in (summed, parts):
        o = torch.full((rows, H * hd), 7.0, dtype=torch.bfloat16, device="cuda")
        kq, vq = dev(kpool), dev(vpool)
        ops.attention_decode_fused(o, given, dev(bias), kq, vq, dev(positions), dev(row_seq), dev(seq_slot),
                                   dev(table), dev(inv), hd, rows, H, KVH, hd, window, 1.0 / math.sqrt(hd), 4096,
                                   write_kv, ws)
        outs.append(o.cpu())
        pools.append((kq.cpu(), vq.cpu()))
    assert torch.equal(outs[0], outs[1])
    assert torch.equal(pools[0][0], pools[1][0]) and torch.equal(pools[0][1], pools[1][1])
    if write_kv:
        assert not torch.equal(pools[0][0], dev(kpool).cpu())      # the new rows did go in


def test_attention_decode_fused_refuses_other_sizes(ops):
    assert not ops.attention_decode_fused_ok(4, 2, 48, 48)      # head size
    assert not ops.attention_decode_fused_ok(4, 2, 64, 32)      # partial rotation
    assert not ops.attention_decode_fused_ok(5, 2, 64, 64)


@pytest.mark.parametrize("where", ["far", "first_in_window", "last_outside_window"])
@pytest.mark.parametrize("copies", [1, 130])
def test_attention_decode_fused_far_key_and_window_edge(ops, where, copies):
    """The one-token kernel with one old key made to dominate the scores of each kv group's
    first head: far back among 900 keys it must be the result; as the oldest key of a window it
    must be the result too; one place further back it must not count at all. Alone (keys cut
    across workgroups, joined by a second launch) and among many sequences (one workgroup each)."""
    H, KVH, hd, n, theta = 4, 2, 64, 900, 10000.0
    window = 0 if where == "far" else 200
    key = {"far": 17, "first_in_window": n - 200, "last_outside_window": n - 201}[where]
    B = copies
    lengths = [n] + [50 + 3 * i for i in range(B - 1)]
    slots, table, kpool, vpool = paged_setup(lengths, KVH, hd, torch.bfloat16, 77)
    width = (H + 2 * KVH) * hd
    qkv = rnd(B, width, seed=120, scale=0.1).to(torch.bfloat16)
    pos = torch.tensor([m - 1 for m in lengths], dtype=torch.int32)
    q_rot = P.rope(qkv[0, :H * hd].double().reshape(1, H, hd), torch.tensor([n - 1]), theta, hd)
    ks = [rnd(m - 1, KVH, hd, seed=121 + i, scale=0.1).to(torch.bfloat16) for i, m in enumerate(lengths)]
    vs = [rnd(m - 1, KVH, hd, seed=171 + i).to(torch.bfloat16) for i, m in enumerate(lengths)]
    ks[0][key] = (q_rot[0, ::H // KVH] * 300).to(torch.bfloat16)
    fill_cache(table, slots, kpool, vpool, ks, vs)
    floats = ops.attention_decode_fused_workspace_floats(B, H, KVH, hd, 4096)
    assert (floats > 0) == (copies == 1)
    ws = torch.empty(floats, device="cuda") if floats else None
    out = torch.empty(B, H * hd, dtype=torch.bfloat16, device="cuda")
    ops.attention_decode_fused(out, dev(qkv), None, dev(kpool), dev(vpool), dev(pos),
                               dev(torch.arange(B, dtype=torch.int32)), dev(torch.tensor(slots, dtype=torch.int32)),
                               dev(table), dev(P.rope_inv_freq(hd, theta)), hd, B, H, KVH, hd, window,
                               1.0 / math.sqrt(hd), 4096, True, ws)
    got = out.cpu().double()[0].reshape(H, hd)
    x = qkv[0].double()
    k_new = P.rope(x[H * hd:(H + KVH) * hd].reshape(1, KVH, hd), torch.tensor([n - 1]), theta, hd).to(torch.bfloat16)
    v_new = x[(H + KVH) * hd:].reshape(1, KVH, hd).to(torch.bfloat16)
    k_all, v_all = torch.cat([ks[0], k_new]).double(), torch.cat([vs[0], v_new]).double()
    want = P.attention(q_rot.to(torch.bfloat16).double(), k_all, v_all, torch.tensor([n - 1]), torch.arange(n),
                       window).reshape(H, hd)
    assert torch.allclose(got, want, rtol=2 ** -6, atol=2 ** -6)
    for h in range(0, H, H // KVH):
        near = torch.allclose(got[h], vs[0][key, h // (H // KVH)].double(), atol=0.05)
        assert near == (where != "last_outside_window"), (where, h)


def test_attention_far_key_stands_out(ops):
    """One far key is made to dominate: a kernel that drops or misplaces it fails."""
    H, KVH, hd, n = 4, 2, 64, 900
    for kind in ("plain", "decode", "prefill"):
        slots, table, kpool, vpool = paged_setup([n], KVH, hd, torch.bfloat16, 50)
        k = rnd(n, KVH, hd, seed=51, scale=0.1).to(torch.bfloat16)
        v = rnd(n, KVH, hd, seed=52).to(torch.bfloat16)
        q = rnd(1, H, hd, seed=53, scale=0.1).to(torch.bfloat16)
        far = 17
        k[far] = (q[0, ::2] * 300).to(torch.bfloat16)      # aligned with the query of each group's first head
        fill_cache(table, slots, kpool, vpool, [k], [v])
        out = torch.empty(1, H * hd, dtype=torch.bfloat16, device="cuda")
        pos = torch.tensor([n - 1], dtype=torch.int32)
        zero = torch.zeros(1, dtype=torch.int32)
        scale = 1 / math.sqrt(hd)
        if kind == "plain":
            ops.attention_plain(out, dev(q.reshape(1, -1)), dev(kpool), dev(vpool), dev(pos), dev(zero),
                                dev(torch.tensor(slots, dtype=torch.int32)), dev(table), 1, H, KVH, hd, 0, scale)
        elif kind == "decode":
            ws = torch.empty(ops.attention_decode_workspace_floats(1, H, KVH, hd, 4096), device="cuda")
            ops.attention_decode(out, dev(q.reshape(1, -1)), dev(kpool), dev(vpool), dev(pos), dev(zero),
                                 dev(torch.tensor(slots, dtype=torch.int32)), dev(table), 1, H, KVH, hd, 0,
                                 scale, 4096, ws)
        else:
            ops.attention_prefill(out, dev(q.reshape(1, -1)), dev(kpool), dev(vpool),
                                  dev(torch.tensor([0, 1], dtype=torch.int32)),
                                  dev(torch.tensor(slots, dtype=torch.int32)),
                                  dev(torch.tensor([n - 1], dtype=torch.int32)), dev(table), 1, 1, 1,
                                  H, KVH, hd, 0, scale)
        want = P.attention(q.double(), k.double(), v.double(), torch.tensor([n - 1]), torch.arange(n), 0)
        got = out.cpu().double()
        assert torch.allclose(got, want, rtol=2 ** -6, atol=2 ** -6), kind
        # heads 0 and 2 must return (almost) the far value
        assert torch.allclose(got.reshape(H, hd)[0], v[far, 0].double(), atol=0.05), kind


# ------------------------------------------------------------------ random sizes
def test_gemm_blocksplit_at_random_sizes(ops):
    """300 products of random sizes (1 to 32 rows, any N up to 6000, K in steps of 8 up to 20000), plain and gated,
    with and without bias, bf16 and fp32 results, row-major and piece-major, against double precision."""
    import random
    rng = random.Random(5)
    for case in range(300):
        M = rng.randint(1, 32)
        K = 8 * rng.randint(1, rng.choice([40, 300, 2500]))
        N = rng.randint(1, rng.choice([64, 700, 6000]))
        gated = rng.random() < 0.3 and M <= 16
        if gated:
            N = 2 * max(1, N // 2)
        x = rnd(M, K, seed=case).to(torch.bfloat16)
        w = rnd(N, K, seed=case + 1, scale=0.05).to(torch.bfloat16)
        bias = None
        if rng.random() < 0.5 and not gated:
            bias = rnd(N, seed=case + 2).to(rng.choice([torch.bfloat16, torch.float32]))
        od = torch.bfloat16 if gated else rng.choice([torch.bfloat16, torch.float32])
        NO = N // 2 if gated else N
        xin = rng.random() < 0.5 and M <= 16
        op = rng.random() < 0.5 and M <= 16 and od == torch.bfloat16 and NO % 8 == 0
        out = torch.full(ops.pieces_shape(M, NO) if op else (M, NO), 7.0, dtype=od, device="cuda")
        xd = dev(x)
        ops.gemm_blocksplit(out, to_pieces(xd) if xin else xd, dev(w), dev(bias) if bias is not None else None, M,
                            gated=gated, x_pieces=xin, out_pieces=op)
        got = (from_pieces(out) if op else out).cpu().double()
        if gated:
            ref = P.silu(x.double() @ w[0::2].double().T) * (x.double() @ w[1::2].double().T)
        else:
            ref = x.double() @ w.double().T + (bias.double() if bias is not None else 0)
        tol = (2 ** -7 if od == torch.bfloat16 else 1e-4) * max(ref.abs().max().item(), 1e-3) * (2 if gated else 1) + 1e-6
        err = (got - ref).abs().max().item()
        assert err <= tol, (case, M, N, K, gated, od, xin, op, err, tol)


def test_attention_kernels_at_random_sizes(ops):
    """400 cases of random head counts, groups, head sizes (16 to 256 in steps of 16), windows, lengths and
    new-token counts through the prompt kernels, the split one-token kernel and the plain kernel."""
    import random
    rng = random.Random(9)
    for case in range(400):
        hd, KVH = 16 * rng.randint(1, 16), rng.randint(1, 4)
        H = KVH * rng.randint(1, 8)
        window = rng.choice([0, 0, 3, 70, 300])
        kind = rng.choice(["prefill", "prefill", "decode", "plain"])
        lengths = [rng.randint(1, rng.choice([5, 80, 400])) for _ in range(rng.randint(1, 5))]
        q_lens = [1 if kind == "decode" else rng.randint(1, n) for n in lengths]
        tiles = 0 if kind != "prefill" else (rng.choice([0, 1, 2]) if hd <= 128 else rng.choice([0, 1]))
        dtype = torch.bfloat16 if kind != "plain" else rng.choice([torch.float32, torch.bfloat16])
        got, want = attention_case(ops, kind, dtype, H, KVH, hd, window, lengths, q_lens, case, tiles=tiles)
        tol = 2 ** -6 if dtype == torch.bfloat16 else 1e-5
        for g, w in zip(got, want):
            assert torch.allclose(g, w, rtol=tol, atol=tol), (case, kind, dtype, H, KVH, hd, window, lengths, q_lens, tiles)


def test_attention_decode_fused_at_random_sizes(ops):
    """150 cases of the one-launch one-token attention: 1 to 40 sequences of 1 to 1500 keys, 1 to 5 kv heads with
    groups of 1 to 9, head size 64 or 128, windows, with and without the cache write."""
    import random
    rng = random.Random(7)
    theta = 10000.0
    for case in range(150):
        hd, KVH = rng.choice([64, 128]), rng.randint(1, 5)
        H = KVH * rng.randint(1, 9)
        B, window, write_kv = rng.randint(1, 40), rng.choice([0, 0, 5, 70, 300]), rng.random() < 0.7
        lengths = [rng.randint(1, rng.choice([3, 70, 400, 1500])) for _ in range(B)]
        slots, table, kpool, vpool = paged_setup(lengths, KVH, hd, torch.bfloat16, case)
        old = [n if not write_kv else n - 1 for n in lengths]
        ks = [rnd(n, KVH, hd, seed=7 * case + i).to(torch.bfloat16) for i, n in enumerate(old)]
        vs = [rnd(n, KVH, hd, seed=7 * case + 500 + i).to(torch.bfloat16) for i, n in enumerate(old)]
        fill_cache(table, slots, kpool, vpool, ks, vs)
        width = (H + 2 * KVH) * hd if write_kv else H * hd
        qkv = rnd(B, width, seed=case + 3, scale=1.5).to(torch.bfloat16)
        bias = rnd(width, seed=case + 4).to(torch.bfloat16)
        floats = ops.attention_decode_fused_workspace_floats(B, H, KVH, hd, 4096)
        ws = torch.empty(floats, device="cuda") if floats else None
        out = torch.full((B, H * hd), 7.0, dtype=torch.bfloat16, device="cuda")
        pos = torch.tensor([n - 1 for n in lengths], dtype=torch.int32)
        ops.attention_decode_fused(out, dev(qkv), dev(bias), dev(kpool), dev(vpool), dev(pos),
                                   dev(torch.arange(B, dtype=torch.int32)), dev(torch.tensor(slots, dtype=torch.int32)),
                                   dev(table), dev(P.rope_inv_freq(hd, theta)), hd, B, H, KVH, hd, window,
                                   1.0 / math.sqrt(hd), 4096, write_kv, ws)
        got = out.cpu().double()
        x = qkv.double() + bias.double()
        for s in rng.sample(range(B), min(B, 3)):
            n = lengths[s]
            p = torch.tensor([n - 1])
            q = P.rope(x[s, :H * hd].reshape(1, H, hd), p, theta, hd).to(torch.bfloat16).double()
            k_all, v_all = ks[s].double(), vs[s].double()
            if write_kv:
                k_new = P.rope(x[s, H * hd:(H + KVH) * hd].reshape(1, KVH, hd), p, theta, hd).to(torch.bfloat16)
                v_new = x[s, (H + KVH) * hd:].reshape(1, KVH, hd).to(torch.bfloat16)
                k_all, v_all = torch.cat([k_all, k_new.double()]), torch.cat([v_all, v_new.double()])
            want = P.attention(q, k_all, v_all, p, torch.arange(n), window).reshape(-1)
            assert torch.allclose(got[s], want, rtol=2 ** -6, atol=2 ** -6), (case, H, KVH, hd, B, window, write_kv, n)


# ------------------------------------------------------------------ sampling
def test_argmax_lowest_index_on_ties(ops):
    V = 1000
    x = rnd(4, V, seed=60)
    x[0, 500] = x[0, 77] = 9.0
    x[1, :] = 1.0                          # all equal -> index 0
    x[2, 999] = 50.0
    x[3, 3] = x[3, 2] = x[3, 998] = 8.0
    out = torch.empty(4, dtype=torch.int32, device="cuda")
    ops.argmax_rows(out, dev(x), 4)
    assert out.tolist() == [77, 0, 999, 2]
    assert out.tolist() == [P.argmax_lowest(r) for r in x]


@pytest.mark.parametrize("V", [8192, 8193, 30001, 152064])
def test_argmax_over_parts(ops, V):
    """Long rows are cut across workgroups: ties across a cut, a maximum at either end, at
    a cut and in the last (short) part; a width that is no multiple of 4."""
    x = rnd(6, V, seed=61)
    x[0, 8191] = x[0, V - 1] = 30.0               # tie across parts: the lower index
    x[1, V - 1] = 40.0
    x[2, 0] = 40.0
    x[3, :] = -3.0                                # all equal
    x[4, min(V - 1, 8192)] = x[4, 5000] = 35.0
    out = torch.empty(6, dtype=torch.int32, device="cuda")
    ops.argmax_rows(out, dev(x), 6)
    assert out.tolist() == [P.argmax_lowest(r) for r in x]
    assert out.tolist()[:5] == [8191, V - 1, 0, 0, 5000]


def test_penalties(ops):
    V = 50
    x = rnd(2, V, seed=61)
    ctx = [[3, 3, 7, 49], [0]]
    ids = torch.tensor([3, 7, 49, 0], dtype=torch.int32)
    counts = torch.tensor([2, 1, 1, 1], dtype=torch.int32)
    offsets = torch.tensor([0, 3, 4], dtype=torch.int32)
    d = dev(x.clone())
    ops.apply_penalties(d, 2, dev(ids), dev(counts), dev(offsets), 1.15, 0.1, 0.05)
    for r in range(2):
        want = P.apply_penalties(x[r], ctx[r], 384, 1.15, 0.1, 0.05)
        assert torch.allclose(d.cpu()[r], want, rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("W", [1, 5, 16, 300])
def test_penalties_from_a_window_on_the_device(ops, W):
    """The window as a ring on the device, fed one token a row and step: after every step the logits
    equal the plain penalties over the last W tokens (ids repeat, some lie outside the vocabulary, the
    ring wraps several times), and equal the kernel that takes the host's counts bit for bit."""
    V, rows, steps = 97, 3, 40
    g = torch.Generator().manual_seed(63)
    start = [[5, 5, 96], [], list(range(10, 10 + 2 * W))]
    ring = torch.zeros(rows, W, dtype=torch.int32)
    appended = torch.zeros(rows, dtype=torch.int32)
    for r, ctx in enumerate(start):
        last = ctx[max(0, len(ctx) - W):]
        ring[r, :len(last)] = torch.tensor(last, dtype=torch.int32)
        appended[r] = len(last)
    ring, appended = dev(ring), dev(appended)
    ctx = [list(c) for c in start]
    fresh = None
    for step in range(steps):
        x = rnd(rows, V, seed=100 + step)
        d = dev(x.clone())
        ops.apply_penalties_window(d, rows, ring, appended, fresh, 1.2, 0.15, 0.05)
        ids, counts, offsets = [], [], [0]
        for r in range(rows):
            want = P.apply_penalties(x[r], ctx[r], W, 1.2, 0.15, 0.05)
            assert torch.allclose(d.cpu()[r], want, rtol=1e-6, atol=1e-6), (step, r)
            seen = {}
            for tok in ctx[r][max(0, len(ctx[r]) - W):]:
                if 0 <= tok < V:
                    seen[tok] = seen.get(tok, 0) + 1
            ids.append(list(seen))
            counts.append(list(seen.values()))
            offsets.append(offsets[-1] + len(seen))
        flat = lambda v: dev(torch.tensor([a for part in v for a in part], dtype=torch.int32))   # noqa: E731
        d2 = dev(x.clone())
        if offsets[-1]:
            ops.apply_penalties(d2, rows, flat(ids), flat(counts), dev(torch.tensor(offsets, dtype=torch.int32)),
                                1.2, 0.15, 0.05)
        assert torch.equal(d2, d)
        new = torch.randint(-2, V + 3, (rows,), generator=g).tolist()    # some ids outside the vocabulary
        if step % 3 == 0:
            new[0] = 5                                                   # repeats
        fresh = dev(torch.tensor(new, dtype=torch.int32))
        for r in range(rows):
            ctx[r].append(new[r])
    assert appended.cpu().tolist() == [min(len(s), W) + steps - 1 for s in start]


@pytest.mark.parametrize("V", [301, 5000, 152064])
@pytest.mark.parametrize("temperature,top_k,top_p", [(0.8, 0, 1.0), (1.0, 50, 0.9), (0.7, 40, 1.0),
                                                     (1.3, 0, 0.5), (0.05, 0, 1.0), (1.0, 1, 1.0)])
def test_sample_rows_equals_plain(ops, V, temperature, top_k, top_p):
    rows = 6
    x = rnd(rows, V, seed=62, scale=2.0)
    x[1, 5] = x[1, 9] = x[1].max() + 1          # a tie at the top
    us = [0, 1, 2 ** 31, 2 ** 32 - 1, 123456789, 3000000000]
    u = torch.tensor(us, dtype=torch.int64).to(torch.uint32)
    out = torch.empty(rows, dtype=torch.int32, device="cuda")
    ops.sample_rows(out, dev(x), rows, dev(u), temperature, top_k, top_p)
    got = out.tolist()
    want = [P.sample(x[r], temperature, top_k, top_p, us[r]) for r in range(rows)]
    if got != want:
        # exp() may differ in the last bit between the GPU and the CPU; then the draw must lie on
        # a boundary: both tokens adjacent in the sorted order
        for r in range(rows):
            if got[r] != want[r]:
                order = torch.argsort(-x[r].double(), stable=True).tolist()
                assert abs(order.index(got[r]) - order.index(want[r])) == 1, (r, got[r], want[r])
    if top_k == 1:
        assert got == [P.argmax_lowest(r) for r in x]


def test_sample_rows_takes_both_zeros_as_equal(ops):
    """+0.0 and -0.0 are equal values: among them the index alone decides, as in the plain implementation
    (as sort keys the two differ)."""
    V = 4096
    g = torch.Generator().manual_seed(3)
    x = torch.where(torch.rand(2, V, generator=g) < 0.5, torch.tensor(0.0), torch.tensor(-0.0))
    x[1, 100:200] = -1.0
    us = [3359715596, 1234567]
    out = torch.empty(2, dtype=torch.int32, device="cuda")
    for temperature, top_k, top_p in ((0.8, 0, 0.1), (1.0, 50, 1.0), (0.7, 0, 1.0)):
        ops.sample_rows(out, dev(x), 2, dev(torch.tensor(us, dtype=torch.int64).to(torch.uint32)), temperature, top_k, top_p)
        assert out.tolist() == [P.sample(x[r], temperature, top_k, top_p, us[r]) for r in range(2)]


@pytest.mark.parametrize("case", ["top_k beyond the list", "all equal", "ties at the threshold", "two values",
                                  "deep nucleus", "a small top_k among thousands of ties",
                                  "a small top_k that cuts through a few ties"])
def test_sample_rows_list_and_whole_row_agree(ops, case):
    """The kernel works on a list of the row's largest elements and falls back to the whole row
    when that is not enough; both must give the plain implementation's token."""
    V = 40000
    x = rnd(4, V, seed=63, scale=2.0)
    temperature, top_k, top_p = 0.9, 0, 1.0
    if case == "top_k beyond the list":
        top_k = 9000
    elif case == "all equal":
        x[:] = 1.5
    elif case == "ties at the threshold":
        x = torch.round(x * 2) / 2                 # a few dozen distinct values, thousands of ties each
        top_k = 500
    elif case == "two values":
        x[:] = -4.0
        x[:, ::7] = 3.0
        top_p = 0.5
    elif case == "a small top_k among thousands of ties":
        x = torch.round(x * 2) / 2                 # more equal values at the top-k's edge than a wavefront has lanes
        top_k, top_p = 40, 0.95
    elif case == "a small top_k that cuts through a few ties":
        for r in range(4):                         # ranks 37 to 43 hold one value: the top-k of 40 keeps the three
            order = torch.argsort(-x[r], stable=True)   # of them with the lowest indices
            x[r, order[37:44]] = x[r, order[37]].item()
        top_k, top_p, temperature = 40, 0.999, 5.0   # flat, so that draws reach the edge
    elif case == "deep nucleus":
        top_p = 0.9999
        temperature = 3.0                          # flat: the nucleus reaches far beyond the list
    us = [0, 2 ** 32 - 1, 123456789, 3000000000]
    u = torch.tensor(us, dtype=torch.int64).to(torch.uint32)
    out = torch.empty(4, dtype=torch.int32, device="cuda")
    ops.sample_rows(out, dev(x), 4, dev(u), temperature, top_k, top_p)
    got = out.tolist()
    want = [P.sample(x[r], temperature, top_k, top_p, us[r]) for r in range(4)]
    for r in range(4):
        if got[r] != want[r]:                      # a last-bit difference of exp(): neighbours in the order
            order = torch.argsort(-x[r].double(), stable=True).tolist()
            assert abs(order.index(got[r]) - order.index(want[r])) == 1, (case, r, got[r], want[r])


def test_sample_frequencies(ops):
    """Empirical frequencies follow softmax(logits / T) on a small vocabulary."""
    V, n = 8, 20000
    logits = torch.tensor([2.0, 1.0, 0.5, 0.0, -1.0, 1.5, -3.0, 0.2])
    x = logits.repeat(n, 1).contiguous()
    u = torch.tensor([P.uniform_u32(7, 0, i) for i in range(n)], dtype=torch.int64).to(torch.uint32)
    out = torch.empty(n, dtype=torch.int32, device="cuda")
    ops.sample_rows(out, dev(x), n, dev(u), 0.8, 0, 1.0)
    freq = torch.bincount(out.cpu().long(), minlength=V).double() / n
    p = torch.softmax(logits.double() / 0.8, 0)
    chi2 = (n * (freq - p) ** 2 / p).sum().item()
    assert chi2 < 30, chi2                        # 7 degrees of freedom; 30 is far in the tail
