"""The matrix product for 17 to 64 rows whose activation rows go through LDS once per workgroup
(gemm_rows): every tiling and every epilogue against float64 torch, at sizes that are no
multiple of a tile or of a k chunk, row-major and piece-major, in one K slice and in several."""
import pytest
import torch

from tests.plain import qwen2_plain as P
from tests.test_kernels_gpu import alternate_rows, dev, from_pieces, rnd, to_pieces

pytestmark = pytest.mark.gpu

PLANS = [(0, 0, 0), (1, 8, 1), (2, 8, 1), (1, 4, 1), (1, 4, 3), (1, 8, 4), (2, 8, 16), (2, 4, 1), (1, 16, 1), (1, 16, 2)]
SHAPES = [(301, 136), (1000, 1544), (37, 4104), (4608, 3584), (2051, 264), (512, 128), (20002, 136)]


@pytest.fixture(scope="module")
def ops():
    import hector_engine_amd  # noqa: F401
    from hector_engine_amd.kernels import lib, ops as _ops
    lib.load()
    return _ops


def product(ops, a, w, bias, M, plan, out_dtype=torch.float32, **kw):
    """The product through gemm_rows whatever the number of K slices: partial sums are added by
    splitk_reduce. Returns (result on the CPU, slices)."""
    N = w.shape[0]
    out = torch.full((M, N), float("nan"), dtype=out_dtype, device="cuda")
    splits = ops.gemm_rows_plan(M, N, w.shape[1])[1] if plan == (0, 0, 0) else max(plan[2], 1)
    partial = torch.full((splits, M, N), float("nan"), device="cuda")
    if splits > 1 and plan[2] > 1 and (w.shape[1] + 127) // 128 < 2:
        splits = 1                                   # K too short to cut: one slice will run
    used = ops.gemm_rows(out, partial, a, dev(w), dev(bias) if bias is not None and splits <= 1 else None,
                         M, plan=plan, **kw)
    if used > 1:
        ops.splitk_reduce(out, partial[:used].contiguous(), dev(bias) if bias is not None else None, M, used)
    elif splits > 1 and bias is not None:            # fewer slices than asked for: one slice, which takes the bias itself
        ops.gemm_rows(out, None, a, dev(w), dev(bias), M, plan=plan, **kw)
    return out.cpu(), used


@pytest.mark.parametrize("M", [1, 16, 17, 20, 32, 33, 47, 48, 49, 64])
@pytest.mark.parametrize("N,K", SHAPES)
@pytest.mark.parametrize("plan", PLANS)
def test_gemm_rows(ops, M, N, K, plan):
    if (N, K) == (4608, 3584) and (M not in (17, 64) or plan not in ((0, 0, 0), (1, 4, 3))):
        pytest.skip("large shape at two row counts and two tilings only")
    if plan == (2, 4, 1) and M <= 32:
        pytest.skip("two tiles a wavefront in four wavefronts: above 32 rows")
    a = rnd(M, K, seed=190).to(torch.bfloat16)
    w = rnd(N, K, seed=191, scale=0.05).to(torch.bfloat16)
    b = rnd(N, seed=192).to(torch.bfloat16)
    ref = a.double() @ w.double().T + b.double()
    outs = [product(ops, dev(a), w, b, M, plan)[0] for _ in range(2)]
    assert torch.equal(outs[0], outs[1])                           # twice the same bits
    assert (outs[0].double() - ref).abs().max().item() <= 1e-4 * ref.abs().max().item()
    out16, _ = product(ops, dev(a), w, None, M, plan, torch.bfloat16)
    ref0 = a.double() @ w.double().T
    assert (out16.double() - ref0).abs().max().item() <= 2 ** -8 * ref0.abs().max().item() + 1e-6
    # the rows piece-major: the same sums in the same order
    if K % 8 == 0:
        outp, _ = product(ops, dev(to_pieces(a)), w, b, M, plan, x_pieces=True)
        assert torch.equal(outp, outs[0])


@pytest.mark.parametrize("M", [1, 17, 32, 40, 50, 64])
@pytest.mark.parametrize("I,K", [(160, 64), (1008, 520), (37, 136), (1515, 264), (4000, 1024), (9475, 264)])
@pytest.mark.parametrize("plan", [(0, 0, 1), (1, 4, 1), (2, 4, 1), (1, 8, 1), (2, 8, 1), (1, 16, 1)])
def test_gemm_rows_gated_epilogue(ops, M, I, K, plan):
    if plan == (2, 4, 1) and M <= 32:
        pytest.skip("two tiles a wavefront in four wavefronts: above 32 rows")
    x = rnd(M, K, seed=193).to(torch.bfloat16)
    g = rnd(I, K, seed=194, scale=0.1).to(torch.bfloat16)
    u = rnd(I, K, seed=195, scale=0.1).to(torch.bfloat16)
    w = alternate_rows(g, u)
    ref = P.silu(x.double() @ g.double().T) * (x.double() @ u.double().T)
    tol = 2 ** -8 * ref.abs().max().item() + 1e-6
    out = torch.full((M, I), float("nan"), dtype=torch.bfloat16, device="cuda")
    assert ops.gemm_rows(out, None, dev(x), dev(w), None, M, gated=True, plan=plan) == 1
    assert (out.cpu().double() - ref).abs().max().item() <= tol
    if I % 8 == 0:      # written piece-major for the product that reads it next
        outp = torch.full(ops.pieces_shape(M, I), float("nan"), dtype=torch.bfloat16, device="cuda")
        ops.gemm_rows(outp, None, dev(x), dev(w), None, M, gated=True, plan=plan, out_pieces=True)
        assert torch.equal(from_pieces(outp).cpu(), out.cpu())


@pytest.mark.parametrize("M", [1, 17, 40, 64])
@pytest.mark.parametrize("D,K,N2,eps", [(80, 136, 301, 3e-6), (3584, 520, 160, 1e-6), (1000, 18944, 64, 1e-5),
                                        (2312, 264, 64, 1e-6)])
@pytest.mark.parametrize("gain_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("pieces", [False, True])
def test_gemm_rows_carries_the_norm(ops, M, D, K, N2, eps, gain_dtype, pieces):
    """A product adds its result to the residual rows and leaves r * gain and the sums of r^2 (in one
    K slice by its own epilogue, in several through splitk_reduce_residual); the next product applies
    the owed scale (in one slice or in several): add + RMS norm + product of the plain implementation."""
    if K == 18944 and (M == 40 or gain_dtype == torch.float32):
        pytest.skip("long K at three row counts, one gain dtype")
    x = rnd(M, K, seed=200).to(torch.bfloat16)
    w1 = rnd(D, K, seed=201, scale=0.05).to(torch.bfloat16)
    b1 = rnd(D, seed=202).to(torch.bfloat16)
    r0 = rnd(M + 1, D, seed=203, scale=3.0)
    gain = (1 + 0.1 * rnd(D, seed=204)).to(gain_dtype)
    r1 = r0[:M].double() + x.double() @ w1.double().T + b1.double()
    shape = ops.pieces_shape(M, D) if pieces else (M, D)
    results = []
    for way in ("epilogue", "slices"):
        resid = dev(r0.clone())
        xg = torch.zeros(shape, dtype=torch.bfloat16, device="cuda")
        if way == "epilogue":
            groups = -(-D // (16 * 1 * 4))
            sq = torch.full((M, groups), float("nan"), device="cuda")
            assert ops.gemm_rows(None, None, dev(x), dev(w1), dev(b1), M, plan=(1, 4, 1),
                                 residual=(resid, dev(gain), xg, sq), out_pieces=pieces) == 1
        else:
            splits = 3
            partial = torch.full((splits, M, D), float("nan"), device="cuda")
            used = ops.gemm_rows(None, partial, dev(x), dev(w1), None, M, plan=(1, 8, splits))
            sq = torch.full((M, ops.splitk_reduce_residual_blocks(D)), float("nan"), device="cuda")
            ops.splitk_reduce_residual(resid, partial[:used].contiguous(), dev(b1), dev(gain), xg, sq, M, used,
                                       out_pieces=pieces)
        got_r = resid.cpu()
        assert torch.equal(got_r[M], r0[M])                                   # the row after the last is untouched
        assert (got_r[:M].double() - r1).abs().max().item() <= 1e-4 * r1.abs().max().item()
        want_xg = (got_r[:M] * gain.float()).to(torch.bfloat16)
        got_xg = from_pieces(xg).cpu() if pieces else xg.cpu()
        assert (got_xg.float() - want_xg.float()).abs().max().item() <= 2 ** -7 * want_xg.float().abs().max().item()
        assert torch.allclose(sq.cpu().double().sum(1), (got_r[:M].double() ** 2).sum(1), rtol=1e-5)
        results.append((got_r, xg, sq))
    got_r, xg, sq = results[1]
    normed = P.rmsnorm(got_r[:M].double(), gain.double(), eps)
    w2 = rnd(N2, D, seed=205, scale=0.05).to(torch.bfloat16)
    b2 = rnd(N2, seed=206).to(torch.bfloat16)
    ref = normed @ w2.double().T + b2.double()
    for plan in ((1, 4, 1), (2, 8, 2)):           # the consumer in one slice, and in two
        out, used = product(ops, xg, w2, b2, M, plan, row_scale=(sq, eps), x_pieces=pieces)
        assert (out.double() - ref).abs().max().item() <= 2 ** -7 * ref.abs().max().item(), (plan, used)
    I = N2 // 2
    g, u = w2[:I], rnd(I, D, seed=207, scale=0.05).to(torch.bfloat16)
    h = torch.empty(M, I, dtype=torch.bfloat16, device="cuda")
    ops.gemm_rows(h, None, xg, dev(alternate_rows(g, u)), None, M, gated=True, plan=(0, 0, 1), row_scale=(sq, eps),
                  x_pieces=pieces)
    ref = P.silu(normed @ g.double().T) * (normed @ u.double().T)
    assert (h.cpu().double() - ref).abs().max().item() <= 2 ** -6 * ref.abs().max().item() + 1e-6
    t = torch.empty(M, D, dtype=torch.bfloat16, device="cuda")
    ops.scale_rows(t, xg, sq, eps, M, pieces)
    assert (t.cpu().double() - normed).abs().max().item() <= 2 ** -6 * normed.abs().max().item()


def test_gemm_rows_refuses_what_it_cannot_do(ops):
    from hector_engine_amd.kernels.lib import KernelLibraryError
    a = dev(rnd(20, 1024, seed=1).to(torch.bfloat16))
    w = dev(rnd(64, 1024, seed=2).to(torch.bfloat16))
    out = torch.empty(20, 64, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ValueError, match="outside"):
        ops.gemm_rows(out, None, a, w, None, 65)
    with pytest.raises(KernelLibraryError, match="one slice"):       # an epilogue with several K slices
        ops.gemm_rows(out[:, :32].contiguous(), torch.empty(2, 20, 64, device="cuda"), a, w, None, 20, gated=True,
                      plan=(1, 4, 2))
    with pytest.raises(KernelLibraryError, match="partial sums"):    # no room for the slices
        ops.gemm_rows(None, torch.empty(1, 20, 64, device="cuda"), a, w, None, 20, plan=(1, 4, 2))
    with pytest.raises(KernelLibraryError, match="multiple of 8"):
        ops.gemm_rows(torch.empty(20, 64, dtype=torch.bfloat16, device="cuda"), None,
                      dev(rnd(20, 100, seed=3).to(torch.bfloat16)), dev(rnd(64, 100, seed=4).to(torch.bfloat16)), None, 20)
    groups, splits = ops.gemm_rows_plan(64, 3584, 18944)
    assert groups * splits >= 192 and splits > 1                      # few rows, long K: cut across workgroups
    # wide products: one slice, the rows dealt out evenly (76 a workgroup, not 64 or 80; 200, not 256;
    # above 32 rows one workgroup of 148 rows a compute unit)
    assert ops.gemm_rows_plan(32, 37888, 3584) == (499, 1) and ops.gemm_rows_plan(64, 152064, 3584) == (761, 1)
    assert ops.gemm_rows_plan(64, 37888, 3584) == (256, 1)
    with pytest.raises(KernelLibraryError, match="more than 32 rows"):
        ops.gemm_rows(out, None, a, w, None, 20, plan=(2, 4, 1))
