"""Helpers shared by the GPU tests."""
import torch


def rand_ids(vocab: int, n: int, seed: int) -> list[int]:
    g = torch.Generator().manual_seed(1000 + seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def close(got: torch.Tensor, want: torch.Tensor, dtype: str) -> None:
    """float32: the engine's fp32 path against the float64 oracle, a few ulp of the
    logits' size. bfloat16: 8 bits of mantissa at every rounding point; the bound is
    1 % of the largest logit, twice the largest error seen over all tests that use it."""
    got = got.detach().cpu().double()
    want = want.double()
    assert got.shape == want.shape, (got.shape, want.shape)
    scale = want.abs().max().item()
    err = (got - want).abs().max().item()
    tol = 2e-5 * max(scale, 1.0) if dtype == "float32" else 0.01 * scale
    assert err <= tol, f"max error {err:.3g} above {tol:.3g} (logit scale {scale:.3g})"


def argmax_agrees_where_clear(got: torch.Tensor, want: torch.Tensor, margin: float) -> None:
    """Where the oracle's best logit leads by more than `margin`, the engine must agree."""
    want = want.double()
    top2 = want.topk(2, -1).values
    clear = (top2[:, 0] - top2[:, 1]) > margin
    g = got.detach().cpu().argmax(-1)
    w = want.argmax(-1)
    assert torch.equal(g[clear], w[clear])
