"""The argmax entry point that allocates nothing (he_argmax_rows_static) against the one that
takes a workspace (he_argmax_rows), called through ctypes: two calls in a row on one GPU, the
second with a smaller input, so that what the first call left in the static array must not
show; then the refusal of an input beyond the array's size. The entry point has no counterpart
in the reference: it is for callers that cannot allocate device memory."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _lib():
    from hector_engine_amd.kernels import lib
    L = lib.load()
    return L, lib


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _with_workspace(L, lib, logits: torch.Tensor, rows: int, V: int) -> torch.Tensor:
    out = torch.full((rows,), -7, dtype=torch.int32, device=logits.device)
    need = int(L.he_argmax_workspace_bytes(rows, V))
    ws = torch.empty(max(need, 1), dtype=torch.uint8, device=logits.device)
    lib.check(L.he_argmax_rows(out.data_ptr(), logits.data_ptr(), rows, V, logits.stride(0),
                               ws.data_ptr(), need, _stream()))
    return out


def _static(L, lib, logits: torch.Tensor, rows: int, V: int) -> torch.Tensor:
    out = torch.full((rows,), -7, dtype=torch.int32, device=logits.device)   # the caller's output
    lib.check(L.he_argmax_rows_static(out.data_ptr(), logits.data_ptr(), rows, V, logits.stride(0),
                                      _stream()))
    return out


def test_static_argmax_equals_workspace_argmax_twice_in_a_row():
    L, lib = _lib()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    assert L.he_argmax_rows_static_setup() == 0
    g = torch.Generator(device=dev).manual_seed(5)
    # first call: 40 rows of 152064 logits (19 parts a row); the best of every row lies in a
    # late part, and ties are planted so that "lowest index" is decided across parts
    rows, V = 40, 152064
    a = torch.randn((rows, V), generator=g, device=dev, dtype=torch.float32)
    for r in range(rows):
        hi = 90000 + 997 * r
        a[r, hi] = 50.0
        if r % 3 == 0:
            a[r, hi + 20000] = 50.0        # a tie in a later part: the earlier index wins
    want_a = _with_workspace(L, lib, a, rows, V)
    got_a = _static(L, lib, a, rows, V)
    # second call at once, smaller in both rows and vocabulary (4 parts a row), with its best
    # elements early: stale parts of the first call would win if they were read
    rows_b, V_b = 7, 30001
    b = torch.randn((rows_b, V_b), generator=g, device=dev, dtype=torch.float32)
    for r in range(rows_b):
        b[r, 11 + r] = 9.0
    want_b = _with_workspace(L, lib, b, rows_b, V_b)
    got_b = _static(L, lib, b, rows_b, V_b)
    torch.cuda.synchronize()
    assert torch.equal(got_a, want_a)
    assert got_a.tolist() == [90000 + 997 * r for r in range(rows)]
    assert torch.equal(got_b, want_b)
    assert got_b.tolist() == [11 + r for r in range(rows_b)]
    # one part a row: no scratch is touched at all
    c = torch.randn((3, 500), generator=g, device=dev, dtype=torch.float32)
    assert torch.equal(_static(L, lib, c, 3, 500), _with_workspace(L, lib, c, 3, 500))
    assert torch.equal(_static(L, lib, c, 3, 500).cpu(), c.argmax(-1).to(torch.int32).cpu())


def test_static_argmax_refuses_what_its_array_cannot_hold():
    L, lib = _lib()
    dev = torch.device("cuda:0")
    limit = ctypes.c_int64(65536).value
    rows, V = 500, 152064                   # 500 * 19 * 8 bytes > 64 KiB
    assert int(L.he_argmax_workspace_bytes(rows, V)) > limit
    x = torch.zeros((rows, V), dtype=torch.float32, device=dev)
    out = torch.zeros(rows, dtype=torch.int32, device=dev)
    rc = L.he_argmax_rows_static(out.data_ptr(), x.data_ptr(), rows, V, V, _stream())
    assert rc != 0
    msg = L.he_last_error().decode()
    assert "static" in msg and "65536" in msg
    # the largest that fits: 431 rows
    rows = 431
    assert int(L.he_argmax_workspace_bytes(rows, V)) <= limit
    x[:rows, 777] = 1.0
    lib.check(L.he_argmax_rows_static(out.data_ptr(), x.data_ptr(), rows, V, V, _stream()))
    torch.cuda.synchronize()
    assert out[:rows].tolist() == [777] * rows
