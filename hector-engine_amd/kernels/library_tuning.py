"""The library matrix product's own autotuner (torch's TunableOp over hipBLASLt / rocBLAS).

Tall products (more than 64 rows: more than the hand-written kernels take) go to the library,
as the reference sends every product to its BLAS library (kernels/matmul_cublas.cu:240-277).
The library's default choice of kernel is not always its best on MI355X: at the
Qwen2.5-7B shapes its tuner finds kernels 17-27 % faster for the 2048-row down and
gate||up products. Tuning runs the first time a shape (rows, N, K) is seen and takes a second
or so per shape, so it is meant for workloads whose shapes repeat (fixed prompt chunks); it is
off unless asked for. Results are kept in a file and read again by the next process (so the
kernels chosen, and with them the last bits of bfloat16 results, follow that file: name one with
HECTOR_TUNING_FILE or enable(path=...) where runs must repeat exactly). Row counts that
are unlikely to come again (a prompt of 1,937 tokens) are not tuned: worth_tuning().
"""
from __future__ import annotations

import contextlib
import os

import torch

from . import lib as _lib

_enabled = False


def results_path(path: str | None = None) -> str:
    """The tuning file: the given path, else HECTOR_TUNING_FILE, else a file in this user's
    private folder under the temporary directory."""
    path = path or os.environ.get("HECTOR_TUNING_FILE")
    if path:
        return os.path.abspath(path)
    return os.path.join(_lib._build_module().private_folder(), "library_gemm_tuning.csv")


def enable(max_seconds_per_shape: int = 30, max_iterations: int = 10, path: str | None = None) -> None:
    global _enabled
    t = torch.cuda.tunable
    t.set_filename(results_path(path))
    t.enable(True)
    t.tuning_enable(True)
    t.set_max_tuning_duration(max_seconds_per_shape)
    t.set_max_tuning_iterations(max_iterations)
    _enabled = True


def enabled() -> bool:
    return _enabled


def worth_tuning(rows: int) -> bool:
    """Whether a product of this many rows is tuned when first seen: multiples of 128 (fixed
    prompt chunks; the one-token step of 65 to 128 sequences, whose graph has 128 rows: 8.40 ->
    7.95 ms at the Qwen2.5-7B shape). Any other count runs with the library's default kernel, or
    with a tuned one if that exact shape was tuned before."""
    return rows > 0 and rows % 128 == 0


@contextlib.contextmanager
def no_new_tuning():
    """Inside: tuned choices are used, but no shape is tuned (graph capture cannot hold the
    tuner's timing runs)."""
    if not _enabled:
        yield
        return
    t = torch.cuda.tunable
    before = t.tuning_is_enabled()     # one such block may stand inside another
    t.tuning_enable(False)
    try:
        yield
    finally:
        t.tuning_enable(before)
