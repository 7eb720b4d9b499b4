"""Loads the gfx950 kernel library through ctypes and declares its C ABI.

torch is imported first so that the HIP runtime already in the process is the
one the library binds to. There is no fallback: without the library (and
without hipcc to build it) loading raises.
"""
from __future__ import annotations

import ctypes
import importlib.util
import os
import threading

_lock = threading.Lock()
_lib = None

_CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")

EXPECTED_ABI = 20

c_int, c_i64, c_f32, c_ptr = ctypes.c_int, ctypes.c_int64, ctypes.c_float, ctypes.c_void_p

# name -> argument types (all return int unless listed in _RESTYPES)
_SIGNATURES = {
    "he_abi_version": [],
    "he_fill_random": [c_ptr, c_i64, c_int, ctypes.c_uint64, c_ptr, c_f32, c_f32, c_ptr],
    "he_fill_random_integers": [c_ptr, c_i64, ctypes.c_uint64, c_i64, c_ptr],
    "he_cast": [c_ptr, c_ptr, c_i64, c_int, c_int, c_ptr],
    "he_embedding": [c_ptr, c_ptr, c_ptr, c_int, c_int, c_int, c_int, c_ptr],
    "he_gather_rows_f32": [c_ptr, c_ptr, c_ptr, c_int, c_int, c_int, c_ptr],
    "he_residual_add": [c_ptr, c_ptr, c_i64, c_int, c_ptr],
    "he_silu_mul": [c_ptr, c_ptr, c_int, c_int, c_int, c_int, c_int, c_ptr],
    "he_add_rmsnorm": [c_ptr, c_ptr, c_ptr, c_ptr, c_int, c_int, c_f32, c_int, c_int, c_ptr],
    "he_rmsnorm_rows": [c_ptr, c_ptr, c_ptr, c_int, c_int, c_i64, c_i64, c_f32, c_int, c_int, c_ptr],
    "he_gemm_plain_workspace_floats": [c_int, c_int, c_int],
    "he_gemm_plain": [c_ptr, c_ptr, c_ptr, c_ptr, c_int, c_int, c_int, c_i64, c_i64, c_i64,
                      c_int, c_int, c_int, c_ptr, c_i64, c_ptr],
    "he_gemm_blocksplit_bf16": [c_ptr, c_ptr, c_ptr, c_ptr, c_int, c_int, c_int, c_int, c_int, c_int,
                                c_int, c_int, c_int, c_ptr],
    "he_gemm_blocksplit_blocks": [c_int, c_int, c_int],
    "he_gemm_blocksplit_fused_bf16": [c_ptr, c_ptr, c_ptr, c_ptr, c_int, c_int, c_int, c_int, c_int, c_int,
                                      c_int, c_int, c_int, c_ptr, c_int, c_f32, c_ptr, c_ptr, c_int,
                                      c_ptr, c_ptr, c_int, c_int, c_int, c_ptr],
    "he_scale_rows_bf16": [c_ptr, c_ptr, c_ptr, c_int, c_int, c_int, c_f32, c_int, c_ptr],
    "he_splitk_reduce": [c_ptr, c_ptr, c_ptr, c_int, c_int, c_int, c_int, c_int, c_ptr],
    "he_gemm_rows_plan": [c_int, c_int, c_int, ctypes.POINTER(c_int), ctypes.POINTER(c_int)],
    "he_gemm_rows_bf16": [c_ptr, c_ptr, c_i64, c_ptr, c_ptr, c_ptr, c_int, c_int, c_int, c_int, c_int, c_int,
                          c_int, c_int, c_int, c_ptr, c_int, c_f32, c_ptr, c_ptr, c_int, c_ptr, c_ptr, c_int,
                          c_int, c_int, ctypes.POINTER(c_int), c_ptr],
    "he_splitk_reduce_residual_blocks": [c_int],
    "he_splitk_reduce_residual": [c_ptr, c_ptr, c_ptr, c_int, c_ptr, c_int, c_ptr, c_ptr, c_int, c_int, c_int,
                                  c_int, c_int, c_ptr],
    "he_qkv_rope_cache": [c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_i64, c_ptr, c_ptr, c_ptr,
                          c_int, c_ptr, c_ptr, c_ptr, c_ptr, c_int, c_int, c_ptr, c_int, c_int,
                          c_int, c_int, c_int, c_int, c_ptr],
    "he_attention_plain_workspace_floats": [c_int, c_int, c_int, c_int, c_int],
    "he_attention_plain": [c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_int, c_int,
                           c_int, c_int, c_int, c_int, c_int, c_f32, c_int, c_int, c_ptr, c_i64, c_ptr],
    "he_attention_decode_bf16": [c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_int,
                                 c_int, c_int, c_int, c_int, c_int, c_int, c_f32, c_int, c_ptr,
                                 c_i64, c_ptr],
    "he_attention_decode_workspace_floats": [c_int, c_int, c_int, c_int, c_int],
    "he_attention_decode_fused_ok": [c_int, c_int, c_int, c_int],
    "he_attention_decode_fused_workspace_floats": [c_int, c_int, c_int, c_int, c_int, c_int],
    "he_attention_decode_fused_bf16": [c_ptr, c_ptr, c_ptr, c_int, c_i64, c_i64, c_ptr, c_int, c_ptr, c_ptr, c_ptr, c_ptr,
                                       c_ptr, c_ptr, c_int, c_int, c_ptr, c_int, c_int, c_int, c_int,
                                       c_int, c_int, c_f32, c_int, c_int, c_int, c_int, c_ptr, c_i64, c_ptr],
    "he_attention_prefill_bf16": [c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_ptr, c_int,
                                  c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_f32, c_int,
                                  c_int, c_int, c_ptr, c_i64, c_ptr],
    "he_attention_prefill_parts": [c_int, c_int, c_int, c_int, c_int],
    "he_attention_prefill_workspace_floats": [c_int, c_int, c_int, c_int],
    "he_argmax_workspace_bytes": [c_int, c_int],
    "he_argmax_rows": [c_ptr, c_ptr, c_int, c_int, c_i64, c_ptr, c_i64, c_ptr],
    "he_argmax_rows_static_setup": [],
    "he_argmax_rows_static": [c_ptr, c_ptr, c_int, c_int, c_i64, c_ptr],
    "he_apply_penalties": [c_ptr, c_int, c_int, c_i64, c_ptr, c_ptr, c_ptr, c_f32, c_f32, c_f32,
                           c_ptr],
    "he_apply_penalties_window": [c_ptr, c_int, c_int, c_i64, c_ptr, c_ptr, c_int, c_ptr, c_f32, c_f32,
                                  c_f32, c_ptr],
    "he_sample_rows": [c_ptr, c_ptr, c_int, c_int, c_i64, c_ptr, c_f32, c_int, c_f32, c_ptr],
}
_RESTYPES = {
    "he_attention_plain_workspace_floats": c_i64,
    "he_gemm_plain_workspace_floats": c_i64,
    "he_attention_decode_workspace_floats": c_i64,
    "he_attention_decode_fused_workspace_floats": c_i64,
    "he_attention_prefill_workspace_floats": c_i64,
    "he_argmax_workspace_bytes": c_i64,
}


def _build_module():
    spec = importlib.util.spec_from_file_location("_hector_csrc_build", os.path.join(_CSRC, "build.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


class KernelLibraryError(RuntimeError):
    pass


def load():
    """Returns the loaded library, building it first if no current build exists."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        import torch  # noqa: F401  (brings the HIP runtime into the process first)
        try:
            path = _build_module().ensure_built()
        except Exception as exc:
            raise KernelLibraryError(
                f"the HIP kernel library is not built and could not be built: {exc}") from exc
        try:
            lib = ctypes.CDLL(path)
        except OSError as exc:
            raise KernelLibraryError(f"cannot load {path}: {exc}") from exc
        lib.he_last_error.restype = ctypes.c_char_p
        lib.he_last_error.argtypes = []
        for name, argtypes in _SIGNATURES.items():
            fn = getattr(lib, name, None)
            if fn is None:
                raise KernelLibraryError(f"{path} lacks the entry point {name}")
            fn.argtypes = argtypes
            fn.restype = _RESTYPES.get(name, c_int)
        abi = lib.he_abi_version()
        if abi != EXPECTED_ABI:
            raise KernelLibraryError(f"{path} has ABI {abi}, expected {EXPECTED_ABI}: rebuild it")
        lib._path = path
        _lib = lib
        return lib


def loaded_path() -> str | None:
    return None if _lib is None else _lib._path


def check(status: int) -> None:
    if status != 0:
        msg = _lib.he_last_error().decode(errors="replace") if _lib is not None else "?"
        raise KernelLibraryError(f"kernel library error {status}: {msg}")
