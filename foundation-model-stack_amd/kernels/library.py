"""Loads the compiled kernel library and declares its C interface for ctypes.

The library must be there on a GPU machine: nothing in this package falls back
to a CPU or to a library model when it is missing.  ``import torch`` happens
first so that the HIP runtime the kernels link against is the one PyTorch has
already loaded.
"""

from __future__ import annotations

import ctypes
import threading
from ctypes import c_char_p, c_float, c_int, c_long, c_void_p
from typing import Optional

import torch  # noqa: F401  (loads libamdhip64 before our library asks for it)

from . import build as _build

ABI_VERSION = 2

_lib: Optional[ctypes.CDLL] = None
_lock = threading.Lock()

P, I, L, F = c_void_p, c_int, c_long, c_float

_SIGNATURES = {
    "fmsamd_embed": [P, P, I, P, I, I, I, P],
    "fmsamd_add_norm": [P, P, I, P, P, I, P, P, I, I, F, I, P],
    "fmsamd_gated_act": [P, P, I, P, I, I, I, I, P],
    "fmsamd_cast": [P, I, P, I, L, P],
    "fmsamd_advance_positions": [P, P, I, P],
    "fmsamd_bias_add": [P, I, P, I, I, I, P],
    "fmsamd_rope_table": [P, P, P, I, I, P],
    "fmsamd_rope_kv_write": [P, I, L, P, P, P, I, P, P, I, I, P, P, I, I, I, I, P],
    "fmsamd_attn_generic": [P, L, P, L, I, P, P, P, I, P, P, I, I, I, I, F, I, P, F, P],
    "fmsamd_attn_prefill_bf16": [P, L, P, L, P, P, P, P, I, I, P, I, P, P, I, I, I, I, F, I, P],
    "fmsamd_attn_decode_bf16": [P, L, P, L, P, L, P, P, P, I, P, P, I, I, I, I, F, I, I, I, I, I, P, P],
    "fmsamd_qkv_rope_skinny_bf16": [P, L, P, P, I, P, L, I, I, P, P, P, I, P, P, I, I, P, P, I, I, I, P, P, L, P],
    "fmsamd_gemm_f32": [P, L, P, P, P, L, I, I, I, P],
    "fmsamd_gemm_bf16": [P, L, P, P, I, P, I, L, I, I, I, P],
    "fmsamd_gemm_bf16_any": [P, L, P, P, I, P, I, L, I, I, I, P],
    "fmsamd_gemm_skinny_workspace": [I, I, I],
    "fmsamd_gemm_skinny_bf16": [P, L, P, P, I, P, I, L, I, I, I, P, P, L, P],
    "fmsamd_gemm_skinny_gated_bf16": [P, L, P, P, I, P, I, L, I, I, I, I, P, P, L, P],
    "fmsamd_gemm_skinny_residual_partials": [I, I, I],
    "fmsamd_gemm_skinny_residual_bf16": [P, L, P, P, I, P, L, P, I, P, L, P, I, I, I, I, P, P, L, P],
    "fmsamd_sample": [P, L, I, I, I, F, I, P, P, P],
    "fmsamd_argmax": [P, L, I, I, P, L, P, P],
    "fmsamd_probe_read": [P, L, I, I, P, P],
    "fmsamd_probe_mfma": [I, I, I, P, P, P],
}


class KernelLibraryMissing(RuntimeError):
    pass


def load(verbose: bool = True) -> ctypes.CDLL:
    """The kernel library, compiled first if no built copy is found."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        try:
            path = _build.ensure_built(verbose=verbose)
            lib = ctypes.CDLL(path)
        except Exception as err:  # no compiler, no writable folder, broken library
            raise KernelLibraryMissing(
                f"the HIP kernel library of fms_amd could not be built or loaded ({err}); "
                "there is no fallback path: build it with `python -m fms_amd.kernels.build` (needs hipcc)"
            ) from err
        lib.fmsamd_last_error.restype = c_char_p
        lib.fmsamd_last_error.argtypes = []
        lib.fmsamd_abi_version.restype = c_int
        lib.fmsamd_abi_version.argtypes = []
        if lib.fmsamd_abi_version() != ABI_VERSION:
            raise KernelLibraryMissing(
                f"{path} has interface version {lib.fmsamd_abi_version()}, this package needs {ABI_VERSION}: rebuild it"
            )
        for name, argtypes in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.argtypes = argtypes
            fn.restype = c_int
        lib.fmsamd_attn_prefill_qblock.restype = c_int
        lib.fmsamd_attn_prefill_qblock.argtypes = [I, I, I, I]
        lib.fmsamd_argmax_workspace.restype = c_long
        lib.fmsamd_argmax_workspace.argtypes = [I, I]
        lib.fmsamd_attn_decode_workspace.restype = c_long
        lib.fmsamd_gemm_skinny_workspace.restype = c_long
        lib.fmsamd_attn_decode_workspace.argtypes = [I, I, I, I]
        lib.path = path
        _lib = lib
    return _lib


class KernelError(RuntimeError):
    pass


def check(code: int) -> None:
    if code != 0:
        raise KernelError(load().fmsamd_last_error().decode())
