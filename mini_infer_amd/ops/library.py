"""Loads the HIP library through ctypes and declares its entry points.

There is no fallback: if the library is missing and cannot be built, loading
raises `ExtensionMissingError`.  A library that exists is loaded as it is when
its stamp matches the sources; a stale or missing one is rebuilt first.
"""

from __future__ import annotations

import ctypes
from ctypes import c_float, c_int, c_int64, c_void_p
from pathlib import Path

from mini_infer_amd.exceptions import ExtensionMissingError, KernelShapeError
from mini_infer_amd.ops import build as _build

ABI_VERSION = 18

_lib: ctypes.CDLL | None = None
_lib_path: Path | None = None

_P = c_void_p
_SIGNATURES: dict[str, list] = {
    "mi_embed_gather": [c_int, _P, _P, _P, c_int, c_int, c_int, _P],
    "mi_take_device_tokens": [_P, _P, _P, c_int, c_int, c_int, _P],
    "mi_begin_step": [_P, _P, _P, c_int, c_int, c_int, _P, _P, _P, c_int, c_int, _P],
    "mi_add_rmsnorm": [c_int, _P, _P, _P, _P, _P, c_int, c_int, c_float, _P, c_int, c_int64, _P],
    "mi_rope_table": [_P, _P, _P, _P, c_int, c_int, _P],
    "mi_rope_kv_write": [
        c_int, _P, c_int64, _P, _P, _P, _P, _P, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
        c_int, c_int, _P,
    ],
    "mi_silu_mul": [c_int, _P, _P, c_int, c_int, _P],
    "mi_gemm_f32": [_P, c_int64, _P, c_int64, _P, c_int64, c_int, c_int, c_int, _P],
    "mi_gemm_skinny_bf16": [_P, c_int64, _P, c_int64, _P, c_int64, c_int, c_int, c_int, _P],
    "mi_gemm_skinny_f32out_bf16": [_P, c_int64, _P, c_int64, _P, c_int64, c_int, c_int, c_int, _P],
    "mi_gemm_mid_partial_bf16": [_P, c_int64, _P, c_int64, _P, c_int, c_int, c_int, _P],
    "mi_gemm_mid_bf16_ranges": [c_int, c_int],
    "mi_gemm_mid_bf16_supported": [c_int, c_int, c_int, c_int64, c_int64],
    "mi_gemm_skinny_attn_bf16_supported": [c_int, c_int, c_int],
    "mi_gemm_skinny_attn_bf16": [_P, _P, c_int, c_int, c_int, _P, c_int64, _P, c_int64, c_int, c_int, _P],
    "mi_gemm_skinny_swiglu_bf16": [_P, c_int64, _P, c_int64, _P, c_int64, c_int, c_int, c_int, _P],
    "mi_gemm_skinny_rope_bf16": [
        _P, c_int64, _P, c_int64, _P, c_int64, _P, _P, _P, _P, _P, c_int, c_int, c_int, c_int, c_int, c_int,
        c_int, c_int, _P,
    ],
    "mi_gemm_skinny_rope_scaled_bf16": [
        _P, c_int64, _P, c_int, c_float, _P, c_int64, _P, c_int64, _P, _P, _P, _P, _P, c_int, c_int, c_int, c_int,
        c_int, c_int, c_int, c_int, _P,
    ],
    "mi_gemm_skinny_bf16_supported": [c_int, c_int, c_int, c_int64, c_int64],
    "mi_gemm_skinny_wide_bf16_supported": [c_int, c_int, c_int, c_int64, c_int64],
    "mi_attn_generic": [
        c_int, _P, c_int64, _P, _P, _P, c_int, _P, _P, _P, c_int64, _P, _P, c_int, c_int, c_int,
        c_int, c_int, c_int, c_float, c_int, c_int, _P, _P,
    ],
    "mi_attn_mfma": [
        _P, c_int64, _P, _P, _P, c_int, _P, _P, c_int, c_int, c_int, _P, c_int64, _P, _P, c_int,
        c_int, c_int, c_int, c_int, c_float, c_int, c_int, c_int, c_int, c_int, c_int, _P,
    ],
    "mi_gemm_skinny_addnorm_pieces": [c_int],
    "mi_gemm_skinny_addnorm_bf16": [
        _P, c_int64, _P, _P, c_int, c_int, c_int, _P, c_int64, _P, c_int64, _P, _P, c_int64, _P, c_int, c_int, c_int, _P,
    ],
    "mi_gemm_skinny_swiglu_scaled_bf16": [_P, c_int64, _P, c_int, c_float, _P, c_int64, _P, c_int64, c_int, c_int, c_int, _P],
    "mi_attn_mfma_tokens_per_tile": [c_int, c_int, c_int],
    "mi_attn_mfma_supported": [c_int, c_int],
    "mi_sample": [c_int, _P, c_int64, c_int, c_int, _P, _P, _P, _P, _P, _P, _P, _P],
    "mi_sample_slots": [c_int, _P, c_int64, c_int, c_int, _P, _P, c_int, _P, _P],
}


def _declare(lib: ctypes.CDLL) -> None:
    lib.mi_last_error.restype = ctypes.c_char_p
    lib.mi_last_error.argtypes = []
    lib.mi_abi_version.restype = c_int
    lib.mi_abi_version.argtypes = []
    for name, argtypes in _SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = c_int
        fn.argtypes = argtypes


def load(rebuild_if_stale: bool = True) -> ctypes.CDLL:
    """The loaded library; built first if there is none (or only a stale one)."""
    global _lib, _lib_path
    if _lib is not None:
        return _lib
    path = _build.find_built(require_fresh=True)
    if path is None:
        stale = _build.find_built(require_fresh=False)
        if stale is None or rebuild_if_stale:
            try:
                path = _build.build()
            except Exception as err:  # noqa: BLE001 - reported as one clear error
                if stale is None:
                    raise ExtensionMissingError(
                        "the HIP library of mini_infer_amd is not built and building it failed: "
                        f"{err}"
                    ) from err
                path = stale
        else:
            path = stale
    try:
        lib = ctypes.CDLL(str(path))
    except OSError as err:
        raise ExtensionMissingError(f"cannot load {path}: {err}") from err
    _declare(lib)
    found = lib.mi_abi_version()
    if found != ABI_VERSION:
        raise ExtensionMissingError(
            f"{path} has ABI version {found}, this package needs {ABI_VERSION}; rebuild it"
        )
    _lib, _lib_path = lib, path
    return lib


def library_path() -> Path | None:
    return _lib_path


def check(status: int) -> None:
    """Raise for a non-zero status of an entry point, with the library's message."""
    if status == 0:
        return
    message = load().mi_last_error().decode(errors="replace")
    if status == -1:
        raise KernelShapeError(message)
    raise RuntimeError(f"HIP kernel call failed ({status}): {message}")
