"""Loads the gfx950 kernel library through ctypes and declares its entry points.

There is no fallback: if the library cannot be built or loaded, the first use
raises. ``import torch`` must come first so that the library binds to the HIP
runtime that torch has already loaded.
"""
from __future__ import annotations

import ctypes
import threading
from ctypes import c_char_p, c_float, c_int, c_long, c_void_p
from typing import Optional

import torch  # noqa: F401  (loads the HIP runtime the library links against)

from ..csrc import build as _build

ABI_VERSION = 17


class KernelLibraryError(RuntimeError):
    pass


_lock = threading.Lock()
_lib: Optional[ctypes.CDLL] = None
_lib_path: Optional[str] = None

P, I, F = c_void_p, c_int, c_float

_SIGNATURES = {
    "ra_embed": [P, I, P, P, I, I, P],
    "ra_add_rmsnorm": [P, P, P, I, P, I, P, I, I, F, P],
    "ra_qk_norm_rope_cache": [P, I, P, P, I, F, P, P, I, I, P, P, P, I, I, I, I, I, P],
    "ra_qk_norm_rope_cache_sums": [P, I, P, I, F, I, P, I, I, P, P, I, F, P, P, I, I, P, P, P, I, I, I, I, I, P],
    "ra_gemm_wide_partial": [P, P, P, c_long, I, I, I, I, P],
    "ra_silu_mul": [P, P, I, I, I, I, P],
    "ra_attention_plain": [P, I, P, I, P, P, I, P, I, P, P, P, I, I, I, I, I, F, I, P],
    "ra_attention_decode": [P, I, P, I, P, P, P, I, P, P, P, I, I, I, I, I, F, I, I, I, I, P, P, P],
    "ra_attention_prefill": [P, I, P, I, P, P, P, I, P, I, I, I, I, I, F, I, P],
    "ra_attention_prefill_split": [P, I, P, I, P, P, P, I, P, I, P, P, I, P, P, I, I, I, I, F, I, P],
    "ra_gemm_skinny": [P, P, P, P, I, I, I, I, I, I, I, P],
    "ra_gemm_wide": [P, P, P, P, I, I, I, I, I, I, I, P, c_long, P],
    "ra_gemm_wide_normed": [P, P, P, P, I, I, I, I, I, I, I, P, c_long, P, I, F, I, P, I, P, I, P, F, P],
    "ra_gemm_skinny_normed": [P, P, P, P, I, I, I, I, I, I, I, P, I, F, I, P, I, P, I, P, P],
    "ra_gemm_plain": [P, P, P, P, I, I, I, I, I, I, I, P],
    "ra_sample": [P, I, I, I, P, P, P, P, P, P, P],
    "ra_sample_static": [P, I, I, I, P, P, P, P, P],
    "ra_filter_logits": [P, I, I, I, P, P, P],
    "ra_stream_read": [P, c_long, P, P],
    "ra_mfma_loop": [I, I, I, P, P, P],
}


def load() -> ctypes.CDLL:
    global _lib, _lib_path
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        try:
            path = _build.ensure_built()
        except Exception as e:
            raise KernelLibraryError(f"gfx950 kernel library unavailable: {e}") from e
        try:
            lib = ctypes.CDLL(path)
        except OSError as e:
            raise KernelLibraryError(f"cannot load {path}: {e}") from e
        lib.ra_last_error.restype = c_char_p
        lib.ra_last_error.argtypes = []
        lib.ra_abi_version.restype = c_int
        lib.ra_sample_slices.restype = c_int
        lib.ra_sample_slices.argtypes = [c_int]
        for name in ("ra_attention_decode_supports", "ra_attention_prefill_supports"):
            getattr(lib, name).restype = c_int
            getattr(lib, name).argtypes = [c_int, c_int, c_int, c_int]
        lib.ra_attention_decode_slots.restype = c_int
        lib.ra_attention_decode_slots.argtypes = [c_int, c_int, c_int, c_int]
        for name in ("ra_attention_prefill_tile", "ra_attention_prefill_columns", "ra_attention_prefill_groups"):
            getattr(lib, name).restype = c_int
            getattr(lib, name).argtypes = [c_int, c_int, c_int]
        lib.ra_attention_prefill_part_floats.restype = c_long
        lib.ra_attention_prefill_part_floats.argtypes = [c_int, c_int, c_int, c_int, c_int]
        lib.ra_sample_static_max_pairs.restype = c_long
        lib.ra_sample_static_max_pairs.argtypes = []
        lib.ra_sample_static_prepare.restype = c_int
        lib.ra_sample_static_prepare.argtypes = []
        lib.ra_gemm_skinny_max_rows.restype = c_int
        lib.ra_gemm_skinny_max_rows.argtypes = []
        lib.ra_gemm_skinny_row_parts.restype = c_int
        lib.ra_gemm_skinny_row_parts.argtypes = [c_int, c_int]
        lib.ra_gemm_wide_scratch.restype = c_long
        lib.ra_gemm_wide_scratch.argtypes = [c_int, c_int, c_int, c_int, c_int]
        lib.ra_gemm_wide_row_parts.restype = c_int
        lib.ra_gemm_wide_row_parts.argtypes = [c_int]
        lib.ra_gemm_wide_ranges.restype = c_int
        lib.ra_gemm_wide_ranges.argtypes = [c_int, c_int, c_int]
        lib.ra_gemm_wide_preferred.restype = c_int
        lib.ra_gemm_wide_preferred.argtypes = [c_int, c_int, c_int, c_int]
        if lib.ra_abi_version() != ABI_VERSION:
            raise KernelLibraryError(f"{path}: interface version {lib.ra_abi_version()}, expected {ABI_VERSION}; "
                                     "rebuild with `python -m reinfer_amd.csrc.build`")
        for name, args in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = c_int
            fn.argtypes = args
        _lib, _lib_path = lib, path
        return lib


def loaded_path() -> Optional[str]:
    return _lib_path


def call(name: str, *args) -> None:
    lib = load()
    rc = getattr(lib, name)(*args)
    if rc != 0:
        raise KernelLibraryError(lib.ra_last_error().decode("utf-8", "replace"))
