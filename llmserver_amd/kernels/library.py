"""Loads the compiled kernel libraries through ctypes and declares their entry points."""
from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_float, c_int, c_long, c_void_p
from typing import Dict

from . import build

_P = c_void_p
_SIGNATURES = {
    "lsa_embedding": [c_int, _P, _P, _P, c_int, c_int, c_int, _P],
    "lsa_add_rmsnorm": [c_int, _P, _P, _P, c_float, _P, _P, c_int, c_int, _P],
    "lsa_add_rmsnorm_partial_sums": [c_int, _P, _P, c_int, c_long, _P, c_float, _P, _P, c_int, c_int, _P],
    "lsa_swiglu": [c_int, _P, _P, c_int, c_int, _P],
    "lsa_add_bias": [c_int, _P, _P, c_int, c_int, _P],
    "lsa_plain_read": [_P, _P, c_long, c_int, c_int, _P],
    "lsa_qk_norm_rope_kv_write": [c_int, _P, _P, _P, _P, c_int, _P, _P, _P, _P, c_float, _P, c_int, c_int, c_int, c_int,
                                  c_int, c_int, _P],
    "lsa_rotary_table": [_P, _P, _P, c_int, c_int, _P],
    "lsa_sample": [_P, _P, _P, _P, _P, c_int, c_int, _P],
    "lsa_sample_chunks": [c_int],
    "lsa_sample_static": [_P, _P, _P, _P, c_int, c_int, _P],
    "lsa_sample_static_max_rows": [],
    "lsa_sample_static_error": [c_int],
    "lsa_paged_attention": [_P, c_long, _P, _P, _P, _P, c_int, _P, _P, _P, _P, _P, c_int, _P, c_int, c_int, _P, _P, _P, _P, c_int,
                            c_float, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, _P, _P, c_float, _P, c_int, c_int, c_int, _P],
    "lsa_attention_workgroup_tiles": [],
    "lsa_attention_tile_page_multiple": [],
    "lsa_attention_tile_halves": [],
    "lsa_attention_most_splits": [],
    "lsa_attention_tile_key_ranges": [],
    "lsa_attention_head_dim": [],
    "lsa_attention_is_bf16": [],
    "lsa_gemm_skinny": [c_int, _P, _P, _P, c_int, c_int, c_int, c_int, _P, c_int, c_float, _P, _P],
    "lsa_gemm_skinny_parts": [c_int, c_int, c_int],
    "lsa_gemm_skinny_stream": [_P, _P, c_int, c_int, c_int, c_int, _P, c_int, c_float, _P, _P, _P, _P, _P, _P],
    "lsa_gemm_skinny_gated": [_P, _P, _P, c_int, c_int, c_int, c_int, _P, c_int, c_float, _P],
    "lsa_gemm_split_parts": [c_int, c_int, c_int],
    "lsa_gemm_split": [_P, _P, _P, c_int, c_int, c_int, _P],
    "lsa_gemm_split_gated_fits": [c_int, c_int, c_int],
    "lsa_gemm_split_gated": [_P, _P, _P, c_int, c_int, c_int, _P],
}

_RESULT_TYPES = {"lsa_sample_static_error": c_char_p}      # every other entry point returns an int (0 or an error code)

_loaded: Dict[str, ctypes.CDLL] = {}


class KernelLibraryMissing(RuntimeError):
    """The HIP extension is not there and cannot be built: the engine does not run without it."""


def load(name: str) -> ctypes.CDLL:
    """The named library, compiled first if it is not there yet.  Fails loudly; there is no fallback."""
    if name in _loaded:
        return _loaded[name]
    try:
        path = build.build([name])[name]
    except build.KernelBuildError as error:
        raise KernelLibraryMissing(f"HIP kernel library {name!r} is missing and could not be built: {error}") from error
    library = ctypes.CDLL(path)
    for symbol, argtypes in _SIGNATURES.items():
        if hasattr(library, symbol):
            function = getattr(library, symbol)
            function.argtypes = argtypes
            function.restype = _RESULT_TYPES.get(symbol, c_int)
    _loaded[name] = library
    return library


def preload(names) -> None:
    """Compile what is missing in one go (in parallel), then load."""
    build.build(list(names))
    for name in names:
        load(name)


def loaded_libraries():
    return {name: library._name for name, library in _loaded.items()}
