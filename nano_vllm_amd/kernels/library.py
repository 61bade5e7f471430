"""Loads the compiled kernel libraries with ctypes and calls their entry points.

Every entry point takes raw device pointers, sizes and a hipStream_t and returns 0 or a
negative code; the message of a refusal is fetched from the library and raised as
KernelError.  There is no fallback: a library that cannot be built or loaded is an error.
"""
from __future__ import annotations

import ctypes
from typing import Dict, Optional, Tuple

from . import build


class KernelError(RuntimeError):
    pass


_LAST_ERROR_SYMBOL = {
    "embed": "nva_embed_last_error", "norm": "nva_norm_last_error",
    "activation": "nva_activation_last_error", "rope": "nva_rope_last_error",
    "attn_generic": "nva_attn_generic_last_error", "gemm": "nva_gemm_last_error",
    "sample": "nva_sample_last_error", "attn_decode": "nva_attn_decode_last_error",
    "gemm_skinny": "nva_gemm_skinny_last_error", "gemm_team": "nva_gemm_team_last_error",
    "attn_prefill": "nva_attn_prefill_last_error", "gemm_tile": "nva_gemm_tile_last_error",
}

_loaded: Dict[Tuple[str, Optional[str]], ctypes.CDLL] = {}


def load(module: str, dtype: Optional[str]) -> ctypes.CDLL:
    key = (module, dtype)
    lib = _loaded.get(key)
    if lib is None:
        path = build.ensure_built([key])[key]
        try:
            lib = ctypes.CDLL(path)
        except OSError as e:
            raise KernelError(f"cannot load kernel library {path}: {e}") from e
        getattr(lib, _LAST_ERROR_SYMBOL[module]).restype = ctypes.c_char_p
        _loaded[key] = lib
    return lib


def preload(dtype: str, quiet: bool = False) -> None:
    """Builds (in parallel) and loads everything a model of this element type calls."""
    targets = build.targets_for(dtype)
    build.ensure_built(targets, quiet=quiet)
    for m, d in targets:
        load(m, d)


def call(module: str, dtype: Optional[str], symbol: str, *args) -> None:
    lib = load(module, dtype)
    name = f"{symbol}_{dtype}" if dtype else symbol
    fn = getattr(lib, name)
    fn.restype = ctypes.c_int
    rc = fn(*args)
    if rc != 0:
        msg = getattr(lib, _LAST_ERROR_SYMBOL[module])()
        raise KernelError(f"{name}: {msg.decode() if msg else 'error ' + str(rc)}")


def loaded_libraries():
    return {k: lib._name for k, lib in _loaded.items()}
