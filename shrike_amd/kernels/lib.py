"""Loads libshrike_hip.so (building it when it is absent) and declares its
entry points for ctypes.  There is no fallback: without the library nothing
in the product path runs."""

from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_float, c_int, c_longlong, c_void_p

_LIB = None


class KernelError(RuntimeError):
    """A launcher refused its arguments or a launch failed."""


_P, _I, _F = c_void_p, c_int, c_float

_SIGNATURES = {
    "shk_copy_words": [_P, _P, _I, _P, _I, _I, _P],
    "shk_gather_rows": [_P, c_longlong, _I, _P, _P, _I, _I, _P],
    "shk_zero_bytes": [_P, c_longlong, _P],
    "shk_embed": [_P, _I, _P, _P, _I, _I, _I, _P],
    "shk_add_rmsnorm": [_P, _P, _P, _F, _P, _I, _P, _I, _I, _I, _I, _I, _P],
    "shk_act_mul": [_P, _P, _I, _I, _I, _I, _P],
    "shk_gemm": [_P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _P],
    "shk_retile_weight": [_P, _I, _I, _P, _P],
    "shk_interleave_gate_up": [_P, _P, _I, _I, _P, _P],
    "shk_gemm_bf16_tiled_weight": [_P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _I, _P],
    "shk_gemm_bf16_splits": [_I, _I, _I],
    "shk_gemm_bf16_parts": [_I, _I, _I, _I],
    "shk_mfma_alone": [_P, _P, _I, _I, _P],
    "shk_rope_kv_store": [_P, _I, _I, _I, _I, _I, _I, _P, _P, _P, _P, _I, _P, _P, _I, _I, _I, _P, _I, _P, _P],
    "shk_attention": [_P, _I, _P, _I, _I, _I, _I, _I, _P, _P, _P, _I, _I, _P, _P, _I, _I, _I, _F, _P],
    "shk_attention_supports_mfma": [_I, _I, _I, _I, _I],
    "shk_attention_decode_bf16": [_P, _I, _P, _I, _I, _I, _I, _P, _P, _I, _P, _P, _I, _I, _F, _P, _I, _I, _P],
    "shk_attention_prefill_bf16": [_P, _I, _P, _I, _I, _I, _I, _P, _P, _P, _P, _P, _I, _P, _P, _I, _I, _F, _P],
    "shk_attention_prefill_shared_tiles": [_I, _I, _I, _I],
    "shk_attention_prefill_shared_bf16": [_P, _I, _P, _I, _I, _I, _I, _P, _P, _P, _P, _P, _I, _P, _P, _I, _I, _F, _I,
                                          _P, _I, _I, _I, _P],
    "shk_argmax": [_P, _P, _I, _I, _I, _P, _P],
    "shk_argmax_scratch_floats": [_I, _I],
    "shk_sample": [_P, _P, _P, _P, _P, _P, c_longlong, _I, _I, _I, _I, _P],
}


def load():
    """The loaded library; compiles it first if no built copy matches the sources."""
    global _LIB
    if _LIB is None:
        from ..csrc.build import ensure_built

        path = ensure_built()
        lib = ctypes.CDLL(str(path))
        lib.shk_last_error.restype = c_char_p
        lib.shk_last_error.argtypes = []
        lib.shk_version.restype = c_int
        for name, argtypes in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.argtypes = argtypes
            fn.restype = c_int
        lib.shk_sample_scratch_floats.argtypes = [_I, _I]
        lib.shk_sample_scratch_floats.restype = c_longlong
        lib._path = str(path)
        _LIB = lib
    return _LIB


def check(status: int) -> None:
    if status != 0:
        raise KernelError(load().shk_last_error().decode())
