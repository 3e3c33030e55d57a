"""Loads libshrike_hip.so (building it when it is absent) and declares its
entry points for ctypes.  There is no fallback: without the library nothing
in the product path runs.

The launchers can be recorded: between `begin_recording()` and `end_recording()`
every launch is also noted as (launcher, arguments), and the `CallList` that
comes back runs the same launches again with one call into the library
(`shk_run_calls`), on whatever stream is current then."""

from __future__ import annotations

import ctypes
import struct
from ctypes import c_char_p, c_float, c_int, c_longlong, c_void_p

_LIB = None
_RECORDING: list | None = None  # (launcher id, argument tuple) while a step is being recorded
CALL_MAX_ARGS = 26


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


class _Call(ctypes.Structure):
    _fields_ = [("launcher", ctypes.c_int32), ("reserved", ctypes.c_int32),
                ("args", ctypes.c_int64 * CALL_MAX_ARGS)]


def _recorded(fn, launcher_id: int):
    """`fn` with a note of every call while a recording is open."""

    def launch(*args):
        if _RECORDING is not None:
            _RECORDING.append((launcher_id, args))
        return fn(*args)

    return launch


class _Library:
    """The entry points by name: the ctypes functions, those that launch on a
    stream wrapped so that they can be recorded."""


def load():
    """The loaded library; compiles it first if no built copy matches the sources."""
    global _LIB
    if _LIB is None:
        from ..csrc.build import ensure_built

        path = ensure_built()
        raw = ctypes.CDLL(str(path))
        lib = _Library()
        raw.shk_last_error.restype = c_char_p
        raw.shk_last_error.argtypes = []
        raw.shk_version.restype = c_int
        raw.shk_call_id.argtypes = [c_char_p]
        raw.shk_call_id.restype = c_int
        raw.shk_run_calls.argtypes = [_P, _I, _P]
        raw.shk_run_calls.restype = c_int
        lib.shk_last_error, lib.shk_version, lib.shk_run_calls = raw.shk_last_error, raw.shk_version, raw.shk_run_calls
        lib._float_slots = {}
        for name, argtypes in _SIGNATURES.items():
            fn = getattr(raw, name)
            fn.argtypes = argtypes
            fn.restype = c_int
            launcher_id = raw.shk_call_id(name.encode())
            if launcher_id >= 0:
                lib._float_slots[launcher_id] = tuple(i for i, t in enumerate(argtypes) if t is c_float)
                fn = _recorded(fn, launcher_id)
            setattr(lib, name, fn)
        raw.shk_sample_scratch_floats.argtypes = [_I, _I]
        raw.shk_sample_scratch_floats.restype = c_longlong
        lib.shk_sample_scratch_floats = raw.shk_sample_scratch_floats
        lib._path = str(path)
        _LIB = lib
    return _LIB


class CallList:
    """The launches of one recording, laid out for shk_run_calls."""

    def __init__(self, calls: list):
        lib = load()
        self.count = len(calls)
        self._array = (_Call * max(1, self.count))()
        for slot, (launcher_id, args) in zip(self._array, calls):
            if len(args) > CALL_MAX_ARGS:
                raise KernelError(f"a launch with {len(args)} arguments does not fit a recorded call")
            slot.launcher = launcher_id
            floats = lib._float_slots[launcher_id]
            for i, a in enumerate(args):
                if i in floats:
                    slot.args[i] = struct.unpack("<I", struct.pack("<f", a.value if isinstance(a, c_float) else a))[0]
                elif a is None:
                    slot.args[i] = 0
                else:
                    slot.args[i] = int(a.value if hasattr(a, "value") else a)
        self._run = lib.shk_run_calls

    def run(self, stream: int) -> None:
        """All the recorded launches again, in order, on `stream`."""
        check(self._run(self._array, self.count, stream))


def begin_recording() -> None:
    global _RECORDING
    if _RECORDING is not None:
        raise KernelError("a recording of launches is already open")
    load()
    _RECORDING = []


def end_recording(keep: bool = True) -> CallList | None:
    """Closes the recording; the list of its launches, or None with keep=False
    (the step failed, or turned out not to be worth keeping)."""
    global _RECORDING
    calls, _RECORDING = _RECORDING, None
    if calls is None:
        raise KernelError("no recording of launches is open")
    return CallList(calls) if keep else None


def check(status: int) -> None:
    if status != 0:
        raise KernelError(load().shk_last_error().decode())
