"""ctypes binding of libolmax_hip.so — the C-ABI boundary of the HIP hot path.

The library is built in-tree by :mod:`olmax_amd.build`.  There is deliberately no
fallback: if the shared object is missing, or a call returns a non-zero code, an
exception is raised.
"""
from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_double, c_float, c_int32, c_int64, c_void_p
from pathlib import Path

_LIB_PATH = Path(__file__).resolve().parent / "libolmax_hip.so"
_lib = None


class OlmaxHipError(RuntimeError):
    pass


def lib_path() -> Path:
    return _LIB_PATH


def load() -> ctypes.CDLL:
    """Load (once) and return the shared library; raise if it has not been built."""
    global _lib
    if _lib is None:
        if not _LIB_PATH.exists():
            raise OlmaxHipError(
                f"{_LIB_PATH} not found: build it with `python -m olmax_amd.build` "
                "(there is no CPU or eager fallback for the HIP path)"
            )
        _lib = ctypes.CDLL(str(_LIB_PATH))
        _lib.olmax_last_error_string.restype = c_char_p
        _lib.olmax_abi_version.restype = c_int32
    return _lib


def check(rc: int) -> None:
    if rc != 0:
        msg = load().olmax_last_error_string().decode()
        raise OlmaxHipError(f"libolmax_hip error {rc}: {msg}")


def ptr(t) -> c_void_p:
    """Raw device pointer of a torch tensor (None -> NULL)."""
    return c_void_p(0 if t is None else t.data_ptr())


def stream_ptr() -> c_void_p:
    import torch

    return c_void_p(torch.cuda.current_stream().cuda_stream)


i32, i64, f32, f64, vp = c_int32, c_int64, c_float, c_double, c_void_p
