"""Loading the compiled HIP kernels and declaring their C signatures.

There is no fallback: if the library is missing it is compiled, and if that fails, or
the device is not a gfx950, the error is raised to the caller.
"""
from __future__ import annotations

import ctypes
import threading
from ctypes import c_char_p, c_float, c_int, c_longlong, c_void_p
from pathlib import Path
from typing import Optional

from ..csrc import build as _build


class KernelError(RuntimeError):
    """A kernel entry point refused its arguments, or its launch failed."""


_lock = threading.Lock()
_lib: Optional[ctypes.CDLL] = None
_lib_path: Optional[Path] = None

P, I, F, L = c_void_p, c_int, c_float, c_longlong

_SIGNATURES = {
    "pylon_embed": [P, P, I, P, P, I, I, I, F, P],
    "pylon_rmsnorm": [P, I, P, I, P, P, I, I, F, P],
    "pylon_add_rmsnorm": [P, I, P, P, I, I, L, P, P, I, I, F, P],
    "pylon_residual_add": [P, P, I, L, P],
    "pylon_silu_gate": [P, I, P, I, I, I, P],
    "pylon_qkv_prepare": [P, P, P, P, I, L, P, P, F, P, I, P, P, I, I, I, I, I, P],
    "pylon_paged_attention": [P, P, P, P, I, P, I, P, P, I, I, I, I, I, I, F, P],
    "pylon_attention_decode": [P, P, P, P, P, I, P, P, I, I, I, I, I, I, F, I, I, P, L, P],
    "pylon_attention_decode_fused": [P, P, L, I, L, P, P, F, P, P, P, P, P, I, P, P, I, I, I, I, I, I, F, I, I, P, L, P],
    "pylon_attention_prefill": [P, P, P, P, P, I, P, I, I, I, I, I, I, F, I, P],
    "pylon_gemm_tiled": [P, I, P, I, P, I, I, I, I, L, L, L, P],
    "pylon_gemm_skinny": [P, I, P, P, I, I, I, L, L, L, I, L, I, P],
    "pylon_gemm_rows": [P, I, P, P, I, I, I, L, L, L, I, L, I, I, I, I, P],
    "pylon_gemm_rows_shape": [I, I, I, I, I, I, I, I, P],
    "pylon_argmax": [P, P, I, I, L, P, P, P, L, P],
    "pylon_argmax_static": [P, P, I, I, L, P, P, P],
    "pylon_probe_read": [P, L, P, P],
    "pylon_sample": [P, P, I, I, L, P, P, P, P, P, P],
}


def _declare(lib: ctypes.CDLL) -> None:
    lib.pylon_last_error.restype = c_char_p
    lib.pylon_last_error.argtypes = []
    lib.pylon_abi_version.restype = c_int
    lib.pylon_check_device.restype = c_int
    lib.pylon_compute_units.restype = c_int
    lib.pylon_compute_units.argtypes = []
    for name, argtypes in _SIGNATURES.items():
        fn = getattr(lib, name, None)
        if fn is None:
            continue
        fn.argtypes = argtypes
        fn.restype = c_int


def register_signature(name: str, argtypes) -> None:
    """Declare one more entry point (used by kernel files added later)."""
    _SIGNATURES[name] = list(argtypes)
    if _lib is not None and hasattr(_lib, name):
        fn = getattr(_lib, name)
        fn.argtypes = list(argtypes)
        fn.restype = c_int


def library_path() -> Optional[Path]:
    return _lib_path


def load(*, quiet: bool = False) -> ctypes.CDLL:
    """The kernel library, compiled first if no current build exists."""
    global _lib, _lib_path
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        path = _build.ensure_built(quiet=quiet)
        lib = ctypes.CDLL(str(path))
        _declare(lib)
        _lib, _lib_path = lib, path
    return _lib


def call(name: str, *args) -> None:
    lib = load()
    fn = getattr(lib, name, None)
    if fn is None:
        raise KernelError(f"the kernel library {_lib_path} has no entry point {name}")
    status = fn(*args)
    if status != 0:
        raise KernelError(lib.pylon_last_error().decode(errors="replace"))


def check_device() -> None:
    lib = load()
    if lib.pylon_check_device() != 0:
        raise KernelError(lib.pylon_last_error().decode(errors="replace"))


_units: Optional[int] = None


def compute_units() -> int:
    """Compute units of the current device, asked of the runtime once."""
    global _units
    if _units is None:
        units = load().pylon_compute_units()
        if units <= 0:
            raise KernelError("the number of compute units of the device is unknown (no GPU?)")
        _units = units
    return _units
