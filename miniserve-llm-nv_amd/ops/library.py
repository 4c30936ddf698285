"""Loads the HIP library through ctypes and declares every entry point.

There is no fallback: when the library cannot be found or built, or an entry
point reports an error, the call raises.
"""

from __future__ import annotations

import ctypes
import sys
import threading
from ctypes import c_char_p, c_float, c_int, c_size_t, c_void_p

from . import build as _build


class KernelError(RuntimeError):
    """An entry point of the HIP library refused its arguments or its launch."""


_P, _I, _F = c_void_p, c_int, c_float

# name -> argument types (the trailing stream argument included).
_SIGNATURES: dict[str, list] = {
    "ms_embedding_gather": [_P, _P, _P, _I, _I, _I, _I, _P],
    "ms_rmsnorm": [_P, _P, _P, _P, _P, _I, _I, _F, _I, _I, _I, _P],
    "ms_residual_add": [_P, _P, _I, _I, _I, _P],
    "ms_rope_table": [_P, _P, _P, _P, _I, _I, _P],
    "ms_qk_norm_rope_append": [_P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _F, _I, _P],
    "ms_attention_generic": [_P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _F, _I, _I, _P],
    "ms_attention_decode": [_P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _F, _I, _I, _P],
    "ms_attention_decode_supported": [_I, _I],
    "ms_attention_prefill": [_P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _F, _I, _P],
    "ms_attention_prefill_supported": [_I, _I],
    "ms_gemm_f32": [_P, _P, _P, _I, _I, _I, _I, _P],
    "ms_gemm_skinny": [_P, _P, _P, _P, _I, _I, _I, _I, _P],
    "ms_gemm_skinny_supported": [_I, _I, _I, _I],
    "ms_gemm_skinny_groups": [_I, _I],
    "ms_gemm_skinny_norm_ahead": [_P, _P, _P, _I, _I, _I, _P, _P, _P, _P],
    "ms_gemm_skinny_scaled": [_P, _P, _P, _P, _I, _I, _I, _I, _P, _I, _F, _P],
    "ms_gemm_skinny_normed": [_P, _P, _F, _P, _P, _I, _I, _I, _I, _P],
    "ms_gemm_library_open": [c_char_p],
    "ms_gemm_library": [_P, _P, _P, _I, _I, _I, _I, _I, _P, c_size_t, _P],
    "ms_gemm_library_pin": [_I, _I, _I, _I, _I],
    "ms_gemm_library_bucket": [_I],
    "ms_gemm_library_time": [_P, _P, _P, _I, _I, _I, _I, _P, c_size_t, _P, c_size_t, _P, _P, _I, _P, _P],
    "ms_silu_mul": [_P, _P, _I, _I, _I, _P],
    "ms_device_compute_units": [],
    "ms_sample_rows": [_P, _P, _P, _P, _P, _P, _I, _I, _P],
    "ms_argmax_rows": [_P, _P, _P, _P, _I, _I, _I, _P],
    "ms_sample_rows_workspace_bytes": [_I, _I],
    "ms_sample_rows_chunked": [_P, _P, _P, _P, _P, _P, _P, c_size_t, _I, _I, _I, _P],
}

_lock = threading.Lock()
_library: ctypes.CDLL | None = None
_library_path: str | None = None


def _declare(lib: ctypes.CDLL) -> None:
    lib.ms_last_error.restype = c_char_p
    lib.ms_last_error.argtypes = []
    lib.ms_target_arch.restype = c_char_p
    lib.ms_target_arch.argtypes = []
    for name, argtypes in _SIGNATURES.items():
        try:
            function = getattr(lib, name)
        except AttributeError:
            raise KernelError(
                f"{_library_path} lacks the entry point {name}; rebuild it "
                "(python -c 'import __graft_entry__ as g; g.build()')."
            ) from None
        function.restype = c_int
        function.argtypes = argtypes
    lib.ms_sample_rows_workspace_bytes.restype = c_size_t      # a size, not a status


def load() -> ctypes.CDLL:
    """The loaded library.  What is built is loaded; it is compiled, with progress
    lines on stderr, only when nothing is built or what is built does not match
    the sources."""

    global _library, _library_path
    if _library is not None:
        return _library
    with _lock:
        if _library is not None:
            return _library
        path = _build.find_built_library()
        if path is None:
            path = _build.build(force=True)
        elif _build.is_stale(path):
            # A library that does not match its sources may disagree with the Python
            # side about argument types; it is never run.
            print(f"[miniserve_amd] {path} does not match its sources; rebuilding.", file=sys.stderr, flush=True)
            path = _build.build(force=True)
        _library_path = str(path)
        try:
            lib = ctypes.CDLL(_library_path)
        except OSError as exc:
            raise KernelError(f"cannot load {_library_path}: {exc}") from exc
        _declare(lib)
        _library = lib
    return _library


def library_path() -> str | None:
    return _library_path


def call(name: str, *args) -> None:
    lib = load()
    status = getattr(lib, name)(*args)
    if status != 0:
        raise KernelError(lib.ms_last_error().decode("utf-8", "replace"))
