"""ctypes binding of libcorope_amd.so (the gfx950 kernels behind a C ABI).

The shared library is built in-tree by ``build.py``; nothing here falls back to another implementation: if
the library is missing or a call fails, an exception is raised."""
from __future__ import annotations

import ctypes
import os
import threading

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libcorope_amd.so")
ABI_VERSION = 3

# status codes of include/corope_amd.h
OK, E_BADARG, E_UNSUPPORTED, E_ALIGN, E_LAUNCH = 0, -1, -2, -3, -4

_P, _I, _F, _L = ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_int64

#: name -> (restype, argtypes); every symbol include/corope_amd.h declares
SIGNATURES = {
    "corope_amd_version": (_I, []),
    "corope_amd_last_error": (ctypes.c_char_p, []),
    "corope_rope_attn_check": (_I, [_I, _I, _I, _I, _L, _F, _I]),
    "corope_gqa_check": (_I, [_I, _I, _I, _I, _I, _F, _F]),
    "corope_rope_freqs": (_I, [_P, _P, _I, _I, _I, _L, _I, _F, _P]),
    "corope_rope_attn_fwd": (_I, [_P, _P, _P, _P, _P, _L, _P, _P, _I, _I, _I, _I, _F, _I, _P]),
    "corope_rope_attn_fwd_workspace_bytes": (_L, [_I, _I, _I, _I]),
    "corope_rope_attn_fwd_ws": (_I, [_P, _P, _P, _P, _P, _L, _P, _P, _I, _I, _I, _I, _F, _I, _P, _L, _P]),
    "corope_rope_attn_fwd_noalloc_max_bytes": (_L, []),
    "corope_rope_attn_fwd_noalloc": (_I, [_P, _P, _P, _P, _P, _L, _P, _P, _I, _I, _I, _I, _F, _I, _P]),
    "corope_rope_attn_fwd_prerotated": (_I, [_P, _P, _P, _P, _P, _P, _L, _P, _P, _P, _I, _I, _I, _I, _F, _I, _P]),
    "corope_rope_attn_fwd_train": (_I, [_P, _P, _P, _P, _P, _L, _P, _P, _P, _P, _P, _I, _I, _I, _I, _F, _I, _P]),
    "corope_rope_rotate": (_I, [_P, _P, _P, _L, _P, _P, _I, _I, _I, _I, _F, _P]),
    "corope_rope_attn_bwd_preprocess": (_I, [_P, _P, _P, _I, _I, _I, _I, _P]),
    "corope_rope_attn_bwd_dv": (_I, [_P] * 6 + [_L, _P, _I, _I, _I, _I, _F, _I, _P]),
    "corope_rope_attn_bwd_dk": (_I, [_P] * 8 + [_L, _P, _I, _I, _I, _I, _F, _I, _P]),
    "corope_rope_attn_bwd_dkdv": (_I, [_P] * 8 + [_L, _P, _P, _I, _I, _I, _I, _F, _I, _P]),
    "corope_rope_attn_bwd_dq": (_I, [_P] * 8 + [_L, _P, _I, _I, _I, _I, _F, _I, _P]),
    "corope_rope_attn_bwd": (_I, [_P] * 9 + [_L, _P, _P, _P, _I, _I, _I, _I, _F, _I, _P]),
    "corope_rope_attn_bwd_dv_prerotated": (_I, [_P] * 6 + [_L, _P, _I, _I, _I, _I, _F, _I, _P]),
    "corope_rope_attn_bwd_dk_prerotated": (_I, [_P] * 8 + [_L, _P, _I, _I, _I, _I, _F, _I, _P]),
    "corope_rope_attn_bwd_dkdv_prerotated": (_I, [_P] * 8 + [_L, _P, _P, _I, _I, _I, _I, _F, _I, _P]),
    "corope_rope_attn_bwd_dq_prerotated": (_I, [_P] * 9 + [_L, _P, _I, _I, _I, _I, _F, _I, _P]),
    "corope_rope_attn_bwd_prerotated": (_I, [_P] * 9 + [_L, _P, _P, _P, _I, _I, _I, _I, _F, _I, _P]),
    "corope_rope_attn_bwd_workspace_bytes": (_L, [_I, _I, _I, _I]),
    "corope_rope_attn_bwd_ws": (_I, [_P] * 9 + [_L, _P, _P, _P, _I, _I, _I, _I, _F, _I, _P, _L, _P]),
    "corope_rope_attn_fwd_f16": (_I, [_P, _P, _P, _P, _P, _L, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _F, _I, _P]),
    "corope_rope_attn_bwd_f16": (_I, [_P, _P, _I] + [_P] * 7 + [_L, _P, _P, _P, _I, _I, _I, _I, _I, _F, _I, _P, _L, _P]),
    "corope_rope_attn_fwd_strided": (_I, [_P] * 8 + [_L] + [_P] * 5 + [_I] * 5 + [_F, _I, _I, _P]),
    "corope_rope_attn_fwd_gqa": (_I, [_P] * 5 + [_L] + [_P] * 5 + [_I] * 5 + [_F, _I, _P]),
    "corope_rope_attn_bwd_gqa": (_I, [_P, _P, _I] + [_P] * 7 + [_L, _P, _P, _P] + [_I] * 5 + [_F, _I, _P]),
    "corope_gqa_fwd": (_I, [_P, _P, _P, _P, _I, _I, _I, _I, _I, _F, _F, _P]),
    "corope_gqa_fwd_f16": (_I, [_P, _P, _P, _P, _I, _I, _I, _I, _I, _F, _F, _P]),
    "corope_gqa_bwd_workspace_bytes": (_L, [_I, _I, _I, _I, _I]),
    "corope_gqa_bwd_min_workspace_bytes": (_L, [_I, _I, _I, _I, _I]),
    "corope_gqa_bwd": (_I, [_P] * 8 + [_I] * 5 + [_F, _F, _P, _L, _P]),
    "corope_gqa_bwd_f16": (_I, [_P] * 8 + [_I] * 5 + [_F, _F, _P, _L, _P]),
}

_lock = threading.Lock()
_lib = None


class CoRopeLibraryError(RuntimeError):
    """The native library is missing, stale, or a launch failed."""


def load():
    """Open the shared library once and type its entry points."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIB_PATH):
            raise CoRopeLibraryError(
                f"{LIB_PATH} not found: build it with `python co-rope_amd/build.py` (needs hipcc); "
                "there is no fallback implementation")
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            try:
                fn = getattr(lib, name)
            except AttributeError as e:
                raise CoRopeLibraryError(f"{LIB_PATH} does not export {name}; rebuild it") from e
            fn.restype, fn.argtypes = res, args
        if lib.corope_amd_version() != ABI_VERSION:
            raise CoRopeLibraryError(f"{LIB_PATH} has ABI version {lib.corope_amd_version()}, expected {ABI_VERSION}")
        _lib = lib
    return _lib


TRACE_LIB_PATH = os.path.join(_HERE, "lib", "libcorope_amd_trace.so")
_trace_lib = None


def load_trace():
    """The measurement build of the library (same kernels with time stamps compiled in; made by build.py beside the shipped
    one): every entry point of the shipped library plus ``corope_debug_trace(buf)`` and
    ``corope_debug_set_forms(tile_rows, fwd_wave_rows)``, which forces kernel forms for the tests."""
    global _trace_lib
    if _trace_lib is None:
        if not os.path.exists(TRACE_LIB_PATH):
            raise CoRopeLibraryError(f"{TRACE_LIB_PATH} not found: `python co-rope_amd/build.py` makes it")
        lib = ctypes.CDLL(TRACE_LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        lib.corope_debug_trace.restype, lib.corope_debug_trace.argtypes = None, [_P]
        lib.corope_debug_set_forms.restype, lib.corope_debug_set_forms.argtypes = _I, [_I, _I]
        _trace_lib = lib
    return _trace_lib


class using:
    """Context in which ``load()`` hands out `lib` (e.g. the measurement build) instead of the shipped library."""

    def __init__(self, lib):
        self.lib, self.prev = lib, None

    def __enter__(self):
        global _lib
        load()
        with _lock:
            self.prev, _lib = _lib, self.lib
        return self.lib

    def __exit__(self, *exc):
        global _lib
        with _lock:
            _lib = self.prev
        return False


def last_error():
    return load().corope_amd_last_error().decode("utf-8", "replace")


def check(rc, what):
    """Map a status code to the exception the reference's Python layer would raise for the same mistake."""
    if rc == OK:
        return
    msg = f"{what}: {last_error()} (status {rc})"
    if rc in (E_BADARG, E_UNSUPPORTED, E_ALIGN):
        raise ValueError(msg)
    raise CoRopeLibraryError(msg)
