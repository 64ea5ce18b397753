"""Loading the kernel library and declaring its C interface (csrc/api.h) to ctypes.

There is no fallback: if the library is missing it is built, and if it cannot be
built or loaded the error is raised to the caller.
"""
import ctypes
import threading
from ctypes import c_char_p, c_float, c_int, c_size_t, c_void_p

from . import build as _build

_lock = threading.Lock()
_lib = None

P, I, F = c_void_p, c_int, c_float
_SIGNATURES = {
    "hfa_embed": [P, I, P, P, I, I, I, P],
    "hfa_rmsnorm": [P, P, P, I, P, I, I, F, P, I, P, P],
    "hfa_gemm": [P, I, I, P, I, I, P, P, I, I, I, I, I, I, I, P, c_size_t, I, P, I, P],
    "hfa_gemm_finish": [P, I, P, P, I, I, I, I, I, I, P],
    "hfa_gemm_rows": [I, P, I, P, I, I, I, I, P, P, I, F, F, P, I, I, P, I, P, P, P, I, P, I, P],
    "hfa_gemm_rows_supports": [I, I, I, I, I, I],
    "hfa_rope_store": [P, I, I, P, P, I, I, I, I, I, P, P, P, I, I, P, I, P, P],
    "hfa_paged_attention": [P, I, I, P, P, I, I, P, I, P, P, P, I, I, I, P, I, I, I, I, I, I, I, I, F, P, P, c_size_t, I, P],
    "hfa_rope_table": [P, P, I, P, I, P],
    "hfa_decode_attention_supports": [I, I, I, I, I, I, I, I],
    "hfa_decode_attention": [P, I, P, P, P, I, P, P, I, P, P, P, I, I, P, I, I, I, I, I, I, F, P, c_size_t, P],
    "hfa_swiglu": [P, P, I, I, I, P],
    "hfa_scatter_i32": [P, P, P, I, P],
    "hfa_move_i32": [P, P, P, P, I, P],
    "hfa_argmax": [P, I, P, I, I, P, c_size_t, P],
    "hfa_argmax_static": [P, I, P, I, I, P],
    "hfa_topk": [P, I, P, P, P, I, I, I, P],
    "hfa_order_rows": [P, I, P, P, P, I, I, P, c_size_t, P],
    "hfa_draw_rows": [P, P, I, I, P, P, P, P],
    "hfa_random_fill": [P, I, c_size_t, ctypes.c_uint64, F, I, I, P],
    "hfa_probe_read": [P, c_size_t, P, I, P],
    "hfa_probe_copy": [P, P, c_size_t, P],
    "hfa_probe_mfma": [P, I, I, P, P],
}


def library():
    """The loaded library (built first if there is none, or if its sources changed)."""
    global _lib
    with _lock:
        if _lib is None:
            path, current = _build.find_library()
            if path is None or not current:
                path = _build.build()
            lib = ctypes.CDLL(path)
            lib.hfa_last_error.restype = c_char_p
            lib.hfa_last_error.argtypes = []
            lib.hfa_version.restype = c_int
            lib.hfa_order_rows_scratch.restype = c_size_t
            lib.hfa_order_rows_scratch.argtypes = [c_int, c_int]
            lib.hfa_gemm_rows_parts.restype = c_int
            lib.hfa_gemm_rows_parts.argtypes = []
            lib.hfa_probe_mfma_threads.restype = c_int
            lib.hfa_probe_mfma_threads.argtypes = []
            lib.hfa_attention_prompt_rows.restype = c_int
            lib.hfa_attention_prompt_rows.argtypes = []
            for name, args in _SIGNATURES.items():
                fn = getattr(lib, name)
                fn.argtypes = args
                fn.restype = c_int
            lib.path = path
            _lib = lib
        return _lib


def load_extension(path, signatures):
    """A shared library with kernels of a part that is not the package's: ``signatures`` maps each
    entry point to its ctypes argument types (the stream last; it returns an int, 0 = done).
    The part calls them through ``Ops.call``."""
    lib = ctypes.CDLL(path)
    for name, args in signatures.items():
        fn = getattr(lib, name)
        fn.argtypes = list(args)
        fn.restype = c_int
    lib.path = path
    return lib


def last_error():
    return library().hfa_last_error().decode("utf-8", "replace")
