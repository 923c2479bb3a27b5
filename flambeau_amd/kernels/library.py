"""Loading of the HIP kernel library through ctypes.

There is no fallback: a missing library is compiled at first use, and when that is
not possible the import of any kernel raises.  The reference does the same with its
code objects: every kernel module is loaded at start-up and a missing one is an
error (crates/ops/src/hip/mod.rs:40-48).
"""
from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_float, c_int, c_long, c_void_p

_lib = None

P, I, F, L = c_void_p, c_int, c_float, c_long

# name -> argument types (all return int)
_SIGNATURES = {
    "fl_embed": [P, I, P, P, I, I, I, P],
    "fl_rmsnorm": [P, P, P, P, P, P, I, I, I, F, P],
    "fl_add_inplace": [P, P, L, P],
    "fl_gemm_plain": [P, P, P, I, I, I, I, I, P],
    "fl_rope_kv_write": [P, I, I, P, P, P, I, P, P, I, I, I, I, I, I, I, I, F, I, P, I, I, L, P],
    "fl_rope_table": [P, I, I, F, P, P],
    "fl_attn_plain": [P, P, P, I, P, P, P, I, I, I, I, I, I, I, F, I, P],
    "fl_silu_mul": [P, I, P, I, I, I, P],
    "fl_feed_tokens": [P, P, P, I, P],
    "fl_argmax": [P, P, I, I, P],
    "fl_sample": [P, P, P, P, I, I, P],
}


class KernelError(RuntimeError):
    """A kernel refused its arguments or its launch failed."""


def load():
    """The loaded library (compiled first if no library of the current sources exists)."""
    global _lib
    if _lib is not None:
        return _lib
    from ..csrc import build as _build
    path = _build.build(force=False)
    lib = ctypes.CDLL(str(path))
    lib.fl_last_error.restype = c_char_p
    lib.fl_last_error.argtypes = []
    lib.fl_abi_version.restype = c_int
    for name, args in _SIGNATURES.items():
        fn = getattr(lib, name)
        fn.argtypes = args
        fn.restype = c_int
    lib._path = str(path)
    _lib = lib
    return lib


def register_signatures(extra: dict) -> None:
    """Further entry points (tuned kernels register theirs next to their wrappers)."""
    _SIGNATURES.update(extra)
    if _lib is not None:
        for name, args in extra.items():
            fn = getattr(_lib, name)
            fn.argtypes = args
            fn.restype = c_int


_functions: dict = {}


def call(name: str, *args) -> None:
    fn = _functions.get(name)
    if fn is None:
        fn = _functions[name] = getattr(load(), name)
    rc = fn(*args)
    if rc != 0:
        raise KernelError(f"{name}: {load().fl_last_error().decode(errors='replace')} (code {rc})")
