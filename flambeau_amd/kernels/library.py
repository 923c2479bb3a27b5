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
    "fl_rope_table_ladder": [P, I, I, P, F, P, P],
    "fl_attn_plain": [P, P, P, I, P, P, P, I, I, I, I, I, I, I, F, I, P],
    "fl_silu_mul": [P, I, P, I, I, I, P],
    "fl_feed_tokens": [P, P, P, I, P],
    "fl_argmax": [P, P, I, I, P],
    "fl_sample": [P, P, P, P, I, I, P],
    "fl_sample_filtered": [P, P, P, P, P, P, P, I, I, P, P],
    "fl_sample_penalise": [P, I, I, P, P, P, P, P, P],
    "fl_sample_bias": [P, I, I, P, P, P, P],
    "fl_sample_count": [P, I, I, P, P, P],
    "fl_sample_history": [P, I, I, P, I, P],
}


_functions: dict = {}     # name -> foreign function (of this library, or of a part's own)


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
        if name in _functions:          # a launch function of a part's own library
            continue
        fn = getattr(lib, name)
        fn.argtypes = args
        fn.restype = c_int
    lib._path = str(path)
    _lib = lib
    return lib


def register_signatures(extra: dict, library=None) -> None:
    """Further entry points (tuned kernels register theirs next to their wrappers).  ``library``: a
    ``ctypes.CDLL`` of the caller's own that holds them (a part that brings kernels of its own); such
    launch functions return 0 or an error code and take the stream last, like this library's, and
    become recordable with ``make_recordable``."""
    _SIGNATURES.update(extra)
    if library is not None:
        for name, args in extra.items():
            fn = getattr(library, name)
            fn.argtypes = args
            fn.restype = c_int
            _functions[name] = fn
    elif _lib is not None:
        for name, args in extra.items():
            fn = getattr(_lib, name)
            fn.argtypes = args
            fn.restype = c_int


def recordable(name: str) -> bool:
    """Whether the recorder of step programs knows the launch function ``name``."""
    lib = load()
    lib.fl_program_knows.argtypes = [c_char_p]
    return lib.fl_program_knows(name.encode()) >= 0


def make_recordable(name: str, trampoline) -> None:
    """Make a launch function of another library known to the recorder.  ``trampoline``: a C function
    of that library, ``int (const FlArg* args, hipStream_t stream)``, that calls the launch function
    with the recorded arguments and the stream given (a ctypes function pointer or an address); the
    number of arguments comes from the signature registered under ``name``."""
    lib = load()
    lib.fl_program_register.argtypes = [c_char_p, c_void_p, c_int]
    lib.fl_program_register.restype = c_int
    address = ctypes.cast(trampoline, c_void_p).value if not isinstance(trampoline, int) else trampoline
    if lib.fl_program_register(name.encode(), address, len(_SIGNATURES[name])) != 0:
        raise KernelError(f"make_recordable {name}: {lib.fl_last_error().decode(errors='replace')}")


_recording = None        # the Program that launches are being appended to, or None


def call(name: str, *args) -> None:
    fn = _functions.get(name)
    if fn is None:
        fn = _functions[name] = getattr(load(), name)
    rc = fn(*args)
    if rc != 0:
        raise KernelError(f"{name}: {load().fl_last_error().decode(errors='replace')} (code {rc})")
    if _recording is not None:
        _recording.append(name, args)


class FlArg(ctypes.Union):
    _fields_ = [("p", c_void_p), ("l", c_long), ("i", c_int), ("f", c_float)]


_FIELD = {P: "p", I: "i", F: "f", L: "l"}


class suspended:
    """``with suspended():`` launches made inside run, but are not appended to the program that is
    being recorded (a part that cannot be replayed runs between two recorded stretches)."""

    def __enter__(self):
        global _recording
        self._was = _recording
        _recording = None

    def __exit__(self, *exc):
        global _recording
        _recording = self._was


class Program:
    """A list of launches recorded while they ran, replayed with one foreign call (csrc/program.hip).
    ``with program.recording():`` appends every ``call`` made inside; ``run(stream)`` launches them
    again with the arguments they had.  Whoever keeps a program answers for its arguments still
    being valid: same buffers, same shapes."""

    def __init__(self):
        lib = load()
        if not hasattr(lib, "_program_ready"):
            lib.fl_program_new.restype = c_void_p
            lib.fl_program_new.argtypes = []
            lib.fl_program_free.restype = None
            lib.fl_program_free.argtypes = [c_void_p]
            lib.fl_program_size.restype = c_int
            lib.fl_program_size.argtypes = [c_void_p]
            lib.fl_program_append.restype = c_int
            lib.fl_program_append.argtypes = [c_void_p, c_char_p, ctypes.POINTER(FlArg), c_int]
            lib.fl_program_run.restype = c_int
            lib.fl_program_run.argtypes = [c_void_p, c_void_p, ctypes.POINTER(c_int)]
            lib._program_ready = True
        self._lib = lib
        self._handle = c_void_p(lib.fl_program_new())
        self._failed = c_int(-1)
        self._names: list = []

    def __del__(self):
        try:
            if self._handle:
                self._lib.fl_program_free(self._handle)
                self._handle = None
        except Exception:
            pass

    def __len__(self):
        return len(self._names)

    def names(self) -> list:
        """The launch functions recorded, in order."""
        return list(self._names)

    def append(self, name: str, args) -> None:
        types = _SIGNATURES[name]
        arr = (FlArg * len(types))()
        for slot, t, v in zip(arr, types, args):
            if v is not None:
                setattr(slot, _FIELD[t], v)
        if self._lib.fl_program_append(self._handle, name.encode(), arr, len(types)) != 0:
            raise KernelError(f"recording {name}: {self._lib.fl_last_error().decode(errors='replace')}")
        self._names.append(name)

    def recording(self):
        prog = self

        class _Recording:
            def __enter__(self_inner):
                global _recording
                if _recording is not None:
                    raise KernelError("a program is already being recorded")
                _recording = prog

            def __exit__(self_inner, *exc):
                global _recording
                _recording = None
        return _Recording()

    def run(self, stream: int) -> None:
        rc = self._lib.fl_program_run(self._handle, stream, ctypes.byref(self._failed))
        if rc != 0:
            at = self._failed.value
            name = self._names[at] if 0 <= at < len(self._names) else "?"
            raise KernelError(f"replay of {name} (call {at}): {self._lib.fl_last_error().decode(errors='replace')} (code {rc})")
