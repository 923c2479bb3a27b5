"""Kernel sets: what a kind of part needs from the device beyond matrix products, in the forms a
runtime can have (plain kernels for the 32-bit path, tuned ones for bfloat16).

A part asks its runtime for its set by name (``rt.kernels("paged_attention")``) and calls the
set's methods; it never asks whether kernels are tuned.  The runtime knows no set: a new kind of
mixer registers its own beside its wrappers, ``register_kernel_set(name, Plain, Tuned)``, and
nothing in ``engine/`` changes.  A set is made once per runtime, with the runtime as its only
argument."""
from __future__ import annotations

_SETS: dict = {}


def register_kernel_set(name: str, plain, tuned=None) -> None:
    """``plain(rt)`` serves every runtime, ``tuned(rt)`` (if given) those whose ``rt.tuned`` is set."""
    _SETS[name] = (plain, tuned)


def make_kernel_set(name: str, rt):
    try:
        plain, tuned = _SETS[name]
    except KeyError:
        raise KeyError(f"unknown kernel set '{name}'; known: {', '.join(sorted(_SETS)) or '(none)'}") from None
    return (tuned if rt.tuned and tuned is not None else plain)(rt)


def known_kernel_sets():
    return sorted(_SETS)
