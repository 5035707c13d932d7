"""Kernel-variant overrides for tests and benchmarks.

``with override(prefill_tile=21): ...`` makes every op called inside the block on this thread pass a ``VaqTuning`` with
those fields to the library's ``*_tuned`` entry points.  The library itself keeps no tuning state: the struct travels
with each call, and leaving the block (normally or through an exception) restores the previous override.
"""
from __future__ import annotations

import contextlib
import ctypes
import threading

from ._lib import VaqTuning

_state = threading.local()


def current() -> VaqTuning | None:
    """The override active on this thread, or None (= the plain entry points, automatic choices)."""
    return getattr(_state, "tuning", None)


def current_ref():
    t = current()
    return None if t is None else ctypes.byref(t)


@contextlib.contextmanager
def override(**fields):
    """Fields of ``VaqTuning`` by name (``exp`` takes a sequence of up to 15 ints); unnamed fields are 0 = automatic."""
    t = VaqTuning()
    for name, value in fields.items():
        if name == "exp":
            for i, v in enumerate(value):
                t.exp[i] = int(v)
        elif not hasattr(t, name):
            raise TypeError(f"VaqTuning has no field {name!r}")
        else:
            setattr(t, name, int(value))
    prev = current()
    _state.tuning = t
    try:
        yield t
    finally:
        _state.tuning = prev
