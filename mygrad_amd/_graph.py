"""Graph-tracking switch and the read-only guard on arrays of a live graph.

A compact counterpart of the reference's ``mygrad/_utils/graph_tracking.py``
and ``mygrad/_utils/lock_management.py``: while an operation that read or
produced an array is alive, the array is not writeable; writeability comes back
when the last such operation is released (``Tensor.backward`` /
``Tensor.clear_graph`` drop the operations).  That invariant is also what makes
the cached device copy of an array trustworthy, so releasing an array tells
the device-mirror cache.
"""

import contextlib
import functools
import weakref

import numpy as np

from . import _device

TRACK_GRAPH = True
MEM_GUARD = True

# id(arr) -> [weakref(arr), number of live ops holding it, writeable before the first lock]
_held = {}


class _Switch(contextlib.ContextDecorator):
    """Context manager / decorator that sets a module flag and restores it."""

    def __init__(self, name, value):
        self._name, self._value, self._saved = name, value, []

    def __call__(self, func):
        @functools.wraps(func)
        def wrapped(*args, **kwargs):
            with type(self)(self._name, self._value):
                return func(*args, **kwargs)

        return wrapped

    def __enter__(self):
        self._saved.append(globals()[self._name])
        globals()[self._name] = self._value
        return self

    def __exit__(self, *exc):
        globals()[self._name] = self._saved.pop()
        return False


no_autodiff = _Switch("TRACK_GRAPH", False)
mem_guard_off = _Switch("MEM_GUARD", False)
mem_guard_on = _Switch("MEM_GUARD", True)


def _forget(key):
    _held.pop(key, None)


def lock(arr):
    """Make ``arr`` read-only on behalf of one more operation; returns a weakref."""
    key = id(arr)
    entry = _held.get(key)
    if entry is None or entry[0]() is not arr:
        ref = weakref.ref(arr, lambda _r, key=key: _forget(key))
        entry = _held[key] = [ref, 0, bool(arr.flags.writeable)]
    entry[1] += 1
    if arr.flags.writeable:
        arr.flags.writeable = False
    _device.note_locked(arr)
    return entry[0]


def release(refs):
    """Undo one ``lock`` for every still-living array in ``refs``.

    Arrays are released bases first is not required here: NumPy only refuses to
    make a view writeable while its base is read-only, so the list is processed
    twice, owners before views."""
    alive = [r() for r in refs]
    alive = [a for a in alive if a is not None]
    pending = []
    for arr in alive:
        entry = _held.get(id(arr))
        if entry is None or entry[0]() is not arr:
            continue
        entry[1] -= 1
        _device.note_released(arr)
        if entry[1] <= 0:
            del _held[id(arr)]
            if entry[2]:
                pending.append(arr)
    # owners first, then views of them
    pending.sort(key=lambda a: 0 if a.base is None or not isinstance(a.base, np.ndarray) else 1)
    for arr in pending:
        try:
            arr.flags.writeable = True
        except ValueError:  # base still held by another live graph
            pass


def arrays_and_bases(tensors):
    """Each tensor's host array, preceded by its ndarray base if it has one (unique).  A
    tensor whose value is on the device only has no host array that could be written to."""
    seen = set()
    for t in tensors:
        arr = t._value
        if not isinstance(arr, np.ndarray):
            continue
        base = arr.base
        for a in (base, arr):
            if isinstance(a, np.ndarray) and id(a) not in seen:
                seen.add(id(a))
                yield a


def held_count():
    """Number of arrays currently held read-only (for tests)."""
    return len(_held)
