"""Device buffers, pinned host arrays and the host-array -> device-mirror cache.

The Operation contract hands NumPy arrays in and out, so an op's result must end
up in host memory.  To keep activations and gradients from crossing PCIe more
than once, every array that enters or leaves an op keeps its device copy (its
"mirror") for as long as the graph holds the array read-only:

* an input is uploaded the first time an op sees it and found again afterwards
  (the forward input ``x`` is still on the device when ``dw`` is computed);
* an op's output keeps the buffer the kernel wrote, so a chained op
  (conv -> pool) and the backward pass read it in place;
* a gradient returned by ``backward_var`` keeps its buffer until it is either
  consumed by the next ``backward_var`` or modified on the host.

A mirror is dropped when the graph releases its lock on the host array (the host
copy may change from then on), when the host array is garbage collected, or
explicitly via :func:`evict`.
"""

import ctypes
import weakref

import numpy as np

from . import _hip

__all__ = [
    "DeviceBuffer",
    "pinned_empty",
    "to_device",
    "attach",
    "attach_transient",
    "hold_gradient",
    "evict",
    "drop_transients",
    "lookup",
    "download",
    "stats",
]

stats = {"h2d_bytes": 0, "d2h_bytes": 0, "mirror_hits": 0, "uploads": 0}


def _free_device(ptr):
    try:
        _hip.load_library().mg_free(ptr)
    except Exception:  # interpreter shutdown
        pass


def _free_pinned(ptr):
    try:
        _hip.load_library().mg_host_free(ptr)
    except Exception:
        pass


class DeviceBuffer:
    """Owns one device allocation; freed when the last reference goes away."""

    __slots__ = ("ptr", "nbytes", "_finalizer", "__weakref__")

    def __init__(self, nbytes):
        handle = ctypes.c_void_p()
        _hip.check(_hip.lib().mg_malloc(ctypes.byref(handle), int(nbytes)))
        self.ptr = handle.value
        self.nbytes = int(nbytes)
        self._finalizer = weakref.finalize(self, _free_device, self.ptr)

    def upload(self, arr):
        arr = np.ascontiguousarray(arr)
        assert arr.nbytes <= self.nbytes
        _hip.check(_hip.lib().mg_memcpy_h2d(self.ptr, arr.ctypes.data, arr.nbytes))
        stats["h2d_bytes"] += arr.nbytes

    def download_into(self, arr):
        assert arr.flags["C_CONTIGUOUS"] and arr.nbytes <= self.nbytes
        _hip.check(_hip.lib().mg_memcpy_d2h(arr.ctypes.data, self.ptr, arr.nbytes))
        stats["d2h_bytes"] += arr.nbytes

    def free(self):
        self._finalizer()


class _PinnedBlock:
    __slots__ = ("ptr", "nbytes", "_finalizer", "__weakref__")

    def __init__(self, nbytes):
        handle = ctypes.c_void_p()
        _hip.check(_hip.lib().mg_host_alloc(ctypes.byref(handle), int(nbytes)))
        self.ptr = handle.value
        self.nbytes = int(nbytes)
        self._finalizer = weakref.finalize(self, _free_pinned, self.ptr)


def pinned_empty(shape, dtype):
    """Uninitialised C-contiguous ndarray over pinned (page-locked) host memory.

    The array can be locked and unlocked like any other (its base is a writable
    buffer); the pinned block is released when the last view dies.
    """
    dtype = np.dtype(dtype)
    count = int(np.prod(shape, dtype=np.int64))
    nbytes = max(count * dtype.itemsize, 1)
    block = _PinnedBlock(nbytes)
    raw = (ctypes.c_char * nbytes).from_address(block.ptr)
    raw._pinned_block = block  # the ctypes object is the array's base; it keeps the block alive
    return np.ndarray(shape, dtype=dtype, buffer=raw)  # .base is `raw` itself, not a view chain


# --------------------------------------------------------------------------- mirrors
_mirrors = {}  # key -> DeviceBuffer, for arrays the graph holds read-only
_transient = {}  # key -> DeviceBuffer, for gradients in flight during one backward()
_locked = {}  # key -> number of graph locks on that memory


def _key(arr):
    return (arr.__array_interface__["data"][0], arr.nbytes, arr.dtype.str)


def _root(arr):
    """Object that owns ``arr``'s memory (end of the ``.base`` chain)."""
    root = arr
    while isinstance(root, np.ndarray) and root.base is not None:
        root = root.base
    return root


def note_locked(arr):
    """The graph now holds ``arr`` read-only: its mirror may be cached."""
    key = _key(arr)
    _locked[key] = _locked.get(key, 0) + 1


def note_released(arr):
    """The graph released ``arr``: the host copy may change, drop the mirror."""
    key = _key(arr)
    left = _locked.get(key, 0) - 1
    if left > 0:
        _locked[key] = left
        return
    _locked.pop(key, None)
    _mirrors.pop(key, None)


def is_locked(arr):
    """True while the graph holds ``arr`` read-only (so nothing derived from its values on
    the device can have gone stale)."""
    return _key(arr) in _locked


def _evict_key(key):
    _mirrors.pop(key, None)
    _transient.pop(key, None)
    _locked.pop(key, None)


def attach(arr, buf):
    """Record ``buf`` as the device copy of ``arr`` (which the graph is about to lock)."""
    key = _key(arr)
    _mirrors[key] = buf
    try:
        weakref.finalize(_root(arr), _evict_key, key)
    except TypeError:  # owner not weak-referenceable: do not cache
        _mirrors.pop(key, None)


def attach_transient(arr, buf):
    """Record ``buf`` as the device copy of a gradient array until backward() ends."""
    _transient[_key(arr)] = buf


def hold_gradient(arr):
    """Upload ``arr`` now and keep the copy until backward() ends: an operation with several
    non-constant inputs is asked for one gradient per input with the same incoming ``arr``,
    which would otherwise cross PCIe once per request."""
    if not isinstance(arr, np.ndarray) or not arr.flags["C_CONTIGUOUS"] or arr.size == 0:
        return
    if arr.dtype not in (np.float32, np.float64) or lookup(arr) is not None:
        return
    buf = DeviceBuffer(arr.nbytes)
    buf.upload(arr)
    stats["uploads"] += 1
    attach_transient(arr, buf)


def evict(arr):
    key = _key(arr)
    _mirrors.pop(key, None)
    _transient.pop(key, None)


def drop_transients():
    _transient.clear()


def lookup(arr):
    if not arr.flags["C_CONTIGUOUS"]:
        return None
    key = _key(arr)
    buf = _transient.get(key)
    if buf is None and key in _locked:
        buf = _mirrors.get(key)
    return buf


def to_device(arr, dtype=None):
    """Device buffer holding ``arr`` (cast to ``dtype`` if given): the cached mirror
    when there is one, else a fresh upload (cached if the graph holds ``arr``)."""
    if dtype is not None and arr.dtype != dtype:
        arr = arr.astype(dtype)
    elif not arr.flags["C_CONTIGUOUS"]:
        arr = np.ascontiguousarray(arr)
    else:
        buf = lookup(arr)
        if buf is not None:
            stats["mirror_hits"] += 1
            return buf
    buf = DeviceBuffer(arr.nbytes)
    buf.upload(arr)
    stats["uploads"] += 1
    if _key(arr) in _locked:
        attach(arr, buf)
    return buf


def download(buf, shape, dtype):
    """Copy a device buffer into a new pinned host array."""
    out = pinned_empty(shape, dtype)
    buf.download_into(out)
    return out
