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

Under the package's own ``Tensor`` no result crosses PCIe until somebody reads it:
while :func:`deferring` is active, :func:`download` hands back a :class:`DeviceArray`
-- shape, dtype and the device buffer -- instead of copying, ``Tensor.data`` /
``Tensor.grad`` turn it into a host array on first read, and operations take such
values from :func:`to_device` without any copy.  Called directly (or from another
caller of the Operation contract) the operations return host arrays as the contract
says.
"""

import ctypes
import weakref

from math import prod

import numpy as np

from . import _hip

__all__ = [
    "DeviceArray",
    "DeviceBuffer",
    "deferring",
    "full",
    "value_of",
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


def _count(shape):
    """Elements of an array of ``shape`` (a sequence of extents, or one extent)."""
    try:
        return prod(int(n) for n in shape)
    except TypeError:
        return int(shape)


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

    __slots__ = ("ptr", "nbytes", "_owned", "__weakref__")

    def __init__(self, nbytes):
        self._owned = None
        handle = ctypes.c_void_p()
        _hip.check(_hip.lib().mg_malloc(ctypes.byref(handle), int(nbytes)))
        self.ptr = self._owned = handle.value
        self.nbytes = int(nbytes)

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
        """Gives the block back (once; ``ptr`` keeps its value for whoever still compares it)."""
        owned, self._owned = self._owned, None
        if owned is not None:
            _free_device(owned)

    __del__ = free


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
    count = _count(shape)
    nbytes = max(count * dtype.itemsize, 1)
    block = _PinnedBlock(nbytes)
    raw = (ctypes.c_char * nbytes).from_address(block.ptr)
    raw._pinned_block = block  # the ctypes object is the array's base; it keeps the block alive
    return np.ndarray(shape, dtype=dtype, buffer=raw)  # .base is `raw` itself, not a view chain


# --------------------------------------------------------------------------- results kept on the device
_defer = 0


class deferring:
    """While active, :func:`download` returns :class:`DeviceArray` objects instead of copying
    results to the host (the package's ``Tensor`` wraps its calls of an operation in it)."""

    def __enter__(self):
        global _defer
        _defer += 1
        return self

    def __exit__(self, *exc):
        global _defer
        _defer -= 1
        return False


class _Flags(dict):
    c_contiguous = True
    writeable = False


_DEVICE_FLAGS = _Flags(C_CONTIGUOUS=True, WRITEABLE=False)


def _resolve_shape(size, shape):
    """``shape`` with a single -1 filled in, checked against ``size`` like ndarray.reshape."""
    shape = [int(n) for n in shape]
    known = 1
    for n in shape:
        if n != -1:
            known *= n
    if shape.count(-1) == 1 and known and size % known == 0:
        shape[shape.index(-1)] = size // known
        known = size
    if -1 in shape or known != size:
        raise ValueError(f"cannot reshape array of size {size} into shape {tuple(shape)}")
    return tuple(shape)


class DeviceArray:
    """A C-contiguous array that so far exists on the device only: shape, dtype and the
    buffer a kernel wrote.  It answers the questions operations ask of an input before
    launching (``shape``, ``dtype``, ``ndim``, ``size``, ``nbytes``, ``reshape``) without
    touching the data; :meth:`host` copies it into pinned host memory, once.

    ``base`` is the array whose buffer this one shares (a reshape), None for the owner of
    a buffer -- the rule ``Operation.backward`` uses to decide whether a gradient must be
    copied before it may be updated in place.
    """

    __slots__ = ("buf", "shape", "dtype", "base", "_host", "__weakref__")
    flags = _DEVICE_FLAGS

    def __init__(self, buf, shape, dtype, base=None):
        self.buf = buf
        self.shape = tuple(int(n) for n in shape)
        self.dtype = np.dtype(dtype)
        self.base = base
        self._host = None

    @property
    def ndim(self):
        return len(self.shape)

    @property
    def size(self):
        return prod(self.shape)  # the shape is a tuple of Python ints

    @property
    def itemsize(self):
        return self.dtype.itemsize

    @property
    def nbytes(self):
        return self.size * self.dtype.itemsize

    def reshape(self, *shape):
        if len(shape) == 1 and not isinstance(shape[0], (int, np.integer)):
            shape = tuple(shape[0])
        shape = _resolve_shape(self.size, shape)
        return DeviceArray(self.buf, shape, self.dtype, base=self if self.base is None else self.base)

    def host(self):
        """The values as a (pinned) host array; copied on the first call."""
        if self._host is None:
            out = pinned_empty(self.shape, self.dtype)
            if self.size:
                self.buf.download_into(out)
            self._host = out
        return self._host

    def __array__(self, dtype=None, copy=None):
        out = self.host()
        if dtype is not None and np.dtype(dtype) != out.dtype:
            return out.astype(dtype)
        return out.copy() if copy else out

    def copy(self):
        """A new array with a buffer of its own (device-to-device copy)."""
        buf = DeviceBuffer(max(self.nbytes, 16))
        if self.nbytes:
            _hip.check(_hip.lib().mg_memcpy_d2d(buf.ptr, self.buf.ptr, self.nbytes))
        return DeviceArray(buf, self.shape, self.dtype)

    def astype(self, dtype):
        """The values cast to float32 / float64 / float16 on the device (a new buffer)."""
        dtype = np.dtype(dtype)
        if dtype == self.dtype:
            return self
        if not (_is_storage_type(dtype) and _is_storage_type(self.dtype)):
            # mg_cast converts between the floating-point storage types only; anything else (the
            # integer or boolean result of a `repeat`) is converted by NumPy and uploaded again
            return from_host(np.ascontiguousarray(self.host().astype(dtype)))
        buf = DeviceBuffer(max(self.size * dtype.itemsize, 16))
        _hip.check(_hip.lib().mg_cast(_hip.storage_code(self.dtype), _hip.storage_code(dtype), self.size, self.buf.ptr, buf.ptr))
        return DeviceArray(buf, self.shape, dtype)

    def add_into(self, other):
        """``self += other`` on the device, with NumPy's rule for a narrower ``self`` (the sum is
        formed in the wider type and rounded once).  ``self`` must own its buffer and must not
        have been copied to the host yet."""
        assert self.base is None and self._host is None and other.shape == self.shape
        _hip.check(_hip.lib().mg_accumulate(_hip.storage_code(self.dtype), _hip.storage_code(other.dtype), self.size,
                                            self.buf.ptr, other.buf.ptr))

    def __repr__(self):
        return f"DeviceArray(shape={self.shape}, dtype={self.dtype})"


def value_of(tensor):
    """What an operation works on: the tensor's DeviceArray while its values exist on the
    device only, else its host array (``tensor.data``; a tensor class other than this
    package's has nothing else)."""
    try:
        return tensor._value
    except AttributeError:
        return tensor.data


def _is_storage_type(dtype):
    return np.dtype(dtype) in (np.dtype(np.float16), np.dtype(np.float32), np.dtype(np.float64))


def from_host(arr):
    """A C-contiguous host array of any dtype as a DeviceArray (one upload)."""
    buf = DeviceBuffer(max(arr.nbytes, 16))
    if arr.nbytes:
        buf.upload(arr)
        stats["uploads"] += 1
    return DeviceArray(buf, arr.shape, arr.dtype)


def full(shape, dtype, value):
    """``np.full(shape, value, dtype)`` made on the device (float32, float64; float16 is filled as
    float32 and narrowed, which is exact for the values that fit)."""
    dtype = np.dtype(dtype)
    if dtype == np.float16:
        return full(shape, np.float32, value).astype(np.float16)
    count = _count(shape)
    buf = DeviceBuffer(max(count * dtype.itemsize, 16))
    _hip.check(_hip.lib().mg_fill_value(_hip.dtype_code(dtype), count, float(value), buf.ptr))
    return DeviceArray(buf, shape, dtype)


# --------------------------------------------------------------------------- mirrors
_mirrors = {}  # key -> DeviceBuffer, for arrays the graph holds read-only
_transient = {}  # key -> DeviceBuffer, for gradients in flight during one backward()
_locked = {}  # key -> number of graph locks on that memory
_pending = {}  # key -> DeviceBuffer offered by the last attach(), a mirror once the array is locked


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
    offered = _pending.pop(key, None)
    if offered is not None:
        _mirrors[key] = offered
        try:
            weakref.finalize(_root(arr), _evict_key, key)
        except TypeError:  # owner not weak-referenceable: do not cache
            _mirrors.pop(key, None)


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
    the device can have gone stale).  A value that exists on the device only cannot be
    written to from the host at all."""
    return isinstance(arr, DeviceArray) or _key(arr) in _locked


def _evict_key(key):
    _mirrors.pop(key, None)
    _transient.pop(key, None)
    _locked.pop(key, None)


def attach(arr, buf):
    """Offer ``buf`` as the device copy of the result ``arr``.  The offer stands only if the
    graph locks ``arr`` next (``Tensor._op`` does, right after the operation returns): an array
    that is handed out writeable -- under ``no_autodiff`` or with the memory guard off -- may
    be edited on the host, and a copy cached for it would go stale unnoticed."""
    if isinstance(arr, DeviceArray):
        return
    _pending.clear()
    _pending[_key(arr)] = buf


def drop_pending():
    """Forget the offer of the last :func:`attach` (its array was not locked)."""
    _pending.clear()


def attach_transient(arr, buf):
    """Record ``buf`` as the device copy of a gradient array until backward() ends or the
    array dies, whichever comes first (its memory may be handed out again after that)."""
    if isinstance(arr, DeviceArray):
        return
    key = _key(arr)
    _transient[key] = buf
    try:
        weakref.finalize(_root(arr), _drop_transient, key, buf)
    except TypeError:  # owner not weak-referenceable: do not cache
        _transient.pop(key, None)


def _drop_transient(key, buf):
    if _transient.get(key) is buf:
        del _transient[key]


def hold_gradient(arr):
    """Upload ``arr`` now and keep the copy until backward() ends: an operation with several
    non-constant inputs is asked for one gradient per input with the same incoming ``arr``,
    which would otherwise cross PCIe once per request."""
    if isinstance(arr, DeviceArray) or not isinstance(arr, np.ndarray) or not arr.flags["C_CONTIGUOUS"] or arr.size == 0:
        return
    if arr.dtype not in (np.float32, np.float64) or lookup(arr) is not None:
        return
    buf = DeviceBuffer(arr.nbytes)
    buf.upload(arr)
    stats["uploads"] += 1
    attach_transient(arr, buf)


def evict(arr):
    if isinstance(arr, DeviceArray):
        return
    key = _key(arr)
    _mirrors.pop(key, None)
    _transient.pop(key, None)


def drop_transients():
    _transient.clear()


def lookup(arr):
    if isinstance(arr, DeviceArray):
        return arr.buf
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
    if isinstance(arr, DeviceArray):
        stats["mirror_hits"] += 1
        return (arr if dtype is None else arr.astype(dtype)).buf
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
    key = _key(arr)
    if key in _locked:
        _mirrors[key] = buf
        try:
            weakref.finalize(_root(arr), _evict_key, key)
        except TypeError:  # owner not weak-referenceable: do not cache
            _mirrors.pop(key, None)
    return buf


def download(buf, shape, dtype, now=False):
    """The result a kernel left in ``buf``: copied into a new pinned host array, or -- while
    :func:`deferring` is active and unless ``now`` -- left where it is as a DeviceArray."""
    if _defer and not now:
        return DeviceArray(buf, shape, dtype)
    out = pinned_empty(shape, dtype)
    buf.download_into(out)
    return out
