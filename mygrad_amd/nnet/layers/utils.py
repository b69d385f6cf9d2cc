"""Host-side window helper (counterpart of the reference's
``mygrad/nnet/layers/utils.py:7-228``).

``sliding_window_view`` is pure stride arithmetic -- it builds a zero-copy,
read-only view -- and stays on the host.  Its index map

    view[g..., lead..., w...] = arr[lead..., g*step + w*dilation]

is the address function the convolution and pooling kernels evaluate on the
device; ``check_window_args`` is the part of it that the operations reuse to
raise the reference's errors before anything is launched.  ``sliding_window_copy``
evaluates the same map on the device and returns the C-contiguous copy of the view
(what ``np.ascontiguousarray(sliding_window_view(...))`` gives).
"""

from numbers import Integral

import numpy as np
from numpy.lib.stride_tricks import as_strided

__all__ = ["sliding_window_view", "sliding_window_copy", "check_window_args"]


def check_window_args(shape, window_shape, step, dilation=None):
    """Validate and normalise ``(window_shape, step, dilation)`` against an array
    of the given ``shape``; returns them as tuples of ints.

    Raises exactly what the reference raises (utils.py:123-196): ``TypeError``
    for a non-sequence / non-positive-integer window, a bad ``step`` type or a
    bad ``dilation`` type; ``ValueError`` for too many window axes, non-positive
    steps, a window larger than the array, a malformed dilation, or
    ``window * dilation`` exceeding the array extent.
    """
    ndim = len(shape)
    if not hasattr(window_shape, "__iter__"):
        raise TypeError(f"`window_shape` must be a sequence of positive integers, got: {window_shape}")
    window_shape = tuple(window_shape)
    if not all(isinstance(i, Integral) and i > 0 for i in window_shape):
        raise TypeError(f"`window_shape` must be a sequence of positive integers, got: {window_shape}")
    if len(window_shape) > ndim:
        raise ValueError(
            f"`window_shape` ({window_shape}) cannot specify more values than `arr.ndim` ({ndim})."
        )
    m = len(window_shape)

    if not isinstance(step, Integral) and not hasattr(step, "__iter__"):
        raise TypeError(f"`step` must be a positive integer or a sequence of positive integers, got: {step}")
    step = (int(step),) * m if isinstance(step, Integral) else tuple(step)
    if not all(isinstance(i, Integral) and i > 0 for i in step):
        raise ValueError(f"`step` must be a positive integer or a sequence of positive integers, got: {step}")

    tail = tuple(shape[ndim - m :]) if m else ()
    if any(w > x for w, x in zip(window_shape[::-1], tuple(shape)[::-1])):
        raise ValueError(
            "Each size of the window-shape must fit within the trailing dimensions of `arr`."
            f"{window_shape} does not fit in {tail}"
        )

    if dilation is not None and not isinstance(dilation, Integral) and not hasattr(dilation, "__iter__"):
        raise TypeError(
            f"`dilation` must be None, a positive integer, or a sequence of positive integers, got: {dilation}"
        )
    if dilation is None:
        dilation = (1,) * m
    else:
        if isinstance(dilation, Integral):
            dilation = (int(dilation),) * m
        if len(dilation) != m or not all(isinstance(i, Integral) and i > 0 for i in dilation):
            raise ValueError(
                "`dilation` must be None, a positive integer, or a sequence of positive integers with the "
                f"same length as `window_shape` ({window_shape}), got: {dilation}"
            )
        if any(w * d > x for w, d, x in zip(window_shape[::-1], tuple(dilation)[::-1], tuple(shape)[::-1])):
            raise ValueError(
                f"The dilated window ({tuple(w * d for w, d in zip(window_shape, dilation))}) must fit within "
                f"the trailing dimensions of `arr` ({tail})"
            )
    return (
        tuple(int(w) for w in window_shape),
        tuple(int(s) for s in step),
        tuple(int(d) for d in dilation),
    )


def sliding_window_view(arr, window_shape, step, dilation=None):
    """Create a sliding-window view over the trailing dimensions of an array.

    No copy is made unless ``arr`` is not C-contiguous.  The windows cover only
    valid regions of ``arr`` and are placed greedily (flooring).

    Parameters
    ----------
    arr : numpy.ndarray, shape=(..., [x, (...), z])
    window_shape : Sequence[int]
        ``(Wx, ..., Wz)``: extent of the window along each trailing axis.
    step : Union[int, Sequence[int]]
        ``(Sx, ..., Sz)``: spacing between window placements.
    dilation : Optional[Union[int, Sequence[int]]]
        ``(Dx, ..., Dz)``: spacing between the elements of one window.

    Returns
    -------
    numpy.ndarray, read-only view, shape ``(X, ..., Z, ..., Wx, ..., Wz)`` with
    ``X = (x - ((Wx - 1) * Dx + 1)) // Sx + 1``; indexing it with
    ``[ix, ..., iz]`` gives ``arr[..., ix*Sx : ix*Sx + Wx*Dx : Dx, ...]``.
    """
    window, step, dilation = check_window_args(arr.shape, window_shape, step, dilation)
    if not arr.flags["C_CONTIGUOUS"]:
        arr = np.ascontiguousarray(arr)

    m = len(window)
    lead = arr.ndim - m
    unit = [1] * arr.ndim  # element strides of a C-contiguous array
    for axis in range(arr.ndim - 2, -1, -1):
        unit[axis] = unit[axis + 1] * arr.shape[axis + 1]

    placements = tuple(
        (arr.shape[lead + k] - ((window[k] - 1) * dilation[k] + 1)) // step[k] + 1 for k in range(m)
    )
    elem_strides = (
        [step[k] * unit[lead + k] for k in range(m)]
        + unit[:lead]
        + [dilation[k] * unit[lead + k] for k in range(m)]
    )
    return as_strided(
        arr,
        shape=placements + arr.shape[:lead] + window,
        strides=tuple(arr.itemsize * s for s in elem_strides),
        writeable=False,
    )


def sliding_window_copy(arr, window_shape, step, dilation=None):
    """C-contiguous copy of ``sliding_window_view(arr, window_shape, step, dilation)``,
    gathered on the device (same arguments, same errors, same shape; writable).

    The view costs nothing and is the right tool on the host; the copy is for consumers
    that need the windows laid out densely, and it is produced at memory speed instead of
    by NumPy's strided copy loop.  At most three windowed axes; elements of 1, 2, 4 or 8
    bytes."""
    from ... import _device, _hip

    arr = np.asarray(arr)
    window, step, dilation = check_window_args(arr.shape, window_shape, step, dilation)
    m = len(window)
    if not 1 <= m <= _hip.MG_MAX_ND:
        raise NotImplementedError(f"sliding_window_copy handles 1 to {_hip.MG_MAX_ND} windowed axes, got {m} (no CPU fallback)")
    if arr.dtype.itemsize not in (1, 2, 4, 8) or arr.dtype.hasobject:
        raise TypeError(f"sliding_window_copy moves elements of 1, 2, 4 or 8 bytes, got {arr.dtype} (no CPU fallback)")
    lead_shape, tail = arr.shape[: arr.ndim - m], arr.shape[arr.ndim - m :]
    grid = tuple((tail[k] - ((window[k] - 1) * dilation[k] + 1)) // step[k] + 1 for k in range(m))
    out_shape = grid + lead_shape + window
    count = int(np.prod(out_shape, dtype=np.int64))
    if count == 0:
        return np.empty(out_shape, dtype=arr.dtype)
    lead = int(np.prod(lead_shape, dtype=np.int64))
    desc = _hip.window_desc(arr.dtype.itemsize, lead, tail, window, step, dilation, grid)
    xb = _device.to_device(arr)
    ob = _device.DeviceBuffer(max(count * arr.dtype.itemsize, 16))
    _hip.check(_hip.lib().mg_window_gather(desc, xb.ptr, ob.ptr))
    return _device.download(ob, out_shape, arr.dtype)
