"""``Repeat`` on the MI355X (reference: ``mygrad/tensor_manip/tiling/ops.py``).

The forward pass is ``np.repeat``: a gather of whole entries along one axis.  The gradient
adds, for every input entry, the run of output entries that came from it.  The reference
forms that sum over a ``sliding_window_view`` of the incoming gradient (equal repeats) or
with ``np.add.at`` over repeated flat indices (unequal repeats); the device kernel walks the
same runs in ascending order."""

import numpy as np

from ... import _device, _hip
from ...operation_base import Operation

__all__ = ["Repeat"]


class Repeat(Operation):
    takes_device_arrays = True

    # Repeat can broadcast in the case:
    #    repeat(1, 2) -> [1 1]

    def __call__(self, a, repeats, axis=None):
        self.variables = (a,)
        self._axis = axis
        self._repeats = repeats
        x = _device.value_of(a)
        if x.dtype.itemsize not in (1, 2, 4, 8) or x.dtype.hasobject:
            raise TypeError(f"repeat runs on the GPU for elements of 1, 2, 4 or 8 bytes, got {x.dtype} (no CPU fallback)")

        # the array as (outer, n, inner) around the repeated axis
        if axis is None:
            outer, n, inner = 1, x.size, 1
        elif x.ndim == 0:
            # np.repeat treats a scalar as a 1-D array of one entry
            np.lib.array_utils.normalize_axis_index(axis, 1)
            outer, n, inner = 1, 1, 1
        else:
            axis = np.lib.array_utils.normalize_axis_index(axis, x.ndim)
            outer = int(np.prod(x.shape[:axis], dtype=np.int64))
            n = x.shape[axis]
            inner = int(np.prod(x.shape[axis + 1 :], dtype=np.int64))

        # np.repeat on n bytes checks `repeats` (type, sign, length) and counts the output entries
        src_of = np.repeat(np.arange(n, dtype=np.int32), repeats)
        total = src_of.size
        counts = np.asarray(repeats)
        self._uniform = counts.ndim == 0 or counts.size == 1
        self._geometry = (outer, n, inner, total)
        if self._uniform:
            self._count = int(counts.reshape(-1)[0]) if counts.size else 0
            self._offsets = None
        else:
            self._count = 0
            self._offsets = np.concatenate([[0], np.cumsum(counts, dtype=np.int64)]).astype(np.int64)

        if axis is None or x.ndim == 0:
            out_shape = (total,)
        else:
            out_shape = (*x.shape[:axis], total, *x.shape[axis + 1 :])
        if x.size == 0 or total == 0:
            return np.empty(out_shape, dtype=x.dtype)

        xb = _device.to_device(x)
        sb = None if self._uniform else _device.to_device(src_of)
        ob = _device.DeviceBuffer(max(outer * total * inner * x.dtype.itemsize, 16))
        _hip.check(
            _hip.lib().mg_repeat_fwd(
                x.dtype.itemsize, outer, n, inner, self._count, total, sb.ptr if sb is not None else None, xb.ptr, ob.ptr
            )
        )
        out = _device.download(ob, out_shape, x.dtype)
        _device.attach(out, ob)
        return out

    def backward_var(self, grad, index, **kwargs):
        a = _device.value_of(self.variables[index])
        outer, n, inner, total = self._geometry
        if grad.dtype not in (np.float32, np.float64):
            raise TypeError(f"repeat's gradient runs on the GPU in float32 or float64, got {grad.dtype} (no CPU fallback)")
        if a.size == 0 or total == 0:
            # nothing was repeated: every entry's run is empty
            return np.zeros(a.shape, dtype=grad.dtype)
        if grad.size != outer * total * inner:
            raise ValueError(f"repeat backward: gradient of shape {grad.shape} does not match the repeated array")
        gb = _device.to_device(grad)
        fb = None if self._uniform else _device.to_device(self._offsets)
        ob = _device.DeviceBuffer(max(a.size * grad.dtype.itemsize, 16))
        _hip.check(
            _hip.lib().mg_repeat_bwd(
                _hip.dtype_code(grad.dtype), outer, n, inner, self._count, total, fb.ptr if fb is not None else None, gb.ptr, ob.ptr
            )
        )
        out = _device.download(ob, a.shape, grad.dtype)
        _device.attach_transient(out, ob)
        return out
