"""``MatMul`` on the MI355X (reference: ``mygrad/math/misc/ops.py:91-126``).

A matrix product is a convolution whose window has one element: ``a @ b`` with ``a:(M, K)``
and ``b:(K, N)`` is the convolution of ``b`` -- K channels, N positions -- with M filters, and
its two gradients are the convolution's.  The operation therefore runs on the convolution's
implicit-GEMM kernels (``mg_matmul*`` in ``libmygrad_hip.so``) with no kernel of its own.

Operand patterns that run: both operands at most 2-D (vectors are promoted like
``np.matmul`` does); one operand a stack and the other at most 2-D (one launch: the stack is
the convolution's batch, or folds into the rows of the left operand); two stacks of the same
batch shape (one launch for all pairs when the matrices are small, ``mg_matmul_batched``,
else one launch of the tiled kernels per matrix pair); two stacks that broadcast against each other
(each is first spread to the common batch shape on the device, and the gradient of a stack
that was spread is summed back over the axes it was spread along)."""

import numpy as np

from ... import _device, _hip, _reduce
from ...operation_base import Operation

__all__ = ["MatMul"]


# Two stacks are multiplied pair by pair on the tiled kernels when a pair has more than this
# many floating-point operations (it then fills the device by itself), else in one launch of the
# kernel that gives every 16 x 16 tile of every product a wavefront.  Measured on float32 squares:
# that kernel sustains 36-49 TFLOP/s from 128^3 up, a launch of the tiled kernels costs 8-12 us
# and reaches 55 TFLOP/s at 1024^3, where the two meet.
SMALL_PAIR_FLOPS = 2 * 768**3


def _prod(shape):
    return int(np.prod(shape, dtype=np.int64))


class MatMul(Operation):
    takes_device_arrays = True

    gradient_on_device = True

    def __call__(self, a, b):
        self.variables = (a, b)
        x, y = _device.value_of(a), _device.value_of(b)
        # NumPy's own checks (scalars, core dimensions, batch broadcasting) on operands
        # without rows and columns: the same errors, the batch shape of the result, no arithmetic
        probe = np.matmul(
            np.empty(x.shape if x.ndim < 2 else (*x.shape[:-2], 0, x.shape[-1]), dtype=np.int8),
            np.empty(y.shape if y.ndim < 2 else (*y.shape[:-2], y.shape[-2], 0), dtype=np.int8),
        )
        dtype = np.dtype(np.result_type(x.dtype, y.dtype))
        if dtype not in (np.float32, np.float64):
            raise TypeError(f"matmul runs on the GPU in float32 or float64, got {x.dtype} and {y.dtype} (there is no CPU fallback)")

        x2_shape = tuple(x.shape) if x.ndim > 1 else (1, *x.shape)  # a vector is promoted like np.matmul promotes it
        y2_shape = tuple(y.shape) if y.ndim > 1 else (*y.shape, 1)
        M, K, N = x2_shape[-2], x2_shape[-1], y2_shape[-1]
        stack_a, stack_b = x2_shape[:-2], y2_shape[:-2]
        # two different stacks: both are spread to the batch shape they broadcast to
        self._spread = bool(stack_a and stack_b and stack_a != stack_b)
        self._own_stacks = (stack_a, stack_b)
        if self._spread:
            stack_a = stack_b = tuple(probe.shape[: probe.ndim - 2])
        batch_shape = stack_a or stack_b
        out_shape = batch_shape + (() if x.ndim == 1 else (M,)) + (() if y.ndim == 1 else (N,))
        assert len(out_shape) == probe.ndim
        self._dtype, self._dims = dtype, (M, K, N)
        self._stacks = (stack_a, stack_b)
        self._promoted = (x2_shape, y2_shape)
        if 0 in out_shape or K == 0:
            return np.zeros(out_shape, dtype=dtype)

        ab, bb = self._operand(x, 0), self._operand(y, 1)
        ob = _device.DeviceBuffer(max(_prod(out_shape) * dtype.itemsize, 16))
        self._launch("mg_matmul", ab, bb, ob, a_like=0, x_like=1, out_like=2)
        out = _device.download(ob, out_shape, dtype)
        _device.attach(out, ob)
        return out

    def _operand(self, arr, index):
        """Device buffer of operand ``index``, spread over the common batch shape if its own
        stack is a different one."""
        buf = _device.to_device(arr, self._dtype)
        own, batch = self._own_stacks[index], self._stacks[index]
        if not self._spread or own == batch:
            return buf
        core = self._promoted[index][-2:]
        return _reduce.broadcast(buf, own + core, batch + core, self._dtype)

    def _launch(self, entry, first, second, result, a_like, x_like, out_like):
        """Call ``entry(dtype, batch, M, K, N, first, second, result)`` once, or once per
        matrix pair for two stacks.  ``*_like`` say which of (a, b, out) each buffer has the
        layout of (0: a, 1: b, 2: out) so that the per-pair offsets can be formed."""
        M, K, N = self._dims
        stack_a, stack_b = self._stacks
        code, item = _hip.dtype_code(self._dtype), self._dtype.itemsize
        fn = getattr(_hip.lib(), entry)
        if not stack_a:
            _hip.check(fn(code, _prod(stack_b), M, K, N, first.ptr, second.ptr, result.ptr))
        elif not stack_b:
            _hip.check(fn(code, 1, _prod(stack_a) * M, K, N, first.ptr, second.ptr, result.ptr))
        elif 2 * M * K * N <= SMALL_PAIR_FLOPS:
            # a stack of small pairs: one launch, the gradients by transposed reads
            # (entry: first, second -> result)   mg_matmul: a, b -> a @ b;
            # mg_matmul_da: grad, b -> grad @ b^T;   mg_matmul_dx: grad, a -> a^T @ grad
            pairs = _prod(stack_a)
            batched = _hip.lib().mg_matmul_batched
            if entry == "mg_matmul":
                _hip.check(batched(code, pairs, M, K, N, 0, 0, first.ptr, second.ptr, result.ptr))
            elif entry == "mg_matmul_da":
                _hip.check(batched(code, pairs, M, N, K, 0, 1, first.ptr, second.ptr, result.ptr))
            else:
                _hip.check(batched(code, pairs, K, M, N, 1, 0, second.ptr, first.ptr, result.ptr))
        else:
            per = (M * K * item, K * N * item, M * N * item)
            for i in range(_prod(stack_a)):
                _hip.check(
                    fn(code, 1, M, K, N, first.ptr + i * per[a_like], second.ptr + i * per[x_like], result.ptr + i * per[out_like])
                )

    def backward_var(self, grad, index, **kwargs):
        a, b = self.variables
        dtype = self._dtype
        var = _device.value_of((a, b)[index])
        if var.size == 0 or grad.size == 0:
            return np.zeros(var.shape, dtype=dtype)
        M, K, N = self._dims
        stack_a, stack_b = self._stacks
        batch = _prod(stack_a or stack_b)
        if grad.size != batch * M * N:
            raise ValueError(f"matmul backward: gradient of shape {grad.shape} does not match the product")
        gb = _device.to_device(grad, dtype)
        own, full = self._own_stacks[index], self._stacks[index]
        widened = self._spread and own != full
        core = self._promoted[index][-2:]
        count = _prod(full + core) if widened else var.size
        ob = _device.DeviceBuffer(max(count * dtype.itemsize, 16))
        if index == 0:
            # d a = grad @ b^T, summed over a batch that `a` was shared by (ops.py:107-114)
            self._launch("mg_matmul_da", gb, self._operand(_device.value_of(b), 1), ob, a_like=2, x_like=1, out_like=0)
        else:
            # d b = a^T @ grad, summed over a stack of left operands that `b` was shared by (ops.py:116-124)
            self._launch("mg_matmul_dx", gb, self._operand(_device.value_of(a), 0), ob, a_like=2, x_like=0, out_like=1)
        if widened:
            # one gradient per matrix pair: add up those of the pairs that shared this operand's matrix
            lead = len(full) - len(own)
            axes = tuple(range(lead)) + tuple(lead + i for i, n in enumerate(own) if n == 1 and full[lead + i] != 1)
            ob = _reduce.sum_axes(ob, full + core, axes, dtype)
        out = _device.download(ob, var.shape, dtype)
        _device.attach_transient(out, ob)
        return out
