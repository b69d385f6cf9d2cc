"""ctypes binding of ``libmygrad_hip.so`` (declared in ``include/mygrad_hip.h``).

The library is loaded lazily on first use.  There is no CPU fallback: when the
shared library is missing or no gfx950 device can be initialised, every kernel
entry point raises :class:`HipUnavailable`.
"""

import ctypes
import os
import threading

MG_MAX_ND = 3
MG_F32, MG_F64, MG_F16 = 0, 1, 2

MG_OK = 0
MG_ERR_BAD_ARG = -1
MG_ERR_UNSUPPORTED = -2
MG_ERR_NO_DEVICE = -3
MG_ERR_OOM = -4
MG_ERR_HIP = -5
MG_ERR_NOT_INIT = -6

_STATUS_NAMES = {
    MG_ERR_BAD_ARG: "MG_ERR_BAD_ARG",
    MG_ERR_UNSUPPORTED: "MG_ERR_UNSUPPORTED",
    MG_ERR_NO_DEVICE: "MG_ERR_NO_DEVICE",
    MG_ERR_OOM: "MG_ERR_OOM",
    MG_ERR_HIP: "MG_ERR_HIP",
    MG_ERR_NOT_INIT: "MG_ERR_NOT_INIT",
}

_I64x3 = ctypes.c_int64 * MG_MAX_ND


class HipUnavailable(RuntimeError):
    """The HIP library could not be loaded or no gfx950 device is usable."""


class HipError(RuntimeError):
    """A library call returned a non-zero status."""

    def __init__(self, status, message):
        super().__init__(f"{_STATUS_NAMES.get(status, status)}: {message}")
        self.status = status


class ConvDesc(ctypes.Structure):
    _fields_ = [
        ("dtype", ctypes.c_int32),
        ("nd", ctypes.c_int32),
        ("N", ctypes.c_int64),
        ("C", ctypes.c_int64),
        ("F", ctypes.c_int64),
        ("X", _I64x3),
        ("W", _I64x3),
        ("G", _I64x3),
        ("stride", _I64x3),
        ("pad", _I64x3),
        ("dil", _I64x3),
    ]


class PoolDesc(ctypes.Structure):
    _fields_ = [
        ("dtype", ctypes.c_int32),
        ("dx_dtype", ctypes.c_int32),
        ("nd", ctypes.c_int32),
        ("reserved", ctypes.c_int32),
        ("lead", ctypes.c_int64),
        ("X", _I64x3),
        ("P", _I64x3),
        ("S", _I64x3),
        ("G", _I64x3),
    ]


class BnDesc(ctypes.Structure):
    _fields_ = [
        ("dtype", ctypes.c_int32),
        ("has_gamma", ctypes.c_int32),
        ("has_beta", ctypes.c_int32),
        ("reserved", ctypes.c_int32),
        ("N", ctypes.c_int64),
        ("C", ctypes.c_int64),
        ("S", ctypes.c_int64),
        ("eps", ctypes.c_double),
    ]


class WindowDesc(ctypes.Structure):
    _fields_ = [
        ("elem_bytes", ctypes.c_int32),
        ("nd", ctypes.c_int32),
        ("lead", ctypes.c_int64),
        ("X", _I64x3),
        ("W", _I64x3),
        ("S", _I64x3),
        ("D", _I64x3),
        ("G", _I64x3),
    ]


class DeviceInfo(ctypes.Structure):
    _fields_ = [
        ("name", ctypes.c_char * 64),
        ("compute_units", ctypes.c_int32),
        ("clock_khz", ctypes.c_int32),
        ("wavefront", ctypes.c_int32),
        ("lds_bytes_per_block", ctypes.c_int32),
        ("hbm_bytes", ctypes.c_int64),
        ("l2_bytes", ctypes.c_int32),
        ("memory_clock_khz", ctypes.c_int32),
        ("memory_bus_bits", ctypes.c_int32),
        ("reserved", ctypes.c_int32),
    ]


_vp = ctypes.c_void_p
_SIGNATURES = {
    "mg_init": [ctypes.c_int],
    "mg_shutdown": [],
    "mg_device_info": [ctypes.POINTER(DeviceInfo)],
    "mg_malloc": [ctypes.POINTER(_vp), ctypes.c_size_t],
    "mg_free": [_vp],
    "mg_host_alloc": [ctypes.POINTER(_vp), ctypes.c_size_t],
    "mg_host_free": [_vp],
    "mg_memcpy_h2d": [_vp, _vp, ctypes.c_size_t],
    "mg_memcpy_d2h": [_vp, _vp, ctypes.c_size_t],
    "mg_memcpy_d2d": [_vp, _vp, ctypes.c_size_t],
    "mg_memset_zero": [_vp, ctypes.c_size_t],
    "mg_sync": [],
    "mg_timing_enable": [ctypes.c_int],
    "mg_timing_pause": [ctypes.c_int],
    "mg_timing_read": [ctypes.POINTER(ctypes.c_int32), ctypes.POINTER(ctypes.c_float), ctypes.c_int,
                       ctypes.POINTER(ctypes.c_int)],
    "mg_probe_mfma": [ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_double)],
    "mg_probe_stream": [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int, ctypes.c_int,
                        ctypes.POINTER(ctypes.c_float)],
    "mg_event_create": [ctypes.POINTER(_vp)],
    "mg_event_record": [_vp],
    "mg_event_elapsed_ms": [_vp, _vp, ctypes.POINTER(ctypes.c_float)],
    "mg_event_destroy": [_vp],
    "mg_conv_fwd": [ctypes.POINTER(ConvDesc), _vp, _vp, _vp],
    "mg_conv_dgrad": [ctypes.POINTER(ConvDesc), _vp, _vp, _vp],
    "mg_conv_wgrad": [ctypes.POINTER(ConvDesc), _vp, _vp, _vp],
    "mg_maxpool_fwd": [ctypes.POINTER(PoolDesc), _vp, _vp],
    "mg_maxpool_bwd": [ctypes.POINTER(PoolDesc), _vp, _vp, _vp],
    "mg_maxpool_fwd_argmax": [ctypes.POINTER(PoolDesc), _vp, _vp, _vp],
    "mg_maxpool_bwd_argmax": [ctypes.POINTER(PoolDesc), _vp, _vp, _vp],
    "mg_maxpool_bwd_argmax_staged": [ctypes.POINTER(PoolDesc), ctypes.POINTER(PoolDesc), _vp, _vp, _vp, _vp],
    "mg_maxpool_bwd_argmax_staged3": [ctypes.POINTER(PoolDesc), ctypes.POINTER(PoolDesc), ctypes.POINTER(PoolDesc), _vp, _vp, _vp, _vp, _vp],
    "mg_multiply": [ctypes.c_int, ctypes.c_int64, _vp, _vp, _vp],
    "mg_multiply_broadcast": [ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_int64), ctypes.POINTER(ctypes.c_int64),
                              ctypes.POINTER(ctypes.c_int64), _vp, _vp, _vp],
    "mg_relu_fwd": [ctypes.c_int, ctypes.c_int64, _vp, _vp],
    "mg_relu_bwd": [ctypes.c_int, ctypes.c_int64, _vp, _vp, _vp],
    "mg_relu_fwd_mask": [ctypes.c_int, ctypes.c_int64, _vp, _vp, _vp],
    "mg_relu_bwd_mask": [ctypes.c_int, ctypes.c_int64, _vp, _vp, _vp],
    "mg_sum_all": [ctypes.c_int, ctypes.c_int64, _vp, _vp],
    "mg_sum_all_static": [ctypes.c_int, ctypes.c_int64, _vp, _vp],
    "mg_fill_from": [ctypes.c_int, ctypes.c_int64, _vp, _vp],
    "mg_cast": [ctypes.c_int, ctypes.c_int, ctypes.c_int64, _vp, _vp],
    "mg_accumulate": [ctypes.c_int, ctypes.c_int, ctypes.c_int64, _vp, _vp],
    "mg_fill_value": [ctypes.c_int, ctypes.c_int64, ctypes.c_double, _vp],
    "mg_sum_over": [ctypes.c_int] + [ctypes.c_int64] * 3 + [ctypes.c_int, _vp, _vp],
    "mg_sum_product_over": [ctypes.c_int] + [ctypes.c_int64] * 3 + [ctypes.c_int, _vp, _vp, _vp],
    "mg_batchnorm_fwd": [ctypes.POINTER(BnDesc), _vp, _vp, _vp, _vp, _vp, _vp],
    "mg_batchnorm_bwd": [ctypes.POINTER(BnDesc), _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp],
    "mg_matmul": [ctypes.c_int] + [ctypes.c_int64] * 4 + [_vp, _vp, _vp],
    "mg_matmul_batched": [ctypes.c_int] + [ctypes.c_int64] * 4 + [ctypes.c_int, ctypes.c_int, _vp, _vp, _vp],
    "mg_matmul_da": [ctypes.c_int] + [ctypes.c_int64] * 4 + [_vp, _vp, _vp],
    "mg_matmul_dx": [ctypes.c_int] + [ctypes.c_int64] * 4 + [_vp, _vp, _vp],
    "mg_repeat_fwd": [ctypes.c_int] + [ctypes.c_int64] * 5 + [_vp, _vp, _vp],
    "mg_repeat_bwd": [ctypes.c_int] + [ctypes.c_int64] * 5 + [_vp, _vp, _vp],
    "mg_window_gather": [ctypes.POINTER(WindowDesc), _vp, _vp],
    "mg_strided_copy": [ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_int64), ctypes.POINTER(ctypes.c_int64), ctypes.c_int64,
                        ctypes.c_int, _vp, _vp],
    "mg_permute": [ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_int64), ctypes.POINTER(ctypes.c_int32), _vp, _vp],
}
EXPORTED_SYMBOLS = tuple(_SIGNATURES) + ("mg_last_error", "mg_last_plan")

_lock = threading.Lock()
_lib = None
_ready = False


def library_path():
    """Path of the shared library: ``$MYGRAD_HIP_LIB`` or the in-tree build."""
    return os.environ.get("MYGRAD_HIP_LIB") or os.path.join(
        os.path.dirname(os.path.abspath(__file__)), "libmygrad_hip.so"
    )


def load_library():
    """dlopen the library and declare the prototypes (no device needed)."""
    global _lib
    with _lock:
        if _lib is None:
            path = library_path()
            if not os.path.exists(path):
                raise HipUnavailable(
                    f"{path} does not exist; build it with `python -m mygrad_amd.build` "
                    "(there is no CPU fallback)"
                )
            try:
                lib = ctypes.CDLL(path)
            except OSError as exc:
                raise HipUnavailable(f"cannot load {path}: {exc}") from exc
            for name, argtypes in _SIGNATURES.items():
                fn = getattr(lib, name)
                fn.argtypes = argtypes
                fn.restype = ctypes.c_int
            lib.mg_last_error.argtypes = []
            lib.mg_last_error.restype = ctypes.c_char_p
            lib.mg_last_plan.argtypes = []
            lib.mg_last_plan.restype = ctypes.c_char_p
            _lib = lib
    return _lib


def last_error():
    return load_library().mg_last_error().decode("utf-8", "replace")


def last_plan():
    """Which kernel family, tile and split the most recent conv / pool call ran on (diagnostics)."""
    return lib().mg_last_plan().decode("utf-8", "replace")


def check(status):
    if status != MG_OK:
        raise HipError(status, last_error())


def lib():
    """The loaded library with the device initialised; raises HipUnavailable otherwise."""
    global _ready
    if _ready:
        return _lib
    handle = load_library()
    if not _ready:
        device = int(os.environ.get("MYGRAD_HIP_DEVICE", "0"))
        status = handle.mg_init(device)
        if status != MG_OK:
            raise HipUnavailable(
                f"mg_init({device}) failed: {_STATUS_NAMES.get(status, status)}: {last_error()} "
                "(there is no CPU fallback)"
            )
        _ready = True
    return handle


def is_available():
    """True when the library loads and a gfx950 device initialises."""
    try:
        lib()
        return True
    except HipUnavailable:
        return False


def device_info():
    info = DeviceInfo()
    check(lib().mg_device_info(ctypes.byref(info)))
    return {name: (getattr(info, name).decode() if name == "name" else getattr(info, name))
            for name, _ in DeviceInfo._fields_ if name != "reserved"}


def synchronize():
    check(lib().mg_sync())


KERNEL_TAGS = {
    1: "conv_fwd",
    2: "conv_dgrad",
    3: "conv_wgrad",
    4: "wgrad_reduce",
    5: "pack_filters",
    6: "maxpool_fwd",
    7: "maxpool_bwd",
    8: "copy",
    9: "elementwise",
    10: "sum_all",
    11: "batchnorm_stats",
    12: "batchnorm_apply",
    13: "batchnorm_bwd_sums",
    14: "batchnorm_bwd_apply",
    15: "repeat_fwd",
    16: "repeat_bwd",
    17: "window_gather",
    18: "sum_over",
    19: "permute",
    20: "batched_product",
}


def timing_enable(on=True):
    """Start (or stop) bracketing every kernel launch with HIP events."""
    check(lib().mg_timing_enable(1 if on else 0))


def timing_pause(paused=True):
    """Suspend / resume the recording of launches without waiting for the stream."""
    check(lib().mg_timing_pause(1 if paused else 0))


def timing_read(capacity=1 << 16):
    """[(kernel name, milliseconds), ...] for the launches since the last read."""
    tags = (ctypes.c_int32 * capacity)()
    ms = (ctypes.c_float * capacity)()
    count = ctypes.c_int()
    check(lib().mg_timing_read(tags, ms, capacity, ctypes.byref(count)))
    n = min(count.value, capacity)
    return [(KERNEL_TAGS.get(tags[i], str(tags[i])), float(ms[i])) for i in range(n)]


MFMA_KINDS = {"f32_16x16x4": 0, "f64_16x16x4": 1, "f64_4x4x4_4b": 2}


def probe_mfma(kind, waves_per_simd=2):
    """TFLOP/s the matrix cores sustain on one MFMA shape with nothing else in the way."""
    out = ctypes.c_double()
    check(lib().mg_probe_mfma(MFMA_KINDS[kind], int(waves_per_simd), ctypes.byref(out)))
    return out.value


def probe_stream(big_ptr, small_ptr, big_bytes, share, store_big):
    """Milliseconds of one launch that stores (or loads) `big_bytes` while the opposite
    stream moves 1 / share of that volume (share 0: no second stream)."""
    out = ctypes.c_float()
    check(lib().mg_probe_stream(big_ptr, small_ptr, int(big_bytes), int(share), int(bool(store_big)), ctypes.byref(out)))
    return out.value


def _right_aligned(values, fill):
    values = [int(v) for v in values]
    if len(values) > MG_MAX_ND:
        raise ValueError(f"rank {len(values)} exceeds {MG_MAX_ND}")
    return _I64x3(*([fill] * (MG_MAX_ND - len(values)) + values))


def dtype_code(dtype):
    import numpy as np

    dtype = np.dtype(dtype)
    if dtype == np.float32:
        return MG_F32
    if dtype == np.float64:
        return MG_F64
    raise TypeError(f"the HIP kernels handle float32 and float64 only, got {dtype}")


def storage_code(dtype):
    """``dtype_code`` for the two conversions (``mg_cast``, ``mg_accumulate``), which also take
    float16: a type arrays are stored in, not one any kernel computes in."""
    import numpy as np

    return MG_F16 if np.dtype(dtype) == np.float16 else dtype_code(dtype)


def conv_desc(dtype, x_shape, w_shape, grid, stride, padding, dilation):
    """Descriptor for x:(N,C,X...) * w:(F,C,W...) -> (N,F,grid...)."""
    m = len(x_shape) - 2
    return ConvDesc(
        dtype=dtype_code(dtype),
        nd=m,
        N=int(x_shape[0]),
        C=int(x_shape[1]),
        F=int(w_shape[0]),
        X=_right_aligned(x_shape[2:], 1),
        W=_right_aligned(w_shape[2:], 1),
        G=_right_aligned(grid, 1),
        stride=_right_aligned(stride, 1),
        pad=_right_aligned(padding, 0),
        dil=_right_aligned(dilation, 1),
    )


def pool_desc(dtype, lead, pooled_shape, pool, stride, grid, dx_dtype=None):
    return PoolDesc(
        dtype=dtype_code(dtype),
        dx_dtype=dtype_code(dtype if dx_dtype is None else dx_dtype),
        nd=len(pool),
        reserved=0,
        lead=int(lead),
        X=_right_aligned(pooled_shape, 1),
        P=_right_aligned(pool, 1),
        S=_right_aligned(stride, 1),
        G=_right_aligned(grid, 1),
    )


_shared_descs = {}


def shared_desc(build, *args, **kwargs):
    """``build(*args, **kwargs)`` (one of the descriptor builders above and below), built once per
    distinct set of arguments and handed out again: for the operations, which describe the same
    layer at every step and never write to a descriptor.  Arguments that do not hash (lists,
    arrays) get a descriptor of their own."""
    try:
        key = (build, args, tuple(kwargs.items()))
        desc = _shared_descs.get(key)
    except TypeError:
        return build(*args, **kwargs)
    if desc is None:
        if len(_shared_descs) >= 4096:
            _shared_descs.clear()
        desc = _shared_descs[key] = build(*args, **kwargs)
    return desc


def bn_desc(shape, dtype, has_gamma, has_beta, eps):
    """Descriptor of a batch normalisation of an array of `shape` = (N, C, ...)."""
    spatial = 1
    for d in shape[2:]:
        spatial *= int(d)
    return BnDesc(
        dtype=dtype_code(dtype),
        has_gamma=int(bool(has_gamma)),
        has_beta=int(bool(has_beta)),
        reserved=0,
        N=int(shape[0]),
        C=int(shape[1]),
        S=spatial,
        eps=float(eps),
    )


def window_desc(itemsize, lead, windowed_shape, window_shape, step, dilation, grid):
    """Descriptor of a sliding-window view over the trailing axes of an array."""
    return WindowDesc(
        elem_bytes=int(itemsize),
        nd=len(window_shape),
        lead=int(lead),
        X=_right_aligned(windowed_shape, 1),
        W=_right_aligned(window_shape, 1),
        S=_right_aligned(step, 1),
        D=_right_aligned(dilation, 1),
        G=_right_aligned(grid, 1),
    )
