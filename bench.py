#!/usr/bin/env python3
"""Benchmark of the conv_nd / max_pool hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--all]

A step is one pass of the hot path over one batch of synthetic input that is
already resident in HBM: forward + data gradient + filter gradient for a
convolution workload, forward + backward for a pooling workload, each through
the C ABI of libmygrad_hip.so.  The script prints ONE JSON line:

* ``value``        whole-step throughput from the host clock around the K steps
                   (algorithmic flops or bytes / wall time, library stream drained
                   on both sides).  Before the W warm-up steps the step runs untimed
                   for ``--prewarm`` seconds (0.4 by default, reported under
                   ``prewarm``) so that the device clock has settled;
* ``roofline``     the dominant kernel of the step: algorithmic flops (or bytes)
                   of one launch / its mean duration between HIP events recorded
                   on the library stream inside the timed region;
* ``cpu_baseline`` the NumPy restatement of the reference algorithm timed on the
                   host cores on a bounded sample of the same workload;
* ``secondary``    the same figures for the hot path's other configurations (the max_pool
                   half of the metric and the other convolution shapes; every workload
                   with --all, none with --no-secondary).

Algorithmic work:  convolution 2*N*F*prod(G)*C*prod(W) flops per pass (padding
taps count, dense definition); pooling |x|+|out| bytes forward and
|x|+|grad|+|dx| bytes backward.
"""

import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_TFLOPS = {"f32": 157.3, "f64": 78.6}  # MI355X dense matrix peaks
PEAK_HBM_GBS = 8000.0

# name -> definition.  "lit" shapes use the flooring placement of the window
# helper (the Operation-level validator of the reference rejects them).
WORKLOADS = {
    "conv1": dict(kind="conv", dtype="f64", seed=1001, x=(32, 3, 32, 32), w=(16, 3, 3, 3), wscale=27 ** -0.5,
                  stride=(1, 1), padding=(1, 1), dilation=(1, 1)),
    "conv3a": dict(kind="conv", dtype="f32", seed=1003, x=(128, 64, 56, 56), w=(64, 64, 3, 3), wscale=(2 / 576) ** 0.5,
                   stride=(1, 1), padding=(1, 1), dilation=(1, 1)),
    "conv3b": dict(kind="conv", dtype="f32", seed=1004, x=(128, 128, 28, 28), w=(256, 128, 3, 3),
                   wscale=(2 / 1152) ** 0.5, stride=(2, 2), padding=(1, 1), dilation=(1, 1)),
    "conv4": dict(kind="conv", dtype="f64", seed=1005, x=(16, 32, 128, 128), w=(32, 32, 5, 5), wscale=800 ** -0.5,
                  stride=(2, 1), padding=(4, 4), dilation=(2, 2)),
    "conv5": dict(kind="conv", dtype="f32", seed=1006, x=(8, 16, 32, 64, 64), w=(32, 16, 3, 3, 3),
                  wscale=(2 / 432) ** 0.5, stride=(1, 1, 1), padding=(1, 1, 1), dilation=(1, 1, 1)),
    # a ResNet stem: three input channels, a 7x7 filter bank, stride 2 (flooring placement: the last
    # padded row and column are never read).  Its input is the data batch, a constant: like the
    # reference (Operation.backward skips constant variables, operation_base.py:216-228) a step
    # computes no dx.  `stem-dx` is the same layer with dx, for an input that does take a gradient.
    "stem": dict(kind="conv", dtype="f32", seed=1017, x=(128, 3, 224, 224), w=(64, 3, 7, 7), wscale=(2 / 147) ** 0.5,
                 stride=(2, 2), padding=(3, 3), dilation=(1, 1), constant_input=True),
    "stem-dx": dict(kind="conv", dtype="f32", seed=1017, x=(128, 3, 224, 224), w=(64, 3, 7, 7), wscale=(2 / 147) ** 0.5,
                    stride=(2, 2), padding=(3, 3), dilation=(1, 1)),
    # the same stem in double precision, the reference's default dtype (half the batch: the same bytes)
    "stem64": dict(kind="conv", dtype="f64", seed=1017, x=(64, 3, 224, 224), w=(64, 3, 7, 7), wscale=(2 / 147) ** 0.5,
                   stride=(2, 2), padding=(3, 3), dilation=(1, 1), constant_input=True),
    "stem64-dx": dict(kind="conv", dtype="f64", seed=1017, x=(64, 3, 224, 224), w=(64, 3, 7, 7), wscale=(2 / 147) ** 0.5,
                      stride=(2, 2), padding=(3, 3), dilation=(1, 1)),
    "pool2": dict(kind="pool", dtype="f64", seed=1002, x=(64, 64, 56, 56), pool=(3, 3), stride=(2, 2)),
    "pool5": dict(kind="pool", dtype="f32", seed=1006, x=(8, 32, 32, 64, 64), pool=(2, 2, 2), stride=(2, 2, 2)),
    # the same two with each window's argmax recomputed from x in the backward pass (the stateless
    # pair of entry points) instead of remembered from the forward pass
    "pool2-recompute": dict(kind="pool", dtype="f64", seed=1002, x=(64, 64, 56, 56), pool=(3, 3), stride=(2, 2),
                            recompute=True),
    "pool5-recompute": dict(kind="pool", dtype="f32", seed=1006, x=(8, 32, 32, 64, 64), pool=(2, 2, 2),
                            stride=(2, 2, 2), recompute=True),
    # The neighbours of configurations 2, 3b and 4 that the reference's validator accepts (an exact
    # window grid: pooling.py:79-86, conv.py:63-74): what max_pool() / conv_nd() can be called with.
    "pool2-valid": dict(kind="pool", dtype="f64", seed=1002, x=(64, 64, 55, 55), pool=(3, 3), stride=(2, 2)),
    "pool2-valid-recompute": dict(kind="pool", dtype="f64", seed=1002, x=(64, 64, 55, 55), pool=(3, 3), stride=(2, 2),
                                  recompute=True),
    "conv3b-valid": dict(kind="conv", dtype="f32", seed=1004, x=(128, 128, 27, 27), w=(256, 128, 3, 3),
                         wscale=(2 / 1152) ** 0.5, stride=(2, 2), padding=(1, 1), dilation=(1, 1)),
    "conv4-valid": dict(kind="conv", dtype="f64", seed=1005, x=(16, 32, 127, 128), w=(32, 32, 5, 5), wscale=800 ** -0.5,
                        stride=(2, 1), padding=(4, 4), dilation=(2, 2)),
    # relu, multiply and sum (forward and gradients) on a tensor of conv5's output size
    "elem5": dict(kind="elem", dtype="f32", seed=1007, x=(8, 32, 32, 64, 64)),
    # batch normalisation (scaled and shifted) of a tensor of conv3a's output size
    "bn3a": dict(kind="bn", dtype="f32", seed=1008, x=(128, 64, 56, 56), eps=1e-5),
    # matrix product on the convolution kernels: one dense layer's three products
    "bmm64": dict(kind="bmm", dtype="f32", seed=1016, batch=512, M=64, K=64, N=64),
    # the same products in a stack sixteen times as tall: 134 MB per launch instead of 8, so that the
    # kernel's rate shows and not the few microseconds any launch takes
    "bmm64-tall": dict(kind="bmm", dtype="f32", seed=1016, batch=8192, M=64, K=64, N=64),
    "mm4k": dict(kind="matmul", dtype="f32", seed=1011, M=4096, K=4096, N=4096),
    # sums over axes of a tensor of conv5's output size: per channel (the gradient of a bias or of a
    # per-channel scale: every axis but axis 1), then over the channel axis alone
    "scale5": dict(kind="scale", dtype="f32", seed=1015, x=(8, 32, 32, 64, 64), others=((32, 1, 1, 1), (64,))),
    "sum5": dict(kind="sumover", dtype="f32", seed=1012, x=(8, 32, 32, 64, 64), axes=((0, 2, 3, 4), (1,))),
    # transposition of a tensor of conv5's output size: channels last (N,C,D,H,W -> N,D,H,W,C) and back
    "perm5": dict(kind="permute", dtype="f32", seed=1013, x=(8, 32, 32, 64, 64), perms=((0, 2, 3, 4, 1), (0, 4, 1, 2, 3))),
    # Einstein summation: a 1x1 convolution written as 'nchw,fc->nfhw' and its two gradients
    # (operands transposed on the device, product on the convolution kernels, result transposed back)
    "ein1x1": dict(kind="einsum", dtype="f32", seed=1014, x=(32, 256, 56, 56), w=(256, 256),
                   subscripts=("nchw", "fc", "nfhw")),
    # repeat: twofold nearest-neighbour upsampling of the rows of a tensor of pool5's input size
    # (forward and gradient), and then of its columns
    "rep5": dict(kind="repeat", dtype="f32", seed=1009, x=(8, 32, 32, 64, 64), repeats=2, axes=(-2, -1)),
    # the dense copy of the window view the 3x3 convolution of config 3a reads (a quarter of its batch)
    "win3a": dict(kind="window", dtype="f32", seed=1010, x=(32, 64, 56, 56), window=(3, 3), step=(1, 1), dilation=(1, 1)),
}
NP_DTYPE = {"f32": np.float32, "f64": np.float64}
# the configurations of the hot path itself: reported by every default run
HOT_PATH = ["conv3a", "conv3b", "conv4", "conv5", "conv1", "pool2", "pool5", "pool2-recompute", "pool5-recompute",
            "pool2-valid", "pool2-valid-recompute", "conv3b-valid", "conv4-valid"]


def _sweep_shapes():
    """Reference-valid shapes around the benchmark's: what `--sweep` runs, pass by pass."""
    he = lambda w: (2.0 / (w[1] * int(np.prod(w[2:])))) ** 0.5
    shapes = {}

    def conv(name, dtype, x, w, stride, padding, dilation):
        m = len(x) - 2
        as_tuple = lambda v: (v,) * m if isinstance(v, int) else tuple(v)
        shapes[name] = dict(kind="conv", dtype=dtype, seed=2000 + len(shapes), x=x, w=w, wscale=he(w), stride=as_tuple(stride),
                            padding=as_tuple(padding), dilation=as_tuple(dilation))

    def pool(name, dtype, x, window, stride):
        for suffix, extra in (("", {}), ("-recompute", {"recompute": True})):
            shapes[name + suffix] = dict(kind="pool", dtype=dtype, seed=2100 + len(shapes), x=x, pool=window,
                                         stride=(stride,) * len(window), **extra)

    # 3x3, stride 1, padding 1: the stages of a residual network
    conv("c3x3-64@56", "f32", (128, 64, 56, 56), (64, 64, 3, 3), 1, 1, 1)
    conv("c3x3-128@28", "f32", (128, 128, 28, 28), (128, 128, 3, 3), 1, 1, 1)
    conv("c3x3-256@14", "f32", (128, 256, 14, 14), (256, 256, 3, 3), 1, 1, 1)
    conv("c3x3-512@7", "f32", (128, 512, 7, 7), (512, 512, 3, 3), 1, 1, 1)
    conv("c3x3-64@56-f64", "f64", (64, 64, 56, 56), (64, 64, 3, 3), 1, 1, 1)
    # 3x3, stride 2, padding 1 on the odd extents an exact grid needs
    conv("c3x3s2-64@55", "f32", (128, 64, 55, 55), (128, 64, 3, 3), 2, 1, 1)
    conv("c3x3s2-128@27", "f32", (128, 128, 27, 27), (256, 128, 3, 3), 2, 1, 1)
    conv("c3x3s2-256@13", "f32", (128, 256, 13, 13), (512, 256, 3, 3), 2, 1, 1)
    # 1x1: the bottleneck's two ends, and a strided shortcut
    conv("c1x1-256to64@56", "f32", (128, 256, 56, 56), (64, 256, 1, 1), 1, 0, 1)
    conv("c1x1-64to256@56", "f32", (128, 64, 56, 56), (256, 64, 1, 1), 1, 0, 1)
    conv("c1x1s2-256to512@55", "f32", (128, 256, 55, 55), (512, 256, 1, 1), 2, 0, 1)
    # 5x5, dilation 2
    conv("c5x5d2-64@56", "f32", (32, 64, 56, 56), (64, 64, 5, 5), 1, 4, 2)
    conv("c5x5d2s21-32@127-f64", "f64", (16, 32, 127, 128), (32, 32, 5, 5), (2, 1), 4, 2)
    # three convolved axes
    conv("c3x3x3-16to32@32x64x64", "f32", (8, 16, 32, 64, 64), (32, 16, 3, 3, 3), 1, 1, 1)
    conv("c3x3x3-32to64@16x32x32", "f32", (8, 32, 16, 32, 32), (64, 32, 3, 3, 3), 1, 1, 1)
    # pooling: 3x3 every other position (odd extents), 2x2 tiling, overlapping 3-D windows
    pool("p3x3s2@55-f64", "f64", (64, 64, 55, 55), (3, 3), 2)
    pool("p3x3s2@55-f32", "f32", (128, 64, 55, 55), (3, 3), 2)
    pool("p3x3s2@113-f32", "f32", (32, 64, 113, 113), (3, 3), 2)
    pool("p3x3s2@113-f64", "f64", (16, 64, 113, 113), (3, 3), 2)
    pool("p2x2s2@14-f32", "f32", (128, 512, 14, 14), (2, 2), 2)
    pool("p2x2s2@28-f32", "f32", (128, 256, 28, 28), (2, 2), 2)
    pool("p2x2s2@112-f32", "f32", (32, 64, 112, 112), (2, 2), 2)
    pool("p2x2s2@14-f64", "f64", (128, 256, 14, 14), (2, 2), 2)
    pool("p3x3x3s2@33x65x65-f32", "f32", (8, 32, 33, 65, 65), (3, 3, 3), 2)
    pool("p2x2x2s2@32x64x64-f32", "f32", (8, 32, 32, 64, 64), (2, 2, 2), 2)
    return shapes


SWEEP = _sweep_shapes()
WORKLOADS.update(SWEEP)


def conv_grid(wl):
    return tuple(
        (x + 2 * p - ((t - 1) * d + 1)) // s + 1
        for x, t, s, p, d in zip(wl["x"][2:], wl["w"][2:], wl["stride"], wl["padding"], wl["dilation"])
    )


def elem_bytes(x):
    """Algorithmic bytes of sum(relu(x) * g) and its gradients: 15 passes over an array of x's
    size and relu's mask, one bit per element, written once and read once."""
    return 15.0 * x.nbytes + 2.0 * ((x.size + 7) // 8)


def conv_passes(wl):
    return "fwd+dw (constant input: no dx)" if wl.get("constant_input") else "fwd+dx+dw"


def conv_flops_per_pass(wl, batch=None):
    n = wl["x"][0] if batch is None else batch
    return 2.0 * n * wl["w"][0] * np.prod(conv_grid(wl)) * wl["x"][1] * np.prod(wl["w"][2:])


def pool_shapes(wl):
    m = len(wl["pool"])
    lead, pooled = wl["x"][: len(wl["x"]) - m], wl["x"][len(wl["x"]) - m:]
    grid = tuple((x - p) // s + 1 for x, p, s in zip(pooled, wl["pool"], wl["stride"]))
    return lead, pooled, grid


def describe(name):
    wl = WORKLOADS[name]
    if wl["kind"] == "elem":
        return f"{name}: relu + multiply + sum {wl['dtype']} x{wl['x']} fwd+bwd (7 kernels, 15 |x| bytes + relu's mask)"
    if wl["kind"] == "bmm":
        return (f"{name}: matmul {wl['dtype']} of two stacks ({wl['batch']},{wl['M']},{wl['K']}) @ ({wl['batch']},{wl['K']},{wl['N']}): "
                "product + both gradients")
    if wl["kind"] == "matmul":
        return f"{name}: matmul {wl['dtype']} ({wl['M']},{wl['K']}) @ ({wl['K']},{wl['N']}): product + both gradients"
    if wl["kind"] == "permute":
        return f"{name}: transpose {wl['dtype']} x{wl['x']} by {wl['perms'][0]}, then the result by {wl['perms'][1]}"
    if wl["kind"] == "einsum":
        a, b, o = wl["subscripts"]
        return f"{name}: einsum '{a},{b}->{o}' {wl['dtype']} x{wl['x']} w{wl['w']} and both gradients"
    if wl["kind"] == "scale":
        return f"{name}: multiply {wl['dtype']} x{wl['x']} by an operand of shape {wl['others'][0]}, then by one of shape {wl['others'][1]}"
    if wl["kind"] == "sumover":
        return f"{name}: sum {wl['dtype']} x{wl['x']} over axes {wl['axes'][0]}, then over axes {wl['axes'][1]}"
    if wl["kind"] == "repeat":
        return f"{name}: repeat {wl['dtype']} x{wl['x']} repeats={wl['repeats']} along axis {wl['axes'][0]}, then along axis {wl['axes'][1]}, fwd+bwd each"
    if wl["kind"] == "window":
        return (f"{name}: contiguous copy of sliding_window_view {wl['dtype']} x{wl['x']} window{wl['window']} "
                f"step{wl['step']} dilation{wl['dilation']}")
    if wl["kind"] == "bn":
        return f"{name}: batchnorm {wl['dtype']} x{wl['x']} with gamma and beta, eps={wl['eps']}, fwd + dx, dgamma, dbeta"
    if wl["kind"] == "conv":
        return (f"{name}: conv_nd {wl['dtype']} x{wl['x']} * w{wl['w']} stride{wl['stride']} pad{wl['padding']} "
                f"dil{wl['dilation']} -> grid{conv_grid(wl)} {conv_passes(wl)}")
    lead, pooled, grid = pool_shapes(wl)
    how = "argmax recomputed from x in bwd" if wl.get("recompute") else "argmax kept from fwd, one byte per window"
    return f"{name}: max_pool {wl['dtype']} x{wl['x']} pool{wl['pool']} stride{wl['stride']} -> grid{grid} fwd+bwd ({how})"


class Step:
    """Device-resident inputs and outputs of one workload and its step function."""

    def __init__(self, name):
        from mygrad_amd import _device, _hip

        self.name, self.wl = name, WORKLOADS[name]
        wl, dt = self.wl, NP_DTYPE[WORKLOADS[name]["dtype"]]
        rng = np.random.default_rng(wl["seed"])
        self.lib = _hip.lib()
        self.check = _hip.check
        item = np.dtype(dt).itemsize

        def resident(arr):
            buf = _device.DeviceBuffer(arr.nbytes)
            buf.upload(arr)
            return buf

        if wl["kind"] == "conv":
            grid = conv_grid(wl)
            out_shape = (wl["x"][0], wl["w"][0], *grid)
            x = rng.standard_normal(wl["x"]).astype(dt)
            w = (rng.standard_normal(wl["w"]) * wl["wscale"]).astype(dt)
            g = rng.standard_normal(out_shape).astype(dt)
            self.desc = _hip.conv_desc(dt, wl["x"], wl["w"], grid, wl["stride"], wl["padding"], wl["dilation"])
            self.x, self.w, self.g = resident(x), resident(w), resident(g)
            self.out = _device.DeviceBuffer(int(np.prod(out_shape)) * item)
            self.dx = _device.DeviceBuffer(x.nbytes)
            self.dw = _device.DeviceBuffer(w.nbytes)
            per_pass = conv_flops_per_pass(wl)
            self.work = {"conv_fwd": per_pass, "conv_dgrad": per_pass, "conv_wgrad": per_pass}
            self.total_work = (2 if wl.get("constant_input") else 3) * per_pass
            self.unit, self.bound, self.peak = "TFLOP/s", "mfma", PEAK_TFLOPS[wl["dtype"]]
            self.scale = 1e-12
        elif wl["kind"] == "bmm":
            B, M, K, N = wl["batch"], wl["M"], wl["K"], wl["N"]
            self.w = resident((rng.standard_normal((B, M, K)) * K ** -0.5).astype(dt))
            self.x, self.g = resident(rng.standard_normal((B, K, N)).astype(dt)), resident(rng.standard_normal((B, M, N)).astype(dt))
            self.out, self.dx, self.dw = (_device.DeviceBuffer(B * n * item) for n in (M * N, K * N, M * K))
            self.code, self.dims = _hip.dtype_code(dt), (B, M, K, N)
            self.work = {"batched_product": 2.0 * B * M * K * N}
            self.total_work = 6.0 * B * M * K * N
            self.unit, self.bound, self.peak = "TFLOP/s", "mfma", PEAK_TFLOPS[wl["dtype"]]
            self.scale = 1e-12
            # Every pair is read and written once: 2MKN flops over (MK + KN + MN) values.  Below the
            # ridge of the two rooflines (peak flops / peak bytes per second) the products are bound
            # by HBM, and the roofline fraction is quoted against that ceiling; `value` stays in flops.
            pair_bytes = float(B * (M * K + K * N + M * N) * item)
            if self.work["batched_product"] / pair_bytes < self.peak * 1e12 / (PEAK_HBM_GBS * 1e9):
                self.roof = dict(bound="hbm", work={"batched_product": pair_bytes}, scale=1e-9, unit="GB/s", peak=PEAK_HBM_GBS)
        elif wl["kind"] == "matmul":
            M, K, N = wl["M"], wl["K"], wl["N"]
            a = (rng.standard_normal((M, K)) * K ** -0.5).astype(dt)
            x = rng.standard_normal((K, N)).astype(dt)
            g = rng.standard_normal((M, N)).astype(dt)
            self.w, self.x, self.g = resident(a), resident(x), resident(g)
            self.out, self.dx, self.dw = (_device.DeviceBuffer(n * item) for n in (M * N, K * N, M * K))
            self.code, self.dims = _hip.dtype_code(dt), (1, M, K, N)
            per_pass = 2.0 * M * K * N
            self.work = {"conv_fwd": per_pass, "conv_dgrad": per_pass, "conv_wgrad": per_pass}
            self.total_work = (2 if wl.get("constant_input") else 3) * per_pass
            self.unit, self.bound, self.peak = "TFLOP/s", "mfma", PEAK_TFLOPS[wl["dtype"]]
            self.scale = 1e-12
        elif wl["kind"] == "permute":
            x = rng.standard_normal(wl["x"]).astype(dt)
            self.x, self.out, self.back = resident(x), _device.DeviceBuffer(x.nbytes), _device.DeviceBuffer(x.nbytes)
            nd = x.ndim
            mid = tuple(wl["x"][p] for p in wl["perms"][0])
            self.calls = [((ctypes.c_int64 * nd)(*wl["x"]), (ctypes.c_int32 * nd)(*wl["perms"][0])),
                          ((ctypes.c_int64 * nd)(*mid), (ctypes.c_int32 * nd)(*wl["perms"][1]))]
            self.nd = nd
            self.work = {"permute": 2.0 * x.nbytes}
            self.total_work = 4.0 * x.nbytes
            self.unit, self.bound, self.peak = "GB/s", "hbm", PEAK_HBM_GBS
            self.scale = 1e-9
        elif wl["kind"] == "einsum":
            x = rng.standard_normal(wl["x"]).astype(dt)
            w = (rng.standard_normal(wl["w"]) * wl["w"][1] ** -0.5).astype(dt)
            la, lb, lo = wl["subscripts"]
            self.sizes = {**dict(zip(la, wl["x"])), **dict(zip(lb, wl["w"]))}
            g = rng.standard_normal(tuple(self.sizes[l] for l in lo)).astype(dt)
            self.x, self.w, self.g = resident(x), resident(w), resident(g)
            self.np_dtype = np.dtype(dt)
            per_pass = 2.0 * np.prod([float(v) for v in self.sizes.values()])
            self.work = {"conv_fwd": per_pass, "conv_wgrad": per_pass}
            self.total_work = 3 * per_pass
            self.unit, self.bound, self.peak = "TFLOP/s", "mfma", PEAK_TFLOPS[wl["dtype"]]
            self.scale = 1e-12
        elif wl["kind"] == "sumover":
            x = rng.standard_normal(wl["x"]).astype(dt)
            outer, n, inner = wl["x"][0], wl["x"][1], int(np.prod(wl["x"][2:]))
            self.dims, self.code = (outer, n, inner), _hip.dtype_code(dt)
            self.x = resident(x)
            self.out = _device.DeviceBuffer(outer * inner * item)
            # each launch reads x once; what it writes is 1/32 of that at most
            self.work = {"sum_over": float(x.nbytes)}
            self.total_work = 2.0 * x.nbytes
            self.unit, self.bound, self.peak = "GB/s", "hbm", PEAK_HBM_GBS
            self.scale = 1e-9
        elif wl["kind"] == "scale":
            from mygrad_amd import _reduce

            x = rng.standard_normal(wl["x"]).astype(dt)
            self.x, self.out, self.code = resident(x), _device.DeviceBuffer(x.nbytes), _hip.dtype_code(dt)
            self.others = []
            for shape in wl["others"]:
                extents, sa, sb = _reduce.multiply_plan(wl["x"], shape, wl["x"])
                as_array = ctypes.c_int64 * len(extents)
                self.others.append((len(extents), as_array(*extents), as_array(*sa), as_array(*sb),
                                    resident(rng.standard_normal(shape).astype(dt))))
            # each launch reads x and writes the product; the other operand is 1/1000 of that at most
            self.work = {"elementwise": 2.0 * x.nbytes}
            self.total_work = 4.0 * x.nbytes
            self.unit, self.bound, self.peak = "GB/s", "hbm", PEAK_HBM_GBS
            self.scale = 1e-9
        elif wl["kind"] == "repeat":
            x = rng.standard_normal(wl["x"]).astype(dt)
            r = wl["repeats"]
            g = rng.standard_normal((*wl["x"][:-1], wl["x"][-1] * r)).astype(dt)  # same size for either axis
            self.x, self.g = resident(x), resident(g)
            self.out, self.dx = _device.DeviceBuffer(g.nbytes), _device.DeviceBuffer(x.nbytes)
            self.geometry = []
            for axis in wl["axes"]:
                axis %= len(wl["x"])
                outer, n, inner = int(np.prod(wl["x"][:axis])), wl["x"][axis], int(np.prod(wl["x"][axis + 1:]))
                self.geometry.append((outer, n, inner, r, n * r))
            self.code = _hip.dtype_code(dt)
            self.work = {"repeat_fwd": float(x.nbytes + g.nbytes), "repeat_bwd": float(x.nbytes + g.nbytes)}
            self.total_work = 4.0 * (x.nbytes + g.nbytes)
            self.unit, self.bound, self.peak = "GB/s", "hbm", PEAK_HBM_GBS
            self.scale = 1e-9
        elif wl["kind"] == "window":
            x = rng.standard_normal(wl["x"]).astype(dt)
            m = len(wl["window"])
            tail = wl["x"][len(wl["x"]) - m:]
            grid = tuple((tail[k] - ((wl["window"][k] - 1) * wl["dilation"][k] + 1)) // wl["step"][k] + 1 for k in range(m))
            lead = int(np.prod(wl["x"][: len(wl["x"]) - m]))
            count = int(np.prod(grid)) * lead * int(np.prod(wl["window"]))
            self.desc = _hip.window_desc(item, lead, tail, wl["window"], wl["step"], wl["dilation"], grid)
            self.x = resident(x)
            self.out = _device.DeviceBuffer(count * item)
            self.work = {"window_gather": float(x.nbytes + count * item)}
            self.total_work = self.work["window_gather"]
            self.unit, self.bound, self.peak = "GB/s", "hbm", PEAK_HBM_GBS
            self.scale = 1e-9
        elif wl["kind"] == "bn":
            channels = wl["x"][1]
            x = (rng.standard_normal(wl["x"]) * 2 + 0.5).astype(dt)
            g = rng.standard_normal(wl["x"]).astype(dt)
            self.desc = _hip.bn_desc(wl["x"], dt, True, True, wl["eps"])
            self.x, self.g = resident(x), resident(g)
            self.gamma = resident(rng.uniform(0.5, 2, channels).astype(dt))
            self.beta = resident(rng.standard_normal(channels).astype(dt))
            self.out, self.dx = _device.DeviceBuffer(x.nbytes), _device.DeviceBuffer(x.nbytes)
            self.mean, self.var, self.dgamma, self.dbeta = (_device.DeviceBuffer(max(channels * item, 16)) for _ in range(4))
            # per launch: what each kernel must read and write; per step: x in and y out, then
            # x and grad in and dx out (a step that never re-read anything would move 5 |x|)
            self.work = {"batchnorm_stats": float(x.nbytes), "batchnorm_apply": 2.0 * x.nbytes,
                         "batchnorm_bwd_sums": 2.0 * x.nbytes, "batchnorm_bwd_apply": 3.0 * x.nbytes}
            self.total_work = 5.0 * x.nbytes
            self.unit, self.bound, self.peak = "GB/s", "hbm", PEAK_HBM_GBS
            self.scale = 1e-9
        elif wl["kind"] == "elem":
            x = rng.standard_normal(wl["x"]).astype(dt)
            g = rng.standard_normal(wl["x"]).astype(dt)
            self.n, self.code = x.size, _hip.dtype_code(dt)
            self.x, self.g = resident(x), resident(g)
            self.out, self.dx = _device.DeviceBuffer(x.nbytes), _device.DeviceBuffer(x.nbytes)
            self.scalar = _device.DeviceBuffer(16)
            self.mask = _device.DeviceBuffer((x.size + 7) // 8)
            # relu fwd and bwd 2|x| + the mask (one bit per element) each, multiply fwd and two
            # gradients 3|x| each, fill |x|: 6 launches
            self.work = {"elementwise": (elem_bytes(x) - x.nbytes) / 6, "sum_all": float(x.nbytes)}
            self.total_work = elem_bytes(x)
            self.unit, self.bound, self.peak = "GB/s", "hbm", PEAK_HBM_GBS
            self.scale = 1e-9
        else:
            lead, pooled, grid = pool_shapes(wl)
            out_shape = (*lead, *grid)
            x = rng.standard_normal(wl["x"]).astype(dt)
            g = rng.standard_normal(out_shape).astype(dt)
            self.desc = _hip.pool_desc(dt, int(np.prod(lead)), pooled, wl["pool"], wl["stride"], grid)
            self.x, self.g = resident(x), resident(g)
            self.out = _device.DeviceBuffer(g.nbytes)
            self.dx = _device.DeviceBuffer(x.nbytes)
            self.argmax = None if wl.get("recompute") else _device.DeviceBuffer(g.size)
            # algorithmic bytes of the stateless definition, |x| + |out| and |x| + |grad| + |dx|, whichever
            # pair runs: remembering the argmax moves fewer bytes than that in the backward pass
            self.work = {"maxpool_fwd": float(x.nbytes + g.nbytes), "maxpool_bwd": float(2 * x.nbytes + g.nbytes)}
            self.total_work = sum(self.work.values())
            # what the pair that keeps the argmax has to move: forward x, out and one byte per window,
            # backward those bytes, grad and dx -- x is not read again
            if self.argmax is not None:
                self.moved = {"maxpool_fwd": float(x.nbytes + g.nbytes + g.size), "maxpool_bwd": float(g.size + g.nbytes + x.nbytes)}
            self.unit, self.bound, self.peak = "GB/s", "hbm", PEAK_HBM_GBS
            self.scale = 1e-9

    def passes(self):
        """(label, callable, key of the pass in self.work) for each pass of a convolution or pooling step."""
        lib, check, d = self.lib, self.check, self.desc
        if self.wl["kind"] == "conv":
            out = [("fwd", lambda: check(lib.mg_conv_fwd(d, self.x.ptr, self.w.ptr, self.out.ptr)), "conv_fwd")]
            if not self.wl.get("constant_input"):
                out.append(("dx", lambda: check(lib.mg_conv_dgrad(d, self.g.ptr, self.w.ptr, self.dx.ptr)), "conv_dgrad"))
            out.append(("dw", lambda: check(lib.mg_conv_wgrad(d, self.g.ptr, self.x.ptr, self.dw.ptr)), "conv_wgrad"))
            return out
        assert self.wl["kind"] == "pool", self.wl["kind"]
        if self.argmax is None:
            return [("fwd", lambda: check(lib.mg_maxpool_fwd(d, self.x.ptr, self.out.ptr)), "maxpool_fwd"),
                    ("bwd", lambda: check(lib.mg_maxpool_bwd(d, self.x.ptr, self.g.ptr, self.dx.ptr)), "maxpool_bwd")]
        return [("fwd", lambda: check(lib.mg_maxpool_fwd_argmax(d, self.x.ptr, self.out.ptr, self.argmax.ptr)), "maxpool_fwd"),
                ("bwd", lambda: check(lib.mg_maxpool_bwd_argmax(d, self.argmax.ptr, self.g.ptr, self.dx.ptr)), "maxpool_bwd")]

    def __call__(self):
        lib, check = self.lib, self.check
        if self.wl["kind"] == "elem":
            c, n = self.code, self.n
            check(lib.mg_relu_fwd_mask(c, n, self.x.ptr, self.out.ptr, self.mask.ptr))
            check(lib.mg_multiply(c, n, self.out.ptr, self.g.ptr, self.dx.ptr))  # relu(x) * g
            check(lib.mg_sum_all(c, n, self.dx.ptr, self.scalar.ptr))
            check(lib.mg_fill_from(c, n, self.scalar.ptr, self.dx.ptr))  # d sum
            check(lib.mg_multiply(c, n, self.dx.ptr, self.g.ptr, self.out.ptr))  # d (a*b) / d a
            check(lib.mg_multiply(c, n, self.dx.ptr, self.x.ptr, self.out.ptr))  # d (a*b) / d b
            check(lib.mg_relu_bwd_mask(c, n, self.mask.ptr, self.dx.ptr, self.out.ptr))
            return
        if self.wl["kind"] == "bmm":
            B, M, K, N = self.dims
            check(lib.mg_matmul_batched(self.code, B, M, K, N, 0, 0, self.w.ptr, self.x.ptr, self.out.ptr))
            check(lib.mg_matmul_batched(self.code, B, M, N, K, 0, 1, self.g.ptr, self.x.ptr, self.dw.ptr))  # grad @ x^T
            check(lib.mg_matmul_batched(self.code, B, K, M, N, 1, 0, self.w.ptr, self.g.ptr, self.dx.ptr))  # a^T @ grad
            return
        if self.wl["kind"] == "matmul":
            check(lib.mg_matmul(self.code, *self.dims, self.w.ptr, self.x.ptr, self.out.ptr))
            check(lib.mg_matmul_dx(self.code, *self.dims, self.g.ptr, self.w.ptr, self.dx.ptr))
            check(lib.mg_matmul_da(self.code, *self.dims, self.g.ptr, self.x.ptr, self.dw.ptr))
            return
        if self.wl["kind"] == "permute":
            item = 4 if self.wl["dtype"] == "f32" else 8
            check(lib.mg_permute(item, self.nd, *self.calls[0], self.x.ptr, self.out.ptr))
            check(lib.mg_permute(item, self.nd, *self.calls[1], self.out.ptr, self.back.ptr))
            return
        if self.wl["kind"] == "einsum":
            from mygrad_amd.linalg.ops import contract

            la, lb, lo = self.wl["subscripts"]
            contract([(self.x, la), (self.w, lb)], lo, self.sizes, self.np_dtype)
            contract([(self.g, lo), (self.w, lb)], la, self.sizes, self.np_dtype)
            contract([(self.g, lo), (self.x, la)], lb, self.sizes, self.np_dtype)
            return
        if self.wl["kind"] == "sumover":
            check(lib.mg_sum_over(self.code, *self.dims, 0, self.x.ptr, self.out.ptr))
            check(lib.mg_sum_over(self.code, *self.dims, 1, self.x.ptr, self.out.ptr))
            return
        if self.wl["kind"] == "scale":
            for nd, extents, sa, sb, other in self.others:
                check(lib.mg_multiply_broadcast(self.code, nd, extents, sa, sb, self.x.ptr, other.ptr, self.out.ptr))
            return
        if self.wl["kind"] == "repeat":
            for outer, n, inner, r, total in self.geometry:
                check(lib.mg_repeat_fwd(4 if self.code == 0 else 8, outer, n, inner, r, total, None, self.x.ptr, self.out.ptr))
                check(lib.mg_repeat_bwd(self.code, outer, n, inner, r, total, None, self.g.ptr, self.dx.ptr))
            return
        d = self.desc
        if self.wl["kind"] == "window":
            check(lib.mg_window_gather(d, self.x.ptr, self.out.ptr))
            return
        if self.wl["kind"] == "bn":
            check(lib.mg_batchnorm_fwd(d, self.x.ptr, self.gamma.ptr, self.beta.ptr, self.out.ptr, self.mean.ptr, self.var.ptr))
            check(lib.mg_batchnorm_bwd(d, self.x.ptr, self.g.ptr, self.gamma.ptr, self.mean.ptr, self.var.ptr,
                                       self.dx.ptr, self.dgamma.ptr, self.dbeta.ptr))
            return
        if self.wl["kind"] == "conv":
            check(lib.mg_conv_fwd(d, self.x.ptr, self.w.ptr, self.out.ptr))
            if not self.wl.get("constant_input"):
                check(lib.mg_conv_dgrad(d, self.g.ptr, self.w.ptr, self.dx.ptr))
            check(lib.mg_conv_wgrad(d, self.g.ptr, self.x.ptr, self.dw.ptr))
        elif self.argmax is None:
            check(lib.mg_maxpool_fwd(d, self.x.ptr, self.out.ptr))
            check(lib.mg_maxpool_bwd(d, self.x.ptr, self.g.ptr, self.dx.ptr))
        else:
            check(lib.mg_maxpool_fwd_argmax(d, self.x.ptr, self.out.ptr, self.argmax.ptr))
            check(lib.mg_maxpool_bwd_argmax(d, self.argmax.ptr, self.g.ptr, self.dx.ptr))


PREWARM_SECONDS = 0.4


TIME_EVERY = 4


def run_gpu(name, steps, warmup, prewarm=None, time_every=None):
    from mygrad_amd import _hip

    step = Step(name)
    # The device clock climbs for a few hundred milliseconds after an idle period (measured:
    # 2.15 - 2.3 GHz during the first tens of milliseconds of work, 2.38 - 2.40 GHz from then on,
    # see profiles/conv3a_sustained.txt): run the step untimed until it has settled, so that the
    # timed steps show the rate a job sustains rather than the ramp.
    prewarm = PREWARM_SECONDS if prewarm is None else prewarm
    t_end = time.perf_counter() + prewarm
    prewarmed = 0
    while time.perf_counter() < t_end:
        for _ in range(10):
            step()
        _hip.synchronize()
        prewarmed += 10
    for _ in range(warmup):
        step()
    _hip.synchronize()
    # The per-kernel durations come from HIP events recorded in the timed region itself, and an
    # event costs about 3 us of stream time (6 events in a conv3a step: 20 of 740 us; 6 of the 46 us
    # of a pool2 step).  Every `time_every`-th step of the region is recorded, the others run as
    # they would in a job.
    every = TIME_EVERY if time_every is None else max(1, time_every)
    if steps < 2 * every:
        every = 1
    _hip.timing_enable(True)
    t0 = time.perf_counter()
    for i in range(steps):
        if every > 1 and i % every < 2:
            _hip.timing_pause(i % every == 1)
        step()
    _hip.synchronize()
    elapsed = time.perf_counter() - t0
    records = _hip.timing_read()
    _hip.timing_enable(False)
    timed_steps = len(range(0, steps, every))

    per_kernel = {}
    for kname, ms in records:
        per_kernel.setdefault(kname, []).append(ms)
    kernels = {
        k: {"launches": len(v), "avg_ms": float(np.mean(v)), "min_ms": float(np.min(v))} for k, v in per_kernel.items()
    }
    # the ceiling the kernels are priced against (a workload may quote its throughput in flops
    # and still be bound by HBM)
    roof = getattr(step, "roof", None) or dict(bound=step.bound, work=step.work, scale=step.scale, unit=step.unit, peak=step.peak)
    # A pooling pair that keeps the argmax does not read x again in its backward pass: it is priced on
    # the bytes it has to move, not on the stateless definition's |x| + |grad| + |dx| (kept beside it).
    moved = getattr(step, "moved", None)
    if moved:
        roof = dict(roof, work=moved)
    for k, info in kernels.items():
        if k in roof["work"]:
            info["achieved"] = roof["work"][k] * roof["scale"] / (info["avg_ms"] * 1e-3)
            info["unit"] = roof["unit"]
            info["frac"] = info["achieved"] / roof["peak"]
            if moved:
                info["on_definition_bytes"] = step.work[k] * roof["scale"] / (info["avg_ms"] * 1e-3)
    dominant = max((k for k in kernels if k in roof["work"]), key=lambda k: kernels[k]["avg_ms"] * kernels[k]["launches"])
    dom = kernels[dominant]
    ms_per_step = elapsed * 1e3 / steps
    traffic = measured_traffic(name, dominant)
    extra = {}
    if roof["bound"] == "hbm" and traffic:
        # the rate at which bytes really crossed HBM: below `achieved` where a kernel avoids part
        # of the algorithmic bytes (the pool backward pass that routes from the recorded argmax)
        extra["moved"] = traffic * roof["scale"] / (dom["avg_ms"] * 1e-3)
        extra["moved_frac"] = extra["moved"] / roof["peak"]
    total = sum(moved.values()) if moved else step.total_work
    if moved:
        extra["priced_on"] = "bytes the argmax-keeping pair has to move (x, out, one byte per window; bytes, grad, dx)"
        extra["on_definition_bytes"] = dom["on_definition_bytes"]
    return {
        "value": total * step.scale / (elapsed / steps),
        **({"value_on_definition_bytes": step.total_work * step.scale / (elapsed / steps)} if moved else {}),
        "unit": step.unit,
        "ms_per_step": ms_per_step,
        "kernel_ms_per_step": float(sum(np.sum(v) for v in per_kernel.values()) / timed_steps),
        "timed_steps": timed_steps,
        "prewarm": {"seconds": prewarm, "steps": prewarmed},
        "roofline": {
            "bound": roof["bound"],
            "kernel": dominant,
            "achieved": dom["achieved"],
            "peak": roof["peak"],
            "unit": roof["unit"],
            "frac": dom["frac"],
            "traffic": traffic,
            "avg_kernel_ms": dom["avg_ms"],
            "work_per_launch": roof["work"][dominant],
            **extra,
        },
        "kernels": kernels,
    }


def short_plan(note):
    """The kernel family, tile and K split out of a plan note of the library."""
    import re

    m = re.match(r"(\w+): (.*?) tile (\d+x\d+x\d+), (\d+) phase\(s\) \((\d+) fused per tile\).*K splits (\d+)", note)
    if not m:
        return note.split(": ", 1)[-1]
    family, tile, phases, fused, splits = m.group(2), m.group(3), int(m.group(4)), int(m.group(5)), int(m.group(6))
    extra = (f", {phases} phases" + (f" ({fused} fused)" if fused > 1 else "")) if phases > 1 else ""
    return f"{family} {tile}{extra}" + (f", {splits} K splits" if m.group(1) == "wgrad" else "")


def run_sweep(names, steps=20, prewarm=0.25):
    """Every pass of every shape on its own: the plan the library chose, the time of `steps`
    back-to-back calls by the host clock (stream drained on both sides) and the kernels' own
    time by HIP events, as a share of the roofline that bounds the pass."""
    from mygrad_amd import _hip

    rows = []
    for name in names:
        step = Step(name)
        wl = step.wl
        t_end = time.perf_counter() + prewarm
        while time.perf_counter() < t_end:
            for _ in range(5):
                step()
            _hip.synchronize()
        work_of = getattr(step, "moved", None) or step.work
        for label, fn, key in step.passes():
            fn()
            plan = _hip.last_plan()
            _hip.synchronize()
            _hip.timing_enable(True)
            for _ in range(steps):
                fn()
            records = _hip.timing_read()
            _hip.timing_enable(False)
            kernel_ms = sum(ms for _, ms in records) / steps
            reps = steps
            while True:
                _hip.synchronize()
                t0 = time.perf_counter()
                for _ in range(reps):
                    fn()
                _hip.synchronize()
                elapsed = time.perf_counter() - t0
                if elapsed >= 0.02 or reps >= 2000:
                    break
                reps *= 4
            host_ms = elapsed / reps * 1e3
            work = work_of[key]
            rows.append({
                "shape": name, "dtype": wl["dtype"], "kind": wl["kind"], "pass": label, "plan": plan, "launches": len(records) / steps,
                "host_us": host_ms * 1e3, "kernel_us": kernel_ms * 1e3, "work": work, "unit": step.unit,
                "achieved": work * step.scale / (host_ms * 1e-3), "frac": work * step.scale / (host_ms * 1e-3) / step.peak,
                "kernel_frac": work * step.scale / (kernel_ms * 1e-3) / step.peak,
                "small": wl["kind"] == "conv" and min(wl["x"][1], wl["w"][0]) < 32,
            })
        if wl["kind"] == "pool":
            # The passes in turn, as a training step runs them: a pass repeated on its own finds its
            # operands in the 256 MB last-level cache when they fit there, a pair that alternates
            # (x, out, grad and dx together) mostly does not.
            reps = max(steps, 50)
            while True:
                _hip.synchronize()
                t0 = time.perf_counter()
                for _ in range(reps):
                    step()
                _hip.synchronize()
                elapsed = time.perf_counter() - t0
                if elapsed >= 0.03 or reps >= 4000:
                    break
                reps *= 4
            pair_ms = elapsed / reps * 1e3
            work = sum(work_of.values())
            rows.append({"shape": name, "dtype": wl["dtype"], "kind": "pool-pair", "pass": "pair", "plan": "", "launches": 0.0,
                         "host_us": pair_ms * 1e3, "kernel_us": None, "work": work, "unit": step.unit,
                         "achieved": work * step.scale / (pair_ms * 1e-3), "frac": work * step.scale / (pair_ms * 1e-3) / step.peak,
                         "kernel_frac": None, "small": False})
        del step
    return rows


def sweep_table(rows):
    """The sweep as text: one line per pass, then one per pooling pair, then the outliers."""
    lines = ["shape                          dtype pass  host us  kernels us  launches  achieved        % of roofline (host clock / kernels)  plan",
             "-" * 170]
    for r in rows:
        if r["kind"] == "pool-pair":
            continue
        lines.append(f"{r['shape']:<30} {r['dtype']:<5} {r['pass']:<4} {r['host_us']:>8.1f} {r['kernel_us']:>11.1f} {r['launches']:>9.1f}  "
                     f"{r['achieved']:>8.1f} {r['unit']:<8} {100 * r['frac']:>6.1f} / {100 * r['kernel_frac']:<6.1f}"
                     f"                          {short_plan(r['plan'])}")
    lines += ["", "pooling pairs (forward and backward pass in turn, as a step runs them: bytes the pair has to move / time by the host clock;",
              "a pass repeated on its own, as in the lines above, finds more of its operands in the 256 MB last-level cache):"]
    outliers = []
    for r in rows:
        if r["kind"] != "pool-pair":
            continue
        lines.append(f"  {r['shape']:<34} {r['work'] / 1e6:>8.1f} MB in {r['host_us']:>7.1f} us = {r['achieved']:>7.0f} GB/s = {100 * r['frac']:5.1f} % of {PEAK_HBM_GBS:.0f} GB/s")
        if r["frac"] < 0.65:
            outliers.append(f"  {r['shape']}: pair at {100 * r['frac']:.1f} % (bar 65 %)")
    for r in rows:
        if r["kind"] == "conv" and not r["small"] and r["frac"] < 0.60:
            outliers.append(f"  {r['shape']} {r['pass']}: {100 * r['frac']:.1f} % (bar 60 %)")
    lines += ["", "below the bar (convolution passes with C, F >= 32 under 60 % of the MFMA peak, pooling pairs under 65 % of HBM):"]
    lines += outliers or ["  none"]
    return "\n".join(lines)


def compact_summary(line):
    """value and the dominant kernel's share of its roofline for the headline workload and every
    secondary one, short enough to survive a truncated record of the JSON line."""
    out = {}
    for name, entry in [(line["config"]["workload"].split(":")[0], line)] + list(line.get("secondary", {}).items()):
        roof = entry["roofline"]
        item = [round(entry["value"], 1 if entry["unit"] == "TFLOP/s" else 0), round(roof["frac"], 3)]
        if "value_on_definition_bytes" in entry:
            item.append("moved")
        out[name] = item
    return out


def measured_traffic(workload, kernel):
    """HBM bytes per launch from committed rocprofv3 --pmc runs, if recorded."""
    path = os.path.join(ROOT, "profiles", "hbm_traffic.json")
    try:
        with open(path) as fh:
            return json.load(fh).get(workload, {}).get(kernel)
    except (OSError, ValueError):
        return None


def blas_threads():
    try:
        from threadpoolctl import threadpool_info

        counts = [p.get("num_threads", 1) for p in threadpool_info() if p.get("user_api") == "blas"]
        return max(counts) if counts else 1
    except Exception:
        return int(os.environ.get("OMP_NUM_THREADS", "1"))


def run_cpu_baseline(name, min_seconds=10.0, max_reps=200):
    """Time the NumPy restatement of the reference on the host cores: the whole
    workload, repeated until at least ``min_seconds`` of CPU work have been done."""
    from oracle import np_oracle as ora

    wl, dt = WORKLOADS[name], NP_DTYPE[WORKLOADS[name]["dtype"]]
    rng = np.random.default_rng(wl["seed"])
    if wl["kind"] == "conv":
        x = rng.standard_normal(wl["x"]).astype(dt)
        w = (rng.standard_normal(wl["w"]) * wl["wscale"]).astype(dt)
        conf = dict(stride=wl["stride"], padding=wl["padding"], dilation=wl["dilation"])
        g = rng.standard_normal((wl["x"][0], wl["w"][0], *conv_grid(wl))).astype(dt)

        def once():
            ora.conv_forward(x, w, validate=False, **conf)
            if not wl.get("constant_input"):
                ora.conv_backward_x(g, x.shape, x.dtype, w, **conf)
            ora.conv_backward_w(g, x, w.shape, **conf)

        work, scale, unit = (2 if wl.get("constant_input") else 3) * conv_flops_per_pass(wl), 1e-12, "TFLOP/s"
        what = conv_passes(wl)
    elif wl["kind"] == "bmm":
        B, M, K, N = wl["batch"], wl["M"], wl["K"], wl["N"]
        a = (rng.standard_normal((B, M, K)) * K ** -0.5).astype(dt)
        x, g = rng.standard_normal((B, K, N)).astype(dt), rng.standard_normal((B, M, N)).astype(dt)

        def once():
            ora.matmul_forward(a, x)
            ora.matmul_backward(g, a, x, 0)
            ora.matmul_backward(g, a, x, 1)

        work, scale, unit = 6.0 * B * M * K * N, 1e-12, "TFLOP/s"
        what = "np.matmul on the two stacks and both gradients"
    elif wl["kind"] == "matmul":
        M, K, N = wl["M"], wl["K"], wl["N"]
        a = (rng.standard_normal((M, K)) * K ** -0.5).astype(dt)
        x = rng.standard_normal((K, N)).astype(dt)
        g = rng.standard_normal((M, N)).astype(dt)

        def once():
            ora.matmul_forward(a, x)
            ora.matmul_backward(g, a, x, 0)
            ora.matmul_backward(g, a, x, 1)

        work, scale, unit = 6.0 * M * K * N, 1e-12, "TFLOP/s"
        what = "product and both gradients (three BLAS sgemm calls)"
    elif wl["kind"] == "permute":
        x = rng.standard_normal(wl["x"]).astype(dt)

        def once():
            mid = np.ascontiguousarray(np.transpose(x, wl["perms"][0]))
            np.ascontiguousarray(np.transpose(mid, wl["perms"][1]))

        work, scale, unit = 4 * x.nbytes, 1e-9, "GB/s"
        what = "np.ascontiguousarray(np.transpose(...)) twice"
    elif wl["kind"] == "einsum":
        x = rng.standard_normal(wl["x"]).astype(dt)
        w = rng.standard_normal(wl["w"]).astype(dt)
        la, lb, lo = wl["subscripts"]
        sizes = {**dict(zip(la, wl["x"])), **dict(zip(lb, wl["w"]))}
        g = rng.standard_normal(tuple(sizes[l] for l in lo)).astype(dt)
        # np.einsum without optimize=True (the reference's default) does not call BLAS: an eighth
        # of the batch keeps one repetition to a few seconds
        part = max(1, wl["x"][0] // 8)
        x, g = np.ascontiguousarray(x[:part]), np.ascontiguousarray(g[:part])
        sizes[la[0]] = part

        def once():
            ora.einsum_forward(f"{la},{lb}", lo, x, w)
            ora.einsum_backward(g, 0, f"{la},{lb}", lo, [x, w])
            ora.einsum_backward(g, 1, f"{la},{lb}", lo, [x, w])

        work, scale, unit = 6.0 * np.prod([float(v) for v in sizes.values()]), 1e-12, "TFLOP/s"
        what = f"np.einsum for the product and both gradients on {part} of the {wl['x'][0]} batch entries"
        whole = False
    elif wl["kind"] == "sumover":
        x = rng.standard_normal(wl["x"]).astype(dt)

        def once():
            for axes in wl["axes"]:
                ora.sum_axes(x, axes)

        work, scale, unit = 2 * x.nbytes, 1e-9, "GB/s"
        what = "np.sum over each of the two sets of axes"
    elif wl["kind"] == "scale":
        x = rng.standard_normal(wl["x"]).astype(dt)
        others = [rng.standard_normal(shape).astype(dt) for shape in wl["others"]]

        def once():
            for other in others:
                ora.multiply(x, other)

        work, scale, unit = 4 * x.nbytes, 1e-9, "GB/s"
        what = "np.multiply by a per-channel scale and by a row"
    elif wl["kind"] == "repeat":
        x = rng.standard_normal(wl["x"]).astype(dt)
        g = rng.standard_normal((*wl["x"][:-1], wl["x"][-1] * wl["repeats"])).astype(dt)

        def once():
            for axis in wl["axes"]:
                out = ora.repeat_forward(x, wl["repeats"], axis)
                ora.repeat_backward(g.reshape(out.shape), x, wl["repeats"], axis)

        work, scale, unit = 4 * (x.nbytes + g.nbytes), 1e-9, "GB/s"
        what = "np.repeat and the windowed-sum gradient along each of the two axes"
    elif wl["kind"] == "window":
        x = rng.standard_normal(wl["x"]).astype(dt)
        count = np.prod(ora.window_view(x, wl["window"], wl["step"], wl["dilation"]).shape)

        def once():
            np.ascontiguousarray(ora.window_view(x, wl["window"], wl["step"], wl["dilation"]))

        work, scale, unit = x.nbytes + int(count) * x.itemsize, 1e-9, "GB/s"
        what = "np.ascontiguousarray of the view"
    elif wl["kind"] == "bn":
        x = (rng.standard_normal(wl["x"]) * 2 + 0.5).astype(dt)
        g = rng.standard_normal(wl["x"]).astype(dt)
        gamma = rng.uniform(0.5, 2, wl["x"][1]).astype(dt)
        beta = rng.standard_normal(wl["x"][1]).astype(dt)

        def once():
            ora.batchnorm_forward(x, gamma, beta, eps=wl["eps"])
            ora.batchnorm_backward(g, x, gamma, eps=wl["eps"])

        work, scale, unit = 5 * x.nbytes, 1e-9, "GB/s"
        what = "forward, then dx, dgamma and dbeta (x_norm recomputed in the backward pass)"
    elif wl["kind"] == "elem":
        x = rng.standard_normal(wl["x"]).astype(dt)
        g = rng.standard_normal(wl["x"]).astype(dt)

        def once():
            r = ora.relu_forward(x)
            p = ora.multiply(r, g)
            total = ora.sum_all(p)
            dp = ora.sum_all_backward(p, total)
            ora.multiply_backward(dp, r, g, 0)
            dr = ora.multiply_backward(dp, r, g, 1)
            ora.relu_backward(x, dr)

        work, scale, unit = elem_bytes(x), 1e-9, "GB/s"
        what = "relu, multiply, sum and their gradients"
    else:
        x = rng.standard_normal(wl["x"]).astype(dt)
        lead, pooled, grid = pool_shapes(wl)
        g = rng.standard_normal((*lead, *grid)).astype(dt)

        def once():
            ora.pool_forward(x, wl["pool"], wl["stride"], validate=False)
            ora.pool_backward(x, g, wl["pool"], wl["stride"])

        work, scale, unit = 3 * x.nbytes + 2 * g.nbytes, 1e-9, "GB/s"
        what = "fwd+bwd"
    whole = locals().get("whole", True)
    reps, t0 = 0, time.perf_counter()
    while True:
        once()
        reps += 1
        elapsed = time.perf_counter() - t0
        if elapsed >= min_seconds or reps >= max_reps:
            break
    return {
        "value": float(reps * work * scale / elapsed),
        "unit": unit,
        "cores": blas_threads() if wl["kind"] in ("conv", "matmul") else 1,
        "kind": "port",
        "sample": f"{'the whole workload' if whole else 'a part of the workload'} ({what}), {reps} repetition(s), {elapsed:.1f} s of host time",
        "numpy": np.__version__,
    }


def run_dropin(name, steps=5):
    """Wall time of the same step through the drop-in API (conv_nd / max_pool / ... called on
    tensors, gradients through Tensor.backward()), two ways:

    ``resident``  inputs are device tensors (uploaded once), nothing is read during the loop;
                  the gradients are read once after the last step (``read_back_ms``).  Next to
                  it the kernel time of the same loop from the library's HIP events.
    ``host``      host ndarrays in and every gradient read on the host after every step: the
                  PCIe-inclusive figure.
    Neither is ever ``value``."""
    import mygrad_amd as mg
    from mygrad_amd import _hip
    from mygrad_amd.nnet import conv_nd, max_pool

    wl, dt = WORKLOADS[name], NP_DTYPE[WORKLOADS[name]["dtype"]]
    rng = np.random.default_rng(wl["seed"])
    x = rng.standard_normal(wl["x"]).astype(dt) if "x" in wl else None
    chain = None
    # every branch defines once(T, C): T wraps an input that takes a gradient, C a constant one
    # (both return tensors); it runs one step and returns the tensors whose gradients it left
    if wl["kind"] == "conv":
        w = (rng.standard_normal(wl["w"]) * wl["wscale"]).astype(dt)
        g = rng.standard_normal((wl["x"][0], wl["w"][0], *conv_grid(wl))).astype(dt)
        valid = all((xx + 2 * p - ((t - 1) * d + 1)) % s == 0
                    for xx, t, s, p, d in zip(wl["x"][2:], wl["w"][2:], wl["stride"], wl["padding"], wl["dilation"]))
        if not valid:
            return {"skipped": "the reference's validator rejects this shape; the drop-in raises ValueError like it"}
        conf = dict(stride=wl["stride"], padding=wl["padding"], dilation=wl["dilation"])

        def once(T, C):
            xt, wt = (C(x) if wl.get("constant_input") else T(x)), T(w)
            conv_nd(xt, wt, **conf).backward(C(g))
            return xt, wt

        work, scale, unit = (2 if wl.get("constant_input") else 3) * conv_flops_per_pass(wl), 1e-12, "TFLOP/s"
        if name == "conv5":
            # the whole of configuration 5: conv -> max_pool (2,2,2) -> loss = sum(pool_out * g)
            g5 = rng.standard_normal((wl["x"][0], wl["w"][0], *(n // 2 for n in conv_grid(wl)))).astype(dt)

            def chain(T, C):
                xt, wt = T(x), T(w)
                mg.sum(max_pool(conv_nd(xt, wt, **conf), (2, 2, 2), 2) * C(g5)).backward()
                return xt, wt
    elif wl["kind"] == "matmul":
        M, K, N = wl["M"], wl["K"], wl["N"]
        a = (rng.standard_normal((M, K)) * K ** -0.5).astype(dt)
        x = rng.standard_normal((K, N)).astype(dt)
        g = rng.standard_normal((M, N)).astype(dt)

        def once(T, C):
            at, xt = T(a), T(x)
            (at @ xt).backward(C(g))
            return at, xt

        work, scale, unit = 6.0 * M * K * N, 1e-12, "TFLOP/s"
    elif wl["kind"] == "bmm":
        B, M, K, N = wl["batch"], wl["M"], wl["K"], wl["N"]
        a = (rng.standard_normal((B, M, K)) * K ** -0.5).astype(dt)
        x, g = rng.standard_normal((B, K, N)).astype(dt), rng.standard_normal((B, M, N)).astype(dt)

        def once(T, C):
            at, xt = T(a), T(x)
            (at @ xt).backward(C(g))
            return at, xt

        work, scale, unit = 6.0 * B * M * K * N, 1e-12, "TFLOP/s"
    elif wl["kind"] == "permute":
        return {"skipped": "transposition is a building block of einsum here, not an operation of its own"}
    elif wl["kind"] == "einsum":
        w = rng.standard_normal(wl["w"]).astype(dt)
        la, lb, lo = wl["subscripts"]
        sizes = {**dict(zip(la, wl["x"])), **dict(zip(lb, wl["w"]))}
        g = rng.standard_normal(tuple(sizes[l] for l in lo)).astype(dt)

        def once(T, C):
            xt, wt = T(x), T(w)
            mg.einsum(f"{la},{lb}->{lo}", xt, wt).backward(C(g))
            return xt, wt

        work, scale, unit = 6.0 * np.prod([float(v) for v in sizes.values()]), 1e-12, "TFLOP/s"
    elif wl["kind"] == "sumover":

        def once(T, C):
            outs = [mg.sum(C(x), axis=axes) for axes in wl["axes"]]
            for out in outs:
                out.clear_graph()
            return ()

        work, scale, unit = 2 * x.nbytes, 1e-9, "GB/s"
    elif wl["kind"] == "scale":
        others = [rng.standard_normal(shape).astype(dt) for shape in wl["others"]]

        def once(T, C):
            for other in others:
                (C(x) * C(other)).clear_graph()
            return ()

        work, scale, unit = 4 * x.nbytes, 1e-9, "GB/s"
    elif wl["kind"] == "repeat":
        g = rng.standard_normal((*wl["x"][:-1], wl["x"][-1] * wl["repeats"])).astype(dt)
        seeds = {}

        def once(T, C):
            leaves = []
            for axis in wl["axes"]:
                xt = T(x)
                out = mg.repeat(xt, wl["repeats"], axis)
                seeds.setdefault(axis, np.ascontiguousarray(g.reshape(out.shape)))
                out.backward(C(seeds[axis]))
                leaves.append(xt)
            return leaves[-1:]

        work, scale, unit = 4 * (x.nbytes + g.nbytes), 1e-9, "GB/s"
    elif wl["kind"] == "window":
        count = int(np.prod(mg.sliding_window_view(x, wl["window"], wl["step"], wl["dilation"]).shape))

        def once(T, C):
            mg.sliding_window_copy(x, wl["window"], wl["step"], wl["dilation"])
            return ()

        work, scale, unit = x.nbytes + count * x.itemsize, 1e-9, "GB/s"
    elif wl["kind"] == "bn":
        from mygrad_amd.nnet import batchnorm

        g = rng.standard_normal(wl["x"]).astype(dt)
        gamma = rng.uniform(0.5, 2, wl["x"][1]).astype(dt)
        beta = rng.standard_normal(wl["x"][1]).astype(dt)

        def once(T, C):
            xt, gt, bt = T(x), T(gamma), T(beta)
            batchnorm(xt, gamma=gt, beta=bt, eps=wl["eps"]).backward(C(g))
            return xt, gt, bt

        work, scale, unit = 5 * x.nbytes, 1e-9, "GB/s"
    elif wl["kind"] == "elem":
        from mygrad_amd.nnet import relu

        g = rng.standard_normal(wl["x"]).astype(dt)

        def once(T, C):
            xt, gt = T(x), T(g)
            mg.sum(relu(xt) * gt).backward()
            return xt, gt

        work, scale, unit = elem_bytes(x), 1e-9, "GB/s"
    else:
        lead, pooled, grid = pool_shapes(wl)
        g = rng.standard_normal((*lead, *grid)).astype(dt)
        if any((xx - p) % s for xx, p, s in zip(pooled, wl["pool"], wl["stride"])):
            return {"skipped": "the reference's validator rejects this shape; the drop-in raises ValueError like it"}

        def once(T, C):
            xt = T(x)
            max_pool(xt, wl["pool"], wl["stride"]).backward(C(g))
            return (xt,)

        work, scale, unit = 3 * x.nbytes + 2 * g.nbytes, 1e-9, "GB/s"

    def measure(step):
        def read(leaves):
            for t in leaves:
                t.grad

        # host arrays in, gradients read every step
        host_T = lambda a: mg.Tensor(a, copy=False)
        host_C = lambda a: mg.Tensor(a, copy=False, constant=True)
        read(step(host_T, host_C))
        t0 = time.perf_counter()
        for _ in range(steps):
            read(step(host_T, host_C))
        host_ms = (time.perf_counter() - t0) / steps * 1e3
        if wl["kind"] == "window":
            return {"host": {"ms_per_step": host_ms, "note": "host ndarray in, host ndarray out"}}

        # device tensors in, nothing read until the loop is over
        held = {}

        def dev_T(a, constant=None):
            if id(a) not in held:
                held[id(a)] = (a, mg.device_tensor(a, constant=constant))
            return held[id(a)][1]

        dev_C = lambda a: dev_T(a, constant=True)
        many = max(steps, 20)
        step(dev_T, dev_C)
        _hip.synchronize()
        warm = time.perf_counter()
        while time.perf_counter() - warm < PREWARM_SECONDS:  # untimed, for the device clock to settle as in the headline loop
            for _ in range(10):
                step(dev_T, dev_C)
            _hip.synchronize()
        t0 = time.perf_counter()
        for _ in range(many):
            leaves = step(dev_T, dev_C)
        _hip.synchronize()
        wall_ms = (time.perf_counter() - t0) / many * 1e3
        t0 = time.perf_counter()
        read(leaves)
        read_ms = (time.perf_counter() - t0) * 1e3
        _hip.timing_enable(True)
        for _ in range(many):
            step(dev_T, dev_C)
        _hip.synchronize()
        kernel_ms = sum(ms for _, ms in _hip.timing_read()) / many
        _hip.timing_enable(False)
        return {
            "resident": {"ms_per_step": wall_ms, "kernel_ms_per_step": kernel_ms, "over_kernels": wall_ms / kernel_ms if kernel_ms else None,
                         "read_back_ms": read_ms, "steps": many,
                         "note": "device tensors in, Tensor.backward() every step, gradients read once after the last step; the loop runs "
                                 "untimed for the pre-warm time first, like the headline loop (compare with its ms_per_step); "
                                 "kernel_ms_per_step is from a second loop with HIP events around every launch, whose recording "
                                 "costs a few microseconds per launch"},
            "host": {"ms_per_step": host_ms, "note": "host ndarrays in, every gradient read on the host after every step (PCIe included)"},
        }

    result = measure(once)
    for entry in result.values():
        entry["value"] = float(work * scale / (entry["ms_per_step"] * 1e-3))
        entry["unit"] = unit
    if chain is not None:
        result["chain"] = measure(chain)
        result["chain"]["what"] = "conv_nd -> max_pool((2,2,2), 2) -> sum(pool_out * g) and backward()"
    return result


def run_copy_calibration(mib=1024, reps=20):
    """A plain 16-byte-per-lane device copy of known size: what the HBM traffic
    counters of a profile are scaled against, and the practical bandwidth ceiling."""
    from mygrad_amd import _device, _hip

    n = mib << 20
    a, b = _device.DeviceBuffer(n), _device.DeviceBuffer(n)
    lib = _hip.lib()
    _hip.check(lib.mg_memset_zero(a.ptr, n))
    for _ in range(3):
        _hip.check(lib.mg_memcpy_d2d(b.ptr, a.ptr, n))
    _hip.timing_enable(True)
    for _ in range(reps):
        _hip.check(lib.mg_memcpy_d2d(b.ptr, a.ptr, n))
    ms = [m for k, m in _hip.timing_read() if k == "copy"]
    _hip.timing_enable(False)
    avg = float(np.mean(ms))
    return {"metric": "device copy", "bytes_read": n, "bytes_written": n, "avg_kernel_ms": avg,
            "value": 2 * n * 1e-9 / (avg * 1e-3), "unit": "GB/s", "launches": len(ms)}


def run_mix_calibration(mib=268, reps=10):
    """One stream over a buffer larger than the last-level cache, stored or loaded 16 bytes
    per lane, with the opposite stream at a fraction of its volume: what the memory system
    sustains per mix of loads and stores -- the practical ceiling of the bandwidth-bound
    kernels, whose passes are such mixes (a pooling gradient stores 7 bytes per byte it loads,
    a 1x1 convolution to four times the channels 4 per byte)."""
    from mygrad_amd import _device, _hip

    n = mib << 20
    big, small, other = _device.DeviceBuffer(n), _device.DeviceBuffer(n), _device.DeviceBuffer(n)
    lib = _hip.lib()
    for buf in (big, small, other):
        _hip.check(lib.mg_memset_zero(buf.ptr, n))
    rows = []
    for store_big in (1, 0):
        for share in (0, 64, 8, 4, 2, 1):
            ms = []
            for _ in range(reps):
                _hip.probe_stream(other.ptr, small.ptr, n, 0, 0)  # reading a third buffer pushes the operands out of the caches
                ms.append(_hip.probe_stream(big.ptr, small.ptr, n, share, store_big))
            avg = float(np.mean(ms[2:]))
            second = n // share if share else 0
            rows.append({"stored_bytes": n if store_big else second, "loaded_bytes": second if store_big else n,
                         "avg_kernel_us": avg * 1e3, "GB/s": (n + second) * 1e-9 / (avg * 1e-3)})
    return {"metric": "one launch of a load stream and a store stream, 16 bytes per lane", "unit": "GB/s", "mixes": rows}


def run_mfma_probe():
    """What the matrix cores sustain per MFMA shape with operands in registers and no
    memory traffic, next to the published peaks: the ceiling of the convolution
    kernels' inner loops on this device."""
    from mygrad_amd import _hip

    published = {"f32_16x16x4": PEAK_TFLOPS["f32"], "f64_16x16x4": PEAK_TFLOPS["f64"], "f64_4x4x4_4b": PEAK_TFLOPS["f64"]}
    out = {}
    for kind in _hip.MFMA_KINDS:
        rates = {w: _hip.probe_mfma(kind, w) for w in (1, 2, 4)}
        best = max(rates.values())
        out[kind] = {"tflops_by_waves_per_simd": rates, "best": best, "published_peak": published[kind],
                     "frac_of_published": best / published[kind]}
    return {"metric": "MFMA issue rate, registers only", "unit": "TFLOP/s", "shapes": out}


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="conv3a", choices=sorted(WORKLOADS))
    ap.add_argument("--all", action="store_true",
                    help="report every other workload under 'secondary', not only the hot path's other configurations")
    ap.add_argument("--no-secondary", action="store_true", help="run the one workload only")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--prewarm", type=float, default=PREWARM_SECONDS,
                    help="seconds of untimed steps before the warm-up steps, for the device clock to settle (0: none)")
    ap.add_argument("--time-every", type=int, default=TIME_EVERY,
                    help="record per-kernel HIP events in every N-th step of the timed region (1: in every step)")
    ap.add_argument("--dropin", action="store_true",
                    help="also time the step through the Python drop-in API (reported under 'dropin', never as value)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="run only a 1 GiB device copy (the reference point for HBM traffic counters)")
    ap.add_argument("--copy-mib", type=int, default=1024, help="size of the --calibrate-copy buffer in MiB (read + written)")
    ap.add_argument("--calibrate-mix", action="store_true",
                    help="time a store (or load) stream with the opposite stream at 0, 1/64 ... 1/1 of its volume and exit")
    ap.add_argument("--mix-mib", type=int, default=268, help="size of the larger stream of --calibrate-mix in MiB")
    ap.add_argument("--sweep", action="store_true",
                    help="run only the sweep over reference-valid shapes around the benchmark's, pass by pass: a text "
                         "table on stdout (what profiles/sweep_hotpath.txt holds), the rows as one JSON line on stderr")
    ap.add_argument("--sweep-only", default="", help="with --sweep: only the shapes whose name contains this text")
    ap.add_argument("--probe-mfma", action="store_true",
                    help="run only the matrix-core rate probe (registers only, per MFMA shape)")
    args = ap.parse_args()

    if args.gpus != 1:
        sys.exit("bench.py: this build runs on exactly one GPU (--gpus 1); the path shards over the batch axis "
                 "by design but no multi-GPU code is part of it")

    if args.calibrate_copy:
        print(json.dumps(run_copy_calibration(args.copy_mib)))
        return
    if args.calibrate_mix:
        print(json.dumps(run_mix_calibration(args.mix_mib)))
        return
    if args.probe_mfma:
        print(json.dumps(run_mfma_probe()))
        return
    if args.sweep:
        rows = run_sweep([n for n in SWEEP if args.sweep_only in n], steps=args.steps)
        print(sweep_table(rows))
        print(json.dumps({"sweep": rows}), file=sys.stderr)
        return

    wl = WORKLOADS[args.workload]
    res = run_gpu(args.workload, args.steps, args.warmup, args.prewarm, args.time_every)
    line = {
        "metric": {"conv": "conv_nd fwd+bwd TFLOP/s", "pool": "max_pool fwd+bwd GB/s",
                   "elem": "relu+multiply+sum fwd+bwd GB/s", "bn": "batchnorm fwd+bwd GB/s",
                   "repeat": "repeat fwd+bwd GB/s", "matmul": "matmul fwd+bwd TFLOP/s", "bmm": "matmul of two stacks fwd+bwd TFLOP/s", "window": "sliding-window copy GB/s",
                   "sumover": "sum over axes GB/s", "scale": "broadcasting multiply GB/s", "permute": "transposition GB/s", "einsum": "einsum fwd+bwd TFLOP/s"}[wl["kind"]],
        "value": res["value"],
        "unit": res["unit"],
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": res["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": wl["dtype"],
        "data": "synthetic (seeded N(0,1) inputs and upstream gradient, He-normal filters), resident in HBM",
        "config": {"workload": describe(args.workload)},
        "roofline": res["roofline"],
        "kernel_ms_per_step": res["kernel_ms_per_step"],
        "timed_steps": res["timed_steps"],
        "prewarm": res["prewarm"],
        "kernels": res["kernels"],
    }
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = run_cpu_baseline(args.workload)
    if args.dropin:
        line["dropin"] = run_dropin(args.workload)
    if not args.no_secondary:
        # the other half of the metric (max_pool GB/s) and the other convolution configurations,
        # each with its own roofline and a short CPU baseline
        names = [n for n in WORKLOADS if n not in SWEEP] if args.all else HOT_PATH
        secondary = {}
        for name in names:
            if name == args.workload:
                continue
            r = run_gpu(name, args.steps, args.warmup, args.prewarm, args.time_every)
            steps = args.steps
            if r["ms_per_step"] * steps < 10.0:
                # A region of a millisecond or so (20 steps of a 40 us pooling pair) is a tenth the drain of
                # the stream at its end and the events of its recorded steps: time about 20 ms of steps
                # instead, five of them with events.
                steps = min(2000, max(steps, int(20.0 / r["ms_per_step"])))
                r = run_gpu(name, steps, args.warmup, 0.05, max(args.time_every, steps // 5))
            entry = {"config": describe(name), "value": r["value"], "unit": r["unit"], "dtype": WORKLOADS[name]["dtype"],
                     "steps": steps, "ms_per_step": r["ms_per_step"], "kernel_ms_per_step": r["kernel_ms_per_step"], "roofline": r["roofline"],
                     "kernels": r["kernels"]}
            if not args.no_cpu_baseline:
                entry["cpu_baseline"] = run_cpu_baseline(name, min_seconds=2.0)
            if args.dropin:
                entry["dropin"] = run_dropin(name)
            secondary[name] = entry
        line["secondary"] = secondary
    line["summary"] = compact_summary(line)  # last: the end of the line is what a truncated record keeps
    print(json.dumps(line))


if __name__ == "__main__":
    main()
