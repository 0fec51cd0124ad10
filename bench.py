#!/usr/bin/env python3
"""Benchmark of the kernel-layer hot path on one MI355X.

Workload (BASELINE.json configs[3], the shape the performance target is stated on):
ConvKernelLayer<float,3> forward + backward (weight, bias and input gradients), batch 256, input
NHWC 56x56x64 drawn from N(0,1), 128 filters 3x3, stride 1, padding 1, He-normal weights, upstream
gradient N(0,1). One step = one pass_forward + one pass_back on tensors already resident in HBM.

Prints one JSON line: whole-step throughput in GFLOP/s (algorithmic FLOP = 6*M*K*F per step),
samples/s, the MFMA roofline of the slowest GEMM kernel (measured with HIP events on the library's
stream) and the CPU baseline (the oracle's restatement of the reference algorithm on the host
cores, on a bounded sample of the same workload).
"""
import argparse
import collections
import csv
import glob
import importlib
import json
import os
import sqlite3
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_TFLOPS = {"f32": 157.3, "f64": 78.6}      # MI355X dense matrix peaks (no sparsity)
SHAPE = dict(H=56, W=56, C=64, F=128, RH=3, RW=3)

# HBM bytes per launch (read + written) of the three GEMM kernels come from rocprofv3 FETCH_SIZE and WRITE_SIZE readings
# of `bench.py --copy-calibration`, each scaled by what the same counter reads for the calibration copy of known size.
# Counters cannot be read while timing, so the figures live in a tracked file that `bench.py summarize traffic --write`
# rewrites from the counter runs, together with a hash of the kernel sources they were measured on; a build from other
# sources reports null.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "conv_cfg4_hbm_traffic.json")
KERNEL_SOURCES = ("c-attl3_amd/csrc/gemm_kernels.hip", "c-attl3_amd/csrc/common.hpp", "c-attl3_amd/csrc/act_math.hpp",
                  "c-attl3_amd/csrc/lstm_math.hpp")


def kernel_sources_hash():
    import hashlib
    h = hashlib.sha256()
    for rel in KERNEL_SOURCES:
        with open(os.path.join(ROOT, rel), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def measured_traffic(dtype_name, batch, kernel):
    """(bytes or None, note) for one GEMM pass of the default workload from the tracked counter summary."""
    try:
        with open(TRAFFIC_FILE) as f:
            rec = json.load(f)
    except (OSError, ValueError):
        return None, "no tracked counter summary"
    if rec.get("kernel_sources_sha256_16") != kernel_sources_hash():
        return None, "the kernel sources changed since the counters were read (%s): re-run the counter passes" % rec.get("kernel_sources_sha256_16")
    entry = rec.get("entries", {}).get("%s:%d" % (dtype_name, batch), {})
    return entry.get(kernel), "rocprofv3 FETCH_SIZE x %.3f + WRITE_SIZE x %.3f, kernel and its reduce launch" % (
        rec.get("fetch_factor", 0.0), rec.get("write_factor", 0.0))


def he_normal(gen, rows, cols, dtype):
    # parameter_initialization/HeParameterInitialization.hpp:34-36: sd = sqrt(2 / fan_in), fan_in = rows
    return np.asfortranarray((gen.standard_normal((rows, cols)) * np.sqrt(2.0 / rows)).astype(dtype))


def gpu_run(args, dtype):
    ch = importlib.import_module("c-attl3_amd")
    ch.init(0)
    N, H, W, C, F = args.batch, SHAPE["H"], SHAPE["W"], SHAPE["C"], SHAPE["F"]
    K = SHAPE["RH"] * SHAPE["RW"] * C
    M = N * H * W
    gen = np.random.default_rng(0xC0FFEE04)
    layer = ch.ConvKernelLayer(dtype, (H, W, C), F)
    layer.get_params()[0].set_values(he_normal(gen, K, F, dtype))
    x = ch.DeviceTensor.from_host(np.asfortranarray(gen.standard_normal((N, H, W, C)).astype(dtype)))
    go = ch.DeviceTensor.from_host(np.asfortranarray(gen.standard_normal((N, H, W, F)).astype(dtype)))
    out = ch.DeviceTensor((N, H, W, F), dtype)
    dx = ch.DeviceTensor((N, H, W, C), dtype)

    def step():
        layer.forward_into(x, out, True)
        layer.backward_into(go, dx)

    for _ in range(args.warmup):
        step()
    # the timed region, `repeats` times over: each is exactly `steps` steps between two synchronisations
    walls = []
    for _ in range(max(1, args.repeats)):
        ch.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step()
        ch.synchronize()
        walls.append((time.perf_counter() - t0) * 1e3 / args.steps)
    wall_ms = float(np.median(walls))

    # per-kernel durations with HIP events on the library's stream
    timer = ch.Timer()
    reps = max(3, args.steps)

    def timed(fn):
        # A pass launched back to back runs a few percent slow for its first 10-20 ms after the other kernels (the
        # durations in a kernel trace fall from about 1.03 to 0.94 ms over twenty forward launches), so each
        # pass gets as many untimed launches first as are timed, and the median of three timed groups is reported.
        for _ in range(reps):
            fn()
        groups = []
        for _ in range(3):
            timer.start()
            for _ in range(reps):
                fn()
            groups.append(timer.stop() / reps)
        return float(np.median(groups))

    t_fwd = timed(lambda: layer.forward_into(x, out, True))
    t_bwd = timed(lambda: layer.backward_into(go, dx))
    layer.set_input_layer(True)
    t_wgrad = timed(lambda: layer.backward_into(go, None))         # weight + bias gradient only
    layer.set_input_layer(False)
    t_dgrad = max(t_bwd - t_wgrad, 1e-6)
    gemm_flop = 2.0 * M * K * F
    kernels = {
        "gather_gemm_kernel (forward)": t_fwd,
        "wgrad_kernel (+ reduce, bias column sums)": t_wgrad,
        "gather_gemm_kernel (input gradient)": t_dgrad,
    }
    es = np.dtype(dtype).itemsize
    in_b, out_b, w_b = N * H * W * C * es, N * H * W * F * es, K * F * es
    nbytes = {
        "gather_gemm_kernel (forward)": in_b + w_b + out_b,
        "wgrad_kernel (+ reduce, bias column sums)": in_b + out_b + w_b,
        "gather_gemm_kernel (input gradient)": out_b + w_b + in_b,
    }
    if args.copy_calibration:
        # a plain copy kernel of known size (identity activation: reads and writes x.nbytes) so that
        # FETCH_SIZE / WRITE_SIZE counter readings of the same profile can be scaled to bytes
        ident = ch.ActivationLayer(dtype, "identity", (H, W, C))
        for _ in range(3):
            ident.forward_into(x, dx, True)
        ch.synchronize()
    for t in (x, go, out, dx):
        t.free()
    return dict(wall_ms=wall_ms, walls=walls, M=M, K=K, F=F, gemm_flop=gemm_flop, kernels=kernels, bytes=nbytes)


def host_tensor_run(args, dtype):
    """The same step through the host-tensor Layer API (pageable numpy arrays in, numpy arrays out: what the drop-in
    adapters do with Eigen tensors): PCIe-inclusive, never the headline value."""
    ch = importlib.import_module("c-attl3_amd")
    ch.init(0)
    N, H, W, C, F = args.batch, SHAPE["H"], SHAPE["W"], SHAPE["C"], SHAPE["F"]
    gen = np.random.default_rng(0xC0FFEE04)
    layer = ch.ConvKernelLayer(dtype, (H, W, C), F)
    layer.get_params()[0].set_values(he_normal(gen, 9 * C, F, dtype))
    x = np.asfortranarray(gen.standard_normal((N, H, W, C)).astype(dtype))
    go = np.asfortranarray(gen.standard_normal((N, H, W, F)).astype(dtype))
    best = None
    for _ in range(3):
        t0 = time.perf_counter()
        layer.pass_forward(x, True)
        layer.pass_back(go)
        dt = time.perf_counter() - t0
        best = dt if best is None else min(best, dt)
    moved = 2.0 * (x.nbytes + go.nbytes)       # x in, out back, out_grad in, in_grad back
    return {"ms_per_step": round(best * 1e3, 2), "GB/s": round(moved / best / 1e9, 1),
            "tflops": round(6.0 * N * H * W * 9 * C * F / best / 1e12, 2), "bytes_moved": moved,
            "note": "pass_forward + pass_back on pageable host arrays, outputs allocated per call, best of 3"}


CALIBRATION_SHAPE = (256, 32, 32, 64)


def copy_calibration(ch, dtype):
    """A plain copy of known size (the identity activation on a 256 x 32 x 32 x 64 tensor: reads and writes
    16,777,216 elements) for scaling the FETCH_SIZE / WRITE_SIZE readings of the same profiler run to bytes."""
    a = ch.DeviceTensor(CALIBRATION_SHAPE, dtype)
    b = ch.DeviceTensor(CALIBRATION_SHAPE, dtype)
    ident = ch.ActivationLayer(dtype, "identity", CALIBRATION_SHAPE[1:])
    for _ in range(3):
        ident.forward_into(a, b, True)
    ch.synchronize()
    a.free()
    b.free()


def small_convs_run(args, dtype):
    """The convolution shapes of the other BASELINE configurations, one layer at a time on device-resident tensors:
    forward, weight + bias gradient and input gradient timed with HIP events. These are small-K or few-row problems,
    so each line carries both bounds: roofline time = max(FLOP / matrix peak, algorithmic bytes / 8 TB/s), and the
    fraction of it that the measured time reaches."""
    ch = importlib.import_module("c-attl3_amd")
    ch.init(0)
    es = np.dtype(dtype).itemsize
    peak = PEAK_TFLOPS[args.dtype] * 1e12
    shapes = [
        ("configs[0] conv 64x32x32x3 -> 16", 64, 32, 32, 3, 16),
        ("configs[2] conv1 128x32x32x3 -> 32", 128, 32, 32, 3, 32),
        ("configs[2] conv2 128x16x16x32 -> 64", 128, 16, 16, 32, 64),
        ("configs[4] input-side gates, all 10 steps, 320x16x16x8 -> 128", 320, 16, 16, 8, 128),
        ("configs[4] recurrent gates, one step, 32x16x16x32 -> 128", 32, 16, 16, 32, 128),
    ]
    gen = np.random.default_rng(11)
    timer = ch.Timer()
    reps = max(20, args.steps)
    rows = []
    if args.only:
        shapes = [sh for sh in shapes if args.only in sh[0]]
    for name, N, H, W, C, F in shapes:
        K, M = 9 * C, N * H * W
        layer = ch.ConvKernelLayer(dtype, (H, W, C), F)
        layer.get_params()[0].set_values(he_normal(gen, K, F, dtype))
        x = ch.DeviceTensor.from_host(np.asfortranarray(gen.standard_normal((N, H, W, C)).astype(dtype)))
        go = ch.DeviceTensor.from_host(np.asfortranarray(gen.standard_normal((N, H, W, F)).astype(dtype)))
        out = ch.DeviceTensor((N, H, W, F), dtype)
        dx = ch.DeviceTensor((N, H, W, C), dtype)

        def timed(fn):
            for _ in range(3):
                fn()
            timer.start()
            for _ in range(reps):
                fn()
            return timer.stop() / reps

        t_fwd = timed(lambda: layer.forward_into(x, out, True)) if args.passes in ("both", "fwd") else float("nan")
        if args.passes in ("both", "bwd"):
            layer.forward_into(x, out, True)
            t_bwd = timed(lambda: layer.backward_into(go, dx))
        else:
            t_bwd = float("nan")
        in_b, out_b, w_b = M * C * es, M * F * es, K * F * es
        flop = 2.0 * M * K * F
        for pass_name, t_ms, launches, nbytes in (("forward", t_fwd, 1, in_b + w_b + out_b),
                                                  ("backward (weight, bias and input gradients)", t_bwd, 2, 2 * (in_b + out_b + w_b))):
            if t_ms != t_ms:
                continue
            roof_s = max(launches * flop / peak, nbytes / 8e12)
            rows.append({"layer": name, "pass": pass_name, "M": M, "K": K, "F": F, "ms": round(t_ms, 4),
                         "gflops": round(launches * flop / (t_ms * 1e-3) / 1e9, 1), "GB/s": round(nbytes / (t_ms * 1e-3) / 1e9, 1),
                         "bound": "mfma" if launches * flop / peak >= nbytes / 8e12 else "hbm",
                         "roofline_us": round(roof_s * 1e6, 2), "frac_of_roofline": round(roof_s / (t_ms * 1e-3), 4)})
        for t in (x, go, out, dx):
            t.free()
    if args.copy_calibration:
        copy_calibration(ch, dtype)
    return {"metric": "small_conv_layer_passes", "unit": "ms", "n_gpus": 1, "dtype": args.dtype, "data": "synthetic",
            "config": {"workload": "convolution layers of BASELINE configs[0], [2] and [4], one pass per line, tensors resident in HBM"},
            "rows": rows}


def conv_shapes_run(args, dtype):
    """Layers that no launch rule was written for: a held-out table of convolution, transposed-convolution and dense
    shapes (two of them in fp64 whatever --dtype says), forward and backward, each against its roofline
    max(FLOP / matrix peak of the precision, algorithmic bytes / 8 TB/s). FLOP = 2 M K F per GEMM with M = batch x
    output positions of the (equivalent) convolution: what a strided or transposed layer needs, not what a kernel
    that multiplies zeros spends."""
    ch = importlib.import_module("c-attl3_amd")
    ch.init(0)
    # name, kind, batch, H, W, C, F, RH, RW, pv, ph, sv, sh, dv, dh, fp64
    shapes = [
        ("conv 3x3 28x28x128 -> 256, batch 64", "conv", 64, 28, 28, 128, 256, 3, 3, 1, 1, 1, 1, 0, 0, False),
        ("conv 3x3 14x14x256 -> 256, batch 256", "conv", 256, 14, 14, 256, 256, 3, 3, 1, 1, 1, 1, 0, 0, False),
        ("conv 3x3 7x7x512 -> 512, batch 256", "conv", 256, 7, 7, 512, 512, 3, 3, 1, 1, 1, 1, 0, 0, False),
        ("conv 1x1 28x28x128 -> 512, batch 64", "conv", 64, 28, 28, 128, 512, 1, 1, 0, 0, 1, 1, 0, 0, False),
        ("conv 5x5 32x32x32 -> 64 pad 2, batch 128", "conv", 128, 32, 32, 32, 64, 5, 5, 2, 2, 1, 1, 0, 0, False),
        ("conv 3x3 stride 2 56x56x64 -> 128, batch 64", "conv", 64, 56, 56, 64, 128, 3, 3, 1, 1, 2, 2, 0, 0, False),
        ("conv 3x3 30x30x24 -> 48, batch 96", "conv", 96, 30, 30, 24, 48, 3, 3, 1, 1, 1, 1, 0, 0, False),
        ("conv 3x3 dilation 1 24x24x32 -> 32 pad 2, batch 64", "conv", 64, 24, 24, 32, 32, 3, 3, 2, 2, 1, 1, 1, 1, False),
        ("dense 4096 -> 1024, batch 512", "dense", 512, 1, 1, 4096, 1024, 1, 1, 0, 0, 1, 1, 0, 0, False),
        ("conv 3x3 28x28x128 -> 256, batch 64, fp64", "conv", 64, 28, 28, 128, 256, 3, 3, 1, 1, 1, 1, 0, 0, True),
        ("conv 3x3 14x14x256 -> 256, batch 128, fp64", "conv", 128, 14, 14, 256, 256, 3, 3, 1, 1, 1, 1, 0, 0, True),
        # the layers of the reference's examples/mnist_autoencoder.cpp:27-30, :40-43 at batch 256
        ("autoencoder conv 4x4 stride 2 28x28x1 -> 3, batch 256", "conv", 256, 28, 28, 1, 3, 4, 4, 0, 0, 2, 2, 0, 0, False),
        ("autoencoder conv 4x4 13x13x3 -> 3, batch 256", "conv", 256, 13, 13, 3, 3, 4, 4, 0, 0, 1, 1, 0, 0, False),
        ("autoencoder transposed conv 4x4 10x10x3 -> 3, batch 256", "transconv", 256, 10, 10, 3, 3, 4, 4, 0, 0, 1, 1, 0, 0, False),
        ("autoencoder transposed conv 4x4 stride 2 13x13x3 -> 1, batch 256", "transconv", 256, 13, 13, 3, 1, 4, 4, 0, 0, 2, 2, 0, 0, False),
        ("transposed conv 3x3 stride 2 14x14x128 -> 64 pad 1, batch 64", "transconv", 64, 14, 14, 128, 64, 3, 3, 1, 1, 2, 2, 0, 0, False),
        # the last layer of an image decoder: many channels in, an image out
        ("conv 3x3 64x64x64 -> 3, batch 64", "conv", 64, 64, 64, 64, 3, 3, 3, 1, 1, 1, 1, 0, 0, False),
    ]
    if args.only:
        shapes = [sh for sh in shapes if args.only in sh[0]]
    gen = np.random.default_rng(23)
    timer = ch.Timer()
    reps = max(20, args.steps)
    rows = []
    for name, kind, N, H, W, C, F, RH, RW, pv, ph, sv, sh, dv, dh, fp64 in shapes:
        dt = np.float64 if (fp64 or args.dtype == "f64") else np.float32
        es, peak = np.dtype(dt).itemsize, PEAK_TFLOPS["f64" if dt == np.float64 else "f32"] * 1e12
        if kind == "dense":
            layer = ch.DenseKernelLayer(dt, (C,), F)
            in_shape, K = (N, C), C
        elif kind == "conv":
            layer = ch.ConvKernelLayer(dt, (H, W, C), F, RH, RW, pv, ph, sv, sh, dv, dh)
            in_shape, K = (N, H, W, C), RH * RW * C
        else:
            layer = ch.TransConvKernelLayer(dt, (H, W, C), F, RH, RW, pv, ph, sv, sh, dv, dh)
            in_shape, K = (N, H, W, C), RH * RW * F        # of the convolution that maps the output back to the input
        out_shape = (N,) + tuple(layer.get_output_dims())
        wp = layer.get_params()[0]
        wp.set_values(he_normal(gen, wp.get_rows(), wp.get_cols(), dt))
        x = ch.DeviceTensor.from_host(np.asfortranarray(gen.standard_normal(in_shape).astype(dt)))
        go = ch.DeviceTensor.from_host(np.asfortranarray(gen.standard_normal(out_shape).astype(dt)))
        out = ch.DeviceTensor(out_shape, dt)
        dx = ch.DeviceTensor(in_shape, dt)
        # rows and columns of the GEMM: a transposed convolution is the convolution from its output to its input
        M = int(np.prod(in_shape[:-1])) if kind == "transconv" else int(np.prod(out_shape[:-1]))
        cols = C if kind == "transconv" else F

        def timed(fn):
            for _ in range(3):
                fn()
            timer.start()
            for _ in range(reps):
                fn()
            return timer.stop() / reps

        t_fwd = timed(lambda: layer.forward_into(x, out, True)) if args.passes in ("both", "fwd") else None
        t_bwd = None
        if args.passes in ("both", "bwd"):
            layer.forward_into(x, out, True)
            t_bwd = timed(lambda: layer.backward_into(go, dx))
        in_b, out_b, w_b = int(np.prod(in_shape)) * es, int(np.prod(out_shape)) * es, wp.get_rows() * wp.get_cols() * es
        flop = 2.0 * M * K * cols
        for pass_name, t_ms, launches, nbytes in (("fwd", t_fwd, 1, in_b + w_b + out_b), ("bwd", t_bwd, 2, 2 * (in_b + out_b + w_b))):
            if t_ms is None:
                continue
            roof_s = max(launches * flop / peak, nbytes / 8e12)
            rows.append({"layer": name, "pass": pass_name, "M": M, "K": K, "F": cols, "dtype": np.dtype(dt).name,
                         "us": round(t_ms * 1e3, 2), "tflops": round(launches * flop / (t_ms * 1e-3) / 1e12, 2),
                         "bound": "mfma" if launches * flop / peak >= nbytes / 8e12 else "hbm",
                         "roofline_us": round(roof_s * 1e6, 2), "frac_of_roofline": round(roof_s / (t_ms * 1e-3), 4)})
        for t in (x, go, out, dx):
            t.free()
    if args.copy_calibration:
        copy_calibration(ch, dtype)
    return {"metric": "held_out_layer_passes", "unit": "us", "n_gpus": 1, "dtype": args.dtype, "data": "synthetic",
            "config": {"workload": "convolution, transposed-convolution and dense layers outside the BASELINE configurations, one pass "
                                   "per line, tensors resident in HBM"}, "rows": rows}


def pointwise_run(args, dtype):
    """HBM-bound layers at the cfg4 activation shape (N x 56 x 56 x 64): achieved GB/s against the
    algorithmic bytes per element of each pass (read x, write y, ...)."""
    ch = importlib.import_module("c-attl3_amd")
    ch.init(0)
    N, H, W, C = args.batch, SHAPE["H"], SHAPE["W"], SHAPE["C"]
    es = np.dtype(dtype).itemsize
    gen = np.random.default_rng(7)
    x = ch.DeviceTensor.from_host(np.asfortranarray(gen.standard_normal((N, H, W, C)).astype(dtype)))
    y = ch.DeviceTensor((N, H, W, C), dtype)
    g = ch.DeviceTensor.from_host(np.asfortranarray(gen.standard_normal((N, H, W, C)).astype(dtype)))
    dx = ch.DeviceTensor((N, H, W, C), dtype)
    yp = ch.DeviceTensor((N, H // 2, W // 2, C), dtype)
    gp = ch.DeviceTensor.from_host(np.asfortranarray(gen.standard_normal((N, H // 2, W // 2, C)).astype(dtype)))
    elems = N * H * W * C
    timer = ch.Timer()
    reps = max(3, args.steps)

    def timed(fn):
        fn()
        timer.start()
        for _ in range(reps):
            fn()
        return timer.stop() / reps

    rows = []

    def add(name, ms, bytes_per_elem):
        gbs = elems * bytes_per_elem / (ms * 1e-3) / 1e9
        rows.append({"kernel": name, "ms": round(ms, 4), "bytes_per_elem": bytes_per_elem, "GB/s": round(gbs, 1),
                     "frac_of_8TB/s": round(gbs / 8000.0, 4)})

    for kind in ("identity", "relu", "sigmoid", "tanh"):
        layer = ch.ActivationLayer(dtype, kind, (H, W, C))
        add(kind + " forward", timed(lambda: layer.forward_into(x, y, True)), 2 * es)
        add(kind + " backward", timed(lambda: layer.backward_into(g, dx)), (2 if kind == "identity" else 3) * es)
    mx = ch.MaxPoolLayer(dtype, (H, W, C))
    add("maxpool 2x2 forward", timed(lambda: mx.forward_into(x, yp, True)), es + (es + 4) / 4.0)
    add("maxpool 2x2 backward", timed(lambda: mx.backward_into(gp, dx)), es + (es + 4) / 4.0)
    mn = ch.MeanPoolLayer(dtype, (H, W, C))
    add("meanpool 2x2 forward", timed(lambda: mn.forward_into(x, yp, True)), es + es / 4.0)
    add("meanpool 2x2 backward", timed(lambda: mn.backward_into(gp, dx)), es + es / 4.0)
    bn = ch.BatchNormLayer(dtype, (H, W, C))
    add("batchnorm forward (training)", timed(lambda: bn.forward_into(x, y, True)), 4 * es)
    add("batchnorm backward", timed(lambda: bn.backward_into(g, dx)), 5 * es)
    dr = ch.DropoutLayer(dtype, (H, W, C), 0.25, seed=1)
    add("dropout forward (training; the mask is regenerated, not stored)", timed(lambda: dr.forward_into(x, y, True)), 2 * es)
    add("dropout backward", timed(lambda: dr.backward_into(g, dx)), 2 * es)
    bc = ch.BroadcastLayer(dtype, (H // 2, W // 2, C), (2, 2, 1))
    add("broadcast 2x2x1 forward (28x28x64 -> 56x56x64)", timed(lambda: bc.forward_into(yp, y, True)), es + es / 4.0)
    add("broadcast 2x2x1 backward", timed(lambda: bc.backward_into(g, yp)), es + es / 4.0)
    # The passes of a fused layer that stream the activation tensor (they run between GEMM launches, so HIP events around a
    # layer call cannot isolate them: their durations and HBM bytes are read from a kernel trace / counter run of this
    # workload): a 1x1 convolution 8 -> 64 channels, so that the tensor behind it has the shape above, followed by
    # batch norm + ReLU + 2x2 max pool (bn_chain_forward / bn_chain_sums / bn_chain_apply kernels), by ReLU + max pool
    # and by sigmoid + mean pool (chain_backward kernels).
    x8 = ch.DeviceTensor.from_host(np.asfortranarray(gen.standard_normal((N, H, W, 8)).astype(dtype)))
    dx8 = ch.DeviceTensor((N, H, W, 8), dtype)
    for members in ((ch.BatchNormLayer(dtype, (H, W, C)), ch.ActivationLayer(dtype, "relu", (H, W, C)), ch.MaxPoolLayer(dtype, (H, W, C))),
                    (ch.ActivationLayer(dtype, "relu", (H, W, C)), ch.MaxPoolLayer(dtype, (H, W, C))),
                    (ch.ActivationLayer(dtype, "sigmoid", (H, W, C)), ch.MeanPoolLayer(dtype, (H, W, C)))):
        conv = ch.ConvKernelLayer(dtype, (H, W, 8), C, 1, 1, 0, 0)
        conv.get_params()[0].set_values(he_normal(gen, 8, C, dtype))
        fused = ch.FusedKernelLayer((conv,) + members)
        for _ in range(reps + 1):
            fused.forward_into(x8, yp, True)
            fused.backward_into(gp, dx8)
        ch.synchronize()
        del fused
    return rows


def convlstm_run(args, dtype):
    """BASELINE configs[4]: ConvLSTM, T=10, batch 32, 16x16x8 input, 32 hidden channels, 3x3 kernels, output = last
    hidden state, full BPTT; one step = propagate + backpropagate on sequences resident in HBM."""
    ch = importlib.import_module("c-attl3_amd")
    ch.init(0)
    N, T, H, W, C, hid = 32, 10, 16, 16, 8, 32
    gen = np.random.default_rng(0xC0FFEE05)
    net = ch.ConvLSTMNetwork(dtype, (H, W, C), hid, output_seq_size_func=lambda t: (1, t - 1))
    for k in range(8):
        w, _ = net.kernel_params(k)
        w.set_values(he_normal(gen, w.get_rows(), hid, dtype))
    x = ch.DeviceTensor.from_host(np.asfortranarray(gen.standard_normal((N, T, H, W, C)).astype(dtype)))
    go = ch.DeviceTensor.from_host(np.asfortranarray(gen.standard_normal((N, 1, H, W, hid)).astype(dtype)))

    def step():
        net.propagate(x)
        net.backpropagate(go)

    for _ in range(args.warmup):
        step()
    ch.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    ch.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps
    # the same propagate + backpropagate recorded once and launched as a HIP graph
    with ch.Graph() as graph:
        step()
    for _ in range(args.warmup):
        graph.launch()
    ch.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        graph.launch()
    ch.synchronize()
    graph_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    graph.destroy()
    M = N * H * W
    fwd = 2.0 * M * hid * 4 * (T * 9 * C + (T - 1) * 9 * hid)          # the 4+4 kernels of every step
    flop = 2 * fwd + 2.0 * M * 4 * hid * 9 * hid * (T - 1)              # + weight gradients + recurrent input gradients
    return {"metric": "convlstm_bptt_sequences_per_s", "value": round(N / (ms * 1e-3), 1), "unit": "sequences/s", "n_gpus": 1,
            "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 4), "higher_is_better": True,
            "dtype": args.dtype, "data": "synthetic", "gflops": round(flop / (ms * 1e-3) / 1e9, 1),
            "recorded_as_hip_graph": {"ms_per_step": round(graph_ms, 4), "sequences_per_s": round(N / (graph_ms * 1e-3), 1)},
            "config": {"workload": "ConvLSTM T=10 batch 32 16x16x8 -> 32 hidden, 3x3, propagate + BPTT (BASELINE configs[4])",
                       "flop_per_step": flop}}


def train_steps_run(args, dtype):
    """BASELINE configs[1] and [2] as whole device-resident training steps (propagate, softmax cross-entropy gradient,
    backpropagate, optimizer update, gradient reset): MLP 784-512-256-10 at batch 256 with vanilla SGD, and
    conv32-ReLU-pool-conv64-BN-ReLU-pool-dense10 on 32x32x3 at batch 128 with Adam."""
    ch = importlib.import_module("c-attl3_amd")
    ch.init(0)
    gen = np.random.default_rng(0xC0FFEE02)

    def mlp():
        return [ch.DenseKernelLayer(dtype, (784,), 512), ch.ActivationLayer(dtype, "relu", (512,)),
                ch.DenseKernelLayer(dtype, (512,), 256), ch.ActivationLayer(dtype, "relu", (256,)),
                ch.DenseKernelLayer(dtype, (256,), 10)]

    def convnet():
        return [ch.ConvKernelLayer(dtype, (32, 32, 3), 32), ch.ActivationLayer(dtype, "relu", (32, 32, 32)),
                ch.MaxPoolLayer(dtype, (32, 32, 32)), ch.ConvKernelLayer(dtype, (16, 16, 32), 64),
                ch.BatchNormLayer(dtype, (16, 16, 64)), ch.ActivationLayer(dtype, "relu", (16, 16, 64)),
                ch.MaxPoolLayer(dtype, (16, 16, 64)), ch.DenseKernelLayer(dtype, (8, 8, 64), 10)]

    rows = []
    for name, build, N, in_shape, out_shape, adam, flop, fuse in (
            ("MLP 784-512-256-10, batch 256, vanilla SGD (BASELINE configs[1])", mlp, 256, (784,), (10,), False, 616300544.0, False),
            ("the same MLP, each dense layer and its ReLU as one fused layer", mlp, 256, (784,), (10,), False, 616300544.0, True),
            ("convnet 32x32x3, batch 128, Adam (BASELINE configs[2])", convnet, 128, (32, 32, 3), (10, 1, 1), True, 4.108e9, False),
            ("the same convnet, conv-ReLU-pool and conv-BN-ReLU-pool as fused layers", convnet, 128, (32, 32, 3), (10, 1, 1), True,
             4.108e9, True)):
        layers = build()
        layers[0].set_input_layer(True)
        params = [p for l in layers for p in l.get_params()]
        if fuse:
            layers = ch.fuse_layers(layers)
        for p in params:
            if p.are_optimizable() and p.get_rows() > 1:
                p.set_values(he_normal(gen, p.get_rows(), p.get_cols(), dtype))
        plist = ch.ParameterList(params)
        x = ch.DeviceTensor.from_host(np.asfortranarray(gen.standard_normal((N,) + in_shape).astype(dtype)))
        obj = np.zeros((N,) + out_shape, dtype, order="F")
        obj.reshape((N, -1), order="F")[np.arange(N), gen.integers(0, 10, N)] = 1
        y = ch.DeviceTensor.from_host(obj)

        def step(t):
            a = x
            for l in layers:
                a = l.pass_forward(a, True)
            g = ch.loss_d_function("softmax_cross_entropy", a, y, scale=1.0 / N)
            for l in reversed(layers):
                g = l.pass_back(g)
            # update + reset_grad of SGDOptimizer::_train over all parameters, sixteen per launch
            if adam:
                plist.optimizer_step("adam", [1e-3, 1e-1, 1e-3, 1e-5], timestep=t)
            else:
                plist.optimizer_step("vanilla_sgd", [1e-3])

        for t in range(args.warmup):
            step(t)
        ch.synchronize()
        t0 = time.perf_counter()
        for t in range(args.steps):
            step(t)
        ch.synchronize()
        ms = (time.perf_counter() - t0) * 1e3 / args.steps
        rows.append({"workload": name, "ms_per_step": round(ms, 4), "samples_per_s": round(N / (ms * 1e-3), 1),
                     "gflops": round(flop / (ms * 1e-3) / 1e9, 1)})
        if fuse:
            # the same step recorded once and launched as a HIP graph (cattle_hip_graph_*); Adam's update depends on the
            # time step, a scalar argument, so it stays outside the recording
            def passes(t):
                a = x
                for l in layers:
                    a = l.pass_forward(a, True)
                g = ch.loss_d_function("softmax_cross_entropy", a, y, scale=1.0 / N)
                for l in reversed(layers):
                    g = l.pass_back(g)
                if not adam:
                    plist.optimizer_step("vanilla_sgd", [1e-3])

            with ch.Graph() as graph:
                passes(0)

            def graph_step(t):
                graph.launch()
                if adam:
                    plist.optimizer_step("adam", [1e-3, 1e-1, 1e-3, 1e-5], timestep=t)

            for t in range(args.warmup):
                graph_step(t)
            ch.synchronize()
            t0 = time.perf_counter()
            for t in range(args.steps):
                graph_step(t)
            ch.synchronize()
            ms = (time.perf_counter() - t0) * 1e3 / args.steps
            rows.append({"workload": name + ", recorded as a HIP graph" + (" (Adam step outside)" if adam else ""),
                         "ms_per_step": round(ms, 4), "samples_per_s": round(N / (ms * 1e-3), 1),
                         "gflops": round(flop / (ms * 1e-3) / 1e9, 1)})
            ch.synchronize()
            graph.destroy()
    line = {"metric": "device_resident_training_step", "unit": "ms", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "dtype": args.dtype, "data": "synthetic",
            "driver": "python (ctypes), one C-ABI call per layer pass, one for the optimizer step", "steps_timed": rows}
    # the same two steps driven from C++ through DeviceNet.hpp (fp32; each batch reads its loss back, as SGDOptimizer::_train does)
    exe = os.path.join(ROOT, "c-attl3_amd", "examples", "train_steps")
    if os.path.exists(exe) and args.dtype == "f32":
        import subprocess
        out = subprocess.run([exe, str(max(args.steps, 20)), str(args.warmup)], stdout=subprocess.PIPE, check=True).stdout
        line["cpp_driver"] = json.loads(out.decode().strip().splitlines()[-1])
    return line


def cpu_baseline(args, dtype):
    """Times the oracle (the restatement of the reference algorithm: explicit patch matrix + GEMMs +
    col2im, OpenMP GEMMs) on a bounded sample: the same layer at a smaller batch."""
    from oracle import oracle
    N = args.cpu_batch
    H, W, C, F = SHAPE["H"], SHAPE["W"], SHAPE["C"], SHAPE["F"]
    K = 9 * C
    gen = np.random.default_rng(0xC0FFEE04)
    w = he_normal(gen, K, F, dtype)
    b = np.zeros((1, F), dtype)
    x = np.asfortranarray(gen.standard_normal((N, H, W, C)).astype(dtype))
    go = np.asfortranarray(gen.standard_normal((N, H, W, F)).astype(dtype))
    best = None
    for _ in range(3):
        t0 = time.perf_counter()
        _, cache = oracle.conv_forward(x, w, b, return_cache=True)
        oracle.conv_backward(x.shape, cache, w, go)
        dt = time.perf_counter() - t0
        best = dt if best is None else min(best, dt)
    flop = 6.0 * N * H * W * K * F
    return {
        "value": round(flop / best / 1e9, 2), "unit": "GFLOP/s", "cores": oracle.num_threads(), "kind": "port",
        "sample": "same layer at batch %d (1/%d of the workload), best of 3, %.2f s per fwd+bwd, %.1f samples/s"
                  % (N, max(1, args.batch // N), best, N / best),
    }


# ---- summaries of rocprofv3 output (what profiles/*.md are made of) -------------------------------------------------

PASSES = ("gather_gemm_kernel (forward)", "wgrad_kernel (+ reduce, bias column sums)", "gather_gemm_kernel (input gradient)")


def short_kernel_name(name):
    return name.replace("void cattle_hip::(anonymous namespace)::", "").split("(")[0]


def summarize_kernels(directory, limit=16):
    """The top_kernels view of a `rocprofv3 --kernel-trace --stats` run as a markdown table (microseconds)."""
    out = ["| kernel | calls | total us | average us | % |", "|---|---|---|---|---|"]
    for db in sorted(glob.glob(os.path.join(directory, "**", "*_results.db"), recursive=True)):
        con = sqlite3.connect(db)
        rows = con.execute("select name, total_calls, total_duration, average, percentage from top_kernels").fetchall()
        for name, calls, total, avg, pct in rows[:limit]:
            out.append("| `%s` | %d | %.1f | %.1f | %.2f |" % (short_kernel_name(name), calls, total, avg, pct))      # the view is in microseconds
    return "\n".join(out)


def read_counters(directory):
    """[(dispatch id, kernel, counter, value)] of a `rocprofv3 --pmc ... --output-format csv` run, in dispatch order."""
    rows = []
    for path in sorted(glob.glob(os.path.join(directory, "**", "*counter_collection.csv"), recursive=True)):
        with open(path) as f:
            for r in csv.DictReader(f):
                rows.append((int(r["Dispatch_Id"]), short_kernel_name(r["Kernel_Name"]), r["Counter_Name"], float(r["Counter_Value"])))
    rows.sort(key=lambda r: r[0])
    return rows


def summarize_counters(directories):
    """Mean counter value per dispatch, per kernel, as a markdown table."""
    agg = collections.OrderedDict()
    names = []
    for d in directories:
        for _, kernel, counter, value in read_counters(d):
            agg.setdefault(kernel, collections.OrderedDict()).setdefault(counter, []).append(value)
            if counter not in names:
                names.append(counter)
    out = ["| kernel | dispatches | " + " | ".join(names) + " |", "|---|---|" + "---|" * len(names)]
    for kernel, per in agg.items():
        n = max(len(v) for v in per.values())
        cells = ["%.6g" % (sum(per[c]) / len(per[c])) if c in per else "" for c in names]
        out.append("| `%s` | %d | %s |" % (kernel, n, " | ".join(cells)))
    return "\n".join(out)


def per_pass(rows, copy_kernel_prefix="act_forward_kernel"):
    """Mean counter value per dispatch for the three GEMM passes (each with its reduce launch) and for the
    calibration copy. A gather launch that follows a weight-gradient launch is the input gradient, any other one the
    forward pass; reduce launches belong to the GEMM launch before them."""
    sums = collections.defaultdict(list)
    last = None
    current = None
    for _, kernel, _, value in rows:
        if kernel.startswith("gather_gemm_kernel"):
            current = PASSES[2] if last == "wgrad" else PASSES[0]
            last = "gather"
            sums[current + " | kernel"].append(value)
        elif kernel.startswith("wgrad_kernel"):
            current = PASSES[1]
            last = "wgrad"
            sums[current + " | kernel"].append(value)
        elif kernel.startswith("reduce_partials"):
            # the weight gradient's slices are summed when the gradient is next needed: by the backward pass after
            sums[PASSES[1] + " | reduce"].append(value)
        elif kernel.startswith("split_reduce_kernel"):
            if current is not None:
                sums[current + " | reduce"].append(value)
        elif kernel.startswith(copy_kernel_prefix):
            sums["copy"].append(value)
    return {k: sum(v) / len(v) for k, v in sums.items()}


def summarize_traffic(fetch_dir, write_dir, dtype, batch, write):
    es = 4 if dtype == "f32" else 8
    copy_bytes = batch * 56 * 56 * 64 * es             # the identity activation reads and writes one input-sized tensor
    fetch, wr = per_pass(read_counters(fetch_dir)), per_pass(read_counters(write_dir))
    if "copy" not in fetch or "copy" not in wr:
        sys.exit("no calibration copy in the counter runs: run bench.py with --copy-calibration")
    f_fac, w_fac = copy_bytes / (fetch["copy"] * 1024.0), copy_bytes / (wr["copy"] * 1024.0)
    entry = {}
    lines = ["| pass | read MB (kernel + reduce) | written MB (kernel + reduce) | total MB |", "|---|---|---|---|"]
    for p in PASSES:
        rk, rr = fetch.get(p + " | kernel", 0.0) * 1024 * f_fac, fetch.get(p + " | reduce", 0.0) * 1024 * f_fac
        wk, wrd = wr.get(p + " | kernel", 0.0) * 1024 * w_fac, wr.get(p + " | reduce", 0.0) * 1024 * w_fac
        entry[p] = round(rk + rr + wk + wrd)
        lines.append("| %s | %.1f + %.1f | %.1f + %.1f | %.1f |" % (p, rk / 1e6, rr / 1e6, wk / 1e6, wrd / 1e6, entry[p] / 1e6))
    print("calibration copy: %d bytes each way; FETCH_SIZE reads %.1f KiB (factor %.3f), WRITE_SIZE %.1f KiB (factor %.3f)"
          % (copy_bytes, fetch["copy"], f_fac, wr["copy"], w_fac))
    print("\n".join(lines))
    if write:
        path = os.path.join(ROOT, "profiles", "conv_cfg4_hbm_traffic.json")
        try:
            with open(path) as f:
                rec = json.load(f)
        except (OSError, ValueError):
            rec = {}
        h = kernel_sources_hash()
        if rec.get("kernel_sources_sha256_16") != h:
            rec = {"entries": {}}
        rec["kernel_sources_sha256_16"] = h
        rec["kernel_sources"] = list(KERNEL_SOURCES)
        rec["fetch_factor"], rec["write_factor"] = round(f_fac, 4), round(w_fac, 4)
        rec["unit"] = "bytes per launch, kernel and its reduce launch, read + written"
        rec["entries"]["%s:%d" % (dtype, batch)] = entry
        with open(path, "w") as f:
            json.dump(rec, f, indent=1, sort_keys=True)
            f.write("\n")
        print("wrote", path)


def summarize_hbm(fetch_dir, write_dir, copy_bytes, copy_kernel):
    """Per kernel: mean FETCH_SIZE and WRITE_SIZE readings per dispatch (KiB) of two `rocprofv3 --pmc` runs and the bytes
    they stand for, each counter scaled by what it reads for the dispatches of `copy_kernel`, which move `copy_bytes` each
    way (a plain copy run in the same process: `--copy-calibration`, or the identity layer of the pointwise workload)."""
    def means(directory):
        agg = collections.OrderedDict()
        for _, kernel, counter, value in read_counters(directory):
            agg.setdefault(kernel, []).append(value)
        return collections.OrderedDict((k, (sum(v) / len(v), len(v))) for k, v in agg.items())
    fetch, wr = means(fetch_dir), means(write_dir)
    fcopy = [v for k, v in fetch.items() if k.startswith(copy_kernel)]
    wcopy = [v for k, v in wr.items() if k.startswith(copy_kernel)]
    if not fcopy or not wcopy:
        sys.exit("no dispatch of %s in the counter runs" % copy_kernel)
    f_fac, w_fac = copy_bytes / (fcopy[0][0] * 1024.0), copy_bytes / (wcopy[0][0] * 1024.0)
    out = ["calibration: `%s` moves %d bytes each way; FETCH_SIZE reads %.1f KiB (factor %.3f), WRITE_SIZE %.1f KiB (factor %.3f)"
           % (copy_kernel, copy_bytes, fcopy[0][0], f_fac, wcopy[0][0], w_fac), "",
           "| kernel | dispatches | FETCH_SIZE KiB | WRITE_SIZE KiB | read MB | written MB | total MB |", "|---|---|---|---|---|---|---|"]
    for kernel, (fv, n) in fetch.items():
        wv = wr.get(kernel, (0.0, 0))[0]
        rb, wb = fv * 1024 * f_fac, wv * 1024 * w_fac
        out.append("| `%s` | %d | %.1f | %.1f | %.3f | %.3f | %.3f |" % (kernel, n, fv, wv, rb / 1e6, wb / 1e6, (rb + wb) / 1e6))
    return "\n".join(out)


def summarize_main(argv):
    """`bench.py summarize ...`: turns rocprofv3 output of bench.py runs into the short summaries kept under profiles/.

        python bench.py summarize kernels  <dir with *_results.db>
        python bench.py summarize counters <dir with *counter_collection.csv> [...]
        python bench.py summarize traffic  <FETCH_SIZE dir> <WRITE_SIZE dir> --dtype f32 --batch 256 [--write]
        python bench.py summarize hbm      <FETCH_SIZE dir> <WRITE_SIZE dir> --copy-bytes B [--copy-kernel PREFIX]

    `traffic` needs the two counter runs to have been made with `bench.py --copy-calibration`, which adds a plain copy
    kernel of known size: each counter is scaled by what it reads for that copy. With --write it rewrites
    profiles/conv_cfg4_hbm_traffic.json, which the default run reads for `roofline.traffic`, together with a hash of the
    kernel sources, so that figures measured on other sources are never reported."""
    ap = argparse.ArgumentParser(prog="bench.py summarize")
    sub = ap.add_subparsers(dest="cmd", required=True)
    k = sub.add_parser("kernels")
    k.add_argument("directory")
    k.add_argument("--limit", type=int, default=16)
    c = sub.add_parser("counters")
    c.add_argument("directories", nargs="+")
    t = sub.add_parser("traffic")
    t.add_argument("fetch_dir")
    t.add_argument("write_dir")
    t.add_argument("--dtype", default="f32")
    t.add_argument("--batch", type=int, default=256)
    t.add_argument("--write", action="store_true")
    h = sub.add_parser("hbm")
    h.add_argument("fetch_dir")
    h.add_argument("write_dir")
    h.add_argument("--copy-bytes", type=int, required=True)
    h.add_argument("--copy-kernel", default="act_forward_kernel<float, 0")
    a = ap.parse_args(argv)
    if a.cmd == "hbm":
        print(summarize_hbm(a.fetch_dir, a.write_dir, a.copy_bytes, a.copy_kernel))
        return
    if a.cmd == "kernels":
        print(summarize_kernels(a.directory, a.limit))
    elif a.cmd == "counters":
        print(summarize_counters(a.directories))
    else:
        summarize_traffic(a.fetch_dir, a.write_dir, a.dtype, a.batch, a.write)


def main():
    if sys.argv[1:2] == ["summarize"]:
        summarize_main(sys.argv[2:])
        return
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--batch", type=int, default=256)
    ap.add_argument("--dtype", choices=["f32", "f64"], default="f32")
    ap.add_argument("--cpu-batch", type=int, default=256)
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also launch a plain copy kernel of x's size (for scaling rocprof byte counters)")
    ap.add_argument("--only", default="", help="small_convs / conv_shapes: only the layers whose name contains this")
    ap.add_argument("--passes", choices=["both", "fwd", "bwd"], default="both", help="small_convs / conv_shapes: which passes to run")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--repeats", type=int, default=5, help="how often the timed loop of --steps steps is repeated (median reported)")
    ap.add_argument("--no-extra", action="store_true", help="skip the fp64 leg and the host-tensor leg of the default run")
    ap.add_argument("--workload", choices=["conv", "pointwise", "convlstm", "train_steps", "small_convs", "conv_shapes"], default="conv",
                    help="conv: the headline benchmark; pointwise: HBM-bound layers, one line of per-kernel GB/s; "
                         "convlstm: the fused-gate ConvLSTM of BASELINE configs[4], sequences/s; "
                         "train_steps: whole device-resident training steps of BASELINE configs[1] and [2]; "
                         "small_convs: the convolution layers of the other configurations against both rooflines; "
                         "conv_shapes: a held-out table of layer shapes that no launch rule was tuned on")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one MI355X: this build has no multi-GPU path, run with --gpus 1")
    dtype = np.float32 if args.dtype == "f32" else np.float64
    if args.workload == "pointwise":
        rows = pointwise_run(args, dtype)
        print(json.dumps({"metric": "pointwise_layer_hbm_bandwidth", "unit": "GB/s", "n_gpus": 1, "dtype": args.dtype,
                          "data": "synthetic", "config": {"workload": "activation / pool / batch-norm layers on a %d x 56 x 56 x 64 "
                                                                      "tensor resident in HBM" % args.batch},
                          "roofline": {"bound": "hbm", "peak": 8000.0, "unit": "GB/s"}, "kernels": rows}))
        return

    if args.workload == "train_steps":
        print(json.dumps(train_steps_run(args, dtype)))
        return
    if args.workload == "convlstm":
        print(json.dumps(convlstm_run(args, dtype)))
        return
    if args.workload == "small_convs":
        print(json.dumps(small_convs_run(args, dtype)))
        return
    if args.workload == "conv_shapes":
        print(json.dumps(conv_shapes_run(args, dtype)))
        return

    r = gpu_run(args, dtype)
    step_flop = 3.0 * r["gemm_flop"]
    gflops = step_flop / (r["wall_ms"] * 1e-3) / 1e9
    peak = PEAK_TFLOPS[args.dtype]
    name, t_ms = max(r["kernels"].items(), key=lambda kv: kv[1])
    achieved = r["gemm_flop"] / (t_ms * 1e-3) / 1e12
    line = {
        "metric": "conv_fwd_bwd_gflops", "value": round(gflops, 1), "unit": "GFLOP/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(r["wall_ms"], 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": args.dtype, "data": "synthetic",
        "config": {"workload": "ConvKernelLayer<%s,3> fwd+bwd, batch %d, NHWC 56x56x64 -> 128 filters 3x3 s1 p1 "
                               "(BASELINE configs[3])" % ("float" if args.dtype == "f32" else "double", args.batch),
                   "M": r["M"], "K": r["K"], "F": r["F"], "flop_per_step": step_flop},
        "samples_per_s": round(args.batch / (r["wall_ms"] * 1e-3), 1),
        "frac_of_mfma_peak": round(gflops / 1e3 / peak, 4),
        "roofline": {"bound": "mfma", "kernel": name, "achieved": round(achieved, 2), "peak": peak, "unit": "TFLOP/s",
                     "frac": round(achieved / peak, 4),
                     "traffic": None,
                     "algorithmic_bytes": r["bytes"][name],
                     "flop_per_launch": r["gemm_flop"], "ms_per_launch": round(t_ms, 4)},
        "kernel_ms": {k: round(v, 4) for k, v in r["kernels"].items()},
    }
    line["roofline"]["traffic"], line["roofline"]["traffic_source"] = measured_traffic(args.dtype, args.batch, name)
    line["repeats"] = {"n": len(r["walls"]), "ms_per_step_min": round(min(r["walls"]), 4),
                       "ms_per_step_median": round(float(np.median(r["walls"])), 4), "ms_per_step_max": round(max(r["walls"]), 4)}
    if not args.no_extra and args.dtype == "f32":
        # BASELINE configs[3] asks for both MFMA paths: the same layer and step count in fp64
        d = gpu_run(args, np.float64)
        d_tflops = 3.0 * d["gemm_flop"] / (d["wall_ms"] * 1e-3) / 1e12
        line["f64"] = {"ms_per_step": round(d["wall_ms"], 4), "tflops": round(d_tflops, 2),
                       "frac_of_mfma_peak": round(d_tflops / PEAK_TFLOPS["f64"], 4), "peak": PEAK_TFLOPS["f64"],
                       "samples_per_s": round(args.batch / (d["wall_ms"] * 1e-3), 1),
                       "ms_per_step_min": round(min(d["walls"]), 4), "ms_per_step_max": round(max(d["walls"]), 4),
                       "kernel_ms": {k: round(v, 4) for k, v in d["kernels"].items()}}
    if not args.no_extra:
        line["host_tensor_api"] = host_tensor_run(args, dtype)
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(args, dtype)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
