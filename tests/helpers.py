"""Shared test helpers: seeded inputs in the reference's memory layout, the error metric, and
definitional (brute-force) versions of the layer maths used to pin the oracle."""
import numpy as np

# Conv geometries exercised by the reference's own gradient tests (test/gradient_test.cpp:166-185),
# re-viewed as 4-D (H,W,C) problems the way ConvKernelLayer<Scalar,1|2> does
# (layer/kernel/ConvKernelLayer.hpp:400-417, :494-508), plus the BASELINE-style 3x3 p1 case.
#   (H, W, C, F, RH, RW, pv, ph, sv, sh, dv, dh)
REFERENCE_CONV_CASES = [
    (32, 1, 1, 5, 3, 1, 2, 0, 1, 1, 1, 0),    # rank 1: length 32, k3 p2 s1 d1
    (30, 1, 5, 1, 3, 1, 1, 0, 1, 1, 0, 0),    # rank 1 second layer (as C=5 re-view)
    (10, 10, 1, 5, 3, 2, 1, 2, 1, 2, 1, 0),   # rank 2: 3x2 receptor, pad (1,2), stride (1,2), dilation (1,0)
    (8, 8, 2, 5, 3, 2, 1, 2, 1, 2, 1, 0),     # rank 3: same on 8x8x2
    (6, 6, 5, 1, 2, 2, 1, 1, 1, 1, 0, 0),     # second layer: 2x2 p1 s1
    (7, 6, 3, 4, 3, 3, 1, 1, 1, 1, 0, 0),     # BASELINE-style 3x3 p1 s1
    (9, 11, 2, 3, 2, 3, 0, 1, 2, 3, 0, 1),    # strides (2,3), dilation (0,1), no vertical padding
]

# Transposed-convolution geometries of the reference's gradient test (test/gradient_test.cpp:194-204), re-viewed as
# 4-D problems the way TransConvKernelLayer<Scalar,1|2> does (layer/kernel/TransConvKernelLayer.hpp:404-417,
# :503-516), plus an up-sampling case.   (IH, IW, C, F, RH, RW, pv, ph, sv, sh, dv, dh)
REFERENCE_TRANSCONV_CASES = [
    (16, 1, 1, 5, 4, 1, 1, 0, 1, 1, 1, 0),    # rank 1: length 16, receptor 4, padding 1, dilation 1
    (100, 1, 1, 1, 1, 1, 1, 0, 1, 1, 0, 0),   # rank 1 second layer: receptor 1, padding 1 (cuts the border)
    (4, 5, 1, 5, 5, 3, 1, 0, 1, 2, 0, 1),     # rank 2: 5x3 receptor, pad (1,0), stride (1,2), dilation (0,1)
    (2, 3, 2, 5, 5, 3, 1, 0, 1, 2, 0, 1),     # rank 3: same on 2x3x2
    (4, 9, 5, 1, 2, 2, 1, 1, 1, 1, 0, 0),     # second layer: 2x2 p1 s1
    (5, 4, 3, 4, 3, 3, 1, 1, 1, 1, 0, 0),     # 3x3 p1 s1 (shape preserving)
    (4, 3, 2, 3, 4, 4, 1, 1, 2, 2, 0, 0),     # 4x4 stride 2 padding 1: doubles the resolution
]


def rng(seed):
    return np.random.default_rng(seed)


def uniform(gen, shape, lo, hi, dtype):
    return np.asfortranarray(gen.uniform(lo, hi, size=shape).astype(dtype))


def normal(gen, shape, dtype, std=1.0):
    return np.asfortranarray((gen.standard_normal(size=shape) * std).astype(dtype))


# label -> (floored error, un-floored error over |ref| > floor, element count): what the labelled comparisons of a
# test run achieved; tests/conftest.py prints the table at the end of the run
ACHIEVED = {}


def rel_err(a, b, floor_frac=0.1, label=None):
    """max_i |a_i - b_i| / max(|b_i|, floor), floor = floor_frac * RMS(b) (tiny if b is all zero).

    The absolute floor keeps the relative error meaningful for elements that are (near) zero by
    cancellation: they are compared relative to a tenth of the tensor's RMS instead. With a label the
    achieved error is recorded, beside the plain relative error max |a_i - b_i| / |b_i| over the
    elements with |b_i| > floor (no floor in the denominator)."""
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    assert a.shape == b.shape, (a.shape, b.shape)
    if a.size == 0:
        return 0.0
    rms = float(np.sqrt(np.mean(b * b)))
    floor = max(floor_frac * rms, 1e-30)
    diff = np.abs(a - b)
    err = float(np.max(diff / np.maximum(np.abs(b), floor)))
    if label is not None:
        big = np.abs(b) > floor
        plain = float(np.max(diff[big] / np.abs(b[big]))) if np.any(big) else 0.0
        old = ACHIEVED.get(label, (0.0, 0.0, 0))
        ACHIEVED[label] = (max(old[0], err), max(old[1], plain), old[2] + a.size)
    return err


def conv_dims(H, W, RH, RW, pv, ph, sv, sh, dv, dh):
    OH = (H - RH - (RH - 1) * dv + 2 * pv) // sv + 1
    OW = (W - RW - (RW - 1) * dh + 2 * ph) // sh + 1
    return OH, OW


def brute_conv_forward(x, w, b, RH, RW, pv, ph, sv, sh, dv, dh):
    """Definitional cross-correlation in float64: the seven nested loops, no matrices."""
    x = np.asarray(x, dtype=np.float64)
    w = np.asarray(w, dtype=np.float64)
    N, H, W, C = x.shape
    F = w.shape[1]
    OH, OW = conv_dims(H, W, RH, RW, pv, ph, sv, sh, dv, dh)
    out = np.zeros((N, OH, OW, F))
    for n in range(N):
        for oh in range(OH):
            for ow in range(OW):
                for f in range(F):
                    s = float(np.reshape(b, (-1,))[f])
                    for c in range(C):
                        for rw in range(RW):
                            for rh in range(RH):
                                h = oh * sv + rh * (dv + 1) - pv
                                ww = ow * sh + rw * (dh + 1) - ph
                                if 0 <= h < H and 0 <= ww < W:
                                    s += x[n, h, ww, c] * w[rh + RH * (rw + RW * c), f]
                    out[n, oh, ow, f] = s
    return out


def brute_maxpool(x, RH, RW, sv, sh):
    x = np.asarray(x)
    N, H, W, C = x.shape
    OH, OW = (H - RH) // sv + 1, (W - RW) // sh + 1
    out = np.empty((N, OH, OW, C), dtype=x.dtype)
    inds = np.empty((OH * OW, C * N), dtype=np.uint32)
    lowest = np.finfo(x.dtype).min
    for ow in range(OW):
        for oh in range(OH):
            for c in range(C):
                for n in range(N):
                    best, bi = lowest, 0
                    for k in range(RW):
                        for l in range(RH):
                            v = x[n, oh * sv + l, ow * sh + k, c]
                            if v > best:
                                best, bi = v, k * RH + l
                    out[n, oh, ow, c] = best
                    inds[ow * OH + oh, c * N + n] = bi
    return out, inds


ALL_LOSSES = ["squared", "softmax_cross_entropy", "absolute", "binary_cross_entropy", "cross_entropy", "kullback_leibler",
              "hinge", "squared_hinge", "multi_label_hinge", "squared_multi_label_hinge", "multi_label_log"]


def loss_inputs(gen, kind, N, dims, dtype, steps=None):
    """Outputs and objectives a loss of this kind accepts (the ranges its class comment in loss/*.hpp names), as
    (N, *dims) tensors or, with `steps`, (N, steps, *dims) sequences; element j of a sample's step is at Fortran
    position j of its `dims`. binary_cross_entropy takes one value per sample and step (dims must multiply to 1)."""
    Ts = 1 if steps is None else steps
    V = int(np.prod(dims))
    shape = (N, Ts, V)
    if kind in ("squared", "absolute"):
        out, obj = gen.standard_normal(shape), gen.standard_normal(shape)
    elif kind == "softmax_cross_entropy":
        out, obj = gen.standard_normal(shape) * 2, np.zeros(shape)
        np.put_along_axis(obj, gen.integers(0, V, (N, Ts, 1)), 1.0, axis=2)
    elif kind == "binary_cross_entropy":
        assert V == 1
        out, obj = gen.uniform(0.05, 0.95, shape), gen.uniform(0, 1, shape)
    elif kind in ("cross_entropy", "kullback_leibler"):
        out = gen.uniform(0.05, 1, shape)
        out /= out.sum(axis=2, keepdims=True)
        obj = gen.uniform(0.05, 1, shape)
        obj /= obj.sum(axis=2, keepdims=True)
    elif kind in ("hinge", "squared_hinge"):
        out, obj = gen.standard_normal(shape), np.zeros(shape)
        np.put_along_axis(obj, gen.integers(0, V, (N, Ts, 1)), 1.0, axis=2)
    elif kind in ("multi_label_hinge", "squared_multi_label_hinge"):
        out, obj = gen.standard_normal(shape), gen.integers(0, 2, shape) * 2.0 - 1.0
    elif kind == "multi_label_log":
        out, obj = gen.uniform(0.05, 0.95, shape), gen.integers(0, 2, shape) * 1.0
    else:
        raise KeyError(kind)
    full = (N,) + (() if steps is None else (steps,)) + tuple(dims)
    return tuple(np.asfortranarray(np.asfortranarray(a.astype(dtype)).reshape(full, order="F")) for a in (out, obj))
