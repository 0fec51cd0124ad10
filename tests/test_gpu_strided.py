"""The input gradient of a strided convolution (and with it the forward pass of a strided transposed convolution) is
computed residue class by residue class of the input positions, each class a stride-1 GEMM over the taps that reach it
(ConvKernelLayer.hpp:159-181 scatters patch by patch; TransConvKernelLayer.hpp:115-151). These are problems large
enough for that path, against the oracle (fp32 1e-4, fp64 1e-10); small ones and strides that share a factor with the
dilation keep the single launch over all taps, which the sweep in test_gpu_conv_sweep.py covers."""
import importlib

import numpy as np
import pytest

import helpers as hp
from oracle import oracle

pytestmark = pytest.mark.gpu

ch = importlib.import_module("c-attl3_amd")

TOL = {np.dtype(np.float32): 1e-4, np.dtype(np.float64): 1e-10}

# N, H, W, C, F, RH, RW, pv, ph, sv, sh, dv, dh
CASES = [
    (128, 32, 32, 32, 64, 3, 3, 1, 1, 2, 2, 0, 0),
    (160, 33, 30, 16, 48, 4, 4, 0, 0, 2, 2, 0, 0),       # odd extents: classes of unequal size
    (96, 24, 24, 32, 32, 3, 3, 1, 1, 1, 2, 0, 0),        # stride along the width only
    (96, 30, 28, 24, 96, 5, 5, 2, 2, 3, 2, 0, 0),
    (192, 32, 32, 16, 64, 3, 3, 3, 3, 2, 2, 2, 2),       # dilated receptor (rows 0, 3, 6) under stride 2
    (128, 32, 32, 64, 256, 1, 1, 0, 0, 2, 2, 0, 0),      # receptor narrower than the stride: three classes get no tap
    (128, 31, 29, 8, 160, 2, 3, 1, 0, 2, 3, 0, 0),
]


def _geom(case):
    N, H, W, C, F, RH, RW, pv, ph, sv, sh, dv, dh = case
    return dict(RH=RH, RW=RW, pv=pv, ph=ph, sv=sv, sh=sh, dv=dv, dh=dh)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("case", CASES, ids=lambda c: "x".join(str(v) for v in c))
def test_strided_input_gradient(case, dtype):
    N, H, W, C, F, RH, RW, pv, ph, sv, sh, dv, dh = case
    if np.dtype(dtype) == np.float64 and case not in (CASES[0], CASES[1], CASES[4]):
        pytest.skip("fp64 on three of the geometries")
    gen = hp.rng(900 + H + C)
    x = hp.normal(gen, (N, H, W, C), dtype)
    w = hp.normal(gen, (RH * RW * C, F), dtype, std=0.2)
    b = hp.normal(gen, (1, F), dtype)
    OH, OW = hp.conv_dims(H, W, RH, RW, pv, ph, sv, sh, dv, dh)
    g = hp.normal(gen, (N, OH, OW, F), dtype)
    layer = ch.ConvKernelLayer(dtype, (H, W, C), F, RH, RW, pv, ph, sv, sh, dv, dh)
    wp, bp = layer.get_params()
    wp.set_values(w)
    bp.set_values(b)
    xd, gd = ch.DeviceTensor.from_host(x), ch.DeviceTensor.from_host(g)
    out = layer.pass_forward(xd, True)
    dx = layer.pass_back(gd).to_host()
    x64, w64, b64, g64 = (np.asarray(a, np.float64) for a in (x, w, b, g))
    o_ref, cache = oracle.conv_forward(x64, w64, b64, return_cache=True, **_geom(case))
    dx_ref, dw_ref, db_ref = oracle.conv_backward(x.shape, cache, w64, g64, **_geom(case))
    tol = TOL[np.dtype(dtype)]
    label = "strided %s %s" % ("x".join(str(v) for v in case), np.dtype(dtype).name)
    assert hp.rel_err(out.to_host(), o_ref) < tol
    assert hp.rel_err(dx, dx_ref, label=label + " dx") < tol
    assert hp.rel_err(wp.get_grad(), dw_ref) < tol
    # positions that no tap reaches get exact zeros, and a second pass reproduces the first bit for bit
    assert np.array_equal(dx == 0, dx_ref == 0) or np.count_nonzero(dx_ref == 0) == 0
    dx2 = layer.pass_back(gd).to_host()
    assert np.array_equal(dx, dx2)
    # the weights change: the prepared layouts of all classes must follow
    wp.set_values(2 * w)
    layer.pass_forward(xd, True)
    dx3 = layer.pass_back(gd).to_host()
    assert hp.rel_err(dx3, 2 * dx_ref) < tol


def test_batch_sizes_on_either_side_of_the_switch():
    """The same layer at a batch that takes the single launch over all taps and at one that goes class by class: the
    prepared weights are laid out differently for the two and must be rebuilt when the layer changes sides."""
    dtype = np.float32
    H, W, C, F = 32, 32, 32, 64
    geom = dict(RH=3, RW=3, pv=1, ph=1, sv=2, sh=2, dv=0, dh=0)
    gen = hp.rng(77)
    w = hp.normal(gen, (9 * C, F), dtype, std=0.2)
    layer = ch.ConvKernelLayer(dtype, (H, W, C), F, 3, 3, 1, 1, 2, 2, 0, 0)
    layer.get_params()[0].set_values(w)
    for N in (8, 128, 8, 128):
        x = hp.normal(gen, (N, H, W, C), dtype)
        g = hp.normal(gen, (N, 16, 16, F), dtype)
        layer.pass_forward(x, True)
        dx = layer.pass_back(g)
        x64, w64, g64 = (np.asarray(a, np.float64) for a in (x, w, g))
        _, cache = oracle.conv_forward(x64, w64, np.zeros((1, F)), return_cache=True, **geom)
        dx_ref, _, _ = oracle.conv_backward(x.shape, cache, w64, g64, **geom)
        assert hp.rel_err(dx, dx_ref) < 1e-4, N


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_strided_transposed_convolution_forward(dtype):
    """96 samples of 16x16x64 -> 31x31x32 through a 3x3 stride-2 padding-1 receptor: the forward pass is the class-by-class
    input gradient of the convolution 31x31x32 -> 16x16x64."""
    IH, IW, C, F = 16, 16, 64, 32
    geom = dict(RH=3, RW=3, pv=1, ph=1, sv=2, sh=2, dv=0, dh=0)
    N = 96
    gen = hp.rng(41)
    OH, OW = oracle.transconv_out_dims(IH, IW, 3, 3, 1, 1, 2, 2, 0, 0)
    x = hp.uniform(gen, (N, IH, IW, C), -1, 1, dtype)
    w = hp.uniform(gen, (C, 9 * F), -1, 1, dtype)
    b = hp.uniform(gen, (1, OH * OW * F), -1, 1, dtype)
    go = hp.uniform(gen, (N, OH, OW, F), -1, 1, dtype)
    layer = ch.TransConvKernelLayer(dtype, (IH, IW, C), F, 3, 3, 1, 1, 2, 2, 0, 0)
    wp, bp = layer.get_params()
    wp.set_values(w)
    bp.set_values(b)
    out = layer.pass_forward(x, True)
    dx = layer.pass_back(go)
    x64, w64, b64, go64 = (np.asarray(a, np.float64) for a in (x, w, b, go))
    o_ref = oracle.transconv_forward(x64, w64, b64, F, **geom)
    dx_ref, dw_ref, db_ref = oracle.transconv_backward(x64, w64, go64, **geom)
    tol = TOL[np.dtype(dtype)]
    assert hp.rel_err(out, o_ref, label="strided transposed convolution %s forward" % np.dtype(dtype).name) < tol
    assert hp.rel_err(dx, dx_ref) < tol
    assert hp.rel_err(wp.get_grad(), dw_ref) < tol
