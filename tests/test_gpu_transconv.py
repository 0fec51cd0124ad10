"""GPU parity of the transposed convolution layer (layer/kernel/TransConvKernelLayer.hpp), called through
the C ABI, against the CPU oracle on identical seeded inputs (fp32 1e-4, fp64 1e-10)."""
import importlib

import numpy as np
import pytest

import helpers as hp
from oracle import oracle

pytestmark = pytest.mark.gpu

ch = importlib.import_module("c-attl3_amd")

TOL = {np.dtype(np.float32): 1e-4, np.dtype(np.float64): 1e-10}
DTYPES = [np.float32, np.float64]


def _geom(case):
    IH, IW, C, F, RH, RW, pv, ph, sv, sh, dv, dh = case
    return dict(RH=RH, RW=RW, pv=pv, ph=ph, sv=sv, sh=sh, dv=dv, dh=dh)


def _layer(dtype, case):
    IH, IW, C, F, RH, RW, pv, ph, sv, sh, dv, dh = case
    return ch.TransConvKernelLayer(dtype, (IH, IW, C), F, RH, RW, pv, ph, sv, sh, dv, dh)


def _inputs(case, N, dtype, seed):
    IH, IW, C, F, RH, RW, pv, ph, sv, sh, dv, dh = case
    g = hp.rng(seed)
    OH, OW = oracle.transconv_out_dims(IH, IW, RH, RW, pv, ph, sv, sh, dv, dh)
    x = hp.uniform(g, (N, IH, IW, C), -1, 1, dtype)
    w = hp.uniform(g, (C, RH * RW * F), -1, 1, dtype)
    b = hp.uniform(g, (1, OH * OW * F), -1, 1, dtype)
    go = hp.uniform(g, (N, OH, OW, F), -1, 1, dtype)
    return x, w, b, go


def _check(case, N, dtype, seed=400):
    x, w, b, go = _inputs(case, N, dtype, seed)
    layer = _layer(dtype, case)
    wp, bp = layer.get_params()
    assert wp.get_values().shape == w.shape and bp.get_values().shape == b.shape
    wp.set_values(w)
    bp.set_values(b)
    out = layer.pass_forward(x, True)
    dx = layer.pass_back(go)
    x64, w64, b64, go64 = (np.asarray(a, np.float64) for a in (x, w, b, go))
    o_ref = oracle.transconv_forward(x64, w64, b64, case[3], **_geom(case))
    dx_ref, dw_ref, db_ref = oracle.transconv_backward(x64, w64, go64, **_geom(case))
    tol = TOL[np.dtype(dtype)]
    assert out.shape == o_ref.shape
    assert hp.rel_err(out, o_ref) < tol, "forward"
    assert hp.rel_err(dx, dx_ref) < tol, "input gradient"
    assert hp.rel_err(wp.get_grad(), dw_ref) < tol, "weight gradient"
    assert hp.rel_err(bp.get_grad(), db_ref) < tol, "bias gradient"
    return layer, (x, w, b, go), (o_ref, dx_ref, dw_ref, db_ref)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("N", [4, 5])         # 4: vector loads along N; 5: scalar path
@pytest.mark.parametrize("case", hp.REFERENCE_TRANSCONV_CASES)
def test_transconv_reference_geometries(case, N, dtype):
    _check(case, N, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_transconv_upsampling_at_a_real_size(dtype):
    """32 samples of 14x14x64 -> 28x28x32 through a 4x4 stride-2 padding-1 receptor (GEMMs of K = 512 / 1024)."""
    _check((14, 14, 64, 32, 4, 4, 1, 1, 2, 2, 0, 0), 32, dtype, seed=401)


def test_transconv_accumulates_skips_and_shares():
    dtype = np.float32
    case = hp.REFERENCE_TRANSCONV_CASES[3]
    layer, (x, w, b, go), (o_ref, dx_ref, dw_ref, db_ref) = _check(case, 4, dtype)
    wp, bp = layer.get_params()
    # a second pass_back adds to the gradients (parameters/StandardParameters.hpp:115-123)
    layer.pass_back(go)
    assert hp.rel_err(wp.get_grad(), 2 * dw_ref) < 1e-4 and hp.rel_err(bp.get_grad(), 2 * db_ref) < 1e-4
    wp.reset_grad()
    bp.reset_grad()
    # an input layer returns a null tensor and still accumulates (TransConvKernelLayer.hpp:209-210)
    layer.set_input_layer(True)
    layer.pass_forward(x, True)
    assert layer.pass_back(go) is None
    assert hp.rel_err(wp.get_grad(), dw_ref) < 1e-4
    layer.set_input_layer(False)
    # a clone with shared parameters sees value changes and adds to the same gradient
    twin = layer.clone_with_shared_params()
    w2 = np.asfortranarray(w * dtype(0.5))
    wp.set_values(w2)
    assert np.array_equal(twin.get_params()[0].get_values(), w2)
    o2 = twin.pass_forward(x, True)
    assert hp.rel_err(o2, oracle.transconv_forward(np.asarray(x, np.float64), np.asarray(w2, np.float64),
                                                   np.asarray(b, np.float64), case[3], **_geom(case))) < 1e-4
    twin.pass_back(go)
    assert hp.rel_err(wp.get_grad(), 2 * dw_ref) < 1e-4
    # a device-side update changes what the next forward pass uses (the transposed weights are rebuilt)
    wp.reset_grad()
    layer.pass_forward(x, True)
    layer.pass_back(go)
    wp.sgd_update(0.1)
    w3 = np.asarray(w2, np.float64) - float(dtype(0.1)) * dw_ref
    assert hp.rel_err(wp.get_values(), w3) < 1e-4
    assert hp.rel_err(layer.pass_forward(x, True),
                      oracle.transconv_forward(np.asarray(x, np.float64), np.asarray(wp.get_values(), np.float64),
                                               np.asarray(b, np.float64), case[3], **_geom(case))) < 1e-4


@pytest.mark.parametrize("dtype", DTYPES)
def test_transconv_rank_1_and_2_views(dtype):
    """TransConvKernelLayer<Scalar,1|2>: data re-viewed as single-column / single-channel, filters folded into the
    last nominal rank of the output (test/gradient_test.cpp:194-199)."""
    g = hp.rng(402)
    tol = TOL[np.dtype(dtype)]
    l1 = ch.TransConvKernelLayer(dtype, (16,), 5, 4, vertical_padding=1, vertical_stride=1, vertical_dilation=1)
    assert l1.get_output_dims() == (100,)
    x = hp.uniform(g, (4, 16), -1, 1, dtype)
    w = hp.uniform(g, (1, 20), -1, 1, dtype)
    l1.get_params()[0].set_values(w)
    ref = oracle.transconv_forward(np.asarray(x, np.float64).reshape((4, 16, 1, 1)), np.asarray(w, np.float64), np.zeros((1, 100)),
                                   5, RH=4, RW=1, pv=1, ph=0, sv=1, sh=1, dv=1, dh=0)
    assert hp.rel_err(l1.pass_forward(x, True), ref.reshape((4, 100), order="F")) < tol
    l2 = ch.TransConvKernelLayer(dtype, (4, 5), 5, 5, 3, 1, 0, 1, 2, 0, 1)
    assert l2.get_output_dims() == (6, 65)
    x = hp.uniform(g, (4, 4, 5), -1, 1, dtype)
    w = hp.uniform(g, (1, 75), -1, 1, dtype)
    l2.get_params()[0].set_values(w)
    ref = oracle.transconv_forward(np.asarray(x, np.float64).reshape((4, 4, 5, 1)), np.asarray(w, np.float64), np.zeros((1, 390)),
                                   5, RH=5, RW=3, pv=1, ph=0, sv=1, sh=2, dv=0, dh=1)
    assert hp.rel_err(l2.pass_forward(x, True), ref.reshape((4, 6, 65), order="F")) < tol


def test_transconv_rejects_bad_geometry():
    with pytest.raises(ch.CattleHipError):
        ch.TransConvKernelLayer(np.float32, (4, 4, 2), 0)                       # assert(filters > 0)
    with pytest.raises(ch.CattleHipError):
        ch.TransConvKernelLayer(np.float32, (1, 1, 2), 3, 1, 1, 1, 1)           # the padding removes the whole output
    layer = ch.TransConvKernelLayer(np.float32, (4, 4, 2), 3)
    with pytest.raises(ch.CattleHipError):
        layer.pass_back(np.zeros((2, 4, 4, 3), np.float32, order="F"))          # pass_back before pass_forward
