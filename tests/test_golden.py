"""Committed known answers (tests/golden/layers_golden.npz, written by tests/golden/make_golden.py from
torch float64 autograd and definitional loops, not from the oracle) checked against the CPU oracle
(no GPU needed) and against the HIP layers through the C ABI (gpu-marked).

Inputs are stored in float64; the float32 runs round them first and compare with the float64 answers
within the float32 tolerance."""
import importlib
import os

import numpy as np
import pytest

import helpers as hp
from oracle import oracle

GOLD = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "layers_golden.npz"))
TOL = {np.dtype(np.float32): 1e-4, np.dtype(np.float64): 1e-10}
DTYPES = [np.float32, np.float64]
N_CONV = len(hp.REFERENCE_CONV_CASES)
ACTS = ["identity", "scaled", "sigmoid", "tanh", "softsign", "softplus", "relu", "leaky_relu", "elu", "swish"]


def _in(name, dtype):
    return np.asfortranarray(GOLD[name].astype(dtype))


def _close(got, name, dtype, slack=1.0):
    err = hp.rel_err(got, GOLD[name])
    assert err < slack * TOL[np.dtype(dtype)], (name, err)


def _geom(case):
    H, W, C, F, RH, RW, pv, ph, sv, sh, dv, dh = (int(v) for v in case)
    return (H, W, C, F), dict(RH=RH, RW=RW, pv=pv, ph=ph, sv=sv, sh=sh, dv=dv, dh=dh)


def test_fixture_covers_reference_conv_cases():
    for i, case in enumerate(hp.REFERENCE_CONV_CASES):
        assert tuple(int(v) for v in GOLD["conv%d_case" % i]) == case


# ---------------------------------------------------------------- oracle vs known answers (CPU)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("i", range(N_CONV))
def test_oracle_conv(i, dtype):
    p = "conv%d_" % i
    _, geom = _geom(GOLD[p + "case"])
    x, w, b, go = (_in(p + k, dtype) for k in ("x", "w", "b", "go"))
    out, cache = oracle.conv_forward(x, w, b, return_cache=True, **geom)
    dx, dw, db = oracle.conv_backward(x.shape, cache, w, go, **geom)
    for got, k in ((out, "out"), (dx, "dx"), (dw, "dw"), (db, "db")):
        _close(got, p + k, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_oracle_dense(dtype):
    x, w, b, go = (_in("dense_" + k, dtype) for k in ("x", "w", "b", "go"))
    _close(oracle.dense_forward(x, w, b), "dense_out", dtype)
    dx, dw, db = oracle.dense_backward(x, w, go)
    for got, k in ((dx, "dx"), (dw, "dw"), (db, "db")):
        _close(got, "dense_" + k, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_oracle_batchnorm(dtype):
    x1, x2, gamma, beta, go = (_in("bn_" + k, dtype) for k in ("x1", "x2", "gamma", "beta", "go"))
    C = gamma.size
    am, ais = np.zeros(C, dtype), np.zeros(C, dtype)
    for k, x in enumerate((x1, x2)):
        y, std, isd = oracle.bn_forward(x, gamma, beta, am, ais, k > 0, True)
        dx, dg, db = oracle.bn_backward(go, gamma, std, isd)
        _close(y, "bn_y%d" % k, dtype)
        _close(dx, "bn_dx%d" % k, dtype, 10)      # dx is a difference of O(L)-sized terms
        _close(dg, "bn_dgamma%d" % k, dtype)
        _close(db, "bn_dbeta%d" % k, dtype)
    _close(am, "bn_run_mean", dtype)
    _close(ais, "bn_run_inv_sd", dtype)
    y, _, _ = oracle.bn_forward(x1, gamma, beta, am, ais, True, False)
    _close(y, "bn_y_infer", dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_oracle_activations(dtype):
    x, go = _in("act_x", dtype), _in("act_go", dtype)
    for name in ACTS:
        p = float(dtype(GOLD["act_%s_p" % name]))
        y = oracle.act_forward(name, x, p)
        _close(y, "act_%s_y" % name, dtype)
        _close(oracle.act_backward(name, x, y, go, p), "act_%s_dx" % name, dtype)
    y = oracle.softmax_forward(x, 1e-5)
    _close(y, "softmax_y", dtype)
    _close(oracle.softmax_backward(y, go), "softmax_dx", dtype)
    for name in ("prelu", "pswish"):
        par = GOLD[name + "_param"].astype(dtype)
        _close(getattr(oracle, name + "_forward")(x, par), name + "_y", dtype)
        dx, dp = getattr(oracle, name + "_backward")(x, par, go)
        _close(dx, name + "_dx", dtype)
        _close(dp, name + "_dparam", dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("i", [0, 1])
def test_oracle_pools(i, dtype):
    p = "pool%d_" % i
    RH, RW, sv, sh = (int(v) for v in GOLD[p + "geom"])
    x, go = _in(p + "x", dtype), _in(p + "go", dtype)
    out, inds = oracle.maxpool_forward(x, RH, RW, sv, sh)
    # float32 rounding of the inputs is monotone, so values round alike; crafted ties stay ties
    assert np.array_equal(out, GOLD[p + "max"].astype(dtype))
    if dtype == np.float64:
        assert np.array_equal(inds, GOLD[p + "inds"])
    _close(oracle.maxpool_backward(x.shape, go, GOLD[p + "inds"], RH, RW, sv, sh), p + "max_dx", dtype)
    _close(oracle.meanpool_forward(x, RH, RW, sv, sh), p + "mean", dtype)
    _close(oracle.meanpool_backward(x.shape, go, RH, RW, sv, sh), p + "mean_dx", dtype)


# ---------------------------------------------------------------- HIP layers vs known answers (GPU)
def _ch():
    return importlib.import_module("c-attl3_amd")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("i", range(N_CONV))
def test_hip_conv(i, dtype):
    ch = _ch()
    p = "conv%d_" % i
    (H, W, C, F), g = _geom(GOLD[p + "case"])
    x, w, b, go = (_in(p + k, dtype) for k in ("x", "w", "b", "go"))
    layer = ch.ConvKernelLayer(dtype, (H, W, C), F, g["RH"], g["RW"], g["pv"], g["ph"], g["sv"], g["sh"], g["dv"],
                               g["dh"])
    wp, bp = layer.get_params()
    wp.set_values(w)
    bp.set_values(b)
    _close(layer.pass_forward(x, True), p + "out", dtype)
    _close(layer.pass_back(go), p + "dx", dtype)
    _close(wp.get_grad(), p + "dw", dtype)
    _close(bp.get_grad(), p + "db", dtype)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", DTYPES)
def test_hip_dense(dtype):
    ch = _ch()
    x, w, b, go = (_in("dense_" + k, dtype) for k in ("x", "w", "b", "go"))
    layer = ch.DenseKernelLayer(dtype, x.shape[1:], w.shape[1])
    wp, bp = layer.get_params()
    wp.set_values(w)
    bp.set_values(b)
    out = layer.pass_forward(x, True)
    _close(out.reshape(GOLD["dense_out"].shape, order="F"), "dense_out", dtype)
    _close(layer.pass_back(go.reshape(out.shape, order="F")), "dense_dx", dtype)
    _close(wp.get_grad(), "dense_dw", dtype)
    _close(bp.get_grad(), "dense_db", dtype)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", DTYPES)
def test_hip_batchnorm(dtype):
    ch = _ch()
    x1, x2, gamma, beta, go = (_in("bn_" + k, dtype) for k in ("x1", "x2", "gamma", "beta", "go"))
    layer = ch.BatchNormLayer(dtype, x1.shape[1:])
    prm = layer.get_params()
    prm[2].set_values(gamma.reshape(1, -1))
    prm[3].set_values(beta.reshape(1, -1))
    for k, x in enumerate((x1, x2)):
        prm[2].reset_grad()
        prm[3].reset_grad()
        _close(layer.pass_forward(x, True), "bn_y%d" % k, dtype)
        _close(layer.pass_back(go), "bn_dx%d" % k, dtype, 10)
        _close(prm[2].get_grad().reshape(-1), "bn_dgamma%d" % k, dtype)
        _close(prm[3].get_grad().reshape(-1), "bn_dbeta%d" % k, dtype)
    _close(prm[0].get_values().reshape(-1), "bn_run_mean", dtype)
    _close(prm[1].get_values().reshape(-1), "bn_run_inv_sd", dtype)
    _close(layer.pass_forward(x1, False), "bn_y_infer", dtype)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", DTYPES)
def test_hip_activations(dtype):
    ch = _ch()
    x, go = _in("act_x", dtype), _in("act_go", dtype)
    for name in ACTS:
        layer = ch.ActivationLayer(dtype, name, x.shape[1:], float(GOLD["act_%s_p" % name]))
        _close(layer.pass_forward(x, True), "act_%s_y" % name, dtype)
        _close(layer.pass_back(go), "act_%s_dx" % name, dtype)
    sm = ch.ActivationLayer(dtype, "softmax", x.shape[1:], 1e-5)
    _close(sm.pass_forward(x, True), "softmax_y", dtype)
    _close(sm.pass_back(go), "softmax_dx", dtype)
    for name in ("prelu", "pswish"):
        layer = ch.ActivationLayer(dtype, name, x.shape[1:], 0.1)
        prm = layer.get_params()[0]
        prm.set_values(GOLD[name + "_param"].astype(dtype).reshape(1, -1))
        _close(layer.pass_forward(x, True), name + "_y", dtype)
        _close(layer.pass_back(go), name + "_dx", dtype)
        _close(prm.get_grad().reshape(-1), name + "_dparam", dtype)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("i", [0, 1])
def test_hip_pools(i, dtype):
    ch = _ch()
    p = "pool%d_" % i
    RH, RW, sv, sh = (int(v) for v in GOLD[p + "geom"])
    x, go = _in(p + "x", dtype), _in(p + "go", dtype)
    mx = ch.MaxPoolLayer(dtype, x.shape[1:], RH, RW, sv, sh)
    assert np.array_equal(mx.pass_forward(x, True), GOLD[p + "max"].astype(dtype))
    if dtype == np.float64:
        assert np.array_equal(mx.max_indices(x.shape[0]), GOLD[p + "inds"])
        _close(mx.pass_back(go), p + "max_dx", dtype)
    mean = ch.MeanPoolLayer(dtype, x.shape[1:], RH, RW, sv, sh)
    _close(mean.pass_forward(x, True), p + "mean", dtype)
    _close(mean.pass_back(go), p + "mean_dx", dtype)
