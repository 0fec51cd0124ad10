"""Pins the CPU oracle's conv and dense routines (oracle/cattle_oracle.cpp) without the reference
being compilable: definitional loops, torch float64 as an independent implementation, closed-form
special cases and adjoint identities. A dropped term, a wrong sign, a transposed operand or a wrong
(rh,rw,c) ordering fails at least one of these."""
import numpy as np
import pytest
import torch

import helpers as hp
from oracle import oracle


def _inputs(case, N, dtype, seed):
    H, W, C, F, RH, RW, pv, ph, sv, sh, dv, dh = case
    g = hp.rng(seed)
    x = hp.uniform(g, (N, H, W, C), -1, 1, dtype)
    w = hp.uniform(g, (RH * RW * C, F), -1, 1, dtype)
    b = hp.uniform(g, (1, F), -1, 1, dtype)
    OH, OW = hp.conv_dims(H, W, RH, RW, pv, ph, sv, sh, dv, dh)
    go = hp.uniform(g, (N, OH, OW, F), -1, 1, dtype)
    return x, w, b, go


def _geom(case):
    H, W, C, F, RH, RW, pv, ph, sv, sh, dv, dh = case
    return dict(RH=RH, RW=RW, pv=pv, ph=ph, sv=sv, sh=sh, dv=dv, dh=dh)


def _torch_conv(x, w, b, go, case):
    """Independent float64 implementation: Eigen order -> NCHW, W[k,f] -> [F,C,RH,RW] with
    k = rh + RH*(rw + RW*c); torch dilation = reference dilation + 1."""
    H, W, C, F, RH, RW, pv, ph, sv, sh, dv, dh = case
    xt = torch.tensor(np.transpose(np.asarray(x, np.float64), (0, 3, 1, 2)).copy(), requires_grad=True)
    w4 = np.asarray(w, np.float64).reshape((RH, RW, C, F), order="F")       # (rh, rw, c, f)
    wt = torch.tensor(np.transpose(w4, (3, 2, 0, 1)).copy(), requires_grad=True)
    bt = torch.tensor(np.asarray(b, np.float64).reshape(-1).copy(), requires_grad=True)
    out = torch.nn.functional.conv2d(xt, wt, bt, stride=(sv, sh), padding=(pv, ph), dilation=(dv + 1, dh + 1))
    got = torch.tensor(np.transpose(np.asarray(go, np.float64), (0, 3, 1, 2)).copy())
    out.backward(got)
    o = np.transpose(out.detach().numpy(), (0, 2, 3, 1))
    dx = np.transpose(xt.grad.numpy(), (0, 2, 3, 1))
    dw = np.transpose(wt.grad.numpy(), (2, 3, 1, 0)).reshape((RH * RW * C, F), order="F")
    db = bt.grad.numpy().reshape(1, F)
    return o, dx, dw, db


@pytest.mark.parametrize("case", hp.REFERENCE_CONV_CASES)
def test_conv_forward_matches_definition(case):
    x, w, b, _ = _inputs(case, 3, np.float64, 11)
    out = oracle.conv_forward(x, w, b, **_geom(case))
    ref = hp.brute_conv_forward(x, w, b, *case[4:])
    assert out.shape == ref.shape
    assert hp.rel_err(out, ref) < 1e-12


@pytest.mark.parametrize("case", hp.REFERENCE_CONV_CASES)
@pytest.mark.parametrize("dtype,tol", [(np.float64, 1e-11), (np.float32, 2e-5)])
def test_conv_forward_backward_match_torch(case, dtype, tol):
    x, w, b, go = _inputs(case, 5, dtype, 12)
    out, cache = oracle.conv_forward(x, w, b, return_cache=True, **_geom(case))
    dx, dw, db = oracle.conv_backward(x.shape, cache, w, go, **_geom(case))
    o_t, dx_t, dw_t, db_t = _torch_conv(x, w, b, go, case)
    assert hp.rel_err(out, o_t) < tol
    assert hp.rel_err(dx, dx_t) < tol
    assert hp.rel_err(dw, dw_t) < tol
    assert hp.rel_err(db, db_t) < tol


def test_conv_patch_matrix_ordering():
    """The cached patch matrix has row n + N*(oh + OH*ow) and column rh + RH*(rw + RW*c)
    (layer/kernel/ConvKernelLayer.hpp:128-142): encode coordinates in the input and decode."""
    N, H, W, C, RH, RW = 2, 4, 5, 3, 2, 3
    x = np.zeros((N, H, W, C), order="F")
    for n in range(N):
        for h in range(H):
            for w_ in range(W):
                for c in range(C):
                    x[n, h, w_, c] = n + 10 * h + 100 * w_ + 1000 * c
    w = np.zeros((RH * RW * C, 1), order="F")
    _, cache = oracle.conv_forward(x, w, np.zeros((1, 1)), RH=RH, RW=RW, pv=0, ph=0, return_cache=True)
    OH, OW = H - RH + 1, W - RW + 1
    assert cache.shape == (N * OH * OW, RH * RW * C)
    for ow in range(OW):
        for oh in range(OH):
            for n in range(N):
                for c in range(C):
                    for rw in range(RW):
                        for rh in range(RH):
                            v = cache[n + N * (oh + OH * ow), rh + RH * (rw + RW * c)]
                            assert v == n + 10 * (oh + rh) + 100 * (ow + rw) + 1000 * c


def test_conv_delta_and_box_kernels():
    g = hp.rng(3)
    x = hp.normal(g, (2, 6, 7, 2), np.float64)
    RH = RW = 3
    # delta at (rh,rw)=(0,2) on channel 1 -> output is the input shifted by (rh-pv, rw-ph) = (-1,+1)
    w = np.zeros((RH * RW * 2, 1), order="F")
    w[0 + RH * (2 + RW * 1), 0] = 1.0
    out = oracle.conv_forward(x, w, np.zeros((1, 1)))
    exp = np.zeros((2, 6, 7, 1))
    exp[:, 1:, :-1, 0] = x[:, :-1, 1:, 1]
    assert np.array_equal(out, exp)
    # all-ones kernel, no padding -> box sum over the window and channels
    w1 = np.ones((RH * RW * 2, 1), order="F")
    out = oracle.conv_forward(x, w1, np.full((1, 1), 0.5), pv=0, ph=0)
    exp = np.zeros((2, 4, 5, 1))
    for oh in range(4):
        for ow in range(5):
            exp[:, oh, ow, 0] = x[:, oh:oh + 3, ow:ow + 3, :].sum(axis=(1, 2, 3)) + 0.5
    assert hp.rel_err(out, exp) < 1e-13


def test_conv_1x1_equals_dense():
    g = hp.rng(4)
    x = hp.normal(g, (4, 1, 1, 9), np.float64)
    w = hp.normal(g, (9, 6), np.float64)
    b = hp.normal(g, (1, 6), np.float64)
    out = oracle.conv_forward(x, w, b, RH=1, RW=1, pv=0, ph=0)
    dense = oracle.dense_forward(x.reshape((4, 9), order="F"), w, b)
    assert np.allclose(out.reshape((4, 6), order="F"), dense, rtol=0, atol=1e-14)
    assert hp.rel_err(dense, x.reshape((4, 9), order="F") @ w + b) < 1e-13


@pytest.mark.parametrize("case", hp.REFERENCE_CONV_CASES)
def test_conv_adjoint_identities(case):
    """<conv(x;W) - b, g> = <x, dgrad(g;W)> = <W, wgrad(x,g)>, bgrad = sum of g."""
    x, w, b, go = _inputs(case, 4, np.float64, 21)
    out, cache = oracle.conv_forward(x, w, np.zeros_like(b), return_cache=True, **_geom(case))
    dx, dw, db = oracle.conv_backward(x.shape, cache, w, go, **_geom(case))
    lhs = float(np.sum(out * go))
    assert abs(lhs - float(np.sum(x * dx))) < 1e-10 * max(1.0, abs(lhs))
    assert abs(lhs - float(np.sum(w * dw))) < 1e-10 * max(1.0, abs(lhs))
    assert np.allclose(db.reshape(-1), go.sum(axis=(0, 1, 2)), rtol=1e-12, atol=1e-12)


def test_conv_backward_accumulates_and_input_layer_skips():
    case = hp.REFERENCE_CONV_CASES[5]
    x, w, b, go = _inputs(case, 3, np.float64, 5)
    _, cache = oracle.conv_forward(x, w, b, return_cache=True, **_geom(case))
    dx, dw, db = oracle.conv_backward(x.shape, cache, w, go, **_geom(case))
    dx2, dw2, db2 = oracle.conv_backward(x.shape, cache, w, go, input_layer=True, wgrad=dw.copy(order="F"),
                                         bgrad=db.copy(order="F"), **_geom(case))
    assert dx2 is None
    assert np.allclose(dw2, 2 * dw) and np.allclose(db2, 2 * db)


def test_conv_central_difference_on_inputs_and_params():
    """The reference's GradientCheck procedure (core/GradientCheck.hpp:64-117, step 1e-5, double),
    extended to the input gradient."""
    case = hp.REFERENCE_CONV_CASES[3]
    x, w, b, go = _inputs(case, 2, np.float64, 6)
    geom = _geom(case)
    _, cache = oracle.conv_forward(x, w, b, return_cache=True, **geom)
    dx, dw, db = oracle.conv_backward(x.shape, cache, w, go, **geom)
    loss = lambda xx, ww, bb: float(np.sum(oracle.conv_forward(xx, ww, bb, **geom) * go))
    step = 1e-5
    g = hp.rng(7)
    for arr, grad in ((x, dx), (w, dw), (b, db)):
        for _ in range(6):
            idx = tuple(int(g.integers(0, s)) for s in arr.shape)
            keep = arr[idx]
            arr[idx] = keep + step
            lp = loss(x, w, b)
            arr[idx] = keep - step
            lm = loss(x, w, b)
            arr[idx] = keep
            num = (lp - lm) / (2 * step)
            assert abs(num - grad[idx]) <= 1e-6 * max(1.0, abs(num))


@pytest.mark.parametrize("dtype,tol", [(np.float64, 1e-12), (np.float32, 1e-5)])
def test_dense_forward_backward(dtype, tol):
    g = hp.rng(8)
    N, V, O = 7, 4 * 4 * 2, 16                      # test/gradient_test.cpp:156-158 (rank-3 dense)
    x = hp.normal(g, (N, 4, 4, 2), dtype)
    w = hp.normal(g, (V, O), dtype)
    b = hp.normal(g, (1, O), dtype)
    go = hp.normal(g, (N, O), dtype)
    X = np.asarray(x, np.float64).reshape((N, V), order="F")
    out = oracle.dense_forward(x, w, b)
    assert hp.rel_err(out, X @ np.asarray(w, np.float64) + np.asarray(b, np.float64)) < tol
    dx, dw, db = oracle.dense_backward(x, w, go)
    G = np.asarray(go, np.float64)
    assert hp.rel_err(dw, X.T @ G) < tol
    assert hp.rel_err(db, G.sum(axis=0, keepdims=True)) < tol
    assert hp.rel_err(dx.reshape((N, V), order="F"), G @ np.asarray(w, np.float64).T) < tol
    dx2, dw2, _ = oracle.dense_backward(x, w, go, input_layer=True, wgrad=dw.copy(order="F"))
    assert dx2 is None and hp.rel_err(dw2, 2 * (X.T @ G)) < tol
