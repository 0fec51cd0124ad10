"""Pins the CPU oracle's batch-norm, activation and pooling routines against closed forms,
invariants, torch float64 and brute force (the reference's own tests hold no known answers for
them: test/gradient_test.cpp:214-373)."""
import numpy as np
import pytest
import torch

import helpers as hp
from oracle import oracle


# ------------------------------------------------------------------------------ batch norm
def _bn_setup(shape, dtype, seed, per_channel=True):
    g = hp.rng(seed)
    x = hp.normal(g, shape, dtype, std=2.0) + dtype(0.7)
    groups = shape[-1] if per_channel else int(np.prod(shape[1:]))
    gamma = (1.0 + 0.3 * g.standard_normal(groups)).astype(dtype)
    beta = (0.2 * g.standard_normal(groups)).astype(dtype)
    go = hp.normal(g, shape, dtype)
    return x, gamma, beta, go, groups


@pytest.mark.parametrize("dtype,tol", [(np.float64, 1e-11), (np.float32, 2e-5)])
def test_bn_per_channel_against_torch_and_invariants(dtype, tol):
    shape = (6, 4, 5, 3)
    x, gamma, beta, go, C = _bn_setup(shape, dtype, 31)
    am, ais = np.zeros(C, dtype), np.zeros(C, dtype)
    y, std, inv_sd = oracle.bn_forward(x, gamma, beta, am, ais, False, True)
    dx, dg, db = oracle.bn_backward(go, gamma, std, inv_sd)
    xt = torch.tensor(np.transpose(np.asarray(x, np.float64), (0, 3, 1, 2)).copy(), requires_grad=True)
    gt = torch.tensor(np.asarray(gamma, np.float64), requires_grad=True)
    bt = torch.tensor(np.asarray(beta, np.float64), requires_grad=True)
    yt = torch.nn.functional.batch_norm(xt, None, None, gt, bt, training=True, eps=1e-5)
    yt.backward(torch.tensor(np.transpose(np.asarray(go, np.float64), (0, 3, 1, 2)).copy()))
    assert hp.rel_err(y, np.transpose(yt.detach().numpy(), (0, 2, 3, 1))) < tol
    assert hp.rel_err(dx, np.transpose(xt.grad.numpy(), (0, 2, 3, 1))) < 20 * tol
    assert hp.rel_err(dg, gt.grad.numpy()) < tol
    assert hp.rel_err(db, bt.grad.numpy()) < tol
    # the statistics the reference keeps: mean and INVERSE standard deviation (biased variance)
    x64 = np.asarray(x, np.float64)
    mean = x64.mean(axis=(0, 1, 2))
    var = x64.var(axis=(0, 1, 2))
    assert hp.rel_err(am, mean) < tol and hp.rel_err(ais, 1 / np.sqrt(var + 1e-5)) < tol
    # invariants of the input gradient per channel
    L = x.size // C
    dx64, std64 = np.asarray(dx, np.float64), np.asarray(std, np.float64)
    scale = np.abs(dx64).sum(axis=(0, 1, 2))
    assert np.all(np.abs(dx64.sum(axis=(0, 1, 2))) <= 50 * tol * scale)
    # sum(dx * x_hat) = inv_sd * sum(x_hat * g * gamma) * (1 - sum(x_hat^2) / L): zero only for eps == 0
    sg = np.asarray(go, np.float64) * np.asarray(gamma, np.float64)
    expect = np.asarray(inv_sd, np.float64) * (std64 * sg).sum(axis=(0, 1, 2)) * \
        (1 - (std64 * std64).sum(axis=(0, 1, 2)) / L)
    assert np.all(np.abs((dx64 * std64).sum(axis=(0, 1, 2)) - expect) <= 50 * tol * scale)
    assert L == 120


def test_bn_running_statistics_and_inference():
    """First training call assigns the running stats, later calls blend with decay
    (layer/BatchNormLayer.hpp:234-243); inference uses them (:246)."""
    dtype = np.float64
    shape = (5, 3, 3, 2)
    x1, gamma, beta, _, C = _bn_setup(shape, dtype, 32)
    x2 = x1 * 1.5 - 0.3
    am, ais = np.full(C, 9.0), np.full(C, 9.0)
    oracle.bn_forward(x1, gamma, beta, am, ais, False, True, decay=0.2)
    m1, s1 = x1.mean(axis=(0, 1, 2)), 1 / np.sqrt(x1.var(axis=(0, 1, 2)) + 1e-5)
    assert np.allclose(am, m1) and np.allclose(ais, s1)
    oracle.bn_forward(x2, gamma, beta, am, ais, True, True, decay=0.2)
    m2, s2 = x2.mean(axis=(0, 1, 2)), 1 / np.sqrt(x2.var(axis=(0, 1, 2)) + 1e-5)
    assert np.allclose(am, 0.8 * m1 + 0.2 * m2) and np.allclose(ais, 0.8 * s1 + 0.2 * s2)
    y, _, _ = oracle.bn_forward(x1, gamma, beta, am, ais, True, False)
    assert np.allclose(y, (x1 - am) * ais * gamma + beta)


def test_bn_per_activation_is_columnwise():
    dtype = np.float64
    shape = (9, 2, 3, 2)
    x, gamma, beta, go, V = _bn_setup(shape, dtype, 33, per_channel=False)
    am, ais = np.zeros(V), np.zeros(V)
    y, std, inv_sd = oracle.bn_forward(x, gamma, beta, am, ais, False, True, per_channel=False)
    X = x.reshape((9, V), order="F")
    mean, var = X.mean(axis=0), X.var(axis=0)
    exp = (X - mean) / np.sqrt(var + 1e-5) * gamma + beta
    assert np.allclose(y.reshape((9, V), order="F"), exp)
    dx, dg, db = oracle.bn_backward(go, gamma, std, inv_sd, per_channel=False)
    xt = torch.tensor(X.copy(), requires_grad=True)
    yt = torch.nn.functional.batch_norm(xt, None, None, torch.tensor(gamma), torch.tensor(beta), training=True,
                                        eps=1e-5)
    yt.backward(torch.tensor(go.reshape((9, V), order="F").copy()))
    assert hp.rel_err(dx.reshape((9, V), order="F"), xt.grad.numpy()) < 1e-9
    assert np.allclose(db, go.reshape((9, V), order="F").sum(axis=0))


# ------------------------------------------------------------------------------ activations
def _np_act(kind, x, p):
    sig = lambda z: 1.0 / (1.0 + np.exp(-z))
    return {
        "identity": lambda: (x, np.ones_like(x)),
        "scaled": lambda: (x * p, np.full_like(x, p)),
        "binary_step": lambda: ((x >= 0).astype(x.dtype), np.zeros_like(x)),
        "sigmoid": lambda: (sig(x), sig(x) * (1 - sig(x))),
        "tanh": lambda: (np.tanh(x), 1 - np.tanh(x) ** 2),
        "softsign": lambda: (x / (1 + np.abs(x)), 1 / (1 + np.abs(x)) ** 2),
        "softplus": lambda: (np.log1p(np.exp(x)), sig(x)),
        "relu": lambda: (np.maximum(x, 0), (x >= 0).astype(x.dtype)),
        "leaky_relu": lambda: (np.maximum(x, p * x), np.where(x >= 0, 1.0, p)),
        "elu": lambda: (np.where(x >= 0, x, p * np.expm1(x)), np.where(x >= 0, 1.0, p * np.exp(x))),
        "swish": lambda: (x * sig(p * x), sig(p * x) + p * x * sig(p * x) * (1 - sig(p * x))),
    }[kind]()


@pytest.mark.parametrize("kind,p", [("identity", 0), ("scaled", 1.7), ("binary_step", 0), ("sigmoid", 0),
                                    ("tanh", 0), ("softsign", 0), ("softplus", 0), ("relu", 0),
                                    ("leaky_relu", 0.1), ("elu", 1.0), ("swish", 1.3)])
@pytest.mark.parametrize("dtype,tol", [(np.float64, 1e-12), (np.float32, 2e-6)])
def test_activation_closed_forms(kind, p, dtype, tol):
    g = hp.rng(41)
    x = hp.normal(g, (5, 3, 4, 2), dtype, std=2.0)
    x[0, 0, 0, 0] = 0.0                                 # derivative-at-zero conventions
    go = hp.normal(g, x.shape, dtype)
    y = oracle.act_forward(kind, x, p)
    dx = oracle.act_backward(kind, x, y, go, p)
    ye, de = _np_act(kind, np.asarray(x, np.float64), float(p))
    assert hp.rel_err(y, ye) < tol
    assert hp.rel_err(dx, de * np.asarray(go, np.float64)) < 10 * tol
    if kind in ("relu", "leaky_relu", "elu"):
        assert dx[0, 0, 0, 0] == go[0, 0, 0, 0]         # gradient 1 at x == 0 (ReLUActivationLayer.hpp:56)


def test_softmax_rows_and_jacobian():
    g = hp.rng(42)
    x = hp.normal(g, (6, 10), np.float64, std=3.0)
    go = hp.normal(g, (6, 10), np.float64)
    y = oracle.softmax_forward(x)
    e = np.exp(x - x.max(axis=1, keepdims=True))
    exp = e / (e.sum(axis=1, keepdims=True) + 1e-5)     # epsilon in the denominator (:57-58)
    assert np.allclose(y, exp, rtol=1e-13, atol=0)
    dx = oracle.softmax_backward(y, go)
    assert np.allclose(dx, y * go - y * (y * go).sum(axis=1, keepdims=True), rtol=1e-12, atol=1e-15)


def test_prelu_and_pswish():
    g = hp.rng(43)
    N, V = 7, 12
    x = hp.normal(g, (N, 3, 4), np.float64)
    go = hp.normal(g, (N, 3, 4), np.float64)
    alpha = g.uniform(0.05, 1.5, V)
    X, G = x.reshape((N, V), order="F"), go.reshape((N, V), order="F")
    y = oracle.prelu_forward(x, alpha)
    assert np.array_equal(y.reshape((N, V), order="F"), np.maximum(X, X * alpha))
    dx, da = oracle.prelu_backward(x, alpha, go)
    assert np.allclose(dx.reshape((N, V), order="F"), np.where(X >= 0, G, alpha * G))
    assert np.allclose(da, np.where(X >= 0, 0.0, X * G).sum(axis=0))
    beta = g.uniform(0.5, 1.5, V)
    sig = 1 / (1 + np.exp(-X * beta))
    y = oracle.pswish_forward(x, beta)
    assert np.allclose(y.reshape((N, V), order="F"), X * sig)
    dx, dbeta = oracle.pswish_backward(x, beta, go)
    assert np.allclose(dx.reshape((N, V), order="F"), sig * ((1 - sig) * beta * X + 1) * G)
    assert np.allclose(dbeta, (sig * (1 - sig) * X * X * G).sum(axis=0))
    # finite-difference check of the parameter gradient
    step = 1e-6
    b2 = beta.copy(); b2[3] += step
    b3 = beta.copy(); b3[3] -= step
    num = (np.sum(oracle.pswish_forward(x, b2) * go) - np.sum(oracle.pswish_forward(x, b3) * go)) / (2 * step)
    assert abs(num - dbeta[3]) < 1e-6 * max(1, abs(num))


# ------------------------------------------------------------------------------ pooling
POOL_CASES = [(8, 8, 3, 2, 2, 2, 2), (16, 16, 2, 3, 2, 1, 2), (7, 9, 2, 3, 2, 2, 3), (32, 1, 2, 3, 1, 1, 1)]


@pytest.mark.parametrize("H,W,C,RH,RW,sv,sh", POOL_CASES)
def test_maxpool_matches_brute_force(H, W, C, RH, RW, sv, sh):
    g = hp.rng(51)
    x = hp.normal(g, (3, H, W, C), np.float32)
    out, inds = oracle.maxpool_forward(x, RH, RW, sv, sh)
    eo, ei = hp.brute_maxpool(x, RH, RW, sv, sh)
    assert np.array_equal(out, eo) and np.array_equal(inds, ei)
    # torch agrees on values; the indices are the reference's own encoding, pinned by brute force
    if (sv, sh) != (0, 0):
        t = torch.nn.functional.max_pool2d(torch.tensor(np.transpose(x, (0, 3, 1, 2)).copy()), (RH, RW), (sv, sh))
        assert np.array_equal(out, np.transpose(t.numpy(), (0, 2, 3, 1)))


def test_maxpool_ties_nan_and_neg_inf():
    """Strict '>' from lowest(): first maximum in (w-major, h-minor) scan order wins; NaN is never
    selected; an all-NaN or all -inf window gives lowest() and index 0
    (layer/pool/MaxPoolLayer.hpp:45-62)."""
    x = np.zeros((1, 4, 4, 1), dtype=np.float32, order="F")
    out, inds = oracle.maxpool_forward(x)
    assert np.all(inds == 0) and np.all(out == 0)
    x[0, 1, 0, 0] = 5      # (h=1,w=0) and (h=0,w=1) tie inside window (0,0): w=0 scanned first
    x[0, 0, 1, 0] = 5
    out, inds = oracle.maxpool_forward(x)
    assert inds[0, 0] == 0 * 2 + 1 and out[0, 0, 0, 0] == 5
    x[0, 0:2, 2:4, 0] = np.nan                      # window (oh=0, ow=1) is all NaN
    x[0, 2:4, 0:2, 0] = -np.inf                     # window (oh=1, ow=0) is all -inf
    x[0, 2, 2, 0] = np.nan                          # NaN next to a finite maximum
    x[0, 3, 3, 0] = 1
    out, inds = oracle.maxpool_forward(x)
    lowest = np.finfo(np.float32).min
    assert out[0, 0, 1, 0] == lowest and inds[1 * 2 + 0, 0] == 0
    assert out[0, 1, 0, 0] == lowest and inds[0 * 2 + 1, 0] == 0
    assert out[0, 1, 1, 0] == 1 and inds[1 * 2 + 1, 0] == 1 * 2 + 1


@pytest.mark.parametrize("H,W,C,RH,RW,sv,sh", POOL_CASES)
def test_pool_backward_accumulates_overlaps(H, W, C, RH, RW, sv, sh):
    g = hp.rng(52)
    x = hp.normal(g, (2, H, W, C), np.float64)
    out, inds = oracle.maxpool_forward(x, RH, RW, sv, sh)
    go = hp.normal(g, out.shape, np.float64)
    dx = oracle.maxpool_backward(x.shape, go, inds, RH, RW, sv, sh)
    xt = torch.tensor(np.transpose(x, (0, 3, 1, 2)).copy(), requires_grad=True)
    torch.nn.functional.max_pool2d(xt, (RH, RW), (sv, sh)).backward(
        torch.tensor(np.transpose(go, (0, 3, 1, 2)).copy()))
    assert np.allclose(dx, np.transpose(xt.grad.numpy(), (0, 2, 3, 1)), rtol=1e-13, atol=1e-13)
    mo = oracle.meanpool_forward(x, RH, RW, sv, sh)
    xt = torch.tensor(np.transpose(x, (0, 3, 1, 2)).copy(), requires_grad=True)
    mt = torch.nn.functional.avg_pool2d(xt, (RH, RW), (sv, sh))
    mt.backward(torch.tensor(np.transpose(go, (0, 3, 1, 2)).copy()))
    assert np.allclose(mo, np.transpose(mt.detach().numpy(), (0, 2, 3, 1)), rtol=1e-13, atol=1e-13)
    mdx = oracle.meanpool_backward(x.shape, go, RH, RW, sv, sh)
    assert np.allclose(mdx, np.transpose(xt.grad.numpy(), (0, 2, 3, 1)), rtol=1e-13, atol=1e-13)
