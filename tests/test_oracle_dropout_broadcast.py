"""Pins the oracle's restatements of the two data-movement layers around the kernel layers, DropoutLayer and
BroadcastLayer (ReshapeLayer changes no value: layer/ReshapeLayer.hpp:77-90), without the reference being
compilable. The reference draws dropout's uniform numbers from Eigen's generator, which is not restated: which
elements are dropped is unpinned by construction; the generator used instead is pinned against its published
outputs, and the mask rule, which is the reference's, on hand-worked values."""
import numpy as np
import pytest
import torch

import helpers as hp
from oracle import oracle

DTYPES = [np.float32, np.float64]


def test_splitmix64_published_outputs():
    """The first outputs of splitmix64 seeded with 1234567, as published with the generator's reference code."""
    want = [6457827717110365317, 3203168211198807973, 9817491932198370423, 4593380528125082431, 16408922859458223821]
    assert [oracle.splitmix64_output(1234567, i) for i in range(5)] == want


@pytest.mark.parametrize("dtype", DTYPES)
def test_dropout_uniforms_are_the_top_bits_of_the_stream(dtype):
    seed, q = 99, 3
    key = oracle.splitmix64_output(seed, q)
    u = oracle.dropout_uniforms(seed, q, (5, 4), dtype)
    flat = u.reshape(-1, order="F")
    for i in range(flat.size):
        if dtype == np.float32:          # one output serves two elements: bits 63..40 the even one, 31..8 the odd one
            bits = oracle.splitmix64_output(key, i // 2)
            want = (((bits >> 8) & 0xFFFFFF) if i % 2 else bits >> 40) / 2.0 ** 24
        else:
            want = (oracle.splitmix64_output(key, i) >> 11) / 2.0 ** 53
        assert flat[i] == dtype(want)
    assert not np.array_equal(u, oracle.dropout_uniforms(seed, q + 1, (5, 4), dtype))        # another pass, another mask
    assert not np.array_equal(u, oracle.dropout_uniforms(seed + 1, q, (5, 4), dtype))


@pytest.mark.parametrize("dtype", DTYPES)
def test_dropout_uniforms_are_uniform(dtype):
    n = 1 << 18
    u = np.asarray(oracle.dropout_uniforms(7, 0, (n,), dtype), np.float64)
    assert u.min() >= 0 and u.max() < 1
    assert abs(u.mean() - 0.5) < 4 * np.sqrt(1 / 12.0 / n)
    assert abs(u.var() - 1 / 12.0) < 4 * np.sqrt(1 / 180.0 / n)
    counts = np.bincount((u * 16).astype(int), minlength=16)
    chi2 = ((counts - n / 16.0) ** 2 / (n / 16.0)).sum()
    assert chi2 < 45                                   # 15 degrees of freedom: 45 is beyond the 99.99th percentile
    assert abs(np.corrcoef(u[:-1], u[1:])[0, 1]) < 4 / np.sqrt(n)


def test_dropout_mask_rule_by_hand():
    """mask = 0 where u <= p (the boundary is dropped), else 1 / (1 - p + eps): layer/DropoutLayer.hpp:78-81."""
    u = np.asfortranarray(np.array([[0.1, 0.25, 0.2500001, 0.9]], np.float64))
    x = np.asfortranarray(np.array([[2.0, 3.0, 4.0, -5.0]], np.float64))
    assert np.array_equal(oracle.dropout_apply(x, u, 0.25, eps=0.25), [[0.0, 0.0, 4.0, -5.0]])          # scale 1 / (1 - .25 + .25)
    assert np.allclose(oracle.dropout_apply(x, u, 0.25, eps=0.0), [[0.0, 0.0, 4.0 / 0.75, -5.0 / 0.75]], rtol=1e-15)
    assert np.array_equal(oracle.dropout_apply(x, u, 1.0, eps=1e-5), np.zeros((1, 4)))                   # p = 1 drops everything


@pytest.mark.parametrize("dtype", DTYPES)
def test_dropout_keeps_the_expectation(dtype):
    g = hp.rng(31)
    x = hp.uniform(g, (64, 4096), 0.5, 1.5, dtype)
    p = 0.3
    y = oracle.dropout_apply(x, oracle.dropout_uniforms(5, 0, x.shape, dtype), p, eps=1e-5)
    dropped = np.mean(y == 0)
    assert abs(dropped - p) < 4 * np.sqrt(p * (1 - p) / x.size)
    assert abs(y.mean(dtype=np.float64) / x.mean(dtype=np.float64) - (1 - dropped) / (1 - p + 1e-5)) < 2e-3


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("dims,reps", [((3, 4, 2), (2, 1, 3)), ((1, 1, 5), (4, 3, 1)), ((2, 3, 1), (1, 1, 1)), ((5, 1, 1), (1, 2, 2))])
def test_broadcast_against_numpy_and_autograd(dims, reps, dtype):
    g = hp.rng(32)
    N = 3
    x = hp.normal(g, (N,) + dims, dtype)
    out = oracle.broadcast_forward(x, *reps)
    assert np.array_equal(out, np.tile(x, (1,) + reps))
    go = hp.normal(g, out.shape, dtype)
    xt = torch.tensor(np.asarray(x, np.float64), requires_grad=True)
    (xt.repeat(1, *reps) * torch.tensor(np.asarray(go, np.float64))).sum().backward()
    dx = oracle.broadcast_backward(x.shape, go, *reps)
    assert hp.rel_err(dx, xt.grad.numpy()) < (1e-5 if dtype == np.float32 else 1e-13)
    # the adjoint identity <B x, g> = <x, B^T g>
    lhs = float(np.sum(np.asarray(out, np.float64) * np.asarray(go, np.float64)))
    rhs = float(np.sum(np.asarray(x, np.float64) * np.asarray(dx, np.float64)))
    assert abs(lhs - rhs) < (1e-4 if dtype == np.float32 else 1e-11) * max(1.0, abs(lhs))


def test_broadcast_backward_sums_rank_by_rank_in_float32():
    """layer/BroadcastLayer.hpp:84-98: the replicas of the first rank are summed first (from zero, in order), then
    those of the second, then the third; in float32 that order is visible."""
    g = hp.rng(33)
    go = hp.normal(g, (1, 3, 2, 2), np.float32, 1e3) + np.float32(1e-3)
    dx = oracle.broadcast_backward((1, 1, 1, 1), go, 3, 2, 2)
    f = np.float32
    by_rank = f(0)
    for c in range(2):
        acc_w = f(0)
        for w in range(2):
            acc_h = f(0)
            for h in range(3):
                acc_h = f(acc_h + go[0, h, w, c])
            acc_w = f(acc_w + acc_h)
        by_rank = f(by_rank + acc_w)
    assert dx[0, 0, 0, 0] == by_rank
