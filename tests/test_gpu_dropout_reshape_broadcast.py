"""GPU parity of the three data-movement layers that sit between kernel layers in the reference's own example networks
(DropoutLayer, ReshapeLayer, BroadcastLayer), through the C ABI, against the CPU oracle on identical seeded inputs.
The dropout mask is a function of the layer's seed, the number of the training pass and the element index, which the
oracle restates: outputs and gradients are compared bit for bit in the layer's own scalar type."""
import importlib

import numpy as np
import pytest

import helpers as hp
from oracle import oracle

pytestmark = pytest.mark.gpu

ch = importlib.import_module("c-attl3_amd")

DTYPES = [np.float32, np.float64]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("N,dims", [(64, (8, 8, 4)), (3, (5, 7, 3)), (1, (1,)), (7, (33,)), (128, (1000,))])
def test_dropout_passes(N, dims, dtype):
    g = hp.rng(1401)
    p, eps, seed = 0.3, 1e-5, 1234
    layer = ch.DropoutLayer(dtype, dims, p, eps, seed)
    assert layer.get_input_dims() == tuple(dims) and layer.get_output_dims() == tuple(dims) and not layer.get_params()
    x = hp.normal(g, (N,) + tuple(dims), dtype)
    go = hp.normal(g, x.shape, dtype)
    for q in range(3):                                              # every training pass draws a new mask
        u = oracle.dropout_uniforms(seed, q, x.shape, dtype)
        assert np.array_equal(layer.pass_forward(x, True), oracle.dropout_apply(x, u, p, eps))
        assert np.array_equal(layer.pass_back(go), oracle.dropout_apply(go, u, p, eps))
    # an inference pass hands the input through and draws nothing: the next training pass is pass 3
    assert np.array_equal(layer.pass_forward(x, False), x)
    u3 = oracle.dropout_uniforms(seed, 3, x.shape, dtype)
    clone = layer.clone()                                           # a copy carries the state of the generator along
    assert np.array_equal(layer.pass_forward(x, True), oracle.dropout_apply(x, u3, p, eps))
    assert np.array_equal(clone.pass_forward(x, True), oracle.dropout_apply(x, u3, p, eps))
    # device-resident tensors, and an input layer returns no gradient
    xd, gd = ch.DeviceTensor.from_host(x), ch.DeviceTensor.from_host(go)
    u4 = oracle.dropout_uniforms(seed, 4, x.shape, dtype)
    assert np.array_equal(layer.pass_forward(xd, True).to_host(), oracle.dropout_apply(x, u4, p, eps))
    assert np.array_equal(layer.pass_back(gd).to_host(), oracle.dropout_apply(go, u4, p, eps))
    layer.set_input_layer(True)
    layer.pass_forward(x, True)
    assert layer.pass_back(go) is None


def test_dropout_at_the_benchmark_activation_shape():
    """256 x 56 x 56 x 64 float32: every output is 0 or the input times the scaling factor, the dropped share is the
    probability, the gradient uses the same mask, and the expectation of the activations is kept."""
    g = hp.rng(1402)
    shape, p = (256, 56, 56, 64), 0.25
    layer = ch.DropoutLayer(np.float32, shape[1:], p, 1e-5, 77)
    x = hp.uniform(g, shape, 0.5, 1.5, np.float32)
    y = layer.pass_forward(x, True)
    scale = np.float32(1) / (np.float32(1) - np.float32(p) + np.float32(1e-5))
    kept = y != 0
    assert np.array_equal(y[kept], x[kept] * scale)
    share = 1.0 - kept.mean()
    assert abs(share - p) < 4 * np.sqrt(p * (1 - p) / x.size)
    assert abs(y.mean(dtype=np.float64) / x.mean(dtype=np.float64) - 1.0) < 1e-3
    dx = layer.pass_back(np.ones(shape, np.float32, order="F"))
    assert np.array_equal(dx != 0, kept) and np.all(dx[kept] == scale)
    # bit for bit against the oracle on a slab of the tensor (the mask depends on the linear index only)
    u = oracle.dropout_uniforms(77, 0, (x.size,), np.float32).reshape(shape, order="F")
    assert np.array_equal(u <= np.float32(p), ~kept)


def test_dropout_errors():
    for bad in (0.0, 1.5, -0.1):
        with pytest.raises(ch.CattleHipError):
            ch.DropoutLayer(np.float32, (4,), bad)                   # layer/DropoutLayer.hpp:39-40
    with pytest.raises(ch.CattleHipError):
        ch.DropoutLayer(np.float32, (4,), 0.5, epsilon=0.0)          # :41
    layer = ch.DropoutLayer(np.float32, (4,), 1.0)                   # probability 1 is allowed and drops everything
    x = np.ones((2, 4), np.float32, order="F")
    assert np.all(layer.pass_forward(x, True) == 0)
    fresh = ch.DropoutLayer(np.float32, (4,), 0.5)
    fresh.pass_forward(x, False)
    with pytest.raises(ch.CattleHipError):
        fresh.pass_back(x)                                           # no training pass, no mask (:91)


@pytest.mark.parametrize("dtype", DTYPES)
def test_reshape_keeps_the_values(dtype):
    g = hp.rng(1403)
    layer = ch.ReshapeLayer(dtype, (100,), (10, 5, 2))               # as in examples/mnist_autoencoder.cpp:38
    x = hp.normal(g, (6, 100), dtype)
    out = layer.pass_forward(x, True)
    assert out.shape == (6, 10, 5, 2) and np.array_equal(out, x.reshape(out.shape, order="F"))
    go = hp.normal(g, out.shape, dtype)
    assert np.array_equal(layer.pass_back(go), go.reshape(x.shape, order="F"))
    xd = ch.DeviceTensor.from_host(x)
    assert np.array_equal(layer.pass_forward(xd, False).to_host(), out)
    layer.set_input_layer(True)
    layer.pass_forward(x, True)
    assert layer.pass_back(go) is None
    with pytest.raises(ch.CattleHipError):
        ch.ReshapeLayer(dtype, (100,), (10, 5, 3))                    # volumes differ (layer/ReshapeLayer.hpp:38)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("dims,reps", [((3, 4, 2), (2, 1, 3)), ((1, 1, 5), (4, 3, 1)), ((2, 3, 1), (1, 1, 1)), ((5,), (3,)),
                                       ((7, 3), (2, 2)), ((14, 14, 8), (2, 2, 1))])
def test_broadcast(dims, reps, dtype):
    g = hp.rng(1404)
    N = 37
    layer = ch.BroadcastLayer(dtype, dims, reps)
    out_dims = tuple(d * r for d, r in zip(dims, reps))
    assert layer.get_output_dims() == out_dims
    x = hp.normal(g, (N,) + tuple(dims), dtype)
    pad = (1,) * (3 - len(dims))
    x4 = x.reshape((N,) + tuple(dims) + pad, order="F")
    out = layer.pass_forward(x, True)
    ref = oracle.broadcast_forward(x4, *(tuple(reps) + pad))
    assert np.array_equal(out, ref.reshape(out.shape, order="F"))
    go = hp.normal(g, out.shape, dtype, 100.0)
    dx = layer.pass_back(go)
    dx_ref = oracle.broadcast_backward(x4.shape, go.reshape(ref.shape, order="F"), *(tuple(reps) + pad))
    assert np.array_equal(dx, dx_ref.reshape(x.shape, order="F"))    # the reference's summation order, bit for bit
    xd, gd = ch.DeviceTensor.from_host(x), ch.DeviceTensor.from_host(go)
    assert np.array_equal(layer.pass_forward(xd, True).to_host(), out)
    assert np.array_equal(layer.pass_back(gd).to_host(), dx)


def test_broadcast_errors():
    with pytest.raises(ch.CattleHipError):
        ch.BroadcastLayer(np.float32, (3, 4, 2), (2, 0, 1))          # layer/BroadcastLayer.hpp:38-39
    with pytest.raises(ValueError):
        ch.BroadcastLayer(np.float32, (3, 4, 2), (2, 2))
