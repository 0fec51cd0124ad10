"""The sums of weight-gradient slices are taken when a gradient is first needed, not in the backward pass: whatever the
caller does in between (reading a gradient, a second backward pass, layers that share parameters, an optimizer step that
takes a few slices along or one that finds them summed already), gradients and updated weights must be those of the
reference's order of events - accumulate_grad in pass_back, update in the optimizer (StandardParameters.hpp:114-123,
SGDOptimizer.hpp:58-70). Data are multiples of 1/8, so every sum is exact and the comparisons are bit for bit against
the oracle's float64 layers."""
import importlib

import numpy as np
import pytest

import helpers as hp
from oracle import oracle

pytestmark = pytest.mark.gpu

ch = importlib.import_module("c-attl3_amd")


def _dyadic(gen, shape, dtype, steps=8):
    return np.asfortranarray(gen.integers(-steps, steps + 1, size=shape).astype(dtype) / steps)


def _conv_case(dtype, N, H, W, C, F, seed):
    gen = hp.rng(seed)
    x = _dyadic(gen, (N, H, W, C), dtype)
    w = _dyadic(gen, (9 * C, F), dtype)
    b = _dyadic(gen, (1, F), dtype)
    g = _dyadic(gen, (N, H, W, F), dtype)
    x64, w64, b64, g64 = (np.asarray(a, np.float64) for a in (x, w, b, g))
    _, cache = oracle.conv_forward(x64, w64, b64, return_cache=True)
    dx, dw, db = oracle.conv_backward(x.shape, cache, w64, g64)
    return x, w, b, g, dw, db.reshape(1, -1)


# batch sizes and shapes that give one slice (the launch adds to the gradient itself), a few slices (they ride with the
# optimizer launch) and many slices (summed by the launch of their own)
CASES = [(8, 4, 4, 3, 5), (64, 8, 8, 4, 8), (128, 16, 16, 8, 16)]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("case", CASES)
def test_gradients_accumulate_over_passes_and_reads(case, dtype):
    N, H, W, C, F = case
    x, w, b, g, dw, db = _conv_case(dtype, N, H, W, C, F, seed=N)
    layer = ch.ConvKernelLayer(dtype, (H, W, C), F)
    wp, bp = layer.get_params()
    wp.set_values(w)
    bp.set_values(b)
    xd, gd = ch.DeviceTensor.from_host(x), ch.DeviceTensor.from_host(g)
    layer.pass_forward(xd, True)
    layer.pass_back(gd)
    assert np.array_equal(wp.get_grad(), dw) and np.array_equal(bp.get_grad(), db)
    assert np.array_equal(wp.get_grad(), dw), "reading a gradient twice"
    layer.pass_back(gd)                       # pending sums of the first pass must not be lost to the second
    layer.pass_back(gd)
    assert np.array_equal(bp.get_grad(), 3 * db) and np.array_equal(wp.get_grad(), 3 * dw)
    wp.reset_grad()
    layer.pass_back(gd)
    wp.reset_grad()                           # a reset right behind a pass: the pending sums go with it
    assert not wp.get_grad().any()
    assert np.array_equal(bp.get_grad(), 4 * db)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("read_first", [False, True])
def test_optimizer_step_finds_whole_gradients(case, dtype, read_first):
    """The same update whether the optimizer launch takes the slices along, a launch before it sums them, or a read of
    the gradient has summed them already."""
    N, H, W, C, F = case
    x, w, b, g, dw, db = _conv_case(dtype, N, H, W, C, F, seed=3 * N)
    layer = ch.ConvKernelLayer(dtype, (H, W, C), F)
    wp, bp = layer.get_params()
    wp.set_values(w)
    bp.set_values(b)
    xd, gd = ch.DeviceTensor.from_host(x), ch.DeviceTensor.from_host(g)
    layer.pass_forward(xd, True)
    layer.pass_back(gd)
    if read_first:
        assert np.array_equal(bp.get_grad(), db)
    ch.ParameterList([wp, bp]).optimizer_step("vanilla_sgd", [0.125])
    assert np.array_equal(wp.get_values(), (np.asarray(w, np.float64) - 0.125 * dw).astype(dtype))
    assert np.array_equal(bp.get_values(), (np.asarray(b, np.float64) - 0.125 * db).astype(dtype))
    assert not wp.get_grad().any() and not bp.get_grad().any()
    # and the next pass starts from zero
    layer.pass_forward(xd, True)
    layer.pass_back(gd)
    layer.pass_back(gd)
    ch.synchronize()
    w2 = np.asarray(wp.get_values(), np.float64)
    _, cache = oracle.conv_forward(np.asarray(x, np.float64), w2, np.asarray(bp.get_values(), np.float64), return_cache=True)
    _, dw2, db2 = oracle.conv_backward(x.shape, cache, w2, np.asarray(g, np.float64))
    assert np.array_equal(wp.get_grad(), 2 * dw2) and np.array_equal(bp.get_grad(), 2 * db2.reshape(1, -1))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_layers_that_share_parameters(dtype):
    """clone_with_shared_params (core/Layer.hpp:62-68): both layers accumulate into the same gradient."""
    N, H, W, C, F = 64, 8, 8, 4, 8
    x, w, b, g, dw, db = _conv_case(dtype, N, H, W, C, F, seed=17)
    a = ch.ConvKernelLayer(dtype, (H, W, C), F)
    twin = a.clone_with_shared_params()
    wp, bp = a.get_params()
    wp.set_values(w)
    bp.set_values(b)
    xd, gd = ch.DeviceTensor.from_host(x), ch.DeviceTensor.from_host(g)
    a.pass_forward(xd, True)
    twin.pass_forward(xd, True)
    a.pass_back(gd)
    twin.pass_back(gd)
    ch.ParameterList([wp, bp]).optimizer_step("vanilla_sgd", [0.0625])
    tw, tb = twin.get_params()
    assert np.array_equal(tw.get_values(), (np.asarray(w, np.float64) - 0.125 * dw).astype(dtype))
    assert np.array_equal(tb.get_values(), (np.asarray(b, np.float64) - 0.125 * db).astype(dtype))
    deep = a.clone()                          # a deep copy takes the gradients as they stand
    a.pass_back(gd)
    got = deep.get_params()[0].get_grad()
    assert not got.any()
    del twin, a
    ch.synchronize()
