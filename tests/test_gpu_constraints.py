"""The value and gradient constraints of device-resident parameters (cattle_hip_layer_param_set_constraints) against the
oracle's restatement of parameters/StandardParameters.hpp:105-123, :150-182: after every accumulation of a gradient, with the
regularization term of an optimizer step, after every update of the values and when values are set."""
import importlib

import numpy as np
import pytest

import helpers as hp
from oracle import oracle

pytestmark = pytest.mark.gpu

ch = importlib.import_module("c-attl3_amd")

TOL = {np.dtype(np.float32): 1e-4, np.dtype(np.float64): 1e-10}
GRAD_LIMITS = [dict(clip=0.05), dict(max_l1_norm=0.7), dict(max_l2_norm=0.3), dict(clip=0.2, max_l1_norm=0.9, max_l2_norm=0.5)]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("limits", GRAD_LIMITS, ids=lambda d: "-".join(sorted(d)))
def test_gradient_constraints_after_every_accumulation(limits, dtype):
    N, V, F = 16, 12, 7
    gen = hp.rng(31)
    layer = ch.DenseKernelLayer(dtype, (V,), F)
    wp, bp = layer.get_params()
    w = hp.uniform(gen, (V, F), -1, 1, dtype)
    wp.set_values(w)
    kw = dict(grad_clip=limits.get("clip", 0.0), grad_max_l1_norm=limits.get("max_l1_norm", 0.0),
              grad_max_l2_norm=limits.get("max_l2_norm", 0.0))
    wp.set_constraints(**kw)
    acc = np.zeros((V, F), np.float64, order="F")
    for _ in range(3):                           # the gradient accumulates over passes; each accumulation is constrained
        x = hp.uniform(gen, (N, V), -1, 1, dtype)
        g = hp.uniform(gen, (N, F), -1, 1, dtype)
        layer.pass_forward(x, True)
        layer.pass_back(g)
        _, dw, _ = oracle.dense_backward(np.asarray(x, np.float64), np.asarray(w, np.float64), np.asarray(g, np.float64))
        acc = oracle.constrain(acc + dw, **limits)
        assert hp.rel_err(wp.get_grad(), acc) < TOL[np.dtype(dtype)]
    assert np.abs(bp.get_grad()).max() > 0       # the bias has no constraints: untouched by them


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("many", [False, True])
def test_value_constraints_and_constrained_regularized_step(dtype, many):
    N, V, F = 8, 10, 6
    gen = hp.rng(32)
    layer = ch.DenseKernelLayer(dtype, (V,), F)
    wp, bp = layer.get_params()
    wp.set_constraints(value_clip=0.6, value_max_l1_norm=3.0, value_max_l2_norm=8.0, grad_max_l1_norm=0.5)
    wp.set_regularization(l1_lambda=0.02, l2_lambda=0.3)
    w0 = hp.uniform(gen, (V, F), -1, 1, dtype)
    wp.set_values(w0)
    w = oracle.constrain(np.asarray(w0, np.float64), clip=0.6, max_l1_norm=3.0, max_l2_norm=8.0)      # set_values constrains
    assert hp.rel_err(wp.get_values(), w) < TOL[np.dtype(dtype)]
    lr = 0.5
    for _ in range(2):
        x = hp.uniform(gen, (N, V), -1, 1, dtype)
        g = hp.uniform(gen, (N, F), -1, 1, dtype)
        layer.pass_forward(x, True)
        layer.pass_back(g)
        _, dw, _ = oracle.dense_backward(np.asarray(x, np.float64), w, np.asarray(g, np.float64))
        grad = oracle.constrain(dw, max_l1_norm=0.5)
        # SGDOptimizer::_train: regularize (an accumulate_grad, constrained again), update through set_values, reset
        grad = oracle.constrain(grad + oracle.regularization(w, l1=0.02, l2=0.3)[1], max_l1_norm=0.5)
        w = oracle.constrain(oracle.sgd_update(w, grad, lr=lr), clip=0.6, max_l1_norm=3.0, max_l2_norm=8.0)
        if many:
            ch.ParameterList([wp, bp]).optimizer_step("vanilla_sgd", [lr])
        else:
            wp.optimizer_step("vanilla_sgd", [lr])
            bp.optimizer_step("vanilla_sgd", [lr])
        assert hp.rel_err(wp.get_values(), w) < TOL[np.dtype(dtype)]
        assert not np.any(wp.get_grad())
    # the next forward pass works from the constrained values (its prepared layout was rebuilt)
    x = hp.uniform(gen, (N, V), -1, 1, dtype)
    out = layer.pass_forward(x, True)
    ref = oracle.dense_forward(np.asarray(x, np.float64), w, np.asarray(bp.get_values(), np.float64))
    assert hp.rel_err(out, ref) < TOL[np.dtype(dtype)]


def test_constraints_are_refused_on_the_fused_lstm():
    net = ch.ConvLSTMNetwork(np.float32, (4, 4, 2), 3)
    with pytest.raises(ch.CattleHipError) as e:
        net.get_params()[0].set_constraints(grad_clip=1.0)
    assert e.value.code == 1
