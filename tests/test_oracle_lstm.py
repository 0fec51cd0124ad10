"""Pins the CPU restatement of LSTMNeuralNetwork (tests/harness.py, SeqConvLSTM over the oracle's layers), which the fused
device network is checked against: torch's LSTM as an independent implementation of the same cell where the two
coincide (vectors, sigmoid gates, tanh candidate and state, an output at every step, no bias on the hidden side), and
central differences of a
scalar function of the output, as the reference's own network tests do (test/gradient_test.cpp:656-744), for the
variants torch does not have: multiplicative integration, delayed and shortened outputs, convolutional kernels."""
import numpy as np
import pytest
import torch

import harness as hn
import helpers as hp

ONE = dict(RH=1, RW=1, pv=0, ph=0)


def _fill(net, gen, scale=0.5):
    for layer in net.kernels():
        for p in layer.get_params():
            p.set_values(hp.normal(gen, p.get_values().shape, np.float64, scale))


def test_dense_lstm_against_torch():
    g = hp.rng(61)
    N, T, V, H = 4, 5, 6, 3
    net = hn.SeqConvLSTM(hn.OracleBackend(np.float64), (1, 1, V), H, conv_kw=ONE, foremost=False)
    _fill(net, g)
    ref = torch.nn.LSTM(V, H, batch_first=True).double()
    k = net.kernels()                                       # in/out pairs of forget, write, candidate, read
    # torch's cell adds its hidden-side bias at the first step too (to W_hh times a zero state); the reference's first
    # step has no output kernel at all (:283-298). With zero biases on the output kernels the two are the same function.
    for j in range(4):
        b = k[2 * j + 1].get_params()[1]
        b.set_values(np.zeros_like(b.get_values()))
    order = (1, 0, 2, 3)                                     # torch stacks its gates as input (write), forget, cell (candidate), output (read)
    with torch.no_grad():
        ref.weight_ih_l0.copy_(torch.tensor(np.concatenate([k[2 * j].get_params()[0].get_values().T for j in order])))
        ref.weight_hh_l0.copy_(torch.tensor(np.concatenate([k[2 * j + 1].get_params()[0].get_values().T for j in order])))
        ref.bias_ih_l0.copy_(torch.tensor(np.concatenate([k[2 * j].get_params()[1].get_values()[0] for j in order])))
        ref.bias_hh_l0.copy_(torch.tensor(np.concatenate([k[2 * j + 1].get_params()[1].get_values()[0] for j in order])))
    x = hp.normal(g, (N, T, 1, 1, V), np.float64)
    go = hp.normal(g, (N, T, 1, 1, H), np.float64)
    xt = torch.tensor(x.reshape(N, T, V), requires_grad=True)
    out_t, _ = ref(xt)
    (out_t * torch.tensor(go.reshape(N, T, H))).sum().backward()
    out = net.propagate(x, T, 0)
    assert hp.rel_err(out.reshape(N, T, H), out_t.detach().numpy()) < 1e-12
    dx = net.backpropagate(go)
    assert hp.rel_err(dx.reshape(N, T, V), xt.grad.numpy()) < 1e-11
    for j, gate in enumerate(order):
        sl = slice(j * H, (j + 1) * H)
        assert hp.rel_err(k[2 * gate].get_params()[0].get_grad().T, ref.weight_ih_l0.grad.numpy()[sl]) < 1e-11
        assert hp.rel_err(k[2 * gate + 1].get_params()[0].get_grad().T, ref.weight_hh_l0.grad.numpy()[sl]) < 1e-11
        assert hp.rel_err(k[2 * gate].get_params()[1].get_grad()[0], ref.bias_ih_l0.grad.numpy()[sl]) < 1e-11


@pytest.mark.parametrize("mul_int", [False, True])
@pytest.mark.parametrize("dims,hidden,conv_kw,T_in,seq", [
    ((1, 1, 5), 3, ONE, 3, (3, 0)),                 # the reference's rank-1 test: an output at every step
    ((1, 1, 5), 3, ONE, 5, (1, 4)),                 # its multiplicative-integration test: the last step only
    ((1, 1, 4), 2, ONE, 2, (3, 1)),                 # runs two steps past the input
    ((4, 3, 2), 2, None, 3, (2, 1)),                # 3 x 3 convolutional kernels, output in the middle
])
def test_lstm_gradients_are_the_derivatives(dims, hidden, conv_kw, T_in, seq, mul_int):
    g = hp.rng(62)
    N = 2
    out_len, delay = seq
    net = hn.SeqConvLSTM(hn.OracleBackend(np.float64), dims, hidden, conv_kw=conv_kw, foremost=False, mul_int=mul_int)
    _fill(net, g)
    x = hp.normal(g, (N, T_in) + dims, np.float64)
    go = hp.normal(g, (N, out_len, dims[0], dims[1], hidden), np.float64)

    def value():
        return float(np.sum(net.propagate(x, out_len, delay) * go))

    net.propagate(x, out_len, delay)
    dx = net.backpropagate(go)
    h = 1e-6
    for idx in [tuple(g.integers(0, s) for s in x.shape) for _ in range(6)]:
        keep = x[idx]
        x[idx] = keep + h
        up = value()
        x[idx] = keep - h
        dn = value()
        x[idx] = keep
        assert abs((up - dn) / (2 * h) - dx[idx]) < 1e-6 * max(1.0, abs(dx[idx])), ("input", idx)
    for ki, layer in enumerate(net.kernels()):
        for pi, p in enumerate(layer.get_params()):
            grad = p.get_grad().copy()
            v = p.get_values().copy()
            idx = tuple(g.integers(0, s) for s in v.shape)
            for sign, store in ((1, "up"), (-1, "dn")):
                w = v.copy()
                w[idx] += sign * h
                p.set_values(w)
                if store == "up":
                    up = value()
                else:
                    dn = value()
            p.set_values(v)
            assert abs((up - dn) / (2 * h) - grad[idx]) < 1e-6 * max(1.0, abs(grad[idx])), (ki, pi, idx)


def test_multiplicative_integration_differs_and_reduces_to_the_sum_rule_at_the_ends():
    """With one input step and one extra step no time step has both an input and a previous output, so the two
    variants coincide (neural_network/LSTMNeuralNetwork.hpp:283-298, :347-361); with two input steps they differ."""
    g = hp.rng(63)
    nets = [hn.SeqConvLSTM(hn.OracleBackend(np.float64), (1, 1, 4), 3, conv_kw=ONE, mul_int=m) for m in (False, True)]
    _fill(nets[0], g)
    for a, b in zip(nets[0].kernels(), nets[1].kernels()):
        for pa, pb in zip(a.get_params(), b.get_params()):
            pb.set_values(pa.get_values())
    x = hp.normal(g, (3, 2, 1, 1, 4), np.float64)
    assert np.array_equal(nets[0].propagate(x[:, :1], 2, 0), nets[1].propagate(x[:, :1], 2, 0))
    assert not np.allclose(nets[0].propagate(x, 2, 0), nets[1].propagate(x, 2, 0))
