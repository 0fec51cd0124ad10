"""Recorded steps (cattle_hip_graph_*): a training step recorded once and launched as a HIP graph must do, at every launch,
exactly what the same calls do when they are issued one by one. The eager calls are what the other GPU tests hold against
the oracle; here the replays are held against the eager calls, bit for bit (same kernels, same arguments, same order), with
the program's own eager work and waits between the launches, and every launch is checked, not only the first."""
import ctypes
import importlib

import numpy as np
import pytest

import helpers as hp

pytestmark = pytest.mark.gpu

ch = importlib.import_module("c-attl3_amd")


def _mlp(dtype, fused):
    layers = [ch.DenseKernelLayer(dtype, (20,), 48), ch.ActivationLayer(dtype, "relu", (48,)),
              ch.DenseKernelLayer(dtype, (48,), 32), ch.ActivationLayer(dtype, "tanh", (32,)),
              ch.DenseKernelLayer(dtype, (32,), 6)]
    layers[0].set_input_layer(True)
    params = [p for l in layers for p in l.get_params()]
    return (ch.fuse_layers(layers) if fused else layers), params, layers


def _convnet(dtype):
    layers = [ch.ConvKernelLayer(dtype, (8, 8, 3), 8), ch.ActivationLayer(dtype, "relu", (8, 8, 8)), ch.MaxPoolLayer(dtype, (8, 8, 8)),
              ch.ConvKernelLayer(dtype, (4, 4, 8), 8), ch.BatchNormLayer(dtype, (4, 4, 8)), ch.ActivationLayer(dtype, "relu", (4, 4, 8)),
              ch.DenseKernelLayer(dtype, (4, 4, 8), 6)]
    layers[0].set_input_layer(True)
    params = [p for l in layers for p in l.get_params()]
    return ch.fuse_layers(layers), params, layers


def _init(params, seed, dtype):
    gen = hp.rng(seed)
    for p in params:
        if p.are_optimizable() and p.get_rows() > 1:
            p.set_values(hp.uniform(gen, (p.get_rows(), p.get_cols()), -0.5, 0.5, dtype))


def _step(net, plist, x, y, N, sgd=True):
    a = x
    for l in net:
        a = l.pass_forward(a, True)
    g = ch.loss_d_function("softmax_cross_entropy", a, y, scale=1.0 / N)
    for l in reversed(net):
        g = l.pass_back(g)
    if sgd:
        plist.optimizer_step("vanilla_sgd", [0.05])
    return a


def _values(params):
    return [p.get_values() for p in params]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("fused", [False, True])
def test_recorded_sgd_step_equals_eager_steps(dtype, fused):
    N, steps = 16, 5
    gen = hp.rng(77)
    x_host = hp.uniform(gen, (N, 20), -1, 1, dtype)
    y_host = np.zeros((N, 6), dtype, order="F")
    y_host[np.arange(N), gen.integers(0, 6, N)] = 1
    other = ch.ActivationLayer(dtype, "sigmoid", (20,))

    # the reference run: `steps` eager steps, outputs and weights after each
    net, params, _ = _mlp(dtype, fused)
    _init(params, 5, dtype)
    plist = ch.ParameterList(params)
    x, y = ch.DeviceTensor.from_host(x_host), ch.DeviceTensor.from_host(y_host)
    want = []
    for _ in range(steps):
        out = _step(net, plist, x, y, N)
        want.append((out.to_host(), _values(params)))

    # one eager step, then the same step recorded and launched steps - 1 times
    net2, params2, _ = _mlp(dtype, fused)
    _init(params2, 5, dtype)
    plist2 = ch.ParameterList(params2)
    x2, y2 = ch.DeviceTensor.from_host(x_host), ch.DeviceTensor.from_host(y_host)
    out = _step(net2, plist2, x2, y2, N)
    assert np.array_equal(out.to_host(), want[0][0])
    with ch.Graph() as graph:
        out = _step(net2, plist2, x2, y2, N)
    for a, b in zip(_values(params2), want[0][1]):
        assert np.array_equal(a, b)                      # recording ran nothing
    for k in range(1, steps):
        graph.launch()
        got_out, got_vals = out.to_host(), _values(params2)
        assert np.array_equal(got_out, want[k][0]), "output of launch %d" % k
        for a, b in zip(got_vals, want[k][1]):
            assert np.array_equal(a, b), "weights after launch %d" % k
        # eager work of the program's own and a wait between the launches
        other.pass_forward(x2, True)
        ch.synchronize()
    graph.destroy()
    # the layers work eagerly again afterwards
    _step(net2, plist2, x2, y2, N)


def test_recorded_convnet_pass_with_the_optimizer_outside():
    """Forward and backward pass of a fused convnet as a graph; Adam, whose update depends on the time step, is called
    eagerly after every launch."""
    dtype, N, steps = np.float32, 16, 4
    gen = hp.rng(78)
    x_host = hp.normal(gen, (N, 8, 8, 3), dtype)
    y_host = np.zeros((N, 6, 1, 1), dtype, order="F")
    y_host[np.arange(N), gen.integers(0, 6, N), 0, 0] = 1
    runs = []
    for recorded in (False, True):
        net, params, _ = _convnet(dtype)
        _init(params, 9, dtype)
        plist = ch.ParameterList(params)
        x, y = ch.DeviceTensor.from_host(x_host), ch.DeviceTensor.from_host(y_host)
        history = []
        graph = None
        for t in range(steps):
            if recorded and t >= 1:
                if graph is None:
                    with ch.Graph() as graph:
                        _step(net, plist, x, y, N, sgd=False)
                graph.launch()
            else:
                _step(net, plist, x, y, N, sgd=False)
            plist.optimizer_step("adam", [1e-2, 1e-1, 1e-3, 1e-5], timestep=t)
            history.append(_values(params))
        runs.append(history)
        if graph is not None:
            graph.destroy()
    for t in range(steps):
        for a, b in zip(runs[0][t], runs[1][t]):
            assert np.array_equal(a, b), "after step %d" % t


def test_recorded_convlstm_sequence():
    dtype, N, T, H, W, C, hid = np.float32, 4, 5, 6, 6, 3, 8
    gen = hp.rng(79)
    x_host = hp.normal(gen, (N, T, H, W, C), dtype)
    g_host = hp.normal(gen, (N, 1, H, W, hid), dtype)
    grads = []
    for recorded in (False, True):
        net = ch.ConvLSTMNetwork(dtype, (H, W, C), hid, output_seq_size_func=lambda t: (1, t - 1))
        wgen = hp.rng(3)
        for k in range(8):
            w, _ = net.kernel_params(k)
            w.set_values(hp.uniform(wgen, (w.get_rows(), hid), -0.3, 0.3, dtype))
        x, g = ch.DeviceTensor.from_host(x_host), ch.DeviceTensor.from_host(g_host)

        def step():
            out = net.propagate(x)
            net.backpropagate(g)
            return out

        out = step()                                 # gradients accumulate: two passes in both runs
        if recorded:
            with ch.Graph() as graph:
                out = step()
            graph.launch()
        else:
            out = step()
        got = [out.to_host()] + [net.kernel_params(k)[0].get_grad() for k in range(8)]
        grads.append(got)
        if recorded:
            graph.destroy()
    for a, b in zip(*grads):
        assert np.array_equal(a, b)


def test_what_cannot_be_recorded_is_refused():
    dtype, N = np.float32, 8
    layer = ch.DenseKernelLayer(dtype, (12,), 5)
    x = ch.DeviceTensor.from_host(hp.uniform(hp.rng(1), (N, 12), -1, 1, dtype))
    layer.pass_forward(x, True)
    with ch.Graph() as graph:
        layer.pass_forward(x, True)
        with pytest.raises(ch.CattleHipError) as e:
            ch.synchronize()
        assert e.value.code == 2
        with pytest.raises(ch.CattleHipError) as e:
            layer.pass_forward(np.zeros((N, 12), dtype, order="F"), True)        # a host tensor
        assert e.value.code == 2
        with pytest.raises(ch.CattleHipError) as e:
            ch.trim()
        assert e.value.code == 2
    graph.launch()
    ch.synchronize()
    graph.destroy()
    h = ctypes.c_void_p()
    assert ch.lib().cattle_hip_graph_end_capture(ctypes.byref(h)) == 2       # no recording in progress
