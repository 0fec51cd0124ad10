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


def test_a_living_graph_pins_the_buffers_it_may_point_into():
    """A graph keeps device addresses. While it exists, nothing that was allocated before its recording ended may move
    or be freed: growth and empty_cache are refused with the state error (no kernel ever runs on freed memory), and
    everything is allowed again once the graph is destroyed."""
    dtype, N = np.float32, 16
    gen = hp.rng(5)
    net, params, _ = _mlp(dtype, True)
    _init(params, 5, dtype)
    plist = ch.ParameterList(params)
    x = ch.DeviceTensor.from_host(hp.uniform(gen, (N, 20), -1, 1, dtype))
    y_host = np.zeros((N, 6), dtype, order="F")
    y_host[np.arange(N), gen.integers(0, 6, N)] = 1
    y = ch.DeviceTensor.from_host(y_host)
    # an unrelated convolution whose cut reduction will want more of the shared scratch buffer than anything so far
    conv = ch.ConvKernelLayer(dtype, (16, 16, 64), 32)
    xc_small = ch.DeviceTensor.from_host(hp.normal(gen, (4, 16, 16, 64), dtype))
    conv.pass_forward(xc_small, True)
    conv.pass_back(ch.DeviceTensor.from_host(hp.normal(gen, (4, 16, 16, 32), dtype)))      # its partial-sum buffer exists now
    ch.trim()                                               # nothing idle that the tests before left behind
    _step(net, plist, x, y, N)
    with ch.Graph() as graph:
        _step(net, plist, x, y, N)
    big = 4 * N
    xb = ch.DeviceTensor.from_host(hp.uniform(gen, (big, 20), -1, 1, dtype))
    # (a) the recorded layers at a larger batch: their buffers would have to grow
    with pytest.raises(ch.CattleHipError) as e:
        a = xb
        for l in net:
            a = l.pass_forward(a, True)
        for l in reversed(net):
            a = l.pass_back(a)
    assert e.value.code == 2 and "graph" in str(e.value)
    # (b) empty_cache of a recorded layer
    with pytest.raises(ch.CattleHipError) as e:
        net[0].empty_cache()
    assert e.value.code == 2 and "graph" in str(e.value)
    # (c) an unrelated, older layer that needs a larger shared scratch buffer (8 tiles cut into many parts)
    xc_big = ch.DeviceTensor.from_host(hp.normal(gen, (64, 16, 16, 64), dtype))
    grew = True
    try:
        conv.pass_forward(xc_big, True)
        conv.pass_back(ch.DeviceTensor.from_host(hp.normal(gen, (64, 16, 16, 32), dtype)))
        grew = False
    except ch.CattleHipError as err:
        assert err.code == 2 and "graph" in str(err)
    assert grew, "the larger problem was expected to need a larger scratch or partials buffer"
    # the graph still launches, on memory of its own
    graph.launch()
    ch.synchronize()
    # a layer created after the recording is free to grow and to empty its caches
    young = ch.DenseKernelLayer(dtype, (20,), 7)
    young.pass_forward(x, True)
    young.pass_forward(xb, True)
    young.empty_cache()
    graph.destroy()
    # and so is everything else once the graph is gone
    a = xb
    for l in net:
        a = l.pass_forward(a, True)
    net[0].empty_cache()
    conv.pass_forward(xc_big, True)
    ch.synchronize()


def test_destroying_a_recorded_layer_keeps_its_buffers_until_the_graph_goes():
    dtype, N = np.float32, 8
    layer = ch.DenseKernelLayer(dtype, (12,), 5)
    x = ch.DeviceTensor.from_host(hp.uniform(hp.rng(1), (N, 12), -1, 1, dtype))
    out = layer.pass_forward(x, True)
    with ch.Graph() as graph:
        layer.forward_into(x, out, True)
    del layer                                   # its parameter buffers are what the recorded kernels read
    graph.launch()                              # must not touch freed memory: the buffers are parked
    ch.synchronize()
    graph.destroy()
    ch.synchronize()


def test_dropout_training_pass_is_not_recorded():
    dtype, N = np.float32, 8
    drop = ch.DropoutLayer(dtype, (12,), 0.5, seed=3)
    x = ch.DeviceTensor.from_host(hp.uniform(hp.rng(1), (N, 12), -1, 1, dtype))
    y = ch.DeviceTensor((N, 12), dtype)
    drop.forward_into(x, y, True)
    with ch.Graph() as graph:
        with pytest.raises(ch.CattleHipError) as e:
            drop.forward_into(x, y, True)
        assert e.value.code == 2 and "dropout" in str(e.value)
        drop.forward_into(x, y, False)          # inference hands the input through: a copy, recordable
    graph.launch()
    ch.synchronize()
    assert np.array_equal(y.to_host(), x.to_host())
    graph.destroy()
