"""The fused-gate convolutional LSTM on the device (one convolution per group of four kernels, all input-side
kernels of all time steps in one launch, gate arithmetic in one kernel per step) against the per-layer
restatement of LSTMNeuralNetwork on the CPU oracle (tests/harness.py, SeqConvLSTM), in float64 on identical
inputs: output sequence, input gradient and all sixteen parameter gradients."""
import importlib

import numpy as np
import pytest

import harness as hn
import helpers as hp

pytestmark = pytest.mark.gpu

ch = importlib.import_module("c-attl3_amd")

TOL = {np.dtype(np.float32): 1e-4, np.dtype(np.float64): 1e-10}
SMOOTH = (("sigmoid", 0), ("sigmoid", 0), ("tanh", 0), ("tanh", 0), ("sigmoid", 0))
EXOTIC = (("softsign", 0), ("swish", 1.3), ("softplus", 0), ("elu", 0.7), ("scaled", 0.5))


def _pair(dtype, dims, hidden, acts, foremost, seq, seed, conv_kw=None, mul_int=False):
    kw = conv_kw or {}
    net = ch.ConvLSTMNetwork(dtype, dims, hidden, kw.get("RH", 3), kw.get("RW", 3), kw.get("pv", 1), kw.get("ph", 1),
                             kw.get("dv", 0), kw.get("dh", 0), activations=[a for a, _ in acts],
                             activation_params=[p for _, p in acts], output_seq_size_func=seq, foremost=foremost,
                             mul_int=mul_int)
    orc = hn.SeqConvLSTM(hn.OracleBackend(np.float64), dims, hidden, acts, conv_kw, foremost, mul_int)
    g = hp.rng(seed)
    for k, layer in enumerate(orc.kernels()):
        rows = layer.get_params()[0].get_values().shape[0]
        w = hn.he_normal(g, rows, hidden, dtype)
        b = hp.normal(g, (1, hidden), dtype, 0.1)
        for host, dev, v in zip(layer.get_params(), net.kernel_params(k), (w, b)):
            dev.set_values(v)
            host.set_values(np.asarray(v, np.float64))
            assert np.array_equal(dev.get_values(), v)
    return net, orc, g


def _check(dtype, N, T_in, dims, hidden, acts, foremost, seq, seed=7, conv_kw=None, mul_int=False):
    net, orc, g = _pair(dtype, dims, hidden, acts, foremost, seq, seed, conv_kw, mul_int)
    out_len, delay = seq(T_in)
    x = hp.normal(g, (N, T_in) + tuple(dims), dtype)
    go = hp.normal(g, (N, out_len, dims[0], dims[1], hidden), dtype)
    tol = TOL[np.dtype(dtype)]
    out = net.propagate(x)
    ref = orc.propagate(np.asarray(x, np.float64), out_len, delay)
    assert out.shape == ref.shape
    assert hp.rel_err(out, ref) < tol, "output sequence"
    dx = net.backpropagate(go)
    dx_ref = orc.backpropagate(np.asarray(go, np.float64))
    if foremost:
        assert dx is None and dx_ref is None
    else:
        assert hp.rel_err(dx, dx_ref) < tol, "input gradient"
    for k, layer in enumerate(orc.kernels()):
        for which, (host, dev) in enumerate(zip(layer.get_params(), net.kernel_params(k))):
            want = host.get_grad()
            if np.all(want == 0):           # a kernel that never ran (no step used it)
                assert np.all(dev.get_grad() == 0)
            else:
                assert hp.rel_err(dev.get_grad(), want) < tol, (net.KERNELS[k], "bias" if which else "weights")
    return net, orc, (x, go)


def test_config5_convlstm_fused():
    """BASELINE config 5: T=10, batch 32, 16x16x8 input, 32 hidden channels, output = last hidden state. At this size
    every step after the first runs its element-wise part inside the output-side convolution (forward) and inside the
    kernel that sums the parts of that convolution's input gradient (backward)."""
    net, _, _ = _check(np.float32, 32, 10, (16, 16, 8), 32, SMOOTH, True, lambda T: (1, T - 1))
    assert net.fused_steps() == (9, 9)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("acts", [SMOOTH, EXOTIC], ids=["smooth", "exotic"])
def test_steps_inside_the_recurrent_kernels(dtype, acts):
    """Hidden sizes that fill the tiles' column groups with whole gate groups (multiples of 8 with 32 output columns,
    of 16 with more) and batch sizes with 16-byte rows: the forward step runs in the convolution's epilogue. Both
    precisions, the usual activations (compile-time kinds) and others (run-time kinds, pre-activation values kept)."""
    # (the unbounded activations of EXOTIC grow from step to step, faster with more hidden channels: fewer steps for them)
    smooth = acts is SMOOTH
    T_in = 4 if smooth else 3
    net, _, _ = _check(dtype, 8, T_in, (6, 5, 3), 8, acts, False, lambda T: (T, 0))
    assert net.fused_steps() == (T_in - 1, T_in - 1)
    if smooth:
        net, _, _ = _check(dtype, 8, 3, (6, 5, 3), 16, acts, False, lambda T: (2, 2))      # runs one step past the input
        assert net.fused_steps() == (3, 3)
        net, _, _ = _check(dtype, 4, 3, (4, 4, 2), 48, acts, True, lambda T: (1, T - 1))   # three column tiles
        assert net.fused_steps() == (2, 2)
    else:
        net, _, _ = _check(dtype, 8, 2, (6, 5, 3), 16, acts, False, lambda T: (T, 0))
        assert net.fused_steps() == (1, 1)
    # a hidden size that does not fill the column groups, a batch size without 16-byte rows: kernels of their own
    net, _, _ = _check(dtype, 8, 2, (6, 5, 3), 12, acts, False, lambda T: (T, 0))
    assert net.fused_steps()[0] == 0
    net, _, _ = _check(dtype, 5, 2, (6, 5, 3), 8, acts, False, lambda T: (T, 0))
    assert net.fused_steps()[0] == 0
    # multiplicative integration keeps the weighted previous outputs for the backward pass: no fused forward step
    net, _, _ = _check(dtype, 8, 2, (6, 5, 3), 8, acts, False, lambda T: (T, 0), mul_int=True)
    assert net.fused_steps()[0] == 0


@pytest.mark.parametrize("mul_int", [False, True])
def test_a_batch_whose_recurrent_input_gradient_runs_as_whole_tiles(mul_int):
    """At config 5's size the input gradient of the output-side kernels is a launch whose reductions are cut into
    parts, and the kernel that sums the parts runs the cell's backward step on the sums. With 131072 rows the same launch
    works on whole tiles and writes the gradient tensor; the backward step is then a kernel of its own."""
    net, _, _ = _check(np.float32, 64, 3, (64, 32, 4), 8, SMOOTH, False, lambda T: (T, 0), mul_int=mul_int)
    assert net.fused_steps() == (0, 0)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("foremost", [True, False])
def test_sequence_alignments(dtype, foremost):
    dims, hidden = (6, 5, 3), 4
    _check(dtype, 5, 4, dims, hidden, SMOOTH, foremost, lambda T: (T, 0))             # an output at every step
    _check(dtype, 4, 3, dims, hidden, SMOOTH, foremost, lambda T: (4, 1))             # runs 2 steps past the input
    _check(dtype, 4, 1, dims, hidden, SMOOTH, foremost, lambda T: (1, 0))             # a single step: no recurrent kernel runs
    _check(dtype, 3, 5, dims, hidden, SMOOTH, foremost, lambda T: (2, 1))             # output in the middle of the sequence


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_other_activations_and_receptors(dtype):
    _check(dtype, 4, 3, (7, 6, 2), 5, EXOTIC, False, lambda T: (T, 0), conv_kw=dict(RH=3, RW=1, pv=1, ph=0))
    _check(dtype, 4, 3, (8, 8, 2), 3, SMOOTH, False, lambda T: (T, 0), conv_kw=dict(RH=3, RW=3, pv=2, ph=2, dv=1, dh=1))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("mul_int", [False, True])
def test_dense_lstm_is_the_one_by_one_case(dtype, mul_int):
    """An LSTM over vectors (the DenseKernelLayer networks of test/gradient_test.cpp:656-699: 32 inputs, 5 hidden units,
    an output at every step of three, and with multiplicative integration only the last of five) is the same network
    on 1 x 1 images with 1 x 1 receptors: the input size is the channel count."""
    one = dict(RH=1, RW=1, pv=0, ph=0)
    _check(dtype, 6, 3, (1, 1, 32), 5, SMOOTH, False, lambda T: (T, 0), conv_kw=one, mul_int=mul_int)
    _check(dtype, 6, 5, (1, 1, 32), 5, SMOOTH, False, lambda T: (1, T - 1), conv_kw=one, mul_int=mul_int)
    _check(dtype, 33, 4, (1, 1, 7), 5, SMOOTH, True, lambda T: (3, 2), conv_kw=one, mul_int=mul_int)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("foremost", [True, False])
def test_multiplicative_integration(dtype, foremost):
    """LSTMNeuralNetwork<Scalar,3,true> (the rank-3 network of test/gradient_test.cpp:735-741 and the alignments above)."""
    dims, hidden = (6, 5, 3), 4
    _check(dtype, 5, 4, dims, hidden, SMOOTH, foremost, lambda T: (T, 0), mul_int=True)
    _check(dtype, 4, 3, dims, hidden, SMOOTH, foremost, lambda T: (4, 1), mul_int=True)       # two steps on the output side only
    _check(dtype, 4, 1, dims, hidden, SMOOTH, foremost, lambda T: (1, 0), mul_int=True)       # a single step: nothing to multiply
    _check(dtype, 3, 5, dims, hidden, EXOTIC, foremost, lambda T: (2, 1), mul_int=True)
    # switching the rule on an existing network empties its caches and takes effect at the next pass
    net, orc, (x, go) = _check(dtype, 4, 3, dims, hidden, SMOOTH, foremost, lambda T: (T, 0), mul_int=False)
    plain = net.propagate(x)
    net.set_multiplicative_integration(True)
    with pytest.raises(ch.CattleHipError):
        net.backpropagate(go)
    assert not np.allclose(net.propagate(x), plain)


def test_gradients_accumulate_and_updates_apply():
    net, orc, (x, go) = _check(np.float32, 4, 3, (6, 5, 3), 4, SMOOTH, True, lambda T: (T, 0))
    w, b = net.kernel_params("output_write")
    g1 = w.get_grad()
    net.propagate(x)
    net.backpropagate(go)
    assert hp.rel_err(w.get_grad(), 2 * g1) < 1e-5                      # a second pass adds to the gradients
    # the fused parameters are ordinary parameters of the handle: optimizer updates and resets work on them
    fused = net.get_params()
    assert [p.get_rows() for p in fused] == [27, 1, 36, 1] and all(p.get_cols() == 16 for p in fused)
    before = w.get_values()
    fused[2].sgd_update(0.1)
    assert hp.rel_err(w.get_values(), np.asarray(before, np.float64) - float(np.float32(0.1)) * np.asarray(w.get_grad(), np.float64)) < 1e-5
    for p in fused:
        p.reset_grad()
    assert np.all(w.get_grad() == 0) and np.all(b.get_grad() == 0)
    # the next pass uses the updated recurrent weights (the fused update moved all four output-side kernels)
    for k in (1, 3, 5, 7):
        for host, dev in zip(orc.kernels()[k].get_params(), net.kernel_params(k)):
            host.set_values(np.asarray(dev.get_values(), np.float64))
    assert hp.rel_err(net.propagate(x), orc.propagate(np.asarray(x, np.float64), 3, 0)) < 1e-4


def test_device_resident_sequences_and_errors():
    net, orc, (x, go) = _check(np.float32, 4, 3, (6, 5, 3), 4, SMOOTH, False, lambda T: (T, 0))
    host_out = net.propagate(x)
    host_dx = net.backpropagate(go)
    xd, gd = ch.DeviceTensor.from_host(x), ch.DeviceTensor.from_host(go)
    assert np.array_equal(net.propagate(xd).to_host(), host_out)
    assert np.array_equal(net.backpropagate(gd).to_host(), host_dx)
    with pytest.raises(ch.CattleHipError):
        net.pass_forward(x[:, 0], True)                                # sequences only
    with pytest.raises(ch.CattleHipError):
        ch.ConvLSTMNetwork(np.float32, (6, 5, 3), 4, 3, 3, 0, 0)       # the kernels must keep the spatial dimensions
    with pytest.raises(ch.CattleHipError):
        ch.ConvLSTMNetwork(np.float32, (6, 5, 3), 4, activations=("softmax", "sigmoid", "tanh", "tanh", "sigmoid"))
    fresh = ch.ConvLSTMNetwork(np.float32, (6, 5, 3), 4)
    with pytest.raises(ch.CattleHipError):
        fresh.backpropagate(go)                                        # no propagate yet


def test_a_network_reused_with_another_sequence_length():
    """The step-shifted device buffers are written slab by slab in every pass, never cleared as a whole: a pass
    after a longer one on the same network gives, bit for bit, what a fresh network gives."""
    dtype, dims, hidden = np.float32, (6, 5, 3), 4
    seq = lambda T: (T, 0)
    used, _, g = _pair(dtype, dims, hidden, SMOOTH, False, seq, 21)
    fresh, _, _ = _pair(dtype, dims, hidden, SMOOTH, False, seq, 21)
    x_long = hp.normal(g, (6, 5) + dims, dtype)
    used.propagate(x_long)
    used.backpropagate(hp.normal(g, (6, 5, dims[0], dims[1], hidden), dtype))
    for p in used.get_params():
        p.reset_grad()
    x = hp.normal(g, (4, 3) + dims, dtype)
    go = hp.normal(g, (4, 3, dims[0], dims[1], hidden), dtype)
    assert np.array_equal(used.propagate(x), fresh.propagate(x))
    assert np.array_equal(used.backpropagate(go), fresh.backpropagate(go))
    for a, b in zip(used.get_params(), fresh.get_params()):
        assert np.array_equal(a.get_grad(), b.get_grad())
