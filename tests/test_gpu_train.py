"""GPU parity of the device-resident ends of a training step: loss kernels and optimizer updates,
called through the C ABI, against the CPU oracle on identical seeded inputs (fp32 1e-4, fp64 1e-10)."""
import importlib

import numpy as np
import pytest

import helpers as hp
from oracle import oracle

pytestmark = pytest.mark.gpu

ch = importlib.import_module("c-attl3_amd")

TOL = {np.dtype(np.float32): 1e-4, np.dtype(np.float64): 1e-10}
DTYPES = [np.float32, np.float64]
KINDS = ["squared", "softmax_cross_entropy"]


def _targets(gen, kind, shape, dtype):
    if kind == "squared":
        return hp.normal(gen, shape, dtype)
    # one-hot over the flattened sample (the last axes), as a classifier's labels are
    N = shape[0]
    V = int(np.prod(shape[1:]))
    y = np.zeros((N, V), dtype=dtype, order="F")
    y[np.arange(N), gen.integers(0, V, N)] = 1
    return np.asfortranarray(y.reshape(shape, order="F"))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("shape", [(256, 10), (37, 3, 5, 2), (1, 1), (70, 1000), (32, 16, 16, 32)])
def test_losses(shape, kind, dtype):
    g = hp.rng(1201)
    out = hp.normal(g, shape, dtype, 2.0)
    obj = _targets(g, kind, shape, dtype)
    o64, y64 = np.asarray(out, np.float64), np.asarray(obj, np.float64)
    eps = float(dtype(1e-5))
    tol = TOL[np.dtype(dtype)]
    # -log p of a probability p known to one ulp carries an absolute error of an ulp of 1 however small the
    # loss is, so losses below 1 are compared absolutely (the reference's float arithmetic is no better)
    l_ref = oracle.loss_function(kind, o64, y64, eps=eps)
    assert np.max(np.abs(ch.loss_function(kind, out, obj) - l_ref) / np.maximum(np.abs(l_ref), 1.0)) < tol
    scale = 1.0 / shape[0]
    g_ref = oracle.loss_d_function(kind, o64, y64, eps=eps, scale=float(dtype(scale)))
    # likewise p - y is a difference of numbers of size <= 1: its error is absolute, of the size of scale * ulp(1)
    got = ch.loss_d_function(kind, out, obj, scale=scale)
    floor = scale if kind == "softmax_cross_entropy" else 0.0
    assert np.max(np.abs(got - g_ref) / np.maximum(np.abs(g_ref), floor + 1e-30)) < tol or hp.rel_err(got, g_ref) < tol
    # the same through device-resident buffers
    od, yd = ch.DeviceTensor.from_host(out), ch.DeviceTensor.from_host(obj)
    assert np.array_equal(ch.loss_function(kind, od, yd), ch.loss_function(kind, out, obj))
    assert np.array_equal(ch.loss_d_function(kind, od, yd, scale=scale).to_host(), ch.loss_d_function(kind, out, obj, scale=scale))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kind", KINDS)
def test_sequential_losses(kind, dtype):
    g = hp.rng(1202)
    shape = (33, 5, 4, 3)              # (N, T, 4, 3)
    out = hp.normal(g, shape, dtype)
    obj = hp.uniform(g, shape, 0, 1, dtype)
    o64, y64 = np.asarray(out, np.float64), np.asarray(obj, np.float64)
    eps = float(dtype(1e-5))
    tol = TOL[np.dtype(dtype)]
    assert hp.rel_err(ch.loss_function(kind, out, obj, sequential=True),
                      oracle.loss_function(kind, o64, y64, eps=eps, sequential=True)) < tol
    assert hp.rel_err(ch.loss_d_function(kind, out, obj, scale=0.25, sequential=True),
                      oracle.loss_d_function(kind, o64, y64, eps=eps, scale=0.25, sequential=True)) < tol


OTHER_LOSSES = hp.ALL_LOSSES[2:]
# losses whose value or gradient switches at a threshold (a margin or difference of zero): their inputs are put
# on a grid of 1/64 so that every margin is computed exactly, in float32 as in the float64 of the oracle, and
# margins of exactly zero occur
THRESHOLD_LOSSES = ("absolute", "hinge", "squared_hinge", "multi_label_hinge", "squared_multi_label_hinge")


def _loss_case(gen, kind, N, dims, dtype, steps=None):
    if kind == "binary_cross_entropy":
        dims = (1,) * len(dims)
    out, obj = hp.loss_inputs(gen, kind, N, dims, dtype, steps)
    if kind in THRESHOLD_LOSSES:
        out = np.asfortranarray(np.round(out * 64) / 64)
        obj = np.asfortranarray(np.round(obj * 64) / 64)
    return out, obj


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kind", OTHER_LOSSES)
@pytest.mark.parametrize("N,dims", [(256, (10,)), (37, (3, 5, 2)), (1, (1,)), (70, (1000,)), (32, (16, 16, 32))])
def test_the_other_losses(N, dims, kind, dtype):
    g = hp.rng(1203)
    out, obj = _loss_case(g, kind, N, dims, dtype)
    o64, y64 = np.asarray(out, np.float64), np.asarray(obj, np.float64)
    eps = float(dtype(1e-5))
    tol = TOL[np.dtype(dtype)]
    l_ref = oracle.loss_function(kind, o64, y64, eps=eps)
    assert np.max(np.abs(ch.loss_function(kind, out, obj) - l_ref) / np.maximum(np.abs(l_ref), 1.0)) < tol
    scale = float(dtype(1.0 / N))
    g_ref = oracle.loss_d_function(kind, o64, y64, eps=eps, scale=scale)
    got = ch.loss_d_function(kind, out, obj, scale=scale)
    assert hp.rel_err(got, g_ref) < tol
    if kind in THRESHOLD_LOSSES:            # which elements are inside the margin is decided identically
        assert np.array_equal(got == 0, g_ref == 0)
    # NegatedLoss: the same values with the opposite sign
    assert np.array_equal(ch.loss_function(kind, out, obj, negated=True), -ch.loss_function(kind, out, obj))
    assert np.array_equal(ch.loss_d_function(kind, out, obj, scale=scale, negated=True), -got)
    # the same through device-resident buffers
    od, yd = ch.DeviceTensor.from_host(out), ch.DeviceTensor.from_host(obj)
    assert np.array_equal(ch.loss_function(kind, od, yd), ch.loss_function(kind, out, obj))
    assert np.array_equal(ch.loss_d_function(kind, od, yd, scale=scale).to_host(), got)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kind", OTHER_LOSSES)
def test_the_other_losses_on_sequences(kind, dtype):
    g = hp.rng(1204)
    out, obj = _loss_case(g, kind, 33, (4, 3), dtype, steps=5)
    o64, y64 = np.asarray(out, np.float64), np.asarray(obj, np.float64)
    eps = float(dtype(1e-5))
    tol = TOL[np.dtype(dtype)]
    assert hp.rel_err(ch.loss_function(kind, out, obj, sequential=True),
                      oracle.loss_function(kind, o64, y64, eps=eps, sequential=True)) < tol
    assert hp.rel_err(ch.loss_d_function(kind, out, obj, scale=0.25, sequential=True),
                      oracle.loss_d_function(kind, o64, y64, eps=eps, scale=0.25, sequential=True)) < tol
    assert hp.rel_err(ch.loss_d_function(kind, out, obj, scale=0.25, sequential=True, negated=True),
                      oracle.loss_d_function(kind, o64, y64, eps=eps, scale=0.25, sequential=True, negated=True)) < tol


@pytest.mark.parametrize("dtype", DTYPES)
def test_loss_corner_values(dtype):
    """The rows worked by hand for the oracle, on the device: margins at the machine epsilon, a zero difference,
    an output of exactly zero under the multi-label log loss, the last one of a row as the hinge class."""
    col = lambda *v: np.asfortranarray(np.array(v, dtype).reshape(1, -1))
    tiny = np.finfo(dtype).eps
    o, y = col(2.0, 1.0, 1.5, 1.0 + tiny), col(1, 0, 0, 0)
    for kind in ("hinge", "squared_hinge"):
        assert np.array_equal(ch.loss_function(kind, o, y), oracle.loss_function(kind, o, y))
        assert np.array_equal(ch.loss_d_function(kind, o, y), [[-1.0, 0.0, 1.0, 0.0]])
    assert np.array_equal(ch.loss_d_function("hinge", col(0.0, 0.0, 5.0), col(0, 1, 0)), [[1.0, -2.0, 1.0]])
    assert np.array_equal(ch.loss_d_function("absolute", col(1.0, 2.0, 0.5), col(1.0, 3.0, 0.25)), [[1.0, -1.0, 1.0]])
    o, y = col(0.5, -2.0, 1.0, -0.25, 1.0 - tiny), col(1, -1, 1, 1, 1)
    assert np.array_equal(ch.loss_d_function("multi_label_hinge", o, y), [[-1.0, 0.0, 0.0, -1.0, 0.0]])
    assert np.array_equal(ch.loss_d_function("squared_multi_label_hinge", o, y), [[-1.0, 0.0, 0.0, -2.5, 0.0]])
    with np.errstate(all="ignore"):
        inf = ch.loss_d_function("multi_label_log", col(0.0, 0.0, 0.25), col(1, 0, 1), epsilon=0.25)
    assert inf[0, 0] == np.inf and inf[0, 1] == -np.inf and inf[0, 2] == 4.0
    # a hinge row without a one (the reference asserts against it): NaN marks the row, other rows are unaffected
    o = np.asfortranarray(np.array([[0.0, 1.0, 2.0], [2.0, 1.0, 1.5]], dtype))
    y = np.asfortranarray(np.array([[0, 0, 0], [1, 0, 0]], dtype))
    for kind in ("hinge", "squared_hinge"):
        l, gr = ch.loss_function(kind, o, y), ch.loss_d_function(kind, o, y)
        assert np.isnan(l[0]) and np.all(np.isnan(gr[0]))
        assert l[1] == oracle.loss_function(kind, o[1:], y[1:])[0]
        assert np.array_equal(gr[1:], oracle.loss_d_function(kind, o[1:], y[1:]))


def test_loss_errors():
    a = np.zeros((4, 3), np.float32, order="F")
    with pytest.raises(ValueError):
        ch.loss_function("squared", a, np.zeros((4, 2), np.float32, order="F"))
    lib = ch.lib()
    import ctypes
    for bad in (11, 0x100 | 11, -1, 0x200):
        rc = lib.cattle_hip_loss_function(0, bad, ctypes.c_void_p(a.ctypes.data), 0, ctypes.c_void_p(a.ctypes.data), 0,
                                          ctypes.c_size_t(4), ctypes.c_size_t(1), ctypes.c_size_t(3), ctypes.c_double(1e-5),
                                          ctypes.c_void_p(a.ctypes.data), 0)
        assert rc != 0 and b"loss kind" in lib.cattle_hip_last_error()
    # the binary cross entropy takes one value per sample and time step (assert in BinaryCrossEntropyLoss.hpp:36,43)
    with pytest.raises(ch.CattleHipError):
        ch.loss_function("binary_cross_entropy", a, a)
    with pytest.raises(ch.CattleHipError):
        ch.loss_d_function("binary_cross_entropy", a, a)


def _dense_with_grads(dtype, seed):
    g = hp.rng(seed)
    layer = ch.DenseKernelLayer(dtype, (24,), 17)
    w = hp.normal(g, (24, 17), dtype, 0.3)
    b = hp.normal(g, (1, 17), dtype, 0.1)
    layer.get_params()[0].set_values(w)
    layer.get_params()[1].set_values(b)
    return layer, g, w, b


def _accumulate(layer, g, dtype):
    x = hp.normal(g, (9, 24), dtype)
    go = hp.normal(g, (9, 17), dtype)
    layer.pass_forward(x, True)
    layer.pass_back(go)
    return x


@pytest.mark.parametrize("dtype", DTYPES)
def test_sgd_update(dtype):
    layer, g, w, b = _dense_with_grads(dtype, 1210)
    _accumulate(layer, g, dtype)
    tol = TOL[np.dtype(dtype)]
    for prm, old in zip(layer.get_params(), (w, b)):
        grad = prm.get_grad()
        prm.sgd_update(0.05)
        ref = oracle.sgd_update(np.asarray(old, np.float64), np.asarray(grad, np.float64), lr=float(dtype(0.05)))
        assert hp.rel_err(prm.get_values(), ref) < tol
        assert np.array_equal(prm.get_grad(), grad)            # the update leaves the gradient alone
    # the forward pass uses the updated weights (kernel-side weight layouts are rebuilt)
    x = hp.normal(g, (5, 24), dtype)
    wn, bn = (np.asarray(p.get_values(), np.float64) for p in layer.get_params())
    assert hp.rel_err(layer.pass_forward(x, False), oracle.dense_forward(np.asarray(x, np.float64), wn, bn)) < tol


@pytest.mark.parametrize("dtype", DTYPES)
def test_adam_updates_over_steps(dtype):
    layer, g, w, b = _dense_with_grads(dtype, 1211)
    tol = TOL[np.dtype(dtype)]
    state = [(np.asarray(v, np.float64), np.zeros(v.shape), np.zeros(v.shape)) for v in (w, b)]
    hyper = dict(lr=2e-3, l1_decay=0.1, l2_decay=0.01, eps=1e-5)
    for t in range(4):
        for prm in layer.get_params():
            prm.reset_grad()
        _accumulate(layer, g, dtype)
        for i, prm in enumerate(layer.get_params()):
            grad = np.asarray(prm.get_grad(), np.float64)
            prm.adam_update(t, learning_rate=hyper["lr"], l1_decay=hyper["l1_decay"], l2_decay=hyper["l2_decay"],
                            epsilon=hyper["eps"])
            state[i] = oracle.adam_update(state[i][0], grad, state[i][1], state[i][2], t,
                                          **{k: float(dtype(v)) for k, v in hyper.items()})
            # teacher-forced: the device continues from its own values, the oracle from the oracle's; compare, then
            # hand the device values to the oracle so that rounding differences do not compound through 1/sqrt(v)
            assert hp.rel_err(prm.get_values(), state[i][0]) < tol, (t, i)
            state[i] = (np.asarray(prm.get_values(), np.float64), state[i][1], state[i][2])
    # AdamOptimizer::_fit starts the averages again from zero
    prm = layer.get_params()[0]
    prm.reset_optimizer_state()
    before = np.asarray(prm.get_values(), np.float64)
    grad = np.asarray(prm.get_grad(), np.float64)
    prm.adam_update(0)
    ref, _, _ = oracle.adam_update(before, grad, np.zeros_like(before), np.zeros_like(before), 0,
                                   lr=float(dtype(1e-3)), l1_decay=float(dtype(1e-1)), l2_decay=float(dtype(1e-3)),
                                   eps=float(dtype(1e-5)))
    assert hp.rel_err(prm.get_values(), ref) < tol


def test_shared_parameters_share_the_update_and_its_state():
    dtype = np.float32
    layer, g, w, b = _dense_with_grads(dtype, 1212)
    twin = layer.clone_with_shared_params()
    _accumulate(layer, g, dtype)
    _accumulate(twin, g, dtype)                       # both accumulate into the one gradient
    layer.get_params()[0].adam_update(0)
    assert np.array_equal(twin.get_params()[0].get_values(), layer.get_params()[0].get_values())
    assert not np.array_equal(layer.get_params()[0].get_values(), w)
    x = hp.normal(g, (3, 24), dtype)
    assert np.array_equal(twin.pass_forward(x, False), layer.pass_forward(x, False))


def test_updates_reject_what_the_reference_skips():
    bn = ch.BatchNormLayer(np.float32, (4, 4, 3))
    running_mean = bn.get_params()[0]                  # not optimizable: optimizers skip it (AdamOptimizer.hpp:72-73)
    with pytest.raises(ch.CattleHipError):
        running_mean.sgd_update(0.1)
    with pytest.raises(ch.CattleHipError):
        running_mean.adam_update(0)
    gamma = bn.get_params()[2]
    with pytest.raises(ch.CattleHipError):
        gamma.sgd_update(0.0)                          # assert(learning_rate > 0)
    with pytest.raises(ch.CattleHipError):
        gamma.adam_update(0, l1_decay=1.5)             # assert(l1_decay >= 0 && l1_decay <= 1)


def _one_hot_labels(gen, N, shape, dtype):
    obj = np.zeros((N,) + shape, dtype, order="F")
    obj.reshape((N, -1), order="F")[np.arange(N), gen.integers(0, int(np.prod(shape)), N)] = 1
    return obj


@pytest.mark.parametrize("config", ["mlp_sgd", "convnet_adam"])
def test_whole_training_steps_stay_on_the_device(config):
    """BASELINE configs 2 and 3 as SGDOptimizer::_train runs them (optimizer/SGDOptimizer.hpp:44-70), three steps
    in a row: once with every tensor, the loss and the update on the device (only the per-sample losses come
    back), once with the same HIP layers fed host tensors and the loss and optimizer done on the host by the
    test harness. Both must tell the same story: same losses, same weights."""
    import harness as hn
    dt = np.float32
    gen = hp.rng(0xC0FFEE20)
    if config == "mlp_sgd":
        N, in_shape, out_shape, build = 256, (784,), (10,), hn.build_mlp
        x = np.asfortranarray(gen.uniform(0, 1, (N,) + in_shape).astype(dt))
    else:
        N, in_shape, out_shape, build = 128, (32, 32, 3), (10, 1, 1), hn.build_convnet
        x = np.asfortranarray(gen.standard_normal((N,) + in_shape).astype(dt))
    obj = _one_hot_labels(gen, N, out_shape, dt)
    dev, host = build(hn.HipBackend(dt)), build(hn.HipBackend(dt))
    hn.init_kernel_weights(dev, 20, dt)
    for pd, ps in zip(dev.params(), host.params()):
        ps.set_values(pd.get_values())
    start = [p.get_values() for p in dev.params()]
    host_adam = hn.Adam(host.params(), lr=1e-3)
    xd, yd = ch.DeviceTensor.from_host(x), ch.DeviceTensor.from_host(obj)
    for step in range(3):
        # device-resident step
        out = dev.propagate(xd, True)
        loss_dev = ch.loss_function("softmax_cross_entropy", out, yd)
        dev.backpropagate(ch.loss_d_function("softmax_cross_entropy", out, yd, scale=1.0 / N))
        for p in dev.params():
            if p.are_optimizable():
                if config == "mlp_sgd":
                    p.sgd_update(1e-3)
                else:
                    p.adam_update(step, learning_rate=1e-3)
                p.reset_grad()
        # host-orchestrated step on the twin network
        out_h = hn.train_step_gradients(host, x, obj, hn.softmax_ce_grad)
        loss_host = oracle.loss_function("softmax_cross_entropy", np.asarray(out_h, np.float64), np.asarray(obj, np.float64))
        if config == "mlp_sgd":
            hn.vanilla_sgd_update(host.params(), 1e-3)
        else:
            host_adam.update(host.params(), step)
        for p in host.params():
            p.reset_grad()
        assert hp.rel_err(loss_dev, loss_host) < 1e-3, step
    for pd, ps, w0 in zip(dev.params(), host.params(), start):
        moved = np.max(np.abs(np.asarray(ps.get_values(), np.float64) - w0))
        diff = np.max(np.abs(np.asarray(pd.get_values(), np.float64) - ps.get_values()))
        # three steps move a weight by up to `moved`; both routes must agree on that movement to 1 % of the
        # largest step (Adam turns rounding-level gradient differences near zero into sign flips of single
        # entries, so entrywise relative agreement is not to be had) and on the values to 1e-4
        assert diff <= 1e-2 * moved + 1e-7, (diff, moved)
        assert np.allclose(pd.get_values(), ps.get_values(), rtol=1e-4, atol=1e-5)


def test_the_reference_cifar_example_network_trains_on_the_device():
    """examples/cifar_convnet.cpp:24-41 (two conv / ReLU / max-pool stages, dropout, two dense layers, softmax,
    CrossEntropyLoss, NadamOptimizer with its default hyper-parameters) on CIFAR-shaped synthetic data: four batches of
    SGDOptimizer::_train with every tensor on the device, against the same network built from the oracle's layers in
    float64 with the oracle's loss and optimizer. The dropout masks are those of the float32 device layers."""
    import harness as hn
    dt, N = np.float32, 200
    gen = hp.rng(0xC0FFEE30)
    x = np.asfortranarray(gen.uniform(0, 1, (N, 32, 32, 3)).astype(dt))
    obj = _one_hot_labels(gen, N, (10, 1, 1), dt)
    dev = hn.build_cifar_example(hn.HipBackend(dt))
    ref = hn.build_cifar_example(hn.OracleBackend(np.float64), mask_dtype=dt)
    hn.init_kernel_weights(dev, 30, dt)
    for pd, pr in zip(dev.params(), ref.params()):
        pr.set_values(np.asarray(pd.get_values(), np.float64))
    hyper = [1e-3, 1e-1, 1e-3, 1e-5]                        # NadamOptimizer's defaults (optimizer/NadamOptimizer.hpp:39-41)
    hyper32 = [float(np.float32(h)) for h in hyper]          # as the float network sees them
    dev_params = ch.ParameterList([p for p in dev.params() if p.are_optimizable()])
    states = [[np.zeros_like(p.get_values()) for _ in range(3)] for p in ref.params()]
    xd, yd = ch.DeviceTensor.from_host(x), ch.DeviceTensor.from_host(obj)
    x64, y64 = np.asarray(x, np.float64), np.asarray(obj, np.float64)
    losses = []
    for step in range(4):
        out = dev.propagate(xd, True)
        loss_dev = ch.loss_function("cross_entropy", out, yd)
        dev.backpropagate(ch.loss_d_function("cross_entropy", out, yd, scale=1.0 / N))
        dev_params.optimizer_step("nadam", hyper, 0, step)
        out_r = ref.propagate(x64, True)
        loss_ref = oracle.loss_function("cross_entropy", out_r, y64, eps=float(np.float32(1e-5)))
        ref.backpropagate(oracle.loss_d_function("cross_entropy", out_r, y64, eps=float(np.float32(1e-5)), scale=float(np.float32(1.0 / N))))
        for p, st in zip(ref.params(), states):
            new, st[:] = oracle.optimizer_update("nadam", p.get_values(), p.get_grad(), st, hyper32, 0, step)
            p.set_values(new)
            p.reset_grad()
        assert hp.rel_err(loss_dev, loss_ref) < 1e-3, step
        losses.append(float(loss_ref.sum()))
    for pd, pr in zip(dev.params(), ref.params()):
        assert np.allclose(pd.get_values(), pr.get_values(), rtol=1e-3, atol=2e-5)
    # inference: dropout hands its input through, the softmax outputs are probabilities
    probs = dev.propagate(xd, False).to_host()
    assert hp.rel_err(probs, ref.propagate(x64, False)) < 1e-3
    assert np.allclose(probs.reshape((N, 10), order="F").sum(axis=1), 1.0, atol=1e-4)


def test_the_reference_autoencoder_example_trains_on_the_device():
    """examples/mnist_autoencoder.cpp:25-53 (strided convolutions without padding, softplus, dense bottleneck, reshape,
    transposed convolutions, SquaredLoss against the input itself, NadamOptimizer) on MNIST-shaped synthetic data: three
    batches on the device against the oracle's layers in float64."""
    import harness as hn
    dt, N = np.float32, 64
    gen = hp.rng(0xC0FFEE32)
    x = hp.uniform(gen, (N, 28, 28, 1), 0, 1, dt)
    dev, ref = hn.build_autoencoder_example(hn.HipBackend(dt)), hn.build_autoencoder_example(hn.OracleBackend(np.float64))
    assert dev.layers[-1].get_output_dims() == (28, 28, 1) and ref.layers[-1].get_output_dims() == (28, 28, 1)
    hn.init_kernel_weights(dev, 50, dt)
    for pd, pr in zip(dev.params(), ref.params()):
        pr.set_values(np.asarray(pd.get_values(), np.float64))
    hyper = [float(np.float32(h)) for h in (1e-3, 1e-1, 1e-3, 1e-5)]
    plist = ch.ParameterList(dev.params())
    states = [[np.zeros_like(p.get_values()) for _ in range(3)] for p in ref.params()]
    xd, x64 = ch.DeviceTensor.from_host(x), np.asarray(x, np.float64)
    for step in range(3):
        out = dev.propagate(xd, True)
        loss_dev = ch.loss_function("squared", out, xd)
        dev.backpropagate(ch.loss_d_function("squared", out, xd, scale=1.0 / N))
        plist.optimizer_step("nadam", hyper, 0, step)
        out_r = ref.propagate(x64, True)
        loss_ref = oracle.loss_function("squared", out_r, x64)
        ref.backpropagate(oracle.loss_d_function("squared", out_r, x64, scale=float(np.float32(1.0 / N))))
        for p, st in zip(ref.params(), states):
            new, st[:] = oracle.optimizer_update("nadam", p.get_values(), p.get_grad(), st, hyper, 0, step)
            p.set_values(new)
            p.reset_grad()
        assert hp.rel_err(loss_dev, loss_ref) < 1e-3, step
    for pd, pr in zip(dev.params(), ref.params()):
        assert np.allclose(pd.get_values(), pr.get_values(), rtol=1e-3, atol=2e-5)
    assert hp.rel_err(dev.propagate(xd, False).to_host(), ref.propagate(x64, False)) < 1e-3


def test_the_reference_gan_example_trains_on_the_device():
    """examples/mnist_gan.cpp:34-107 on MNIST-shaped synthetic data: two rounds of its training loop - the discriminator
    on a generated and on a real batch, then the generator through the frozen discriminator (whose gradients accumulate
    and are reset, but whose values stay: optimizer/SGDOptimizer.hpp:58-70, optimizer/AdamOptimizer.hpp:71) - with
    BinaryCrossEntropyLoss and two AdamOptimizers (learning rate 2e-4, first decay .5), every tensor on the device,
    against the same two networks built from the oracle's layers in float64."""
    import harness as hn
    dt, m = np.float32, 100
    gen = hp.rng(0xC0FFEE31)
    f32 = lambda v: float(np.float32(v))
    hyper = [f32(2e-4), f32(0.5), f32(1e-3), f32(1e-5)]
    eps = f32(1e-5)

    class Side(object):
        """One implementation of the pair of networks with its losses and optimizers."""
        def __init__(self, device):
            self.device = device
            self.G, self.D = hn.build_gan_example(hn.HipBackend(dt)) if device else \
                hn.build_gan_example(hn.OracleBackend(np.float64), mask_dtype=dt)
            self.steps = {"G": 0, "D": 0}
            if device:
                self.lists = {"G": ch.ParameterList(self.G.params()), "D": ch.ParameterList(self.D.params())}
            else:
                self.states = {k: [[np.zeros_like(p.get_values()) for _ in range(3)] for p in net.params()]
                               for k, net in (("G", self.G), ("D", self.D))}

        def tensor(self, a):
            return ch.DeviceTensor.from_host(a) if self.device else np.asarray(a, np.float64)

        def loss(self, out, obj):
            if self.device:
                return ch.loss_function("binary_cross_entropy", out, obj), \
                    ch.loss_d_function("binary_cross_entropy", out, obj, scale=1.0 / m)
            return oracle.loss_function("binary_cross_entropy", out, obj, eps=eps), \
                oracle.loss_d_function("binary_cross_entropy", out, obj, eps=eps, scale=f32(1.0 / m))

        def update(self, which):
            net = self.G if which == "G" else self.D
            if self.device:
                self.lists[which].optimizer_step("adam", hyper, 0, self.steps[which])
            else:
                for p, st in zip(net.params(), self.states[which]):
                    new, st[:] = oracle.optimizer_update("adam", p.get_values(), p.get_grad(), st, hyper, 0, self.steps[which])
                    p.set_values(new)
                    p.reset_grad()
            self.steps[which] += 1

        def round(self, z_fake, real, real_labels, z_gen):
            losses = []
            fake = self.G.propagate(self.tensor(z_fake), False)                       # infer
            for data, labels in ((fake, np.zeros((m, 1, 1, 1), dt)), (self.tensor(real), real_labels)):
                out = self.D.propagate(data, True)
                l, g = self.loss(out, self.tensor(labels))
                self.D.backpropagate(g)
                self.update("D")
                losses.append(np.asarray(l, np.float64))
            out = self.D.propagate(self.G.propagate(self.tensor(z_gen), True), True)
            l, g = self.loss(out, self.tensor(np.ones((m, 1, 1, 1), dt)))
            self.G.backpropagate(self.D.backpropagate(g))
            self.update("G")
            for p in self.D.params():                                                 # frozen: reset, not updated
                p.reset_grad()
            losses.append(np.asarray(l, np.float64))
            return losses

    dev, ref = Side(True), Side(False)
    for net_d, net_r, seed in ((dev.G, ref.G, 40), (dev.D, ref.D, 41)):
        hn.init_kernel_weights(net_d, seed, dt)
        for pd, pr in zip(net_d.params(), net_r.params()):
            pr.set_values(np.asarray(pd.get_values(), np.float64))
    for rnd in range(2):
        z_fake = hp.normal(gen, (m, 1, 1, 100), dt)
        real = hp.uniform(gen, (m, 28, 28, 1), -1, 1, dt)
        real_labels = hp.uniform(gen, (m, 1, 1, 1), 0.9, 1.0, dt)                     # the example's smoothed labels
        z_gen = hp.normal(gen, (m, 1, 1, 100), dt)
        for k, (a, b) in enumerate(zip(dev.round(z_fake, real, real_labels, z_gen), ref.round(z_fake, real, real_labels, z_gen))):
            assert hp.rel_err(a, b) < 1e-3, (rnd, k)
    for net_d, net_r in ((dev.G, ref.G), (dev.D, ref.D)):
        for pd, pr in zip(net_d.params(), net_r.params()):
            assert np.allclose(pd.get_values(), pr.get_values(), rtol=1e-3, atol=2e-5)
            assert np.all(pd.get_grad() == 0)


ALL_OPTIMIZERS = [("vanilla_sgd", [1e-2]), ("momentum_sgd", [1e-2, 1e-3, 0.9]), ("nesterov_momentum_sgd", [1e-2, 1e-3, 0.9]),
                  ("adagrad", [1e-2, 1e-5]), ("rmsprop", [1e-3, 1e-1, 1e-5]), ("adadelta", [5e-2, 1e-5]),
                  ("adam", [1e-3, 1e-1, 1e-3, 1e-5]), ("adamax", [1e-3, 1e-1, 1e-3, 1e-5]), ("nadam", [1e-3, 1e-1, 1e-3, 1e-5]),
                  ("amsgrad", [1e-3, 1e-1, 1e-3, 1e-5])]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rule,hyper", ALL_OPTIMIZERS)
def test_every_optimizer_over_steps(rule, hyper, dtype):
    """Each optimizer's _update_params on the device against the oracle, four steps with fresh gradients, epoch 2
    (the annealed learning rate), default hyper-parameters of the reference. After each comparison the oracle
    continues from the device's values and state estimate so that rounding does not compound through 1/sqrt(v)."""
    layer, g, w, b = _dense_with_grads(dtype, 1220)
    prm = layer.get_params()[0]
    tol = TOL[np.dtype(dtype)]
    hyper_t = [float(dtype(h)) for h in hyper]
    values = np.asarray(w, np.float64)
    states = [np.zeros_like(values) for _ in range(3)]
    for t in range(4):
        prm.reset_grad()
        _accumulate(layer, g, dtype)
        grad = np.asarray(prm.get_grad(), np.float64)
        prm.optimizer_update(rule, hyper, epoch=2, timestep=t)
        values, states = oracle.optimizer_update(rule, values, grad, states, hyper_t, epoch=2, timestep=t)
        got = np.asarray(prm.get_values(), np.float64)
        assert hp.rel_err(got, values) < tol, (rule, t)
        values = got
    # _fit: the state starts again from zero
    prm.reset_optimizer_state()
    before = np.asarray(prm.get_values(), np.float64)
    grad = np.asarray(prm.get_grad(), np.float64)
    prm.optimizer_update(rule, hyper, epoch=0, timestep=0)
    ref, _ = oracle.optimizer_update(rule, before, grad, [np.zeros_like(before) for _ in range(3)], hyper_t, 0, 0)
    assert hp.rel_err(prm.get_values(), ref) < tol


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rule,hyper", [ALL_OPTIMIZERS[0], ALL_OPTIMIZERS[2], ALL_OPTIMIZERS[6], ALL_OPTIMIZERS[9]])
def test_optimizer_step_is_update_then_reset(rule, hyper, dtype):
    """optimizer_step (update and reset_grad in one kernel) leaves the same values, bit for bit, as optimizer_update
    followed by reset_grad over three batches, and a zero gradient after each."""
    a, ga, _, _ = _dense_with_grads(dtype, 1222)
    c, gc, _, _ = _dense_with_grads(dtype, 1222)       # same seed: the same stream of inputs
    pa, pc = a.get_params()[0], c.get_params()[0]
    for t in range(3):
        _accumulate(a, ga, dtype)
        _accumulate(c, gc, dtype)
        assert np.any(pa.get_grad()) and np.array_equal(pa.get_grad(), pc.get_grad())
        pa.optimizer_update(rule, hyper, epoch=1, timestep=t)
        pa.reset_grad()
        pc.optimizer_step(rule, hyper, epoch=1, timestep=t)
        assert np.array_equal(pa.get_values(), pc.get_values()), (rule, t)
        assert not np.any(pc.get_grad())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rule,hyper", [ALL_OPTIMIZERS[0], ALL_OPTIMIZERS[1], ALL_OPTIMIZERS[6]])
def test_optimizer_step_of_a_whole_network(rule, hyper, dtype):
    """ParameterList.optimizer_step (every parameter of a network in one launch per sixteen, prepared weight
    layouts rewritten by the same kernel) against optimizer_step parameter by parameter on a twin network: the same
    values bit for bit after each of three batches, zero gradients, and the next passes (which use the prepared
    layouts) agree as well. conv - ReLU - conv (shared with a clone) - dense layers."""
    def build():
        c1 = ch.ConvKernelLayer(dtype, (8, 8, 3), 6)
        c2 = ch.ConvKernelLayer(dtype, (8, 8, 6), 6, 3, 3, 2, 2, 1, 1, 1, 1)          # dilated, same size out
        layers = [c1, ch.ReLUActivationLayer(dtype, (8, 8, 6)), c2, c2.clone_with_shared_params(),
                  ch.DenseKernelLayer(dtype, (8, 8, 6), 5)]
        layers += [ch.DenseKernelLayer(dtype, (5, 1, 1), 5) for _ in range(7)]        # more than sixteen parameters
        g = hp.rng(1230)
        for l in layers:
            for p in l.get_params():
                if p.get_rows() > 1:
                    p.set_values(hp.normal(g, (p.get_rows(), p.get_cols()), dtype, 0.3))
        return layers

    def passes(layers, x, go):
        a = x
        for l in layers:
            a = l.pass_forward(a, True)
        g = go
        for l in reversed(layers):
            g = l.pass_back(g)
        return a, g

    one, many = build(), build()
    plist = ch.ParameterList([p for l in many for p in l.get_params()])
    assert len(plist) == 22                       # 20 distinct Parameters objects, two of them listed twice
    g = hp.rng(1231)
    for t in range(3):
        x = hp.normal(g, (8, 8, 8, 3), dtype)
        go = hp.normal(g, (8, 5, 1, 1), dtype)
        out_a, dx_a = passes(one, x, go)
        out_b, dx_b = passes(many, x, go)
        assert np.array_equal(out_a, out_b) and np.array_equal(dx_a, dx_b), t
        seen = set()
        for l in one:
            for p in l.get_params():
                assert np.any(p.get_grad())
        for i, l in enumerate(one):
            if i == 3:
                continue                      # the clone shares layer 2's parameters: update them once
            for p in l.get_params():
                p.optimizer_step(rule, hyper, epoch=1, timestep=t)
        plist.optimizer_step(rule, hyper, epoch=1, timestep=t)
        for la, lb in zip(one, many):
            for pa, pb in zip(la.get_params(), lb.get_params()):
                assert np.array_equal(pa.get_values(), pb.get_values()), (rule, t)
                assert not np.any(pb.get_grad())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("l1,l2", [(0.03, 0.0), (0.0, 0.2), (0.03, 0.2)])
@pytest.mark.parametrize("rule,hyper", [ALL_OPTIMIZERS[0], ALL_OPTIMIZERS[6]])
def test_regularized_optimizer_steps(rule, hyper, l1, l2, dtype):
    """Parameters with an L1, L2 or elastic-net regularization: optimizer_step and the step of a whole network add its
    gradient before the update (SGDOptimizer::_train: regularize, update, reset), the plain update does not, and the
    penalty is Parameters::get_regularization_penalty."""
    tol = TOL[np.dtype(dtype)]
    layer, g, _, _ = _dense_with_grads(dtype, 1301)
    _accumulate(layer, g, dtype)
    conv = ch.ConvKernelLayer(dtype, (6, 5, 3), 4)
    x = hp.normal(g, (8, 6, 5, 3), dtype)
    conv.get_params()[0].set_values(hp.normal(g, (27, 4), dtype, 0.3))
    conv.pass_forward(x, True)                                   # builds the prepared weight layout the step rewrites
    conv.pass_back(hp.normal(g, (8, 6, 5, 4), dtype))
    params = [layer.get_params()[0], conv.get_params()[0], conv.get_params()[1]]
    for p in params:
        p.set_regularization(l1, l2)
    lam1, lam2 = float(dtype(l1)), float(dtype(l2))
    hyper32 = [float(dtype(h)) for h in hyper]
    want = []
    for p in params:
        v64, g64 = np.asarray(p.get_values(), np.float64), np.asarray(p.get_grad(), np.float64)
        pen, reg = oracle.regularization(v64, lam1, lam2)
        assert abs(p.get_regularization_penalty() - pen) <= tol * max(1.0, abs(pen))
        new, _ = oracle.optimizer_update(rule, v64, g64 + reg, [np.zeros_like(v64)] * 3, hyper32, 0, 0)
        want.append(new)
    params[0].optimizer_step(rule, hyper, 0, 0)                  # one parameter
    ch.ParameterList(params[1:]).optimizer_step(rule, hyper, 0, 0)         # several in one launch
    for p, w in zip(params, want):
        assert hp.rel_err(p.get_values(), w) < tol
        assert np.all(p.get_grad() == 0)
    # the convolution uses the regularized weights (its prepared layout was rewritten by the step)
    ref, _ = oracle.conv_forward(np.asarray(x, np.float64), want[1], want[2], return_cache=True)
    assert hp.rel_err(conv.pass_forward(x, True), ref) < tol
    # the plain update is _update_params alone: no regularization
    other, g2, _, _ = _dense_with_grads(dtype, 1302)
    _accumulate(other, g2, dtype)
    q = other.get_params()[0]
    q.set_regularization(l1, l2)
    v64, g64 = np.asarray(q.get_values(), np.float64), np.asarray(q.get_grad(), np.float64)
    plain, _ = oracle.optimizer_update(rule, v64, g64, [np.zeros_like(v64)] * 3, hyper32, 0, 0)
    q.optimizer_update(rule, hyper, 0, 0)
    assert hp.rel_err(q.get_values(), plain) < tol
    # none: penalty 0; a clone keeps the regularization
    q.set_regularization(0.0, 0.0)
    assert q.get_regularization_penalty() == 0.0
    assert conv.clone().get_params()[0].get_regularization_penalty() == pytest.approx(conv.get_params()[0].get_regularization_penalty())


def test_optimizer_argument_checks():
    layer, g, w, b = _dense_with_grads(np.float32, 1221)
    prm = layer.get_params()[0]
    with pytest.raises(ch.CattleHipError):
        prm.optimizer_update("momentum_sgd", [1e-2, 1e-3, 1.0])        # assert(momentum > 0 && momentum < 1)
    with pytest.raises(ch.CattleHipError):
        prm.optimizer_update("adadelta", [1.5, 1e-5])                   # assert(decay >= 0 && decay <= 1)
    with pytest.raises(ch.CattleHipError):
        prm.optimizer_update("rmsprop", [1e-3, 1e-1, 0.0])              # assert(epsilon > 0)
    import ctypes
    h = (ctypes.c_double * 4)(1e-3, 0, 0, 0)
    assert ch.lib().cattle_hip_layer_param_optimizer_update(layer._h, ctypes.c_size_t(0), ctypes.c_int(17), h, ctypes.c_size_t(0),
                                                            ctypes.c_size_t(0)) != 0


def test_device_memory_does_not_grow_over_steps_and_network_lifetimes():
    """Activation buffers, staging areas and optimizer state come from the library's pooling allocator: after a first
    network has trained, further networks of the same shape and any number of steps take no more device memory, and
    cattle_hip_trim hands the pooled buffers back."""
    import harness as hn
    dt, N = np.float32, 64
    gen = hp.rng(0xC0FFEE33)
    xd = ch.DeviceTensor.from_host(hp.normal(gen, (N, 32, 32, 3), dt))
    yd = ch.DeviceTensor.from_host(_one_hot_labels(gen, N, (10, 1, 1), dt))

    def used_mib():
        free, total = ch.memory_info()
        return (total - free) / 2.0 ** 20

    def lifetime(steps):
        net = hn.build_convnet(hn.HipBackend(dt))
        hn.init_kernel_weights(net, 60, dt)
        plist = ch.ParameterList(net.params())
        for t in range(steps):
            out = net.propagate(xd, True)
            net.backpropagate(ch.loss_d_function("softmax_cross_entropy", out, yd, scale=1.0 / N))
            plist.optimizer_step("adam", [1e-3, 1e-1, 1e-3, 1e-5], 0, t)

    lifetime(5)
    base = used_mib()
    for _ in range(3):
        lifetime(40)
        assert used_mib() - base <= 2.0            # MiB; the driver allocates in 2 MiB granules
    ch.trim()
    assert used_mib() <= base

