"""The device-resident C++ front end (c-attl3_amd/include/cattle_hip/DeviceNet.hpp) driven by
tests/compat/device_net_test (built by __graft_entry__.build()): three training batches of an MLP with
vanilla SGD and of a small convnet with Adam, every tensor staying on the GPU. The recorded inputs and
initial parameters are replayed here on the CPU oracle with the host-side counterparts of the
reference's callers (tests/harness.py), and batch losses, final parameters and the inference output
are compared."""
import os
import subprocess

import numpy as np
import pytest

import harness as hn
import helpers as hp
from oracle import oracle
from test_gpu_adapters import _read_records

HERE = os.path.dirname(os.path.abspath(__file__))
BINARY = os.path.join(HERE, "compat", "device_net_test")


def test_device_net_compiles_as_cpp11():
    """CPU check: the header needs nothing but the C ABI and is valid C++11."""
    subprocess.check_call(["g++", "-std=c++11", "-fsyntax-only", "-Wall", "-I" + os.path.join(HERE, "..", "include"),
                           "-I" + os.path.join(HERE, "..", "c-attl3_amd", "include"),
                           os.path.join(HERE, "compat", "device_net_test.cpp")])


@pytest.fixture(scope="module")
def records(tmp_path_factory):
    if not os.path.exists(BINARY):
        pytest.fail("tests/compat/device_net_test is not built: run __graft_entry__.build()")
    tmp = tmp_path_factory.mktemp("device_net")
    out = str(tmp / "records.bin")
    subprocess.check_call([BINARY, out, str(tmp)], timeout=120)
    recs = _read_records(out)
    recs["__dir__"] = str(tmp)
    return recs


def _replay(r, net, lr, adam, steps=3):
    """SGDOptimizer::_train's batch body on the oracle network, in float64."""
    for li, layer in enumerate(net.layers):
        for pi, p in enumerate(layer.get_params()):
            p.set_values(np.asarray(r["init.%d.%d" % (li, pi)], np.float64))
    x, y = np.asarray(r["x"], np.float64), np.asarray(r["y"], np.float64)
    opt = hn.Adam(net.params(), lr=lr) if adam else None
    losses = []
    for t in range(steps):
        out = hn.train_step_gradients(net, x, y.reshape((x.shape[0],) + out_shape(net), order="F"), hn.softmax_ce_grad)
        losses.append(oracle.loss_function("softmax_cross_entropy", out, y.reshape(out.shape, order="F")).sum())
        if adam:
            opt.update(net.params(), t)
        else:
            hn.vanilla_sgd_update(net.params(), lr)
        for p in net.params():
            p.reset_grad()
    return np.array(losses)


def out_shape(net):
    return tuple(net.layers[-1].get_output_dims())


@pytest.mark.gpu
@pytest.mark.parametrize("tag", ["f32", "f64"])
def test_network_init_is_the_reference_initialization(records, tag):
    """DeviceFeedforwardNetwork::init(He): bit for bit what GaussianParameterInitialization::apply makes of the same standard
    library (checked inside the C++ driver), zero biases, untouched batch-norm parameters; here the moments of the
    recorded weights (standard deviation 0.1 sqrt(2 / fan_in)) and the transposed convolution's output dimensions."""
    assert np.all(records[tag + ".init_he.ok"] == 1) and records[tag + ".init_he.ok"].size == 7
    assert tuple(records[tag + ".init_he.transconv_dims"]) == oracle.transconv_out_dims(6, 6, 4, 4, 1, 1, 2, 2, 0, 0) + (2,)
    for key, fan_in in ((".init_he.w0", 27), (".init_he.w2", 4), (".init_he.w3", 12 * 12 * 2)):
        w = np.asarray(records[tag + key], np.float64)
        assert w.shape[0] == fan_in
        sd = 0.1 * np.sqrt(2.0 / fan_in)
        assert abs(w.std() / sd - 1) < 4 / np.sqrt(2 * w.size) + 0.02 and abs(w.mean()) < 4 * sd / np.sqrt(w.size)
    # every matrix starts a fresh default-seeded engine: matrices draw the same stream, scaled by their own deviation
    a, b = records[tag + ".init_he.w0"], records[tag + ".init_he.w2"]
    n = min(a.size, b.size)
    ra = a.reshape(-1, order="F")[:n] / (0.1 * np.sqrt(2.0 / 27))
    rb = b.reshape(-1, order="F")[:n] / (0.1 * np.sqrt(2.0 / 4))
    assert np.allclose(ra, rb, rtol=1e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("tag", ["f32", "f64"])
def test_stacked_network_with_a_frozen_module(records, tag):
    """DeviceStackedNetwork and set_frozen against the same training loop spelled out on two separate networks."""
    spelled = {k[len(tag) + 6:]: v for k, v in records.items() if k.startswith(tag + ".gan0.")}
    stacked = {k[len(tag) + 6:]: v for k, v in records.items() if k.startswith(tag + ".gan1.")}
    assert set(spelled) == set(stacked) and len(spelled) == 2 * 4 * 2 + 1
    for k in spelled:
        assert np.array_equal(spelled[k], stacked[k]), k
    assert np.all(np.isfinite(spelled["losses"])) and len(spelled["losses"]) == 6
    # the generator moved in its own steps, the frozen discriminator only in the discriminator's
    assert not np.array_equal(spelled["g.final.0.0"], spelled["g.init.0.0"])
    assert not np.array_equal(spelled["d.final.0.0"], spelled["d.init.0.0"])


@pytest.mark.gpu
@pytest.mark.parametrize("tag,dtype", [("f32", np.float32), ("f64", np.float64)])
def test_reshape_broadcast_dropout_stack(records, tag, dtype):
    x, go = records[tag + ".move.x"], records[tag + ".move.go"]
    assert x.dtype == dtype
    tiled = oracle.broadcast_forward(x.reshape((5, 3, 2, 2), order="F"), 2, 1, 3)
    u = oracle.dropout_uniforms(321, 0, tiled.shape, dtype)
    assert np.array_equal(records[tag + ".move.out"], oracle.dropout_apply(tiled, u, 0.4, 1e-5))
    back = oracle.broadcast_backward((5, 3, 2, 2), oracle.dropout_apply(go, u, 0.4, 1e-5), 2, 1, 3)
    assert np.array_equal(records[tag + ".move.dx"], back.reshape((5, 12), order="F"))
    assert np.array_equal(records[tag + ".move.infer"], tiled)


@pytest.mark.gpu
@pytest.mark.parametrize("tag,tol", [("f32", 1e-5), ("f64", 1e-12)])
def test_parameter_constraints_through_the_front_end(records, tag, tol):
    """DeviceLayer::set_constraints: the values as StandardParameters::set_values leaves them, the gradient as
    accumulate_grad leaves it (clip, then the two norm limits)."""
    r = {k[len(tag) + 6:]: v for k, v in records.items() if k.startswith(tag + ".cons.")}
    values = oracle.constrain(r["w"], 0.3, 0.9, 0.5)
    assert not np.array_equal(values, r["w"])                     # the limits do bite on these values
    assert hp.rel_err(r["values"], values) < tol
    raw = np.asarray(r["x"], np.float64).T @ np.asarray(r["go"], np.float64)      # dense weight gradient: x^T g
    grad = oracle.constrain(np.asfortranarray(raw.astype(r["w"].dtype)), 0.2, 0.6, 0.25)
    assert hp.rel_err(r["grad"], grad) < 10 * tol


@pytest.mark.gpu
@pytest.mark.parametrize("tag,tol", [("f32", 1e-4), ("f64", 1e-10)])
def test_device_loss_of_another_kind_negated(records, tag, tol):
    out, obj = np.asarray(records[tag + ".loss.out"], np.float64), np.asarray(records[tag + ".loss.obj"], np.float64)
    assert hp.rel_err(records[tag + ".loss.values"], oracle.loss_function("squared_hinge", out, obj, negated=True)) < tol
    assert hp.rel_err(records[tag + ".loss.grad"], oracle.loss_d_function("squared_hinge", out, obj, scale=0.5, negated=True)) < tol


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["mlp", "mlpf", "mlpg"])       # layer by layer, with DeviceFeedforwardNetwork::fuse(), and recorded as a graph
@pytest.mark.parametrize("tag,tol", [("f32", 1e-4), ("f64", 1e-9)])
def test_mlp_sgd_batches(records, tag, tol, name):
    r = {k[len(tag) + len(name) + 2:]: v for k, v in records.items() if k.startswith(tag + "." + name + ".")}
    if name != "mlp":
        assert r["groups"][0] == 1                      # dense + ReLU
    be = hn.OracleBackend(np.float64)
    net = hn.FeedforwardNet([be.dense((20,), 16), be.act("relu", (16,)), be.dense((16,), 6)])
    lr = float(np.float32(0.05)) if tag == "f32" else 0.05
    losses = _replay(r, net, lr, adam=False)
    assert hp.rel_err(r["losses"], losses) < tol
    assert losses[2] < losses[0]                                  # the steps do reduce the loss
    for li, layer in enumerate(net.layers):
        for pi, p in enumerate(layer.get_params()):
            assert hp.rel_err(r["final.%d.%d" % (li, pi)], p.get_values()) < tol, (li, pi)


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["convnet", "convnetf"])
@pytest.mark.parametrize("tag,tol", [("f32", 1e-4), ("f64", 1e-9)])
def test_convnet_adam_batches(records, tag, tol, name):
    r = {k[len(tag) + len(name) + 2:]: v for k, v in records.items() if k.startswith(tag + "." + name + ".")}
    if name == "convnetf":
        assert r["groups"][0] == 1                      # conv + ReLU + max pool
    be = hn.OracleBackend(np.float64)
    net = hn.FeedforwardNet([be.conv((8, 8, 3), 8), be.act("relu", (8, 8, 8)), be.maxpool((8, 8, 8)),
                             be.batchnorm((4, 4, 8)), be.dense((4, 4, 8), 5)])
    lr = float(np.float32(0.01)) if tag == "f32" else 0.01
    losses = _replay(r, net, lr, adam=True)
    assert hp.rel_err(r["losses"], losses) < 10 * tol             # three Adam steps deep
    for li, layer in enumerate(net.layers):
        for pi, p in enumerate(layer.get_params()):
            got, want = np.asarray(r["final.%d.%d" % (li, pi)], np.float64), p.get_values()
            # an Adam step moves every weight by about lr whatever the gradient's size, so agreement is
            # measured against the step (1 % of three steps of lr), not against the weight
            assert np.max(np.abs(got - want)) < max(10 * tol, 1e-2 * 3 * lr if tag == "f32" else 1e-7), (li, pi)
    x = np.asarray(r["x"], np.float64)
    infer = net.propagate(x, False)
    assert hp.rel_err(r["infer"], infer.reshape(r["infer"].shape, order="F")) < (1e-2 if tag == "f32" else 1e-6)


@pytest.mark.gpu
@pytest.mark.parametrize("tag,tol", [("f32", 1e-4), ("f64", 1e-10)])
def test_convlstm_sequence(records, tag, tol):
    """DeviceConvLSTM: 4 input steps, the last two hidden states as output, not foremost; against the per-layer LSTM
    on the oracle."""
    r = {k[len(tag) + 6:]: np.asarray(v, np.float64) for k, v in records.items() if k.startswith(tag + ".lstm.")}
    orc = hn.SeqConvLSTM(hn.OracleBackend(np.float64), (5, 4, 3), 6, foremost=False)
    for k, layer in enumerate(orc.kernels()):
        layer.get_params()[0].set_values(r["w%d" % k])
        layer.get_params()[1].set_values(r["b%d" % k])
    out = orc.propagate(np.asfortranarray(r["x"]), 2, 2)
    assert hp.rel_err(r["out"], out) < tol
    dx = orc.backpropagate(np.asfortranarray(r["go"]))
    assert hp.rel_err(r["dx"], dx) < tol
    for k, layer in enumerate(orc.kernels()):
        assert hp.rel_err(r["dw%d" % k], layer.get_params()[0].get_grad()) < tol, k
        assert hp.rel_err(r["db%d" % k], layer.get_params()[1].get_grad()) < tol, k
    lr = float(np.float32(0.05)) if tag == "f32" else 0.05
    assert hp.rel_err(r["w3_updated"], r["w3"] - lr * orc.kernels()[3].get_params()[0].get_grad()) < tol


@pytest.mark.gpu
@pytest.mark.parametrize("tag,dtype", [("f32", np.float32), ("f64", np.float64)])
def test_parameter_files_have_the_reference_format(records, tag, dtype):
    """save_all_unique_params_values writes what core/EigenProxy.hpp:147-159 writes (unsigned short scalar size,
    unsigned rows, unsigned cols, column-major coefficients), one file per matrix of get_params() - the per-channel
    batch norm as four 1x1 matrices per channel - and a fresh network that loads them infers bit for bit alike."""
    import struct
    r = {k[len(tag) + 9:]: v for k, v in records.items() if k.startswith(tag + ".convnet.")}
    mats = []
    i = 0
    while True:
        path = os.path.join(records["__dir__"], "%s_params_%d.prms" % (tag, i))
        if not os.path.exists(path):
            break
        raw = open(path, "rb").read()
        size, rows, cols = struct.unpack("<HII", raw[:10])
        assert size == np.dtype(dtype).itemsize and len(raw) == 10 + size * rows * cols
        mats.append(np.frombuffer(raw[10:], dtype=dtype).reshape((rows, cols), order="F"))
        i += 1
    # conv (weights, bias), 8 channels x (mean, inverse sd, gamma, beta), dense (weights, bias)
    assert [m.shape for m in mats] == [(27, 8), (1, 8)] + [(1, 1)] * 32 + [(128, 5), (1, 5)]
    assert np.array_equal(mats[0], r["final.0.0"]) and np.array_equal(mats[1], r["final.0.1"])
    for c in range(8):
        for k in range(4):
            assert mats[2 + 4 * c + k][0, 0] == r["final.3.%d" % k][0, c]
    assert np.array_equal(mats[34], r["final.4.0"]) and np.array_equal(mats[35], r["final.4.1"])
    assert np.array_equal(r["reloaded_infer"], r["infer"])


@pytest.mark.gpu
@pytest.mark.parametrize("tag,dtype", [("f32", np.float32), ("f64", np.float64)])
def test_lstm_parameter_files_follow_the_layer_order(records, tag, dtype):
    """DeviceConvLSTM::save_all_unique_params_values: sixteen files in the order of LSTMNeuralNetwork::get_layers()
    (neural_network/LSTMNeuralNetwork.hpp:521-529: input and output kernel of the forget, write, candidate and read
    gates, weights before bias), each in the binary format of core/EigenProxy.hpp:147-159; a fresh network that
    loads them gives the same output bit for bit."""
    import struct
    r = {k[len(tag) + 6:]: v for k, v in records.items() if k.startswith(tag + ".lstm.")}
    for i in range(16):
        raw = open(os.path.join(records["__dir__"], "%s_lstm_params_%d.prms" % (tag, i)), "rb").read()
        size, rows, cols = struct.unpack("<HII", raw[:10])
        assert size == np.dtype(dtype).itemsize and len(raw) == 10 + size * rows * cols
        m = np.frombuffer(raw[10:], dtype=dtype).reshape((rows, cols), order="F")
        want = r["%s%d" % ("b" if i % 2 else "w", i // 2)]
        assert m.shape == want.shape and np.array_equal(m, want), i
    assert not os.path.exists(os.path.join(records["__dir__"], "%s_lstm_params_16.prms" % tag))
    assert np.array_equal(r["out_reloaded"], r["out"])


@pytest.mark.gpu
def test_the_cpp_example_runs():
    """c-attl3_amd/examples/train_steps (built by __graft_entry__.build()): the two benchmark networks and the network of
    the reference's cifar_convnet example train from C++ and report their time per step."""
    import json
    exe = os.path.join(HERE, "..", "c-attl3_amd", "examples", "train_steps")
    if not os.path.exists(exe):
        pytest.fail("c-attl3_amd/examples/train_steps is not built: run __graft_entry__.build()")
    out = subprocess.run([exe, "3", "1"], stdout=subprocess.PIPE, check=True, timeout=120).stdout.decode()
    line = json.loads(out.strip().splitlines()[-1])
    for key in ("mlp_784_512_256_10_batch256_sgd_ms", "convnet_32x32x3_batch128_adam_ms", "reference_cifar_example_batch200_nadam_ms"):
        assert 0 < line[key] < 100

