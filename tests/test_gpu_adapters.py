"""The header-only C++ layers (c-attl3_amd/include/cattle_hip/HIPLayers.hpp) driven through the
cattle::Layer interface by tests/compat/adapter_test (built by __graft_entry__.build()); every tensor
it records is checked here against the CPU oracle. Same tolerances as the C-ABI tests."""
import os
import struct
import subprocess

import numpy as np
import pytest

import helpers as hp
from oracle import oracle

HERE = os.path.dirname(os.path.abspath(__file__))
BINARY = os.path.join(HERE, "compat", "adapter_test")
TOL = {"f32": 1e-4, "f64": 1e-10}


def _read_records(path):
    recs = {}
    with open(path, "rb") as f:
        while True:
            head = f.read(4)
            if not head:
                break
            (n,) = struct.unpack("<I", head)
            name = f.read(n).decode()
            ss, rank = struct.unpack("<II", f.read(8))
            dims = struct.unpack("<%dQ" % rank, f.read(8 * rank))
            count = int(np.prod(dims)) if rank else 1
            dt = np.uint32 if name.endswith(".inds") else {4: np.float32, 8: np.float64}[ss]
            data = np.frombuffer(f.read(ss * count), dtype=dt)
            recs[name] = data.reshape(dims, order="F")
    return recs


def test_adapters_compile_as_cpp11():
    """CPU check: the adapters are valid header-only C++11 against the interface double."""
    subprocess.check_call(["g++", "-std=c++11", "-fsyntax-only", "-Wall", "-I" + os.path.join(HERE, "compat"),
                           "-I" + os.path.join(HERE, "..", "include"),
                           "-I" + os.path.join(HERE, "..", "c-attl3_amd", "include"),
                           os.path.join(HERE, "compat", "adapter_test.cpp")])


@pytest.fixture(scope="module")
def records(tmp_path_factory):
    if not os.path.exists(BINARY):
        pytest.fail("tests/compat/adapter_test is not built: run __graft_entry__.build()")
    out = str(tmp_path_factory.mktemp("adapters") / "records.bin")
    subprocess.check_call([BINARY, out], timeout=120)
    return _read_records(out)


@pytest.mark.gpu
@pytest.mark.parametrize("tag", ["f32", "f64"])
def test_kernel_layers(records, tag):
    r = {k[len(tag) + 1:]: np.asarray(v, np.float64) for k, v in records.items() if k.startswith(tag + ".")}
    tol = TOL[tag]
    geom = dict(RH=3, RW=2, pv=1, ph=2, sv=1, sh=2, dv=1, dh=0)
    out, cache = oracle.conv_forward(r["conv.x"], r["conv.w"], r["conv.b"], return_cache=True, **geom)
    dx, dw, db = oracle.conv_backward(r["conv.x"].shape, cache, r["conv.w"], r["conv.go"], **geom)
    assert hp.rel_err(r["conv.out"], out) < tol and hp.rel_err(r["conv.dx"], dx) < tol
    assert hp.rel_err(r["conv.dw"], dw) < tol and hp.rel_err(r["conv.db"], db) < tol
    assert hp.rel_err(r["conv.dw3"], 3 * dw) < tol        # three pass_backs accumulated in the shared Parameters
    # transposed convolution (rank 3 with full backward, rank 1 forward)
    tg = dict(RH=5, RW=3, pv=1, ph=0, sv=1, sh=2, dv=0, dh=1)
    out = oracle.transconv_forward(r["trans.x"], r["trans.w"], r["trans.b"], 5, **tg)
    dx, dw, db = oracle.transconv_backward(r["trans.x"], r["trans.w"], r["trans.go"], **tg)
    assert hp.rel_err(r["trans.out"], out) < tol and hp.rel_err(r["trans.dx"], dx) < tol
    assert hp.rel_err(r["trans.dw"], dw) < tol and hp.rel_err(r["trans.db"], db) < tol
    x1 = r["trans1.x"]
    out1 = oracle.transconv_forward(x1.reshape(x1.shape + (1, 1)), r["trans1.w"], np.zeros((1, 100)), 5, RH=4, RW=1, pv=1, ph=0,
                                    sv=1, sh=1, dv=1, dh=0)
    assert hp.rel_err(r["trans1.out"], out1.reshape(r["trans1.out"].shape, order="F")) < tol
    X = r["dense.x"]
    out = oracle.dense_forward(X, r["dense.w"], r["dense.b"])
    dx, dw, db = oracle.dense_backward(X, r["dense.w"], r["dense.go"].reshape(out.shape, order="F"))
    assert hp.rel_err(r["dense.out"].reshape(out.shape, order="F"), out) < tol
    assert hp.rel_err(r["dense.dx"], dx) < tol and hp.rel_err(r["dense.dw"], dw) < tol and hp.rel_err(r["dense.db"], db) < tol
    out2 = oracle.dense_forward(X, r["dense.w2"], r["dense.b2"])          # after the host values changed
    assert hp.rel_err(r["dense.out2"].reshape(out2.shape, order="F"), out2) < tol


@pytest.mark.gpu
@pytest.mark.parametrize("tag", ["f32", "f64"])
def test_batchnorm_activations_pools(records, tag):
    r = {k[len(tag) + 1:]: v for k, v in records.items() if k.startswith(tag + ".")}
    f = lambda k: np.asarray(r[k], np.float64)
    tol = TOL[tag]
    gamma, beta = f("bn.gamma").reshape(-1), f("bn.beta").reshape(-1)
    am, ais = np.zeros(3), np.zeros(3)
    y1, std, isd = oracle.bn_forward(f("bn.x1"), gamma, beta, am, ais, False, True, decay=float(np.float32(0.2)) if tag == "f32" else 0.2)
    dx, dg, dbeta = oracle.bn_backward(f("bn.go"), gamma, std, isd)
    assert hp.rel_err(r["bn.y1"], y1) < tol and hp.rel_err(r["bn.dx1"], dx, label="adapter batchnorm dx " + tag) < tol
    assert hp.rel_err(f("bn.dgamma").reshape(-1), dg) < tol and hp.rel_err(f("bn.dbeta").reshape(-1), dbeta) < tol
    oracle.bn_forward(f("bn.x2"), gamma, beta, am, ais, True, True, decay=float(np.float32(0.2)) if tag == "f32" else 0.2)
    assert hp.rel_err(f("bn.avg_mean").reshape(-1), am) < tol and hp.rel_err(f("bn.avg_inv_sd").reshape(-1), ais) < tol
    yi, _, _ = oracle.bn_forward(f("bn.x1"), gamma, beta, am, ais, True, False)
    assert hp.rel_err(r["bn.y_infer"], yi) < tol
    x, go = f("act.x"), f("act.go")
    sc = np.float32 if tag == "f32" else np.float64
    for kind, p in (("relu", 0), ("sigmoid", 0), ("tanh", 0), ("leaky_relu", float(sc(1e-1))), ("elu", 1.0), ("swish", 1.0),
                    ("softplus", 0), ("softsign", 0), ("identity", 0), ("scaled", 1.5), ("binary_step", 0)):
        y = oracle.act_forward(kind, x, p)
        assert hp.rel_err(r["act.%s.y" % kind], y) < tol, kind
        assert hp.rel_err(r["act.%s.dx" % kind], oracle.act_backward(kind, x, y, go, p)) < tol, kind
        assert np.array_equal(r["act.%s.y_clone" % kind], r["act.%s.y" % kind])
    y = oracle.softmax_forward(x, float(sc(1e-5)))
    assert hp.rel_err(r["act.softmax.y"], y) < tol and hp.rel_err(r["act.softmax.dx"], oracle.softmax_backward(y, go)) < tol
    alpha = f("act.prelu.alpha").reshape(-1)
    assert hp.rel_err(r["act.prelu.y"], oracle.prelu_forward(x, alpha)) < tol
    pdx, pda = oracle.prelu_backward(x, alpha, go)
    assert hp.rel_err(r["act.prelu.dx"], pdx) < tol and hp.rel_err(f("act.prelu.dalpha").reshape(-1), pda) < tol
    xp = r["pool.x"]
    out, inds = oracle.maxpool_forward(xp, 3, 2, 1, 2)
    assert np.array_equal(r["pool.max.out"], out)
    assert np.array_equal(r["pool.max.inds"].reshape(inds.shape), inds)          # bit-exact argmax cache
    assert np.array_equal(r["pool.max.dx"], oracle.maxpool_backward(xp.shape, r["pool.go"], inds, 3, 2, 1, 2))
    assert hp.rel_err(r["pool.mean.out"], oracle.meanpool_forward(f("pool.x"), 3, 2, 1, 2)) < tol
    assert hp.rel_err(r["pool.mean.dx"], oracle.meanpool_backward(xp.shape, f("pool.go"), 3, 2, 1, 2)) < tol
    x1 = r["pool1.x"]
    o1, _ = oracle.maxpool_forward(x1.reshape(x1.shape + (1, 1), order="F"), 3, 1, 1, 1)
    assert np.array_equal(r["pool1.out"], o1.reshape(r["pool1.out"].shape, order="F"))


@pytest.mark.gpu
@pytest.mark.parametrize("tag", ["f32", "f64"])
def test_feedforward_stack(records, tag):
    """conv -> ReLU -> max pool -> conv -> BN -> ReLU -> max pool -> dense, first layer an input layer."""
    r = {k[len(tag) + 1:]: np.asarray(v, np.float64) for k, v in records.items() if k.startswith(tag + ".")}
    tol = TOL[tag]
    x = r["net.x"]
    N = x.shape[0]
    z = lambda n: np.zeros((1, n))
    c1, cache1 = oracle.conv_forward(x, r["net.w0"], z(4), return_cache=True)
    a1 = oracle.act_forward("relu", c1)
    p1, i1 = oracle.maxpool_forward(a1)
    c2, cache2 = oracle.conv_forward(p1, r["net.w3"], z(6), return_cache=True)
    am, ais = np.zeros(6), np.zeros(6)
    b2, std, isd = oracle.bn_forward(c2, np.ones(6), np.zeros(6), am, ais, False, True)
    a2 = oracle.act_forward("relu", b2)
    p2, i2 = oracle.maxpool_forward(a2)
    out = oracle.dense_forward(p2, r["net.w7"], z(10))
    assert hp.rel_err(r["net.out"].reshape(out.shape, order="F"), out) < tol
    g = r["net.go"].reshape(out.shape, order="F")
    g, dw7, _ = oracle.dense_backward(p2, r["net.w7"], g)
    g = oracle.maxpool_backward(a2.shape, g.reshape(p2.shape, order="F"), i2)
    g = oracle.act_backward("relu", b2, a2, g)
    g, _, _ = oracle.bn_backward(g, np.ones(6), std, isd)
    g, dw3, _ = oracle.conv_backward(p1.shape, cache2, r["net.w3"], g)
    g = oracle.maxpool_backward(a1.shape, g, i1)
    g = oracle.act_backward("relu", c1, a1, g)
    _, dw0, db0 = oracle.conv_backward(x.shape, cache1, r["net.w0"], g, input_layer=True)
    # gradients that flowed through batch norm carry its cancellation: one decade of slack
    assert hp.rel_err(r["net.dw7"], dw7) < tol
    assert hp.rel_err(r["net.dw3"], dw3) < tol
    assert hp.rel_err(r["net.dw0"], dw0) < 10 * tol and hp.rel_err(r["net.db0"], db0) < 10 * tol
    assert N == 6
